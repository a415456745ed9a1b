"""Writes tests/golden/reference_vectors.json: inputs (or the seeds that regenerate them) and the outputs
of the UNMODIFIED reference headers (oracle/_ref/libref_headers.so, built by oracle/Makefile from
/root/reference/src/{sampling_distribution,speculative_sampling,softmax}.h) for the hot path's
floating-point and draw-accounting behaviour -- the things only running the reference can pin:
fp32 bit patterns of the kept probabilities, softmax rows, and what std::mt19937 draws yield.

Run where /root/reference exists:  python tests/golden/make_reference_vectors.py
The committed JSON is what the CPU and GPU tests compare against (tests/test_golden_vectors.py); the
reference itself is not needed to run them.  Floats are stored as uint32 / uint64 bit patterns."""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import orc_lib  # noqa: E402


def tie_free(rng, v, scale):
    x = np.unique((rng.standard_normal(int(v * 1.3) + 8) * scale).astype(np.float32))
    return rng.permutation(x)[:v].copy()


def bits32(a):
    return np.asarray(a, np.float32).view(np.uint32).tolist()


def digest(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    ref = orc_lib.Reference.load()
    assert ref is not None, "build oracle/_ref first (make -C oracle)"
    out = {"sampled_categorical": [], "softmax": [], "penalties": [], "sparse_round": [], "target_selection": []}

    # ComputeSampledCategorical + SampleCategoricalToken(std::mt19937{seed})
    cases = [(70, 5, 0.0, 1.0), (300, 50, 0.9, 0.7), (5000, 40, 0.95, 0.8), (32064, 50, 0.9, 0.7), (32064, 2, 0.5, 1.3),
             (128256, 50, 0.9, 0.7), (128256, 64, 1.0, 1.0), (201088, 40, 0.6, 0.9),
             (33, 0, 0.6, 1.0), (64, 0, 0.9, 1.0), (65, 0, 0.9, 1.0), (5000, 0, 0.9, 1.0), (40000, 0, 0.95, 0.7),
             (128256, 0, 0.5, 1.0), (201088, 1, 0.9, 1.1), (3000, 0, 0.0, 1.0)]
    for n, (v, k, p, t) in enumerate(cases):
        rng = np.random.default_rng(100 + n)
        x = tie_free(rng, v, 3.0)
        if n % 3 == 0:
            x[rng.choice(v, min(8, v), replace=False)] += 10
        idx, probs = ref.sampled_categorical(x, k, p, t)
        draws = []
        for seed in (1, 2, 3, 12345):
            tok, u, used = ref.sample_categorical(idx, probs, seed)
            draws.append({"seed": seed, "u_bits": int(np.float64(u).view(np.uint64)), "consumed": int(used), "token": int(tok)})
        # long kept sets are stored as their first 64 entries plus digests of the whole arrays
        out["sampled_categorical"].append({
            "rng_seed": 100 + n, "vocab": v, "peaks": n % 3 == 0, "k": k, "p": p, "t": t, "input_sha256": digest(x),
            "kept": len(idx), "ids": [int(i) for i in idx[:64]], "prob_bits": bits32(probs[:64]),
            "ids_sha256": digest(np.asarray(idx, np.int32)), "probs_sha256": digest(np.asarray(probs, np.float32)),
            "draws": draws})

    # constant rows: the missed stop on the last element of a sort batch (lengths only; tie order is unspecified)
    out["batch_end"] = []
    for v in (32, 128, 130, 512, 2048, 8192, 32768, 131072):
        idx, probs = ref.sampled_categorical(np.full(v, 0.75, np.float32), 0, 0.5, 1.0)
        out["batch_end"].append({"vocab": v, "kept": len(idx), "prob_bits": bits32(probs[:1])})

    # Softmax / LogSoftMax rows
    for n, (v, t) in enumerate([(7, 2.0), (1000, 1.0), (32064, 0.7), (151936, 1.0)]):
        rng = np.random.default_rng(200 + n)
        x = (rng.standard_normal(v) * 2).astype(np.float32)
        sm, lsm = ref.softmax(x, t), ref.log_softmax(x, t)
        out["softmax"].append({"rng_seed": 200 + n, "vocab": v, "t": t, "input_sha256": digest(x),
                               "softmax_sha256": digest(sm), "log_softmax_sha256": digest(lsm),
                               "softmax_head_bits": bits32(sm[:8]), "log_softmax_head_bits": bits32(lsm[:8])})

    # penalties: min-length -> repetition -> n-gram (LogitsPenaltyProcessor order) on one row each
    for n, (v, pen, ngram) in enumerate([(100, 1.3, 0), (5000, 0.8, 2), (32064, 1.2, 3), (300, 1.0, 1)]):
        rng = np.random.default_rng(300 + n)
        x = (rng.standard_normal(v) * 3).astype(np.float32)
        hist = rng.integers(0, 6, 40).astype(np.int32)
        eos = [3, v - 1]
        y = ref.apply_min_length(x, 2, 5, eos)
        y = ref.apply_repetition_penalty(y, hist, pen)
        y = ref.apply_no_repeat_ngram(y, hist, ngram)
        out["penalties"].append({"rng_seed": 300 + n, "vocab": v, "penalty": pen, "ngram": ngram, "eos": eos,
                                 "input_sha256": digest(x), "history": hist.tolist(), "output_sha256": digest(y),
                                 "touched": {str(int(i)): int(np.float32(y[i]).view(np.uint32)) for i in np.nonzero(y != x)[0]}})

    # ComputeTargetTokenSelection (greedy and sampled)
    for n, greedy in enumerate([True, False, False]):
        rng = np.random.default_rng(400 + n)
        v = 32064
        x = tie_free(rng, v, 3.0)
        prefix = rng.integers(0, 8, 30 + n).astype(np.int32)
        g, idx, probs = ref.target_selection(x, len(prefix), prefix, greedy, 50, 0.9, 0.8, rep_pen=1.2, min_len=40, ngram=2, eos=[5, 7])
        out["target_selection"].append({"rng_seed": 400 + n, "vocab": v, "greedy": greedy, "prefix": prefix.tolist(),
                                        "input_sha256": digest(x), "greedy_token": int(g), "ids": [int(i) for i in idx],
                                        "prob_bits": bits32(probs)})

    # the sparse accept loop with a real engine
    rng = np.random.default_rng(500)
    for n in range(24):
        K = int(rng.integers(1, 7))
        def rows(m):
            r = []
            for _ in range(m):
                ids = rng.choice(200, int(rng.integers(1, 9)), replace=False).astype(np.int32)
                w = rng.random(ids.size).astype(np.float32) + np.float32(0.05)
                r.append((ids, (w / w.sum(dtype=np.float32)).astype(np.float32)))
            return r
        target, draft = rows(K + 1), rows(K)
        for i in range(K):
            if rng.random() < 0.6:
                draft[i] = (target[i][0].copy(), target[i][1][::-1].copy())
        proposal = np.array([d[0][rng.integers(0, len(d[0]))] for d in draft], np.int32)
        seed = int(rng.integers(0, 2 ** 31))
        acc, tok, used, au, su = ref.spec_round_sparse(proposal, target, draft, seed)
        out["sparse_round"].append({
            "seed": seed, "proposal": proposal.tolist(),
            "target": [[r[0].tolist(), bits32(r[1])] for r in target], "draft": [[r[0].tolist(), bits32(r[1])] for r in draft],
            "accept_u_bits": bits32(au), "sample_u_bits": [int(v) for v in np.asarray(su, np.float64).view(np.uint64)],
            "accepted": acc, "final_token": tok, "engine_draws": used})

    path = os.path.join(HERE, "reference_vectors.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
