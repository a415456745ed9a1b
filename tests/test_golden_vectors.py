"""The committed reference vectors (tests/golden/reference_vectors.json, produced by the unmodified
reference headers: see tests/golden/make_reference_vectors.py) against the CPU oracle (no GPU needed)
and against the HIP kernels through the C ABI (marked gpu).  Everything is compared bit for bit."""
import hashlib
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
VEC = json.load(open(os.path.join(HERE, "golden", "reference_vectors.json")))


def tie_free(rng, v, scale):
    x = np.unique((rng.standard_normal(int(v * 1.3) + 8) * scale).astype(np.float32))
    return rng.permutation(x)[:v].copy()


def digest(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def f32(bits):
    return np.asarray(bits, np.uint32).view(np.float32)


def categorical_input(c):
    rng = np.random.default_rng(c["rng_seed"])
    x = tie_free(rng, c["vocab"], 3.0)
    if c["peaks"]:
        x[rng.choice(c["vocab"], min(8, c["vocab"]), replace=False)] += 10
    assert digest(x) == c["input_sha256"], "numpy no longer regenerates the fixture's input"
    return x


def check_kept(c, ids, probs):
    ids, probs = np.asarray(ids, np.int32), np.asarray(probs, np.float32)
    assert len(ids) == c["kept"]
    assert ids[:64].tolist() == c["ids"]
    assert probs[:64].view(np.uint32).tolist() == c["prob_bits"]
    assert digest(ids) == c["ids_sha256"] and digest(probs) == c["probs_sha256"]


def canonical_u(d):
    return float(np.asarray([d["u_bits"]], np.uint64).view(np.float64)[0])


# ---- CPU: the oracle reproduces the reference's vectors -------------------------------------------------

@pytest.mark.parametrize("n", range(len(VEC["sampled_categorical"])))
def test_oracle_sampled_categorical(orc, n):
    c = VEC["sampled_categorical"][n]
    x = categorical_input(c)
    ids, probs = orc.sampled_categorical(x, c["k"], c["p"], c["t"])
    check_kept(c, ids, probs)
    for d in c["draws"]:  # the draw std::mt19937{seed} yields, and whether it was taken at all
        assert d["consumed"] == (2 if c["kept"] >= 2 else 0)
        assert ids[orc.discrete_draw(probs, canonical_u(d))] == d["token"]


def test_oracle_batch_end_rows(orc):
    for c in VEC["batch_end"]:
        ids, probs = orc.sampled_categorical(np.full(c["vocab"], 0.75, np.float32), 0, 0.5, 1.0)
        assert len(ids) == c["kept"] and probs[:1].view(np.uint32).tolist() == c["prob_bits"]


def softmax_input(c):
    x = (np.random.default_rng(c["rng_seed"]).standard_normal(c["vocab"]) * 2).astype(np.float32)
    assert digest(x) == c["input_sha256"]
    return x


@pytest.mark.parametrize("n", range(len(VEC["softmax"])))
def test_oracle_softmax(orc, n):
    c = VEC["softmax"][n]
    x = softmax_input(c)
    assert digest(orc.softmax(x, c["t"])) == c["softmax_sha256"]
    assert digest(orc.log_softmax(x, c["t"])) == c["log_softmax_sha256"]


def penalty_case(c):
    x = (np.random.default_rng(c["rng_seed"]).standard_normal(c["vocab"]) * 3).astype(np.float32)
    assert digest(x) == c["input_sha256"]
    return x, np.asarray(c["history"], np.int32)


@pytest.mark.parametrize("n", range(len(VEC["penalties"])))
def test_oracle_penalties(orc, n):
    c = VEC["penalties"][n]
    x, hist = penalty_case(c)
    y = orc.apply_no_repeat_ngram(orc.apply_repetition_penalty(orc.apply_min_length(x, 2, 5, c["eos"]), hist, c["penalty"]),
                                  hist, c["ngram"])
    assert digest(y) == c["output_sha256"]


def target_case(c):
    x = tie_free(np.random.default_rng(c["rng_seed"]), c["vocab"], 3.0)
    assert digest(x) == c["input_sha256"]
    return x, np.asarray(c["prefix"], np.int32)


@pytest.mark.parametrize("n", range(len(VEC["target_selection"])))
def test_oracle_target_selection(orc, n):
    c = VEC["target_selection"][n]
    x, prefix = target_case(c)
    g, ids, probs = orc.target_selection(x, len(prefix), prefix, c["greedy"], 50, 0.9, 0.8, rep_pen=1.2, min_len=40, ngram=2,
                                         eos=[5, 7])
    assert g == c["greedy_token"] and ids.tolist() == c["ids"] and probs.view(np.uint32).tolist() == c["prob_bits"]


def sparse_rows(rows):
    return [(np.asarray(r[0], np.int32), f32(r[1])) for r in rows]


@pytest.mark.parametrize("n", range(len(VEC["sparse_round"])))
def test_oracle_sparse_round(orc, n):
    c = VEC["sparse_round"][n]
    su = np.asarray(c["sample_u_bits"], np.uint64).view(np.float64)
    got = orc.spec_verify_sparse(c["proposal"], sparse_rows(c["target"]), sparse_rows(c["draft"]), f32(c["accept_u_bits"]), su)
    assert got == (c["accepted"], c["final_token"], c["engine_draws"])


# ---- GPU: the kernels reproduce the reference's vectors ------------------------------------------------

@pytest.fixture(scope="module")
def ctx():
    from gpu_common import pkg
    c = pkg().SearchContext(16, 201088)
    yield c
    c.close()


@pytest.mark.gpu
@pytest.mark.parametrize("n", range(len(VEC["sampled_categorical"])))
def test_gpu_sampled_categorical(ctx, n):
    import torch
    from gpu_common import say
    c = VEC["sampled_categorical"][n]
    say("golden categorical", n, c["vocab"], c["k"], c["p"], c["t"])
    x = categorical_input(c)
    rows = np.tile(x, (len(c["draws"]), 1))
    u = np.array([canonical_u(d) for d in c["draws"]])
    cap = max(64, c["kept"])
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(rows).cuda(), torch.from_numpy(u).cuda(), k=c["k"], p=c["p"],
                                 temperature=c["t"], kept_capacity=cap)
    for r, d in enumerate(c["draws"]):
        assert kc[r].item() == c["kept"]
        check_kept(c, ki[r, :c["kept"]].cpu().numpy(), kp[r, :c["kept"]].cpu().numpy())
        assert tok[r].item() == d["token"]


@pytest.mark.gpu
def test_gpu_batch_end_rows(ctx):
    import torch
    from gpu_common import say
    for c in VEC["batch_end"]:
        say("golden batch end", c["vocab"])
        x = torch.full((1, c["vocab"]), 0.75, device="cuda")
        _, kc, _, kp = ctx.sample(x, torch.zeros(1, dtype=torch.float64, device="cuda"), k=0, p=0.5, temperature=1.0,
                                  kept_capacity=8)
        assert kc[0].item() == c["kept"] and kp[0, :1].cpu().numpy().view(np.uint32).tolist() == c["prob_bits"]


@pytest.mark.gpu
@pytest.mark.parametrize("n", range(len(VEC["softmax"])))
def test_gpu_softmax(ctx, n):
    import torch
    from gpu_common import say
    c = VEC["softmax"][n]
    say("golden softmax", c["vocab"], c["t"])
    x = softmax_input(c)
    sm = ctx.softmax(torch.from_numpy(x.copy())[None].cuda(), c["t"], log=False).cpu().numpy()[0]
    lsm = ctx.softmax(torch.from_numpy(x.copy())[None].cuda(), c["t"], log=True).cpu().numpy()[0]
    assert digest(sm) == c["softmax_sha256"] and digest(lsm) == c["log_softmax_sha256"]


@pytest.mark.gpu
@pytest.mark.parametrize("n", range(len(VEC["penalties"])))
def test_gpu_penalties(ctx, n):
    import torch
    from gpu_common import pkg, say
    c = VEC["penalties"][n]
    say("golden penalties", c["vocab"], c["penalty"], c["ngram"])
    x, hist = penalty_case(c)
    xf = pkg().LogitsXform(history=torch.from_numpy(hist[None]).cuda(), repetition_penalty=c["penalty"], eos_ids=c["eos"],
                           apply_min_length=True, no_repeat_ngram_size=c["ngram"])
    y = ctx.process_logits(torch.from_numpy(x.copy())[None].cuda(), xf).cpu().numpy()[0]
    assert digest(y) == c["output_sha256"]


@pytest.mark.gpu
@pytest.mark.parametrize("n", range(len(VEC["target_selection"])))
def test_gpu_target_selection(ctx, n):
    import torch
    from gpu_common import pkg, say
    c = VEC["target_selection"][n]
    say("golden target selection", n)
    x, prefix = target_case(c)
    lens = torch.tensor([len(prefix)], dtype=torch.int32, device="cuda")
    xf = pkg().LogitsXform(history=torch.from_numpy(prefix[None]).cuda(), history_lens=lens, repetition_penalty=1.2,
                           eos_ids=[5, 7], min_length=40, no_repeat_ngram_size=2)
    row = torch.from_numpy(x)[None].cuda()
    if c["greedy"]:
        assert ctx.argmax(row, xf=xf)[0].item() == c["greedy_token"]
    else:
        _, kc, ki, kp = ctx.sample(row, torch.zeros(1, dtype=torch.float64, device="cuda"), k=50, p=0.9, temperature=0.8,
                                   xf=xf, kept_capacity=64)
        n_kept = kc[0].item()
        assert ki[0, :n_kept].cpu().numpy().tolist() == c["ids"]
        assert kp[0, :n_kept].cpu().numpy().view(np.uint32).tolist() == c["prob_bits"]


@pytest.mark.gpu
def test_gpu_sparse_rounds(ctx):
    import torch
    from gpu_common import say
    say("golden sparse rounds")
    for c in VEC["sparse_round"]:
        target, draft = sparse_rows(c["target"]), sparse_rows(c["draft"])
        K = len(c["proposal"])

        def pack(rows):
            cnt = np.zeros((1, len(rows)), np.int32)
            ids = np.zeros((1, len(rows), 8), np.int32)
            pr = np.zeros((1, len(rows), 8), np.float32)
            for r, (ix, p) in enumerate(rows):
                cnt[0, r] = len(ix)
                ids[0, r, :len(ix)] = ix
                pr[0, r, :len(ix)] = p
            return tuple(torch.from_numpy(t).cuda() for t in (cnt, ids, pr))

        su = np.asarray(c["sample_u_bits"], np.uint64).view(np.float64)
        acc, tok, used = ctx.spec_verify_sparse(pack(target), pack(draft),
                                                torch.tensor([c["proposal"]], dtype=torch.int32, device="cuda"),
                                                torch.from_numpy(f32(c["accept_u_bits"]).reshape(1, K).copy()).cuda(),
                                                torch.from_numpy(su.reshape(1, K + 1).copy()).cuda(), mode=0)
        assert (acc[0].item(), tok[0].item(), used[0].item()) == (c["accepted"], c["final_token"], c["engine_draws"])
