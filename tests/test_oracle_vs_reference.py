"""Validates the CPU oracle against the UNMODIFIED reference headers (oracle/_ref, built from
/root/reference where it is present).  Bit-exact on continuous random inputs (no ties, so
std::partial_sort's unspecified tie order cannot matter).  CPU only."""
import numpy as np
import pytest


def bits(a):
    return np.asarray(a, np.float32).view(np.uint32)


def tie_free(rng, v, scale):
    """v distinct float32 values ~ N(0, scale^2) in random order."""
    x = np.unique((rng.standard_normal(int(v * 1.3) + 8) * scale).astype(np.float32))
    assert x.size >= v
    return rng.permutation(x)[:v].copy()


def test_sampled_categorical_topk_bit_exact(orc, ref):
    rng = np.random.default_rng(10)
    for _ in range(40):
        v = int(rng.integers(70, 3000))
        x = tie_free(rng, v, 3)
        k = int(rng.integers(2, 80))
        p = float(rng.choice([0.0, 0.5, 0.9, 0.99, 1.0]))
        t = float(rng.choice([0.7, 1.0, 1.3]))
        i1, p1 = orc.sampled_categorical(x, k, p, t)
        i2, p2 = ref.sampled_categorical(x, k, p, t)
        assert np.array_equal(i1, i2) and np.array_equal(bits(p1), bits(p2))


def test_sampled_categorical_nucleus_bit_exact(orc, ref):
    rng = np.random.default_rng(11)
    for v in (5, 33, 64, 65, 300, 5000, 40000):
        for p in (0.05, 0.6, 0.9, 0.95):
            x = tie_free(rng, v, 3)
            i1, p1 = orc.sampled_categorical(x, 0, p, 1.0)
            i2, p2 = ref.sampled_categorical(x, 0, p, 1.0)
            assert np.array_equal(i1, i2) and np.array_equal(bits(p1), bits(p2))


def test_nucleus_stop_on_last_element_of_a_sort_batch(orc, ref):
    """A constant row of V logits with p = 0.5 satisfies the tail-bound stop first at element V/2.  When
    V/2 is the end of a sort batch (16, 64, 256, ... elements) the reference does not notice the stop until
    the next batch, so V/2 + 1 elements are kept; otherwise V/2.  Rows of at most 64 logits take the
    exact-partition override and keep V/2.  Only lengths and probabilities are compared: the order of
    tied ids under std::partial_sort is unspecified."""
    for v, want in ((32, 16), (128, 65), (512, 257), (2048, 1025), (8192, 4097), (32768, 16385), (131072, 65537),
                    (130, 65), (1000, 500), (2046, 1023)):
        x = np.full(v, 0.75, np.float32)
        i1, p1 = orc.sampled_categorical(x, 0, 0.5, 1.0)
        i2, p2 = ref.sampled_categorical(x, 0, 0.5, 1.0)
        assert len(i1) == len(i2) == want, (v, len(i1), len(i2))
        assert np.array_equal(bits(p1), bits(p2))
        assert np.array_equal(i1, np.arange(want))  # the oracle's tie rule: lowest index first


def test_config_shaped_rows_bit_exact(orc, ref):
    rng = np.random.default_rng(12)
    # C2-like: V=128256, 8 peaks at +10, T=0.7, k=50, p=0.9
    x = tie_free(rng, 128256, 3)
    x[rng.choice(128256, 8, replace=False)] += 10
    i1, p1 = orc.sampled_categorical(x, 50, 0.9, 0.7)
    i2, p2 = ref.sampled_categorical(x, 50, 0.9, 0.7)
    assert np.array_equal(i1, i2) and np.array_equal(bits(p1), bits(p2))
    # C5-like: V=201088, 5 % allowed, penalty 1.2 over 1024 ids, p=0.95
    v = 201088
    x = tie_free(rng, v, 3)
    allowed = rng.random(v) < 0.05
    x[~allowed] = np.finfo(np.float32).min
    hist = rng.integers(0, v, 1024).astype(np.int32)
    x1 = orc.apply_repetition_penalty(x, hist, 1.2)
    x2 = ref.apply_repetition_penalty(x, hist, 1.2)
    assert np.array_equal(bits(x1), bits(x2)) and np.isinf(x1).any()
    # ties among the masked lowest()/-inf entries lie beyond the nucleus, so the kept set is tie-free
    i1, p1 = orc.sampled_categorical(x1, 0, 0.95, 1.0)
    i2, p2 = ref.sampled_categorical(x2, 0, 0.95, 1.0)
    assert len(i1) > 1000
    assert np.array_equal(i1, i2) and np.array_equal(bits(p1), bits(p2))


def test_discrete_draw_protocol_matches_mt19937(orc, ref):
    # The explicit-u draw equals std::discrete_distribution under mt19937 when u is the canonical
    # double the engine would produce; a one-entry distribution consumes no draw.
    rng = np.random.default_rng(13)
    for seed in range(300):
        n = int(rng.integers(1, 40))
        idx = rng.permutation(1000)[:n].astype(np.int32)
        probs = rng.random(n).astype(np.float32)
        tok, u, draws = ref.sample_categorical(idx, probs, seed)
        assert draws == (0 if n < 2 else 2)
        assert tok == idx[orc.discrete_draw(probs, u)]
    for seed in range(50):
        assert ref.lib.ref_uniform_float(seed) >= 0  # float uniform = float(x)/2^32 as documented


def test_softmax_family_bit_exact(orc, ref):
    rng = np.random.default_rng(14)
    for n in (7, 1000, 151936):
        x = (rng.standard_normal(n) * 2).astype(np.float32)
        for t in (1.0, 0.7):
            assert np.array_equal(bits(orc.softmax(x, t)), bits(ref.softmax(x, t)))
            assert np.array_equal(bits(orc.log_softmax(x, t)), bits(ref.log_softmax(x, t)))


def test_penalties_bit_exact(orc, ref):
    rng = np.random.default_rng(15)
    for _ in range(30):
        v = int(rng.integers(4, 500))
        x = (rng.standard_normal(v) * 3).astype(np.float32)
        hist = rng.integers(-2, v + 2, int(rng.integers(0, 60))).astype(np.int32)
        pen = float(rng.choice([1.0, 1.1, 2.0, 0.5]))
        assert np.array_equal(bits(orc.apply_repetition_penalty(x, hist, pen)),
                              bits(ref.apply_repetition_penalty(x, hist, pen)))
        eos = rng.integers(-1, v + 1, 2).astype(np.int32)
        assert np.array_equal(bits(orc.apply_min_length(x, 3, 5, eos)), bits(ref.apply_min_length(x, 3, 5, eos)))
        assert np.array_equal(bits(orc.apply_min_length(x, 5, 5, eos)), bits(ref.apply_min_length(x, 5, 5, eos)))
        small = rng.integers(0, 4, int(rng.integers(0, 30))).astype(np.int32)
        for ng in (0, 1, 2, 3):
            assert np.array_equal(bits(orc.apply_no_repeat_ngram(x, small, ng)),
                                  bits(ref.apply_no_repeat_ngram(x, small, ng)))


def test_speculative_math_bit_exact(orc, ref):
    rng = np.random.default_rng(16)
    for _ in range(200):
        a, b = np.float32(rng.random()), np.float32(rng.random() * rng.choice([0, 1]))
        assert orc.accept_prob(a, b) == ref.accept_prob(a, b)
    for _ in range(30):
        n = int(rng.integers(2, 200))
        p = rng.random(n).astype(np.float32)
        q = rng.random(n).astype(np.float32)
        assert np.array_equal(bits(orc.build_correction(p, q)), bits(ref.build_correction(p, q)))
    for seed in range(100):
        nt, nd = int(rng.integers(1, 20)), int(rng.integers(1, 20))
        ti = rng.permutation(40)[:nt].astype(np.int32)
        di = rng.permutation(40)[:nd].astype(np.int32)
        tp = rng.random(nt).astype(np.float32)
        dp = rng.random(nd).astype(np.float32)
        tok, u = ref.sample_correction(ti, tp, di, dp, seed)
        assert tok == orc.sample_correction(ti, tp, di, dp, u)


def test_target_selection_bit_exact(orc, ref):
    rng = np.random.default_rng(17)
    for _ in range(40):
        v = int(rng.integers(70, 800))
        x = (rng.standard_normal(v) * 3).astype(np.float32)
        prefix = rng.integers(0, v, int(rng.integers(0, 40))).astype(np.int32)
        kw = dict(rep_pen=float(rng.choice([1.0, 1.3])), min_len=int(rng.choice([0, 100])),
                  ngram=int(rng.choice([0, 2])), eos=[int(rng.integers(0, v))])
        greedy = bool(rng.random() < 0.3)
        k, p = int(rng.choice([0, 5, 40])), float(rng.choice([0.0, 0.8]))
        if not greedy and k <= 1 and p == 0.0:
            p = 0.8
        a = orc.target_selection(x, len(prefix), prefix, greedy, k, p, 0.9, **kw)
        b = ref.target_selection(x, len(prefix), prefix, greedy, k, p, 0.9, **kw)
        assert a[0] == b[0] and np.array_equal(a[1], b[1]) and np.array_equal(bits(a[2]), bits(b[2]))


def test_verify_deterministic_matches_reference(orc, ref):
    rng = np.random.default_rng(18)
    for seed in range(150):
        n = int(rng.integers(1, 5))
        sels = []
        for _ in range(n + 1):
            m = int(rng.integers(1, 4))
            sels.append((rng.permutation(6)[:m].astype(np.int32), rng.random(m).astype(np.float32)))
        proposal = rng.integers(0, 6, n).astype(np.int32)
        r = ref.verify_deterministic(proposal, sels, seed)
        o = orc.verify_deterministic(proposal, sels, list(r["draws"]) + [0.5] * 4)
        for key in ("accepted", "evaluated", "final_token", "used_bonus"):
            assert o[key] == r[key], (seed, key)
        assert o["draws_used"] == len(r["draws"])


def random_sparse_round(rng, vocab, K, orc):
    """K+1 target rows and K draft rows as kept sets of random logits, plus proposal tokens drawn from the
    draft rows (sometimes replaced by ids the target does not hold)."""
    def rows(n, scale):
        out = []
        for _ in range(n):
            x = (rng.standard_normal(vocab) * scale).astype(np.float32)
            k = int(rng.choice([1, 2, 5, 50]))
            p = float(rng.choice([0.0, 0.6, 0.95]))
            out.append(orc.sampled_categorical(x, k, p, float(rng.choice([0.7, 1.0]))))
        return out
    target = rows(K + 1, 2.0)
    draft = rows(K, 2.0)
    for i in range(K):  # correlate drafts with targets so that accepts and rejects both occur
        if rng.random() < 0.6:
            draft[i] = (target[i][0].copy(), target[i][1].copy())
            if len(draft[i][0]) > 2 and rng.random() < 0.5:
                draft[i] = (draft[i][0][::-1].copy(), draft[i][1].copy())  # same ids, different probabilities
    proposal = np.array([d[0][rng.integers(0, len(d[0]))] for d in draft], np.int32)
    for i in range(K):
        if rng.random() < 0.1:
            proposal[i] = rng.integers(0, vocab)
    return proposal, target, draft


def test_sparse_accept_loop_matches_reference_with_real_engine(orc, ref):
    """orc_spec_verify_sparse (explicit uniforms) against the reference's ComputeAcceptProb /
    SampleCorrectionToken / SampleSparseToken driven by std::mt19937: accepted length, final token and the
    number of engine outputs consumed (one per evaluated position, two for a categorical draw over at least
    two entries)."""
    rng = np.random.default_rng(21)
    outcomes = set()
    for case in range(300):
        K = int(rng.integers(1, 9))
        vocab = int(rng.choice([3, 60, 500]))
        proposal, target, draft = random_sparse_round(rng, vocab, K, orc)
        seed = int(rng.integers(0, 2 ** 31))
        acc2, tok2, used2, au, su = ref.spec_round_sparse(proposal, target, draft, seed)
        acc1, tok1, used1 = orc.spec_verify_sparse(proposal, target, draft, au, su)
        assert (acc1, tok1, used1) == (acc2, tok2, used2), case
        outcomes.add((acc1 == K, used1 - min(acc1 + 1, K)))
    assert outcomes == {(True, 0), (True, 2), (False, 0), (False, 2)}  # bonus / correction, with and without a draw


def test_dense_accept_loop_matches_reference_with_real_engine(orc, ref):
    """orc_spec_verify_dense as a loop against the reference: selections that list the whole vocabulary (ids
    0 .. V-1) make the reference's accept loop -- its own ComputeAcceptProb, SampleCorrectionToken and
    SampleSparseToken with a real std::mt19937 -- work on dense distributions; the dense oracle gets the same
    uniforms in its explicit form (the categorical draw is the one the engine yields after the accept draws the
    round has taken).  Accepted length and final token agree on rounds that accept everything, reject early and
    reject late."""
    rng = np.random.default_rng(22)
    outcomes = set()
    for case in range(200):
        K = int(rng.integers(1, 9))
        vocab = int(rng.choice([2, 17, 300]))
        ids = np.arange(vocab, dtype=np.int32)
        sharp = float(rng.choice([0.3, 1.0, 3.0]))
        p = np.stack([orc.softmax((rng.standard_normal(vocab) * sharp).astype(np.float32), 1.0) for _ in range(K + 1)])
        q = np.stack([orc.softmax((rng.standard_normal(vocab) * sharp).astype(np.float32), 1.0) for _ in range(K + 1)])
        if case % 3 == 0:
            q[:K] = p[:K]  # identical distributions: every proposal is accepted, and a correction would find no residual
        if case % 7 == 0:
            q[0] = 0.0
            q[0, 0] = 1.0  # a draft certain of one token the target hardly wants
        proposal = np.array([rng.choice(vocab, p=q[i].astype(np.float64) / q[i].astype(np.float64).sum())
                             for i in range(K)], np.int32)
        target = [(ids, p[i]) for i in range(K + 1)]
        draft = [(ids, q[i]) for i in range(K)]
        seed = int(rng.integers(0, 2 ** 31))
        acc2, tok2, used2, au, su = ref.spec_round_sparse(proposal, target, draft, seed)
        evaluated = min(acc2 + 1, K)
        acc1, tok1 = orc.spec_verify_dense(p[None], q[None], proposal[None], np.asarray(au, np.float32)[None, :K],
                                           np.array([su[evaluated]]))
        assert (int(acc1[0]), int(tok1[0])) == (acc2, tok2), case
        outcomes.add((acc2 == K, acc2 == 0))
    assert outcomes >= {(True, False), (False, True), (False, False)}
