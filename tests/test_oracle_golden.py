"""Pins the CPU oracle (oracle/search_oracle.cpp) against the known-answer vectors held by the
reference's own tests, closed forms, textbook routines and brute force.  CPU only.

Reference tests restated here (paths under the reference tree):
  test/sampling_distribution_tests.cpp:14-40, test/speculative_sampling_tests.cpp:348-704,
  test/sampling_tests.cpp:22-49, test/cuda_batched_sampler_tests/cuda_batched_sampler_tests.cpp:63-96.
"""
import math

import numpy as np
import pytest

LOWEST = np.finfo(np.float32).min


# ---------------- penalties / mask (a3-a6) ----------------
def test_min_length_and_repetition_known_answer(orc):
    # sampling_distribution_tests.cpp:14-27
    row = np.array([4.0, -2.0, 3.0, 5.0], np.float32)
    row = orc.apply_min_length(row, 2, 5, [3])
    row = orc.apply_repetition_penalty(row, [0, 1], 2.0)
    assert row[0] == 2.0 and row[1] == -4.0 and row[2] == 3.0 and row[3] == LOWEST


def test_no_repeat_ngram_known_answer(orc):
    # sampling_distribution_tests.cpp:29-40
    row = orc.apply_no_repeat_ngram(np.arange(5, dtype=np.float32), [1, 2, 3, 4, 1, 2], 3)
    assert row[3] == LOWEST and row[4] == 4.0 and list(row[:3]) == [0.0, 1.0, 2.0]


def test_repetition_penalty_once_per_distinct_token_and_overflow(orc):
    row = np.array([8.0, LOWEST, -1.0], np.float32)
    out = orc.apply_repetition_penalty(row, [0, 0, 0, 1, 2, 7, -3], 2.0)
    assert out[0] == 4.0  # applied once although the id appears three times
    assert out[1] == -np.inf  # lowest()*2 overflows, as in the reference
    assert out[2] == -2.0
    assert np.array_equal(orc.apply_repetition_penalty(row, [0, 1], 1.0), row)  # penalty 1 is a no-op


def test_mask_padded_row_stride_v33(orc):
    # cuda_batched_sampler_tests.cpp:63-96 (bit set = allowed, two words per row for V=33)
    logits = np.ones((2, 33), np.float32)
    mask = np.array([[1 << 0, 1 << 0], [1 << 1, 1 << 0]], np.uint32)
    out = orc.apply_mask(logits, mask)
    for r in range(2):
        for t in range(33):
            assert out[r, t] == (1.0 if (t == 32 or t == r) else LOWEST)


# ---------------- argmax (a2) ----------------
def test_argmax_ties_and_nan(orc):
    assert orc.argmax([1, 5, 5, 2]) == 1  # lowest index on ties
    assert orc.argmax([np.nan, 9, 9]) == 0  # NaN at index 0 is never beaten
    assert orc.argmax([1, np.nan, 3]) == 2  # NaN elsewhere never wins
    assert orc.argmax([-np.inf, -np.inf]) == 0
    rng = np.random.default_rng(0)
    for _ in range(50):
        x = rng.integers(-3, 4, size=rng.integers(1, 200)).astype(np.float32)
        assert orc.argmax(x) == int(np.argmax(x))  # numpy's argmax is also first-maximum


def test_exact_tokens_topk1_topp(orc):
    # sampling_tests.cpp:22-49: top_k==1 resolves to greedy; expected tokens {1,2,3,4}
    logits = np.full((4, 5), 0.1, np.float32)
    for r in range(4):
        logits[r, r + 1] = 0.6
    assert list(orc.argmax_batch(logits)) == [1, 2, 3, 4]


# ---------------- sampled categorical (a7, a8) ----------------
def dense(orc, logits, k, p, t):
    idx, probs = orc.sampled_categorical(logits, k, p, t)
    out = np.zeros(len(logits), np.float32)
    out[idx] = probs
    return out


def test_sampling_dist_known_answers(orc):
    # speculative_sampling_tests.cpp:450-493
    out = dense(orc, [1, 2, 3, 4, 5], 2, 0.0, 1.0)
    assert abs(out[4] - 0.7310586) < 1e-5 and abs(out[3] - 0.2689414) < 1e-5
    assert out[0] == out[1] == out[2] == 0 and abs(out.sum() - 1) < 1e-6
    out = dense(orc, [0, 2], 5, 0.0, 2.0)
    assert abs(out[0] - 0.2689414) < 1e-5 and abs(out[1] - 0.7310586) < 1e-5
    lg = np.log(np.array([0.5, 0.3, 0.15, 0.05], np.float32))
    out = dense(orc, lg, 0, 0.6, 1.0)
    assert abs(out[0] - 0.625) < 1e-5 and abs(out[1] - 0.375) < 1e-5 and out[2] == 0 and out[3] == 0
    lg = np.log(np.array([0.5, 0.3, 0.15, 0.04, 0.01], np.float32))
    out = dense(orc, lg, 2, 0.6, 1.0)
    assert abs(out[0] - 1.0) < 1e-5 and not out[1:].any()


def test_sampling_dist_boundaries(orc):
    # speculative_sampling_tests.cpp:669-704
    out = dense(orc, [1, 5, 2, 4, 3], 1, 0.0, 1.0)  # top_k==1 -> nucleus branch with p=0 -> argmax only
    assert out[1] == 1.0 and out.sum() == 1.0
    lg = np.log(np.array([0.5, 0.3, 0.15, 0.05], np.float32))
    out = dense(orc, lg, 0, 0.01, 1.0)
    assert out[0] == 1.0 and not out[1:].any()
    a = dense(orc, [1, 2, 3], 100, 0.0, 1.0)
    b = dense(orc, [1, 2, 3], 3, 0.0, 1.0)
    assert np.allclose(a, b, atol=1e-6) and abs(a.sum() - 1) < 1e-6
    assert dense(orc, [0, 1, 2], 3, 0.0, 0.05)[2] > 0.99
    assert np.allclose(dense(orc, [0, 1, 2], 3, 0.0, 1000.0), 1 / 3, atol=0.02)


def test_topk_matches_textbook_softmax_and_bruteforce_order(orc):
    rng = np.random.default_rng(1)
    for _ in range(30):
        v = int(rng.integers(3, 400))
        k = int(rng.integers(2, v + 5))
        t = float(np.float32(rng.uniform(0.3, 2.0)))
        x = (rng.standard_normal(v) * 3).astype(np.float32)
        if rng.random() < 0.5:
            x = np.round(x)  # many ties
        idx, probs = orc.sampled_categorical(x, k, 0.0, t)
        m = min(k, v)
        order = np.lexsort((np.arange(v), -x.astype(np.float64)))[:m]  # score desc, index asc
        assert np.array_equal(idx, order)
        z = (x[order].astype(np.float64) - x[order[0]]) / t
        ref = np.exp(z) / np.exp(z).sum()
        assert np.allclose(probs, ref, rtol=1e-5, atol=1e-12)


def test_nucleus_small_vocab_exact_partition(orc):
    # V <= 64 takes the exact-partition path (sampling_distribution.h:186-203): smallest prefix whose
    # softmax mass reaches p.
    rng = np.random.default_rng(2)
    for _ in range(40):
        v = int(rng.integers(2, 65))
        p = float(rng.uniform(0.05, 0.98))
        x = (rng.standard_normal(v) * 2).astype(np.float32)
        idx, probs = orc.sampled_categorical(x, 0, p, 1.0)
        order = np.lexsort((np.arange(v), -x.astype(np.float64)))
        sm = np.exp(x[order].astype(np.float64) - x.max())
        cum = np.cumsum(sm) / sm.sum()
        want = int(np.searchsorted(cum, p - 1e-9, "left")) + 1
        assert abs(len(idx) - want) <= 1  # +-1 only where fp32 rounding sits on the boundary
        assert np.array_equal(idx, order[:len(idx)])
        assert abs(probs.sum() - 1) < 1e-5


def test_nucleus_large_vocab_tail_bound_rule(orc):
    # V > 64: cut at the first sorted position i with prefix >= p*(prefix + (V-i-1)*e_i)
    # (sampling_distribution.h:164-174), evaluated here in float64 as an independent statement.
    rng = np.random.default_rng(3)
    for _ in range(10):
        v = int(rng.integers(200, 5000))
        p = float(rng.uniform(0.5, 0.95))
        x = (rng.standard_normal(v) * 3).astype(np.float32)
        idx, probs = orc.sampled_categorical(x, 0, p, 1.0)
        order = np.lexsort((np.arange(v), -x.astype(np.float64)))
        e = np.exp(x[order].astype(np.float64) - float(x.max()))
        prefix = np.cumsum(e)
        tail = (v - np.arange(v) - 1) * e
        stop = np.nonzero(prefix >= p * (prefix + tail))[0][0] + 1
        assert abs(len(idx) - stop) <= 1
        assert np.array_equal(idx, order[:len(idx)])
        assert np.allclose(probs, e[:len(idx)] / e[:len(idx)].sum(), rtol=1e-5)


# ---------------- discrete draw (a9) ----------------
def test_discrete_draw_is_inverse_cdf(orc):
    rng = np.random.default_rng(4)
    assert orc.discrete_draw([0.3], 0.99) == 0  # single weight: always 0
    for _ in range(200):
        n = int(rng.integers(2, 60))
        w = rng.random(n).astype(np.float32)
        u = float(rng.random())
        cp = np.cumsum(w.astype(np.float64) / w.astype(np.float64).sum())
        cp[-1] = 1.0
        assert orc.discrete_draw(w, u) == int(np.searchsorted(cp, u, "left"))
    assert orc.discrete_draw([0.5, 0.5], 0.5) == 0  # lower_bound: cp[j] >= u
    assert orc.discrete_draw([0.5, 0.5], np.nextafter(0.5, 1)) == 1


# ---------------- softmax family (a11) ----------------
def test_softmax_family_against_float64(orc):
    rng = np.random.default_rng(5)
    for t in (1.0, 0.7, 2.5):
        x = (rng.standard_normal(3000) * 2).astype(np.float32)
        z = (x.astype(np.float64) - x.max()) / t
        sm = np.exp(z) / np.exp(z).sum()
        assert np.allclose(orc.softmax(x, t), sm, rtol=1e-5, atol=1e-12)
        lsm = z - math.log(np.exp(z).sum())
        assert np.allclose(orc.log_softmax(x, t), lsm, rtol=1e-5, atol=1e-5)
    assert np.allclose(orc.softmax_plain(x), orc.softmax(x, 1.0), rtol=1e-6)
    assert np.allclose(orc.log_softmax_plain(x), orc.log_softmax(x, 1.0), rtol=1e-6, atol=1e-6)
    assert abs(np.exp(orc.log_softmax(x, 1.0).astype(np.float64)).sum() - 1) < 1e-4


def test_fp16_conversion_matches_ieee_for_finite_values(orc):
    h = np.arange(0, 1 << 16, dtype=np.uint32).astype(np.uint16)
    got = orc.fp16_to_fp32(h)
    want = h.view(np.float16).astype(np.float32)
    finite = np.isfinite(want)
    assert np.array_equal(got[finite].view(np.uint32), want[finite].view(np.uint32))
    # Inf/NaN encodings (exponent 31) come out as finite values 65536*(1+m/1024), a reference quirk.
    assert got[0x7C00] == 65536.0 and got[0xFC00] == -65536.0


# ---------------- beam top-2B (a12) ----------------
def test_beam_select_top_bruteforce(orc):
    rng = np.random.default_rng(6)
    for _ in range(20):
        batch, beams, vocab = int(rng.integers(1, 4)), int(rng.integers(2, 5)), int(rng.integers(3, 60))
        x = (rng.standard_normal((batch * beams, vocab)) * 2).astype(np.float32)
        if rng.random() < 0.5:
            x = np.round(x * 2) / 2
        bs = (rng.standard_normal(batch * beams)).astype(np.float32)
        sc, tok, idx, full = orc.beam_select_top(x, batch, beams, bs)
        # independent statement of the scores
        ls = np.stack([orc.log_softmax(r, 1.0) for r in x]) + bs[:, None]
        assert np.array_equal(full.view(np.uint32), ls.astype(np.float32).view(np.uint32))
        flat = full.reshape(batch, beams * vocab)
        for b in range(batch):
            order = np.lexsort((np.arange(beams * vocab), -flat[b].astype(np.float64)))[:2 * beams]
            assert np.array_equal(idx[b], order // vocab)
            assert np.array_equal(tok[b], order % vocab)
            assert np.array_equal(sc[b], flat[b][order])


# ---------------- KV gather (a15) ----------------
def test_kv_gather_is_take(orc):
    rng = np.random.default_rng(7)
    present = rng.integers(0, 1 << 16, size=(6, 2, 5, 8)).astype(np.uint16)
    idx = np.array([3, 3, 0, 5, 1, 1], np.int32)
    assert np.array_equal(orc.kv_gather(present, idx), np.take(present, idx, axis=0))


# ---------------- speculative math (a16-a18) ----------------
def test_accept_prob_known_answers(orc):
    # speculative_sampling_tests.cpp:348-368
    assert orc.accept_prob(0.8, 0.4) == 1.0 and orc.accept_prob(0.5, 0.5) == 1.0
    assert orc.accept_prob(0.2, 0.4) == np.float32(0.5) and orc.accept_prob(0.1, 1.0) == np.float32(0.1)
    assert orc.accept_prob(0.0, 0.5) == 0.0 and orc.accept_prob(0.5, 0.0) == 1.0


def test_correction_distribution_known_answers(orc):
    # speculative_sampling_tests.cpp:372-415
    out = orc.build_correction([0.1, 0.5, 0.2, 0.2], [0.3, 0.2, 0.3, 0.2])
    assert list(out) == [0.0, 1.0, 0.0, 0.0]
    out = orc.build_correction([0.4, 0.1, 0.3, 0.1, 0.1], [0.1, 0.3, 0.1, 0.4, 0.1])
    assert abs(out.sum() - 1) < 1e-6 and out[1] == out[3] == out[4] == 0
    out = orc.build_correction([0.5, 0.3, 0.2], [0.5, 0.3, 0.2])
    assert np.array_equal(out, np.array([0.5, 0.3, 0.2], np.float32))


def test_sparse_correction_only_positive_residual(orc):
    # speculative_sampling_tests.cpp:425-437
    for u in np.linspace(0.001, 0.999, 20):
        assert orc.sample_correction([1, 4, 8], [0.2, 0.5, 0.3], [1, 8], [0.4, 0.6], float(u)) == 4


def test_target_selection_known_answers(orc):
    # speculative_sampling_tests.cpp:497-554
    g, idx, probs = orc.target_selection([1, 2, 8, 3], 4, [], True, 0, 0.0, 1.0, min_len=5, eos=[2])
    assert g == 3 and len(idx) == 0
    g, idx, probs = orc.target_selection([6, 5, 4, 1], 1, [0], False, 2, 0.0, 1.0, rep_pen=2.0, eos=[3])
    assert g == -1 and list(idx) == [1, 2] and probs[0] > probs[1]
    g, idx, probs = orc.target_selection([1, 4, 3, 2], 0, [], False, 2, 0.0, 1.0, eos=[3])
    assert list(idx) == [1, 2] and abs(probs.sum() - 1) < 1e-6


def test_verify_deterministic_known_answers(orc):
    # speculative_sampling_tests.cpp:556-660 (single-entry distributions consume no draw)
    r = orc.verify_deterministic([7], [([7], [1.0]), ([9], [1.0])], [])
    assert r == dict(accepted=1, evaluated=1, final_token=9, used_bonus=True, draws_used=0)
    r = orc.verify_deterministic([7], [([5], [1.0]), ([9], [1.0])], [])
    assert (r["accepted"], r["evaluated"], r["final_token"], r["used_bonus"]) == (0, 1, 5, False)
    r = orc.verify_deterministic([1, 9], [([1], [1.0]), ([2], [1.0]), ([3], [1.0])], [])
    assert (r["accepted"], r["evaluated"], r["final_token"], r["used_bonus"]) == (1, 2, 2, False)
    sels = [([1, 2], [0.4, 0.6]), ([3, 4], [0.3, 0.7]), ([5, 6], [0.2, 0.8])]
    r = orc.verify_deterministic([99, 4], sels, [0.9, 0.9, 0.9])
    assert r["evaluated"] == 1 and not r["used_bonus"] and r["draws_used"] == 1  # stops drawing after mismatch


def test_spec_verify_dense_statistics_match_target(orc):
    # speculative_sampling_tests.cpp:749-878: accept/correct must reproduce the target distribution.
    rng = np.random.default_rng(8)
    v, n = 6, 40000
    p = rng.random(v).astype(np.float32)
    p /= p.sum()
    q = rng.random(v).astype(np.float32)
    q /= q.sum()
    pt = np.broadcast_to(p, (n, 2, v)).copy()
    qd = np.broadcast_to(q, (n, 2, v)).copy()
    draft = rng.choice(v, size=(n, 1), p=q.astype(np.float64) / q.astype(np.float64).sum()).astype(np.int32)
    acc, tok = orc.spec_verify_dense(pt, qd, draft, rng.random((n, 1)).astype(np.float32), rng.random(n))
    first = np.where(acc == 1, draft[:, 0], tok)  # the first committed token
    freq = np.bincount(first, minlength=v) / n
    assert np.abs(freq - p).max() < 0.015


def test_cast_known_answers(orc):
    """DeviceInterface::Cast on the CPU (src/cpu/interface.cpp:74-106).  fp32->fp16 is
    FastFloat32ToFloat16: it equals IEEE round-to-nearest for values that are not exact ties (numpy
    agrees there), rounds ties up, keeps -0, and saturates beyond the fp16 range to 0x7FFF.  bf16->fp32
    moves the bits up and canonicalises NaN; fp32->bf16 truncates; int32->int64 sign-extends."""
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(20000) * 50).astype(np.float32)
    x = x[(np.abs(x) > 1e-3) & ((x.view(np.uint32) & 0x1FFF) != 0x1000)]  # no exact ties
    got = orc.cast(x, 2, np.uint16)
    ieee = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, ieee)
    assert list(orc.cast(np.array([0.0, -0.0, 1.0, -2.0, 65504.0, 1e6, -1e6], np.float32), 2, np.uint16)) == \
        [0x0000, 0x8000, 0x3C00, 0xC000, 0x7BFF, 0x7FFF, 0xFFFF]
    tie = np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11], np.float32)  # halfway between fp16 neighbours
    assert list(orc.cast(tie, 2, np.uint16)) == [0x3C01, 0x3C02]  # up, where IEEE would give 0x3C00, 0x3C02
    b = np.array([0x3F80, 0xC000, 0x0001, 0x7F80, 0xFF80, 0x7FC1, 0xFFFF, 0x0000, 0x8000], np.uint16)
    f = orc.cast(b, 1, np.float32).view(np.uint32)
    assert list(f) == [0x3F800000, 0xC0000000, 0x00010000, 0x7F800000, 0xFF800000, 0x7FC00000, 0x7FC00000, 0, 0x80000000]
    assert list(orc.cast(np.array([1.0, -1.5, 3.14159], np.float32), 3, np.uint16)) == [0x3F80, 0xBFC0, 0x4049]
    assert list(orc.cast(np.array([-1, 2 ** 31 - 1, -2 ** 31], np.int32), 4, np.int64)) == [-1, 2 ** 31 - 1, -2 ** 31]
    h = np.arange(65536, dtype=np.uint16)
    assert np.array_equal(orc.cast(h, 0, np.float32), orc.fp16_to_fp32(h))
