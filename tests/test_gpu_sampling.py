"""GPU parity: argmax, logits processing and top-k / top-p sampling through the C ABI against the CPU
oracle on the same seeded inputs.  Bit-exact token ids and indices; probabilities compared bitwise
too (tolerance stated by the task: 1e-5 relative -- the kernels meet it with zero difference)."""
import os

import numpy as np
import pytest
import torch

from gpu_common import LOWEST, make_mask, pkg, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = pkg().SearchContext(256, 201088)
    yield c
    c.close()


def bits(a):
    return np.asarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("rows,vocab", [(1, 32064), (3, 33), (4, 8192), (2, 8193), (5, 50257), (64, 128256), (3, 201088)])
def test_argmax_matches_oracle(ctx, orc, rows, vocab):
    say("argmax", rows, vocab)
    rng = np.random.default_rng(rows * 1000 + vocab)
    x = (rng.standard_normal((rows, vocab)) * 2).astype(np.float32)
    x[0] = np.round(x[0])  # ties
    got = ctx.argmax(torch.from_numpy(x).cuda()).cpu().numpy()
    assert np.array_equal(got, orc.argmax_batch(x))


def test_argmax_special_values(ctx, orc):
    say("argmax special")
    x = np.zeros((6, 1000), np.float32)
    x[0, :] = -np.inf
    x[1, 0] = np.nan
    x[1, 5] = 7
    x[2, 3] = np.nan
    x[2, 9] = 1
    x[3, 10] = -0.0
    x[3, :] *= -1  # all -0/+0
    x[4, :] = LOWEST
    x[5, 999] = np.inf
    got = ctx.argmax(torch.from_numpy(x).cuda()).cpu().numpy()
    assert np.array_equal(got, orc.argmax_batch(x))


@pytest.mark.parametrize("vocab", [40000, 131072, 201088])
def test_argmax_special_values_across_chunks(ctx, orc, vocab):
    """Rows of several 32768-id chunks: equal maxima in different chunks (the lowest id wins), a maximum in the last
    partial chunk, NaN at id 0 (wins outright), NaN elsewhere (never wins), rows without a finite value."""
    say("argmax special, chunks", vocab)
    rng = np.random.default_rng(vocab)
    x = (rng.standard_normal((10, vocab)) * 2).astype(np.float32)
    x[0, [vocab - 1, 33000, 5]] = 50.0
    x[1, [vocab - 1, 33000]] = 50.0
    x[2, vocab - 1] = 50.0
    x[3, 0] = np.nan
    x[3, 35000] = 60.0
    x[4, 35000] = np.nan
    x[4, 36000] = np.nan
    x[5, :] = -np.inf
    x[6, :] = np.nan
    x[7, :] = -np.inf
    x[7, 39999] = LOWEST
    x[8, :] = 3.0
    x[9, :] = np.nan
    x[9, 0] = 1.0
    x[9, 39000] = 1.0
    want = orc.argmax_batch(x)
    assert np.array_equal(ctx.argmax(torch.from_numpy(x).cuda()).cpu().numpy(), want)
    xf = pkg().LogitsXform(history=torch.from_numpy(np.tile(np.array([[5, 33000, 35000, 0]], np.int32), (10, 1))).cuda(),
                           repetition_penalty=1.3)
    proc = np.stack([orc.apply_repetition_penalty(x[r], np.array([5, 33000, 35000, 0], np.int32), 1.3) for r in range(10)])
    assert np.array_equal(ctx.argmax(torch.from_numpy(x).cuda(), xf=xf).cpu().numpy(), orc.argmax_batch(proc))
    with np.errstate(over="ignore"):  # lowest() becomes -inf in fp16
        h = x.astype(np.float16)
    assert np.array_equal(ctx.argmax(torch.from_numpy(h).cuda()).cpu().numpy(), orc.argmax_batch(orc.fp16_to_fp32(h)))


def test_argmax_of_rows_longer_than_the_chunked_path_holds(orc):
    """More than 16 chunks per row (vocabulary above 524288): the exact path answers; exactly 16: the chunked one."""
    say("argmax very long rows")
    rng = np.random.default_rng(77)
    for vocab in (524288, 524289 + 4096):
        ctx = pkg().SearchContext(2, vocab)
        x = (rng.standard_normal((2, vocab)) * 2).astype(np.float32)
        x[1, vocab - 1] = 40.0
        assert np.array_equal(ctx.argmax(torch.from_numpy(x).cuda()).cpu().numpy(), orc.argmax_batch(x))
        ctx.close()


def test_argmax_fp16(ctx, orc):
    say("argmax fp16")
    rng = np.random.default_rng(5)
    h = (rng.standard_normal((7, 151936)) * 2).astype(np.float16)
    got = ctx.argmax(torch.from_numpy(h).cuda()).cpu().numpy()
    assert np.array_equal(got, orc.argmax_batch(orc.fp16_to_fp32(h)))


def test_config1_greedy_with_repetition_penalty(ctx, orc):
    """Benchmark configuration 1: batch 1, vocab 32064, N(0,2^2) logits with a +8 spike, repetition penalty
    1.1 over 512 history ids, greedy argmax per step (16 of the 256 steps here)."""
    rng = np.random.default_rng(1)
    vocab = 32064
    for step in range(16):
        say("config1 step", step)
        x = (rng.standard_normal((1, vocab)) * 2).astype(np.float32)
        x[0, rng.integers(0, vocab)] += 8
        hist = rng.integers(0, vocab, (1, 512)).astype(np.int32)
        xf = pkg().LogitsXform(history=torch.from_numpy(hist).cuda(), repetition_penalty=1.1)
        got = ctx.argmax(torch.from_numpy(x).cuda(), xf=xf).cpu().numpy()
        want = orc.argmax(orc.apply_repetition_penalty(x[0], hist[0], 1.1))
        assert got[0] == want


@pytest.mark.parametrize("rows,vocab,dtype", [(2, 5000, np.float32), (3, 40000, np.float16), (40, 70001, np.float32),
                                              (33, 128256, np.float16)])
def test_argmax_with_fused_logits_processing(ctx, orc, rows, vocab, dtype):
    """Greedy selection with grammar mask, min-length and repetition penalty fused, on the
    single-workgroup-per-row kernel (small shapes) and the chunked kernel (large shapes)."""
    say("argmax fused", rows, vocab, dtype.__name__)
    rng = np.random.default_rng(rows + vocab)
    x = (rng.standard_normal((rows, vocab)) * 2).astype(dtype)
    x32 = orc.fp16_to_fp32(x) if dtype == np.float16 else x
    mask = make_mask(rng, rows, vocab, 0.5)
    hist = rng.integers(-2, vocab + 2, (rows, 300)).astype(np.int32)
    top = np.argmax(x32, axis=1)
    hist[:, 0] = top  # the raw maximum is penalised
    eos = [int(np.argsort(x32[0])[-2]), vocab - 1]
    xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(), history=torch.from_numpy(hist).cuda(),
                           repetition_penalty=1.7, eos_ids=eos, apply_min_length=True)
    got = ctx.argmax(torch.from_numpy(x).cuda(), xf=xf).cpu().numpy()
    proc = orc.apply_mask(x32, mask)
    for r in range(rows):
        row = orc.apply_min_length(proc[r], 0, 1, eos)
        row = orc.apply_repetition_penalty(row, hist[r], 1.7)
        assert got[r] == orc.argmax(row), r


@pytest.mark.parametrize("vocab", [33, 1000, 8192, 40000])
def test_process_logits_in_place(ctx, orc, vocab):
    say("process_logits", vocab)
    rng = np.random.default_rng(vocab)
    rows = 3
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    mask = make_mask(rng, rows, vocab, 0.3)
    hist = rng.integers(-2, vocab + 2, (rows, 100)).astype(np.int32)
    eos = [1, vocab - 1, vocab + 5]
    xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(), history=torch.from_numpy(hist).cuda(),
                           history_len=77, repetition_penalty=1.3, eos_ids=eos, apply_min_length=True)
    got = ctx.process_logits(torch.from_numpy(x).cuda(), xf).cpu().numpy()
    want = orc.apply_mask(x, mask)
    for r in range(rows):
        want[r] = orc.apply_min_length(want[r], 0, 1, eos)
        want[r] = orc.apply_repetition_penalty(want[r], hist[r, :77], 1.3)
    assert np.array_equal(bits(got), bits(want))
    assert np.isinf(got).any() or vocab < 100  # lowest()*1.3 overflows to -inf, as in the reference


def sample_and_check(ctx, orc, x, u, k, p, t, cap=64):
    rows = x.shape[0]
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=k, p=p, temperature=t,
                                 kept_capacity=cap)
    tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    for r in range(rows):
        idx, probs = orc.sampled_categorical(x[r], k, p, t)
        assert kc[r] == len(idx), (r, kc[r], len(idx))
        n = min(len(idx), cap)
        assert np.array_equal(ki[r, :n], idx[:n]), r
        assert np.array_equal(bits(kp[r, :n]), bits(probs[:n])), r
        assert tok[r] == idx[orc.discrete_draw(probs, u[r])], r


@pytest.mark.parametrize("rows,vocab,k,p,t", [
    (4, 4099, 50, 0.9, 0.7), (3, 8192, 2, 0.0, 1.0), (2, 20000, 64, 0.5, 1.3), (5, 128256, 50, 0.9, 0.7),
    (2, 128256, 50, 1.0, 1.0), (3, 201088, 40, 0.95, 0.8), (2, 65, 64, 0.9, 1.0), (2, 300, 50, 0.9, 1.0),
])
def test_sample_topk_topp_small_k(ctx, orc, rows, vocab, k, p, t):
    say("sample topk", rows, vocab, k, p, t)
    rng = np.random.default_rng(vocab + k)
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    u = rng.random(rows)
    before = ctx.fallback_rows()
    sample_and_check(ctx, orc, x, u, k, p, t)
    assert ctx.fallback_rows() == before  # all rows stayed on the single-pass path


@pytest.mark.parametrize("vocab,k,p,t", [(128256, 50, 0.9, 0.7), (5000, 30, 0.0, 1.0), (201088, 0, 0.9, 1.0)])
def test_draw_on_cdf_boundaries(ctx, orc, vocab, k, p, t):
    """Uniform draws placed exactly on, just below and just above values of the cumulative distribution
    std::discrete_distribution builds (double quotients summed in sequence): the kernels' tree-order
    CDF cannot decide these and must fall back to the sequential construction."""
    say("cdf boundaries", vocab, k, p, t)
    rng = np.random.default_rng(vocab + k)
    base = (rng.standard_normal(vocab) * 3).astype(np.float32)
    idx, probs = orc.sampled_categorical(base, k, p, t)
    assert len(idx) >= 3
    total = 0.0
    for q in probs:  # libstdc++: sum in double, in order
        total += float(q)
    cp, run = [], 0.0
    for q in probs[:-1]:
        run += float(q) / total
        cp.append(run)
    picks = [0, len(cp) // 2, len(cp) - 1]
    us = []
    for j in picks:
        us += [cp[j], np.nextafter(cp[j], 0.0), np.nextafter(cp[j], 1.0)]
    us = np.array([v for v in us if 0.0 <= v < 1.0], np.float64)
    x = np.tile(base, (len(us), 1))
    sample_and_check(ctx, orc, x, us, k, p, t, cap=64)


def tokens_only(ctx, x, u, k, p, t):
    """A call that asks for the tokens alone (no kept sets): the route the benchmark times."""
    return ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(np.asarray(u, np.float64)).cuda(), k=k, p=p,
                      temperature=t).cpu().numpy()


@pytest.mark.parametrize("rows,vocab,k,p,t", [
    (64, 128256, 50, 0.9, 0.7), (32, 128256, 64, 0.95, 1.0), (16, 201088, 40, 0.5, 1.3), (8, 4099, 50, 0.0, 1.0),
    (8, 32064, 2, 0.9, 0.25), (8, 70001, 17, 1.0, 2.0), (4, 300, 50, 0.9, 1.0),
])
def test_token_only_calls_match_the_oracle(ctx, orc, rows, vocab, k, p, t):
    """Calls without kept-set outputs decide the nucleus cut and the draw from one fp64 prefix sum with guard
    bands; the tokens must be the ones the sequential arithmetic of the reference yields."""
    say("token only", rows, vocab, k, p, t)
    rng = np.random.default_rng(vocab * 7 + k)
    for rep in range(3):
        x = (rng.standard_normal((rows, vocab)) * (1.0 + 2.0 * rep)).astype(np.float32)
        if rep == 2:
            x = np.round(x * 4) / 4  # heavy ties
        u = rng.random(rows)
        got = tokens_only(ctx, x, u, k, p, t)
        assert np.array_equal(got, orc.sample_batch(x, k, p, t, u)), rep


@pytest.mark.parametrize("vocab,k,t", [(128256, 50, 0.7), (5000, 30, 1.0), (40000, 64, 1.5)])
def test_token_only_calls_on_the_edges_of_their_guard_bands(ctx, orc, vocab, k, t):
    """Token-only calls with draws placed on, just below and just above the values of the cumulative
    distribution, and with top-p masses placed on, just below and just above the fp32 cumulative probabilities
    of the reference's cut loop: none of these can be decided from the prefix sum in tree order, so the kernel
    must notice and run the sequential epilogue."""
    say("token only edges", vocab, k, t)
    rng = np.random.default_rng(vocab + k)
    base = (rng.standard_normal(vocab) * 3).astype(np.float32)
    # draws on the boundaries of the final distribution, for a cut in the middle and for no cut
    for p in (0.9, 0.0):
        idx, probs = orc.sampled_categorical(base, k, p, t)
        assert len(idx) >= 3
        total = 0.0
        for q in probs:
            total += float(q)
        cp, run = [], 0.0
        for q in probs[:-1]:
            run += float(q) / total
            cp.append(run)
        us = []
        for j in sorted({0, 1, len(cp) // 2, len(cp) - 1}):
            us += [cp[j], np.nextafter(cp[j], 0.0), np.nextafter(cp[j], 1.0)]
        us = np.array([v for v in us if 0.0 <= v < 1.0], np.float64)
        x = np.tile(base, (len(us), 1))
        assert np.array_equal(tokens_only(ctx, x, us, k, p, t), orc.sample_batch(x, k, p, t, us))
    # masses on the boundaries of the cut: the reference adds the fp32 probabilities in rank order
    _, pr = orc.sampled_categorical(base, k, 0.0, t)
    cum, run = [], np.float32(0.0)
    for q in pr:
        run = np.float32(run + q)
        cum.append(run)
    u = rng.random(8)
    x = np.tile(base, (len(u), 1))
    for j in sorted({0, 1, len(cum) // 3, len(cum) // 2, len(cum) - 2}):
        for mass in (cum[j], np.nextafter(cum[j], np.float32(0)), np.nextafter(cum[j], np.float32(1))):
            mass = float(mass)
            if not 0.0 < mass < 1.0:
                continue
            kept = len(orc.sampled_categorical(base, k, mass, t)[0])
            assert kept in (j + 1, j + 2), (j, mass, kept)  # the cut really falls where the mass was placed
            assert np.array_equal(tokens_only(ctx, x, u, k, mass, t), orc.sample_batch(x, k, mass, t, u)), (j, mass)


def test_results_written_straight_to_pinned_host_memory(ctx, orc):
    """The output pointers may name pinned host memory that the device can address (the reference mirrors its
    results through pinned memory, src/cuda/interface.cpp:51-60): the kernels store the tokens there themselves, no
    copy follows, and a host that has filled the buffer with -1 sees a step's tokens arrive without synchronising the
    stream.  Sampling, argmax and the EOS / append tail."""
    import time
    say("pinned outputs")
    rng = np.random.default_rng(404)
    rows, vocab = 64, 128256
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    u = rng.random(rows)
    xd, ud = torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda()
    torch.cuda.synchronize()
    out = torch.full((rows,), -1, dtype=torch.int32).pin_memory()
    view = out.numpy()

    def wait_for_tokens():
        t0 = time.perf_counter()
        while (view < 0).any():
            assert time.perf_counter() - t0 < 10.0, "tokens never arrived in pinned memory"

    ctx.sample(xd, ud, k=50, p=0.9, temperature=0.7, out=out)
    wait_for_tokens()  # no synchronisation: the kernel's own stores are what the host sees
    assert np.array_equal(view, orc.sample_batch(x, 50, 0.9, 0.7, u))
    torch.cuda.synchronize()
    view[:] = -1
    ctx.argmax(xd, out=out)
    wait_for_tokens()
    assert np.array_equal(view, orc.argmax_batch(x))
    torch.cuda.synchronize()
    # the tail of a greedy step with its tokens and its all-finished flag in pinned memory
    eos, pad, max_len, cur = [7, 9], 0, 8, 3
    tokens = torch.tensor([5, 7, 9, 11], dtype=torch.int32).pin_memory()
    done = torch.zeros(1, dtype=torch.int32).pin_memory()
    seen = torch.tensor([0, 0, 1, 1], dtype=torch.int32).cuda()
    seqs = torch.zeros((4, max_len), dtype=torch.int32).cuda()
    pkg().SearchContext.greedy_tail(ctx, tokens, seen, eos, pad, seqs, cur, done, allow_host=True)
    torch.cuda.synchronize()
    assert tokens.tolist() == [5, 7, pad, pad] and seen.cpu().tolist() == [0, 1, 1, 1] and done.item() == 0
    assert seqs[:, cur].cpu().tolist() == [5, 7, pad, pad]


def test_prepared_sample_calls_give_the_same_tokens(ctx, orc):
    """SearchContext.prepared_sample marshals a call once; issuing it -- repeatedly, on its stream, into pinned host
    memory or device memory, fp32 or fp16 rows -- gives the tokens of the same call made through `sample`."""
    say("prepared calls")
    rng = np.random.default_rng(405)
    rows, vocab = 64, 40000
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    u = rng.random(rows)
    xd, ud = torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda()
    want = orc.sample_batch(x, 50, 0.9, 0.7, u)
    out_dev = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    out_pin = torch.full((rows,), -1, dtype=torch.int32).pin_memory()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    calls = [ctx.prepared_sample(xd, ud, out_dev, k=50, p=0.9, temperature=0.7),
             ctx.prepared_sample(xd, ud, out_pin, k=50, p=0.9, temperature=0.7, stream=side)]
    for _ in range(3):
        out_dev.fill_(-1)
        out_pin.fill_(-1)
        torch.cuda.synchronize()
        for call in calls:  # (one after the other: calls on one context must not overlap, whatever their streams)
            call()
            torch.cuda.synchronize()
        assert np.array_equal(out_dev.cpu().numpy(), want)
        assert np.array_equal(out_pin.numpy(), want)
    xh = torch.from_numpy(x.astype(np.float16)).cuda()
    call16 = ctx.prepared_sample(xh, ud, out_dev, k=0, p=0.9, temperature=1.0)
    call16()
    torch.cuda.synchronize()
    assert np.array_equal(out_dev.cpu().numpy(), orc.sample_batch(xh.float().cpu().numpy(), 0, 0.9, 1.0, u))


def test_config2_topk_topp_batch64(ctx, orc):
    """Benchmark configuration 2 at full size: batch 64, vocab 128256, N(0,3^2) logits + 8 peaks/row at +10,
    T=0.7, k=50, p=0.9, shared uniforms; 4 of the 128 steps."""
    rng = np.random.default_rng(2)
    rows, vocab = 64, 128256
    for step in range(4):
        say("config2 step", step)
        x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
        for r in range(rows):
            x[r, rng.choice(vocab, 8, replace=False)] += 10
        u = rng.random(rows)
        tok = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=50, p=0.9, temperature=0.7)
        assert np.array_equal(tok.cpu().numpy(), orc.sample_batch(x, 50, 0.9, 0.7, u))


def test_sample_ties_and_degenerate_rows(ctx, orc):
    """Heavy ties (rounded logits, constant rows) push rows onto the exact general path; results must
    still equal the oracle's lowest-index tie rule."""
    say("sample ties")
    rng = np.random.default_rng(3)
    rows, vocab = 4, 20000
    x = np.round(rng.standard_normal((rows, vocab)) * 2).astype(np.float32)
    x[1, :] = 1.5
    x[2, :] = LOWEST
    x[2, 77] = 0.0
    u = rng.random(rows)
    sample_and_check(ctx, orc, x, u, 50, 0.9, 0.7)
    sample_and_check(ctx, orc, x, u, 10, 0.0, 1.0)


def test_sparse_mask_rows_with_heavy_ties(ctx, orc):
    """Nucleus rows under a sparse mask whose allowed logits are quantised (hundreds of ids per score, more than a
    bucket of the counting sort holds), constant, or carry a block of equal values at the top: the row leaves the
    bucket sort for the sorting network inside the same kernel; kept ids, probability bits and tokens equal the
    oracle's, with and without the promise about the mask."""
    say("sparse mask, heavy ties")
    rng = np.random.default_rng(77)
    rows, vocab = 5, 201088
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    x[0] = np.round(x[0] * 2) / 2
    x[1] = np.round(x[1])
    x[2, :] = np.float32(-1.25)
    x[3, : vocab // 3] = np.float32(9.5)
    mask = make_mask(rng, rows, vocab, 0.05)
    allowed = np.unpackbits(mask.view(np.uint8), axis=1, bitorder="little")[:, :vocab].astype(bool)
    hist = rng.integers(0, vocab, (rows, 300)).astype(np.int32)
    u = rng.random(rows)
    xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(), history=torch.from_numpy(hist).cuda(),
                           repetition_penalty=1.3)
    proc = orc.apply_mask(x, mask)
    cap = 16384
    for promise in (0, int(allowed.sum(axis=1).max())):
        xf.c.mask_allowed_max = promise
        tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=0.9, temperature=1.0,
                                     xf=xf, kept_capacity=cap)
        tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
        for r in range(rows):
            idx, probs = orc.sampled_categorical(orc.apply_repetition_penalty(proc[r], hist[r], 1.3), 0, 0.9, 1.0)
            n = min(len(idx), cap)
            assert kc[r] == len(idx), (promise, r, kc[r], len(idx))
            assert np.array_equal(ki[r, :n], idx[:n]), (promise, r)
            assert np.array_equal(bits(kp[r, :n]), bits(probs[:n])), (promise, r)
            assert tok[r] == idx[orc.discrete_draw(probs, u[r])], (promise, r)


def test_grammar_rows_with_15_63_or_255_allowed_ids_stay_off_the_exact_path(ctx, orc):
    """A grammar that lets 15, 63 or 255 ids through, all of them inside the nucleus: the search only stops on the
    first masked id, which is the 16th, 64th, 256th element, and the reference notices such a stop one element later
    (src/sampling_distribution.h:166-181): the kept set ends with two masked ids.  The sparse-mask kernel knows the
    second one (and the elements behind the first in general); kept sets and tokens equal the oracle's, with and
    without a repetition penalty over ids that include masked ones, and no row takes the exact path."""
    say("grammar rows whose list ends on a batch end")
    rng = np.random.default_rng(1563)
    vocab = 201088
    words = (vocab - 1) // 32 + 1
    sizes = [15, 63, 255, 15, 63, 14, 16]
    rows = len(sizes)
    x = (rng.standard_normal((rows, vocab)) * 2).astype(np.float32)
    bits_ = np.zeros((rows, words * 32), bool)
    for r, n in enumerate(sizes):
        ids = rng.choice(vocab, n, replace=False)
        if r == 3:
            ids[0] = 1  # id 0 is masked: the first masked id is 0, the second 2
            ids[1] = 3
        bits_[r, ids] = True
        x[r, ids] = (5.0 + 0.1 * rng.standard_normal(n)).astype(np.float32)  # near-equal: the nucleus needs all of them
    mask = np.ascontiguousarray(np.packbits(bits_.reshape(rows, words, 32), axis=-1, bitorder="little").view(np.uint32).reshape(rows, words))
    proc = orc.apply_mask(x, mask)
    u = rng.random(rows)
    u[1] = 0.99999999
    hist = rng.integers(0, 40, (rows, 24)).astype(np.int32)  # low ids: masked ones among them, 0 and 2 included
    for penalty in (None, 1.3):
        for promise in (0, 256):
            xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(),
                                   history=torch.from_numpy(hist).cuda() if penalty else None,
                                   repetition_penalty=penalty or 1.0, mask_allowed_max=promise)
            before = ctx.fallback_rows()
            tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=0.9, temperature=1.0,
                                         xf=xf, kept_capacity=512)
            took_exact = ctx.fallback_rows() - before
            tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
            for r in range(rows):
                want = orc.apply_repetition_penalty(proc[r], hist[r], penalty) if penalty else proc[r]
                idx, probs = orc.sampled_categorical(want, 0, 0.9, 1.0)
                assert kc[r] == len(idx), (penalty, promise, r, kc[r], len(idx))
                assert np.array_equal(ki[r, :len(idx)], idx), (penalty, promise, r)
                assert np.array_equal(bits(kp[r, :len(idx)]), bits(probs)), (penalty, promise, r)
                assert tok[r] == idx[orc.discrete_draw(probs, u[r])], (penalty, promise, r)
            if penalty is None:
                assert [int(k) for k in kc] == [17, 65, 257, 17, 65, 15, 17], kc
            assert took_exact == 0, (penalty, promise, took_exact)


@pytest.mark.parametrize("sigma,p,t", [(4.0, 0.95, 1.0), (1.0, 0.9, 1.0), (5.0, 0.9, 1.0), (3.0, 0.5, 0.7)])
def test_nucleus_rows_with_lists_near_and_beyond_the_sort(ctx, orc, sigma, p, t):
    """Unmasked nucleus rows of 128256 ids whose chunks list a few thousand to tens of thousands of keys: nuclei that
    fit the finish kernel's sort with room to spare, that fill it almost completely, and that exceed it (sorted in
    rounds).  Kept counts, the first kept ids with their probability bits, and tokens equal the
    oracle's."""
    say("nucleus near the sort's capacity", sigma, p, t)
    rng = np.random.default_rng(int(sigma * 10 + p * 100))
    rows, vocab = 6, 128256
    x = (rng.standard_normal((rows, vocab)) * sigma).astype(np.float32)
    x[1] += np.float32(0.7)
    x[2, : vocab // 2] -= np.float32(2.0)  # one half of the row lower: chunk thresholds differ
    u = rng.random(rows)
    cap = 4096
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=p, temperature=t,
                                 kept_capacity=cap)
    tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    for r in range(rows):
        idx, probs = orc.sampled_categorical(x[r], 0, p, t)
        n = min(len(idx), cap)
        assert kc[r] == len(idx), (r, kc[r], len(idx))
        assert np.array_equal(ki[r, :n], idx[:n]), r
        assert np.array_equal(bits(kp[r, :n]), bits(probs[:n])), r
        assert tok[r] == idx[orc.discrete_draw(probs, u[r])], r


def test_nucleus_whose_stop_falls_on_a_batch_end_stays_off_the_exact_path(ctx, orc):
    """Peaked rows whose nucleus search stops on the 16th, 64th or 256th element: the reference notices such a stop
    only one element later (src/sampling_distribution.h:166-181), so the kept set has 17, 65, 257 tokens, and a
    candidate list trimmed right behind the stop would be one element short.  The finish kernel then takes the next
    run of buckets along; the rows are finished on the fast path with the oracle's kept sets and tokens."""
    say("nucleus stop on a batch end, peaked rows")
    rng = np.random.default_rng(1664)
    vocab, p, t = 128256, 0.9, 1.0
    # (tokens at the top, depth of the element the search stops on, elements behind it and their depth); in the last
    # three rows the stop's element already lies below the candidates' threshold: the list ends with it, and the
    # element behind it is in no list at all
    shapes = [(15, 11.5, 50, 11.6), (63, 10.0, 30, 10.2), (255, 8.8, 30, 9.3), (15, 11.5, 0, 0.0),
              (15, 12.5, 3, 13.0), (63, 11.0, 3, 11.5), (15, 12.5, 0, 0.0)]
    x = (rng.standard_normal((len(shapes), vocab)) - 15.0).astype(np.float32)
    for r, (n_top, stop_depth, n_after, after_depth) in enumerate(shapes):
        ids = rng.choice(32768, n_top + 1 + n_after, replace=False)  # all in the first chunk
        x[r, ids[:n_top]] = 20.0
        x[r, ids[n_top]] = np.float32(20.0 - stop_depth)
        x[r, ids[n_top + 1:]] = (20.0 - after_depth - 0.01 * rng.random(n_after)).astype(np.float32)
    u = rng.random(len(shapes))
    u[0] = 0.9999999  # the draw reaches the element behind the stop
    before = ctx.fallback_rows()
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=p, temperature=t,
                                 kept_capacity=512)
    took_exact = ctx.fallback_rows() - before
    tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    for r, (n_top, _, _, _) in enumerate(shapes):
        idx, probs = orc.sampled_categorical(x[r], 0, p, t)
        assert len(idx) == n_top + 2, (r, len(idx))  # the stop's element and the one behind it
        assert kc[r] == len(idx), (r, kc[r], len(idx))
        assert np.array_equal(ki[r, :len(idx)], idx), r
        assert np.array_equal(bits(kp[r, :len(idx)]), bits(probs)), r
        assert tok[r] == idx[orc.discrete_draw(probs, u[r])], r
    assert took_exact == 0, took_exact
    # the same rows as fp16
    x16 = x.astype(np.float16)
    before = ctx.fallback_rows()
    tok16 = ctx.sample(torch.from_numpy(x16).cuda(), torch.from_numpy(u).cuda(), k=0, p=p, temperature=t).cpu().numpy()
    assert np.array_equal(tok16, orc.sample_batch(x16.astype(np.float32), 0, p, t, u))
    assert ctx.fallback_rows() == before


@pytest.mark.parametrize("sigma,p,t,wide_rows", [(3.0, 0.95, 1.0, 6), (2.0, 0.9, 1.0, 5), (4.0, 0.99, 1.5, 5), (1.0, 0.9, 1.0, 5)])
def test_nucleus_rows_wider_than_the_sort(ctx, orc, sigma, p, t, wide_rows):
    """Unmasked nucleus rows of 128256 ids whose nuclei hold 30000 to 90000 tokens, several times what the finish
    kernel sorts at once: it sorts them in rounds into global memory.  One row is quantised to steps of 1/64 (dozens of
    equal scores per step: buckets beyond the usual ranking), one to steps of 1/4 (thousands: those rows are the exact
    path's).  Every kept id and probability bit, to the nucleus' last element, and the tokens equal the oracle's;
    the rows without heavy ties stay off the exact path."""
    say("nucleus wider than the sort", sigma, p, t)
    rng = np.random.default_rng(int(sigma * 10 + p * 1000))
    rows, vocab = 7, 128256
    x = (rng.standard_normal((rows, vocab)) * sigma).astype(np.float32)
    x[1] += np.float32(0.7)
    x[2, : vocab // 2] -= np.float32(1.0)  # one half of the row lower: chunk thresholds differ
    x[3, 1000:1040] = np.nan
    x[4, 5] = 40.0  # one token far above the rest
    x[5] = (np.round(x[5] * 64) / 64).astype(np.float32)
    x[6] = (np.round(x[6] * 4) / 4).astype(np.float32)
    u = rng.random(rows)
    u[0] = 0.999999  # a draw from the nucleus' far end
    before = ctx.fallback_rows()
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=p, temperature=t,
                                 kept_capacity=vocab)
    took_exact = ctx.fallback_rows() - before
    tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    for r in range(rows):
        idx, probs = orc.sampled_categorical(x[r], 0, p, t)
        n = len(idx)
        assert kc[r] == n, (r, kc[r], n)
        assert np.array_equal(ki[r, :n], idx), r
        assert np.array_equal(bits(kp[r, :n]), bits(probs)), r
        assert tok[r] == idx[orc.discrete_draw(probs, u[r])], r
    assert took_exact <= rows - wide_rows, took_exact


@pytest.mark.parametrize("k", [100, 512, 2048, 6000])
def test_large_k_rows_with_ties_nans_and_clustered_best_tokens(ctx, orc, k):
    """Top-k rows with 64 < k <= 8192 at 128256 ids: fewer numbers than k (NaNs fill the rest), a score shared by
    thousands of ids at the k-th place, the best tokens all in one chunk or in one thread's run of ids, one chunk
    without a number.  Kept sets, probability bits and tokens equal the oracle's."""
    say("large k, ties and NaNs", k)
    rng = np.random.default_rng(k)
    rows, vocab = 6, 128256
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    x[0, :] = np.nan
    x[0, rng.integers(0, vocab, k // 2)] = rng.standard_normal(k // 2).astype(np.float32)
    x[1] = np.round(x[1])
    x[2, 40000:40000 + 3 * k] = 30.0 + rng.standard_normal(3 * k).astype(np.float32)
    x[3, 70000:70032] = 50.0
    x[4, 32768:65536] = np.nan
    u = rng.random(rows)
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=k, p=0.9, temperature=0.8,
                                 kept_capacity=2048)
    tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    for r in range(rows):
        idx, probs = orc.sampled_categorical(x[r], k, 0.9, 0.8)
        n = min(len(idx), 2048)
        assert kc[r] == len(idx), (r, kc[r], len(idx))
        assert np.array_equal(ki[r, :n], idx[:n]), r
        assert np.array_equal(bits(kp[r, :n]), bits(probs[:n])), r
        assert tok[r] == idx[orc.discrete_draw(probs, u[r])], r


@pytest.mark.parametrize("vocab,k", [(128256, 50), (70000, 64), (40000, 2), (128256, 1)])
def test_rows_that_tie_at_their_kth_score_are_selected_not_sorted(ctx, orc, vocab, k):
    """Rows whose k best cannot be told from a chunk's bound -- all ids masked to lowest() but a few, NaNs needed to
    fill the k, one score shared by thousands of ids, a few large values in one thread's run of ids -- leave the
    single-pass path inside the streaming kernel; there the k best are selected exactly (the keys above the k-th
    score, then the first ties in id order) and the tokens, kept ids and probabilities equal the oracle's."""
    say("sample selection", vocab, k)
    rng = np.random.default_rng(vocab + k)
    rows = 6
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    x[0, :] = LOWEST
    x[0, rng.integers(0, vocab, 5)] = [0.0, 1.0, -1.0, 0.5, 0.25]
    x[1, :] = np.nan
    x[1, rng.integers(0, vocab, 20)] = rng.standard_normal(20).astype(np.float32)
    x[2, :] = 1.5
    x[3, : vocab // 2] = 7.0   # above everything else: half the row ties for every place
    x[4, 1000:1200] = 40.0 + rng.standard_normal(200).astype(np.float32)  # the best 200 in consecutive ids
    u = rng.random(rows)
    before = ctx.fallback_rows()
    if k == 1:
        got = ctx.argmax(torch.from_numpy(x).cuda()).cpu().numpy()
        assert np.array_equal(got, orc.argmax_batch(x))
    else:
        sample_and_check(ctx, orc, x, u, k, 0.9, 0.7)
        sample_and_check(ctx, orc, x, u, k, 0.0, 1.0)
        assert ctx.fallback_rows() > before  # (rows 0 and 1 at least cannot stay on the single-pass path)


@pytest.mark.parametrize("vocab", [2, 70, 5000, 40000])
def test_sample_rows_without_finite_logits(ctx, orc, vocab):
    """A row of -inf logits (everything masked, then a penalty above 1 applied to lowest()) has NaN
    weights; the reference's draw then lands on position 0 of its kept list whatever the uniform is."""
    say("sample all -inf", vocab)
    x = np.full((2, vocab), -np.inf, np.float32)
    x[1, vocab // 2] = 0.0
    u = np.array([0.73, 0.41])
    for k, p in ((0, 0.9), (1, 0.0), (5, 0.5), (50, 0.0), (200, 0.9)):
        tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=k, p=p, temperature=0.8,
                                     kept_capacity=64)
        for r in range(2):
            idx, probs = orc.sampled_categorical(x[r], k, p, 0.8)
            assert kc[r].item() == len(idx), (k, p, r)
            assert tok[r].item() == idx[orc.discrete_draw(probs, u[r])], (k, p, r)
        assert tok[0].item() == 0 and tok[1].item() == vocab // 2


def test_sample_large_k_general_path(ctx, orc):
    say("sample k=200")
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((2, 5000)) * 3).astype(np.float32)
    u = rng.random(2)
    sample_and_check(ctx, orc, x, u, 200, 0.95, 0.9, cap=256)
    sample_and_check(ctx, orc, x, u, 6000, 0.0, 1.0, cap=64)  # k > vocab clamps


@pytest.mark.parametrize("vocab,k,p,t,quantum", [
    (128256, 65, 0.9, 0.7, 0.0), (128256, 100, 1.0, 1.0, 0.0), (128256, 512, 0.95, 1.3, 0.0), (201088, 300, 0.0, 0.8, 0.0),
    (128256, 513, 0.95, 1.3, 0.0),  # from here four offers per thread bound the chunk
    (128256, 2048, 0.9, 1.0, 0.0), (201088, 2048, 0.0, 1.0, 0.0), (128256, 1500, 0.99, 0.8, 0.25), (5000, 2048, 0.9, 1.0, 0.0),
    (128256, 2049, 0.95, 1.3, 0.0), (128256, 8192, 0.9, 1.0, 0.0), (201088, 5000, 0.0, 0.9, 0.0), (70000, 6000, 0.95, 1.1, 0.5),
    (128256, 8193, 0.95, 1.3, 0.0),  # beyond the limit of this route: the full-sort path
    (33000, 100, 0.9, 1.0, 0.0),    # the short last chunk holds fewer than k threads' worth of elements
    (40000, 500, 0.99, 1.0, 0.25),  # ties across the cut
    (700, 500, 0.9, 1.0, 0.0),      # k close to the vocabulary
])
def test_sample_large_k_through_the_candidate_lists(ctx, orc, vocab, k, p, t, quantum):
    """Top-k rows with 64 < k <= 8192 are streamed like nucleus rows (candidates = elements at or above
    the k-th best of the per-thread offers of their chunk: the maxima up to k = 512, beyond that the maxima of
    the quarters or eighths of every thread's elements) and finished by the sorting kernel, not by the full-sort
    path; kept sets, probabilities and tokens equal the oracle's."""
    say("sample large k", vocab, k, p, t, quantum)
    rng = np.random.default_rng(vocab + k)
    rows = 5
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    if quantum:
        x = (np.round(x / quantum) * quantum).astype(np.float32)
    x[1, :] = np.float32(0.5)            # a constant row: heavy ties, the exact path is allowed here
    x[2, rng.integers(0, vocab, 50)] = -np.inf
    u = rng.random(rows)
    before = ctx.fallback_rows()
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=k, p=p, temperature=t,
                                 kept_capacity=2048)
    tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    for r in range(rows):
        idx, probs = orc.sampled_categorical(x[r], k, p, t)
        n = min(len(idx), 2048)
        assert kc[r] == len(idx), r
        assert np.array_equal(ki[r, :n], idx[:n]), r
        assert np.array_equal(bits(kp[r, :n]), bits(probs[:n])), r
        assert tok[r] == idx[orc.discrete_draw(probs, u[r])], r
    if k <= 8192 and not quantum:
        assert ctx.fallback_rows() - before <= 1  # at most the constant row


@pytest.mark.parametrize("rows,vocab,p,t", [(3, 5000, 0.9, 1.0), (2, 128256, 0.95, 0.7), (2, 40, 0.6, 1.0),
                                            (2, 64, 0.9, 1.0), (2, 65, 0.9, 1.0), (3, 3000, 0.0, 1.0),
                                            (2, 3000, 0.3, 2.0)])
def test_sample_nucleus(ctx, orc, rows, vocab, p, t):
    say("sample nucleus", rows, vocab, p, t)
    rng = np.random.default_rng(vocab + int(p * 100))
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    u = rng.random(rows)
    sample_and_check(ctx, orc, x, u, 0, p, t, cap=128)


@pytest.mark.parametrize("vocab,sigma,p,fast", [(128256, 4.0, 0.95, True), (201088, 5.0, 0.9, True), (128256, 2.0, 0.95, False),
                                                (40000, 4.0, 0.999, False)])
def test_nucleus_with_more_candidates_than_the_sort_holds(ctx, orc, vocab, sigma, p, fast):
    """Unmasked rows: nearly the whole vocabulary lies within the candidate depth of the maximum.  The finish
    kernel then keeps the best ~16000 by raising its threshold; when they contain the nucleus (peaked rows)
    the row stays on the fast path, otherwise the exact path takes it.  Results equal the oracle's either way."""
    say("nucleus trim", vocab, sigma, p)
    rng = np.random.default_rng(int(vocab + sigma * 10))
    rows = 4
    x = (rng.standard_normal((rows, vocab)) * sigma).astype(np.float32)
    x[3] = (np.round(x[3] * 2) / 2).astype(np.float32)  # ties at the raised threshold
    u = rng.random(rows)
    before = ctx.fallback_rows()
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=p, temperature=1.0,
                                 kept_capacity=4096)
    tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    for r in range(rows):
        idx, probs = orc.sampled_categorical(x[r], 0, p, 1.0)
        assert kc[r] == len(idx), (r, kc[r], len(idx))
        n = min(len(idx), 4096)
        assert np.array_equal(ki[r, :n], idx[:n]), r
        assert np.array_equal(bits(kp[r, :n]), bits(probs[:n])), r
        assert tok[r] == idx[orc.discrete_draw(probs, u[r])], r
    took_exact = ctx.fallback_rows() - before
    assert took_exact == 0 if fast else took_exact > 0, took_exact


@pytest.mark.parametrize("vocab", [32, 128, 130, 512, 2048, 8192, 32768, 131072])
def test_nucleus_stop_on_last_element_of_a_sort_batch(ctx, orc, vocab):
    """Constant rows with p = 0.5 meet the tail-bound stop at element vocab/2; where that is the end of one of
    the reference's sort batches (16, 64, 256, ...) the stop is only noticed one element later
    (src/sampling_distribution.h:166-181), so vocab/2 + 1 tokens are kept."""
    say("nucleus batch end", vocab)
    rng = np.random.default_rng(vocab)
    x = np.full((3, vocab), -0.5, np.float32)
    x[1, :] = 0.0
    x[2, vocab // 2:] = -0.5000001  # a second, slightly lower level
    u = rng.random(3)
    sample_and_check(ctx, orc, x, u, 0, 0.5, 1.0, cap=256)
    idx, _ = orc.sampled_categorical(x[0], 0, 0.5, 1.0)
    quirk = vocab > 64 and vocab // 2 in (16, 64, 256, 1024, 4096, 16384, 65536)
    assert len(idx) == vocab // 2 + (1 if quirk else 0)


@pytest.mark.parametrize("frac,quantum", [(0.004, 0.0), (0.012, 0.0), (0.03, 0.0), (0.012, 0.5), (0.03, 0.5),
                                           (0.06, 0.25)])
def test_nucleus_candidate_counts_and_ties(ctx, orc, frac, quantum):
    """Masked nucleus rows whose candidate lists fall in every size class of the finish kernel's sort
    (about 800 to 12000 keys); a quantum > 0 rounds the logits to a coarse grid so that hundreds of
    candidates tie and the sort must fall back from score buckets to the sorting network."""
    say("nucleus sizes", frac, quantum)
    rng = np.random.default_rng(int(frac * 1000) + int(quantum * 8))
    rows, vocab = 3, 201088
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    if quantum:
        x = (np.round(x / quantum) * quantum).astype(np.float32)
    mask = make_mask(rng, rows, vocab, frac)
    u = rng.random(rows)
    xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda())
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=0.95,
                                 temperature=1.0, xf=xf, kept_capacity=16384)
    tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    proc = orc.apply_mask(x, mask)
    for r in range(rows):
        idx, probs = orc.sampled_categorical(proc[r], 0, 0.95, 1.0)
        assert kc[r] == len(idx)
        assert np.array_equal(ki[r, :len(idx)], idx)
        assert np.array_equal(bits(kp[r, :len(idx)]), bits(probs))
        assert tok[r] == idx[orc.discrete_draw(probs, u[r])]


def test_config5_constrained_nucleus(ctx, orc):
    """Benchmark configuration 5 shape (8 of 256 rows per step, 2 steps): vocab 201088, 5 % grammar mask,
    T=1.0, top-p 0.95, repetition penalty 1.2 over 1024 ids."""
    rng = np.random.default_rng(5)
    rows, vocab = 8, 201088
    for step in range(2):
        say("config5 step", step)
        x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
        mask = make_mask(rng, rows, vocab, 0.05)
        hist = rng.integers(0, vocab, (rows, 1024)).astype(np.int32)
        u = rng.random(rows)
        xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(),
                               history=torch.from_numpy(hist).cuda(), repetition_penalty=1.2)
        tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=0.95,
                                     temperature=1.0, xf=xf, kept_capacity=16384)
        tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
        proc = orc.apply_mask(x, mask)
        for r in range(rows):
            row = orc.apply_repetition_penalty(proc[r], hist[r], 1.2)
            idx, probs = orc.sampled_categorical(row, 0, 0.95, 1.0)
            assert kc[r] == len(idx) and len(idx) > 1000
            assert np.array_equal(ki[r, :len(idx)], idx)
            assert np.array_equal(bits(kp[r, :len(idx)]), bits(probs))
            assert tok[r] == idx[orc.discrete_draw(probs, u[r])]


@pytest.mark.parametrize("vocab,hist_len,span,k,p", [
    (40000, 2200, 40000, 50, 0.9),    # a history longer than two ids per thread, spread over two chunks
    (40000, 2200, 40000, 0, 0.9),
    (70001, 8000, 2500, 40, 1.0),     # more distinct history ids in one chunk than its list holds: exact path
    (70001, 8000, 2500, 0, 0.95),
    (33000, 300, 232, 8, 0.0),        # the short last chunk holds history ids
    (33000, 300, 232, 0, 0.8),
])
def test_sample_long_and_dense_histories(ctx, orc, vocab, hist_len, span, k, p):
    """History ids are processed apart from the other logits (a list per 32768-id chunk): long histories,
    duplicates, ids outside the vocabulary, lists that overflow, ids in a short last chunk."""
    say("sample histories", vocab, hist_len, span, k, p)
    rng = np.random.default_rng(hist_len + span + k)
    rows = 3
    scale = 2.0 if k else 6.0           # nucleus rows stay peaked, so that their candidates fit the fast path
    x = (rng.standard_normal((rows, vocab)) * scale).astype(np.float32)
    hist = (vocab - span + rng.integers(0, span, (rows, hist_len))).astype(np.int32)
    hist[:, :40] = hist[:, 40:80]       # duplicates
    hist[0, 5] = vocab + 3              # beyond the vocabulary: ignored
    hist[1, 7] = -2                     # negative: ignored
    x[:, hist[2, 100:110]] = 4.6 * scale  # penalised ids among the best of their rows
    mask = make_mask(rng, rows, vocab, 0.7)
    u = rng.random(rows)
    before = ctx.fallback_rows()
    for pen in (1.3, 0.75):
        xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(), history=torch.from_numpy(hist).cuda(),
                               repetition_penalty=pen)
        tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=k, p=p, temperature=0.9,
                                     xf=xf, kept_capacity=4096)
        tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
        proc = orc.apply_mask(x, mask)
        for r in range(rows):
            valid = hist[r][(hist[r] >= 0) & (hist[r] < vocab)]
            row = orc.apply_repetition_penalty(proc[r], valid, pen)
            idx, probs = orc.sampled_categorical(row, k, p, 0.9)
            assert kc[r] == len(idx), (r, pen)
            n = min(len(idx), 4096)
            assert np.array_equal(ki[r, :n], idx[:n]), (r, pen)
            assert np.array_equal(bits(kp[r, :n]), bits(probs[:n])), (r, pen)
            assert tok[r] == idx[orc.discrete_draw(probs, u[r])], (r, pen)
    took_exact = ctx.fallback_rows() - before
    assert (took_exact > 0) == (span == 2500), took_exact  # only the overflowing lists go to the exact path


@pytest.mark.parametrize("vocab", [40001, 40002, 40003, 65539, 98305, 98308])
def test_logits_processing_on_rows_of_any_alignment_and_end(ctx, orc, vocab):
    """The kernels with logits processing request a chunk's fp32 logits as sixteen 128-bit loads per thread whatever
    the row's alignment and end (a quad that straddles the end is read as the row's last four elements and put right
    afterwards): rows that start on every 4-byte offset of a 16-byte line, vocabularies that end one, two and three
    elements into a quad, a last chunk of a single element, history ids and masked ids on the row's last elements.
    Argmax, top-k, k = 300 and nucleus rows against the oracle."""
    say("rows of any alignment", vocab)
    rng = np.random.default_rng(vocab)
    rows = 6
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    x[0, vocab - 1] = 30.0   # the row's best on its last element ...
    x[1, vocab - 2] = 30.0   # ... on the one before, penalised below
    x[2, vocab - 3] = 30.0   # ... masked below
    hist = rng.integers(0, vocab, (rows, 200)).astype(np.int32)
    hist[:, 0] = vocab - 2
    hist[:, 1] = vocab - 1
    mask = make_mask(rng, rows, vocab, 0.8)
    words = mask.reshape(rows, -1)
    words[2, (vocab - 3) >> 5] &= ~np.uint32(1 << ((vocab - 3) & 31))
    u = rng.random(rows)
    xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(), history=torch.from_numpy(hist).cuda(),
                           repetition_penalty=1.6)
    xd = torch.from_numpy(x).cuda()
    proc = orc.apply_mask(x, mask)
    want = [orc.apply_repetition_penalty(proc[r], hist[r], 1.6) for r in range(rows)]
    got = ctx.argmax(xd, xf=xf).cpu().numpy()
    for r in range(rows):
        assert got[r] == orc.argmax(want[r]), r
    for k, p, t in ((50, 0.9, 0.7), (300, 0.95, 1.0), (0, 0.9, 1.0)):
        tok, kc, ki, kp = ctx.sample(xd, torch.from_numpy(u).cuda(), k=k, p=p, temperature=t, xf=xf, kept_capacity=2048)
        tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
        for r in range(rows):
            idx, probs = orc.sampled_categorical(want[r], k, p, t)
            n = min(len(idx), 2048)
            assert kc[r] == len(idx), (k, r)
            assert np.array_equal(ki[r, :n], idx[:n]), (k, r)
            assert np.array_equal(bits(kp[r, :n]), bits(probs[:n])), (k, r)
            assert tok[r] == idx[orc.discrete_draw(probs, u[r])], (k, r)


@pytest.mark.parametrize("hist_len", [1500, 2500, 3400, 5000])
def test_sparse_mask_rows_with_thousands_of_distinct_history_ids(orc, hist_len):
    """Nucleus rows under a sparse grammar mask whose history holds more distinct ids than the sparse-mask kernel's
    threads take on as processed candidates (two each): such rows must leave that kernel, not lose ids.  Half of
    the history ids are allowed and strong, so that every one of them is inside the nucleus."""
    say("sparse mask, long history", hist_len)
    rng = np.random.default_rng(hist_len)
    rows, vocab = 2, 201088
    c = pkg().SearchContext(rows, vocab)
    try:
        x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
        mask = make_mask(rng, rows, vocab, 0.04)
        hist = np.stack([rng.choice(vocab, hist_len, replace=False) for _ in range(rows)]).astype(np.int32)
        for r in range(rows):
            ids = hist[r, :hist_len // 2]
            np.bitwise_or.at(mask.reshape(rows, -1)[r], ids >> 5, np.uint32(1) << (ids & 31).astype(np.uint32))
            x[r, ids] += 6.0
        u = rng.random(rows)
        xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(), history=torch.from_numpy(hist).cuda(),
                               repetition_penalty=1.2)
        tok, kc, ki, kp = c.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=0.95, temperature=1.0,
                                   xf=xf, kept_capacity=16384)
        tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
        proc = orc.apply_mask(x, mask)
        for r in range(rows):
            row = orc.apply_repetition_penalty(proc[r], hist[r], 1.2)
            idx, probs = orc.sampled_categorical(row, 0, 0.95, 1.0)
            assert kc[r] == len(idx), r
            assert np.array_equal(ki[r, :len(idx)], idx), r
            assert np.array_equal(bits(kp[r, :len(idx)]), bits(probs)), r
            assert tok[r] == idx[orc.discrete_draw(probs, u[r])], r
    finally:
        c.close()


@pytest.mark.parametrize("vocab", [5000, 70001])
def test_nucleus_with_minus_infinity_below_the_threshold(ctx, orc, vocab):
    """Rows whose elements outside the candidate range are all -inf: the element after the nucleus, which a
    stop on a sort-batch end keeps, is then a -inf one (probability 0) with the lowest id."""
    say("nucleus -inf tail", vocab)
    rng = np.random.default_rng(vocab)
    rows = 4
    x = np.full((rows, vocab), -np.inf, np.float32)
    for r, n in enumerate([16, 64, 15, 256]):   # 16, 64, 256: the nucleus ends on a batch end when p is near 1
        ids = rng.choice(vocab, n, replace=False)
        x[r, ids] = rng.standard_normal(n).astype(np.float32)
    u = rng.random(rows)
    for p in (0.9999999, 0.5):
        tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=p, temperature=1.0,
                                     kept_capacity=1024)
        tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
        for r in range(rows):
            idx, probs = orc.sampled_categorical(x[r], 0, p, 1.0)
            assert kc[r] == len(idx), (r, p, kc[r], len(idx))
            assert np.array_equal(ki[r, :len(idx)], idx), (r, p)
            assert np.array_equal(bits(kp[r, :len(idx)]), bits(probs)), (r, p)
            assert tok[r] == idx[orc.discrete_draw(probs, u[r])], (r, p)


@pytest.mark.parametrize("rows,vocab", [(6, 30000), (64, 40000), (70, 9000)])
def test_sample_heterogeneous_rows(ctx, orc, rows, vocab):
    """BatchedSampler semantics: per-row (k, p, T), greedy = (1, 0, 1).  Up to 64 rows the parameters
    travel inside the kernel arguments, above that through a table on the device: both sides of that edge."""
    say("sample heterogeneous", rows, vocab)
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    u = rng.random(rows)
    kinds = [(1, 0.0, 1.0), (50, 0.9, 0.7), (0, 0.9, 1.0), (8, 1.0, 1.5), (-1, 0.5, 0.8), (100, 0.0, 1.0)]
    params = [kinds[(r * 5 + r // 6) % 6] for r in range(rows)]
    params[0] = kinds[0]
    tok = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), per_row=params).cpu().numpy()
    for r, (k, p, t) in enumerate(params):
        assert tok[r] == orc.sample_row(x[r], k, p, t, u[r]), r
    assert tok[0] == orc.argmax(x[0])


@pytest.mark.parametrize("seed", range(int(os.environ.get("MI355X_RANDOM_FIRST", "0")),
                                        int(os.environ.get("MI355X_RANDOM_FIRST", "0")) +
                                        int(os.environ.get("MI355X_RANDOM_CASES", "300"))))
def test_sample_randomised_shapes_and_parameters(ctx, orc, seed):
    """Differential test over random shapes (vocabularies around the 32768-logit chunk edges included),
    per-row (k, p, T) mixes, logit scales, coarse grids (ties), grammar masks, repetition penalties and
    min-length masking: tokens of every row and the kept sets of uniform-parameter cases must equal
    the oracle's."""
    rng = np.random.default_rng(1000 + seed)
    edges = [1, 2, 63, 64, 65, 255, 4097, 32767, 32768, 32769, 65536, 65537, 98304, 131071, 131073, 196608, 201088]
    vocab = int(rng.choice(edges)) if seed % 2 else int(rng.integers(2, 140000))
    rows = int(rng.integers(1, 7))
    scale = float(rng.choice([0.05, 1.0, 3.0, 30.0]))
    x = (rng.standard_normal((rows, vocab)) * scale).astype(np.float32)
    if seed % 3 == 0:
        x = (np.round(x * 2) / 2).astype(np.float32)  # heavy ties
    if seed % 5 == 0:
        x[0, :] = 1.25  # a constant row
    # the logits as fp32, fp16 or bf16 (the oracle sees the widened values)
    kind = ("f32", "f16", "bf16")[seed % 7 % 3]
    if kind == "f16":
        with np.errstate(over="ignore"):
            x_dev = torch.from_numpy(x.astype(np.float16)).cuda()
        x = x_dev.float().cpu().numpy()
    elif kind == "bf16":
        x_dev = torch.from_numpy(x).to(torch.bfloat16).cuda()
        x = x_dev.float().cpu().numpy()
    else:
        x_dev = torch.from_numpy(x).cuda()
    say("sample random", seed, rows, vocab, scale, kind)
    xf, proc = None, x
    if seed % 4 in (1, 2):
        mask = make_mask(rng, rows, vocab, float(rng.choice([0.02, 0.5, 0.98])))
        hist_len = int(rng.integers(1, 200)) if seed % 9 else int(rng.integers(1500, 6000))  # now and then a long one
        hist = rng.integers(0, vocab, (rows, hist_len)).astype(np.int32)
        pen = float(rng.choice([1.0, 1.3, 0.8]))
        eos = [int(rng.integers(0, vocab))]
        allowed = int(np.unpackbits(mask.view(np.uint8)).reshape(rows, -1).sum(axis=1).max())
        promise = int(rng.choice([0, allowed, 3]))  # none, the true bound, a broken promise (still exact)
        xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(), history=torch.from_numpy(hist).cuda(),
                               repetition_penalty=pen, eos_ids=eos, apply_min_length=bool(seed % 8 == 1),
                               mask_allowed_max=promise)
        proc = orc.apply_mask(x, mask)
        proc = np.stack([orc.apply_repetition_penalty(orc.apply_min_length(proc[r], 0, 1 if seed % 8 == 1 else 0, eos),
                                                       hist[r], pen) for r in range(rows)])
    u = rng.random(rows)

    def params():
        k = int(rng.choice([0, 1, 2, 5, 40, 50, 64, 65, 200, 513, 2048, 2049, vocab, vocab + 7]))
        p = float(rng.choice([0.0, 0.1, 0.5, 0.9, 0.999, 1.0]))
        return k, p, float(rng.uniform(0.3, 2.0))

    if seed % 2:  # heterogeneous rows
        per_row = [params() for _ in range(rows)]
        tok = ctx.sample(x_dev, torch.from_numpy(u).cuda(), per_row=per_row, xf=xf).cpu().numpy()
        for r, (k, p, t) in enumerate(per_row):
            assert tok[r] == orc.sample_row(proc[r], k, p, t, u[r]), (r, k, p, t)
    else:
        k, p, t = params()
        cap = 256
        tok, kc, ki, kp = ctx.sample(x_dev, torch.from_numpy(u).cuda(), k=k, p=p, temperature=t,
                                     xf=xf, kept_capacity=cap)
        tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
        for r in range(rows):
            idx, probs = orc.sampled_categorical(proc[r], k, p, t)
            n = min(len(idx), cap)
            assert kc[r] == len(idx), (r, k, p, t)
            assert np.array_equal(ki[r, :n], idx[:n]), (r, k, p, t)
            assert np.array_equal(bits(kp[r, :n]), bits(probs[:n])), (r, k, p, t)
            assert tok[r] == idx[orc.discrete_draw(probs, u[r])], (r, k, p, t)


@pytest.mark.parametrize("k", [50, 57, 64])
def test_topk_with_clustered_best_tokens_stays_on_the_fast_path(ctx, orc, k):
    """The per-chunk bound pools the best eight per-thread maxima of every wave; rows whose best tokens
    sit next to each other (one wave holds most of them) or whose k is close to 64 let many more than k
    elements past it.  The kernel then takes the exact bound and lists again: results equal the oracle's
    and no row needs the full-sort path."""
    say("clustered top-k", k)
    rng = np.random.default_rng(900 + k)
    rows, vocab = 12, 128256
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    for r in range(rows // 2):
        start = int(rng.integers(0, vocab - 1024)) // 256 * 256
        if r % 2:   # 24 neighbouring ids hold the row's best tokens (six threads with four of them each)
            x[r, start:start + 24] = 14.0 + rng.standard_normal(24).astype(np.float32)
        else:       # 60 of the best tokens at every fourth id of one 256-id strip: one each in 60 threads of one wave
            x[r, start:start + 240:4] = 14.0 + rng.standard_normal(60).astype(np.float32)
    u = rng.random(rows)
    before = ctx.fallback_rows()
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=k, p=0.95, temperature=0.8,
                                 kept_capacity=64)
    tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    for r in range(rows):
        idx, probs = orc.sampled_categorical(x[r], k, 0.95, 0.8)
        assert kc[r] == len(idx), r
        assert np.array_equal(ki[r, :len(idx)], idx), r
        assert np.array_equal(bits(kp[r, :len(idx)]), bits(probs)), r
        assert tok[r] == idx[orc.discrete_draw(probs, u[r])], r
    assert ctx.fallback_rows() == before


def test_wait_that_gives_up_hands_rows_to_the_exact_path(orc):
    """Failure handling of the top-k hand-over between workgroups, forced from the host: with a poll limit
    of 0 a finishing workgroup gives up on every list that has not arrived yet.  Its row must come out of
    the exact path unchanged, the context must report the event, and every later call must still be right
    (all its top-k rows then take the exact path)."""
    say("poll limit 0")
    rng = np.random.default_rng(77)
    rows, vocab = 128, 201088  # seven workgroups per row, far more workgroups than the GPU runs at once
    c = pkg().SearchContext(rows, vocab)
    try:
        x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
        u = rng.random(rows)
        want = np.array([orc.sample_row(x[r], 50, 0.9, 0.7, u[r]) for r in range(rows)], np.int32)
        xd, ud = torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda()
        assert np.array_equal(c.sample(xd, ud, k=50, p=0.9, temperature=0.7).cpu().numpy(), want)
        assert not c.wait_gave_up() and c.fallback_rows() == 0
        c.set_poll_limit(0)
        assert np.array_equal(c.sample(xd, ud, k=50, p=0.9, temperature=0.7).cpu().numpy(), want)
        assert c.wait_gave_up()
        assert 0 < c.fallback_rows() <= rows
        c.set_poll_limit(1 << 21)
        before = c.fallback_rows()
        assert np.array_equal(c.sample(xd, ud, k=50, p=0.9, temperature=0.7).cpu().numpy(), want)
        assert c.fallback_rows() - before == rows  # the fast path stays off for this context
        tk, ts = c.topk_scores(xd[:4], 8)
        for r in range(4):
            order = np.lexsort((np.arange(vocab), -x[r].astype(np.float64)))[:8]
            assert np.array_equal(tk[r].cpu().numpy(), order.astype(np.int32))
    finally:
        c.close()


def test_argument_errors(ctx):
    x = torch.zeros((2, 100), device="cuda")
    u = torch.zeros(2, dtype=torch.float64, device="cuda")
    with pytest.raises(RuntimeError, match="temperature"):
        ctx.sample(x, u, k=5, p=0.5, temperature=0.0)
    big = torch.zeros((257, 10), device="cuda")
    with pytest.raises(RuntimeError, match="capacity"):
        ctx.argmax(big)


@pytest.mark.parametrize("vocab,ngram,hist_len", [(1000, 2, 60), (40000, 3, 300), (70001, 1, 17), (300, 4, 2), (5000, 2, 1500)])
def test_no_repeat_ngram_ban(ctx, orc, vocab, ngram, hist_len):
    """ApplyNoRepeatNgramToLogits after mask, min-length and penalty (LogitsPenaltyProcessor::Apply order):
    in-place processing, greedy argmax and sampling all see the banned ids as lowest()."""
    say("no-repeat ngram", vocab, ngram, hist_len)
    rng = np.random.default_rng(vocab + ngram)
    rows = 4
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    hist = rng.integers(0, 6, (rows, hist_len)).astype(np.int32)  # six distinct ids: every n-gram repeats
    hist[1, :] = rng.integers(0, vocab, hist_len)  # a row whose n-grams hardly ever repeat
    x[:, :6] += 8.0  # the banned ids would otherwise win
    mask = make_mask(rng, rows, vocab, 0.9)
    eos = [3, vocab - 1]
    for pen in (1.0, 1.3):
        xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(), history=torch.from_numpy(hist).cuda(),
                               repetition_penalty=pen, eos_ids=eos, apply_min_length=True, no_repeat_ngram_size=ngram)
        want = orc.apply_mask(x, mask)
        for r in range(rows):
            w = orc.apply_min_length(want[r], 0, 1, eos)
            w = orc.apply_repetition_penalty(w, hist[r], pen)
            want[r] = orc.apply_no_repeat_ngram(w, hist[r], ngram)
        got = ctx.process_logits(torch.from_numpy(x.copy()).cuda(), xf).cpu().numpy()
        assert np.array_equal(bits(got), bits(want))
        if hist_len >= ngram:
            assert (want[0] != orc.apply_repetition_penalty(orc.apply_min_length(orc.apply_mask(x, mask)[0], 0, 1, eos),
                                                             hist[0], pen)).any()  # something was banned
        tok = ctx.argmax(torch.from_numpy(x).cuda(), xf=xf).cpu().numpy()
        assert np.array_equal(tok, orc.argmax_batch(want))
        u = rng.random(rows)
        for k, p in ((40, 0.9), (0, 0.8)):
            tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=k, p=p, temperature=0.9,
                                         xf=xf, kept_capacity=64)
            for r in range(rows):
                idx, probs = orc.sampled_categorical(want[r], k, p, 0.9)
                n = min(len(idx), 64)
                assert kc[r].item() == len(idx)
                assert np.array_equal(ki[r, :n].cpu().numpy(), idx[:n])
                assert np.array_equal(bits(kp[r, :n].cpu().numpy()), bits(probs[:n]))
                assert tok[r].item() == idx[orc.discrete_draw(probs, u[r])]


@pytest.mark.parametrize("vocab,K,seed_len,greedy", [(32064, 8, 40, False), (32064, 8, 40, True), (5000, 3, 2, False),
                                                     (140000, 5, 700, False)])
def test_target_selection_of_verify_rows(ctx, orc, vocab, K, seed_len, greedy):
    """ComputeTargetTokenSelection for the K+1 verify rows of one sequence (src/speculative_sampling.h:59-79,
    src/speculative_decoding_strategy.cpp:632-656): row i is processed with current_length = seed + i and
    the prefix seed tokens + the first i proposal tokens -- one shared history buffer, per-row lengths --
    then reduced to the greedy token or the kept (ids, probabilities)."""
    say("target selection", vocab, K, seed_len, greedy)
    rng = np.random.default_rng(vocab + K + seed_len)
    rows = K + 1
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    seq = rng.integers(0, 8, seed_len + K).astype(np.int32)  # few distinct ids: n-grams repeat
    x[:, :8] += 6.0
    eos = [5, 7]
    min_len = seed_len + 3  # the first rows are still too short for EOS
    lens = (seed_len + np.arange(rows)).astype(np.int32)
    xf = pkg().LogitsXform(history=torch.from_numpy(seq[None, :]).cuda(), shared_history=True,
                           history_lens=torch.from_numpy(lens).cuda(), repetition_penalty=1.2, eos_ids=eos,
                           min_length=min_len, no_repeat_ngram_size=2)
    k, p, t = 50, 0.9, 0.8
    u = rng.random(rows)
    if greedy:
        tok = ctx.argmax(torch.from_numpy(x).cuda(), xf=xf).cpu().numpy()
    else:
        tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=k, p=p, temperature=t,
                                     xf=xf, kept_capacity=64)
        tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    for i in range(rows):
        g, idx, probs = orc.target_selection(x[i], int(lens[i]), seq[:lens[i]], greedy, k, p, t, rep_pen=1.2,
                                             min_len=min_len, ngram=2, eos=eos)
        if greedy:
            assert tok[i] == g, i
        else:
            assert kc[i] == len(idx), i
            assert np.array_equal(ki[i, :len(idx)], idx), i
            assert np.array_equal(bits(kp[i, :len(idx)]), bits(probs)), i
            assert tok[i] == idx[orc.discrete_draw(probs, u[i])], i


@pytest.mark.parametrize("batch", [1, 7, 300])
def test_greedy_tail_eos_pad_append(ctx, batch):
    """CheckForEOSAndPad + AppendNextTokensToSequences against the CPU search's PadIfAlreadyEOS / SetNextToken /
    AppendNextTokensToSequences loop (src/search.cpp:194-201,256-296) over a whole generation."""
    say("greedy tail", batch)
    rng = np.random.default_rng(batch)
    max_length, eos, pad = 12, [3, 9], 1
    seq = np.zeros((batch, max_length), np.int32)
    seen = np.zeros(batch, bool)
    d_seq = torch.zeros((batch, max_length), dtype=torch.int32, device="cuda")
    d_seen = torch.zeros(batch, dtype=torch.int32, device="cuda")
    d_done = torch.zeros(1, dtype=torch.int32, device="cuda")
    length, done = 0, False
    while not done and length < max_length:
        tokens = rng.integers(0, 12 if length > 3 else 40, batch).astype(np.int32)
        d_tok = torch.from_numpy(tokens).cuda()
        ctx.greedy_tail(d_tok, d_seen, eos, pad, d_seq, length, d_done)
        want = np.where(seen, pad, tokens)
        seen |= np.isin(want, eos) & ~seen
        done = bool(seen.all())
        assert np.array_equal(d_tok.cpu().numpy(), want)
        assert np.array_equal(d_seen.cpu().numpy().astype(bool), seen)
        assert bool(d_done.item()) == done
        if not done:  # the CPU search appends only while some row is alive; the device writes the column anyway
            seq[:, length] = want
            length += 1
            assert np.array_equal(d_seq.cpu().numpy()[:, :length], seq[:, :length])
    assert done or length == max_length
    before = d_seq.clone()
    ctx.greedy_tail(torch.zeros(batch, dtype=torch.int32, device="cuda"), d_seen, eos, pad, d_seq, max_length, d_done)
    assert torch.equal(before, d_seq)  # nothing is written beyond max_length


@pytest.mark.parametrize("vocab,frac,penalty,p", [
    (201088, 0.05, 1.2, 0.95),     # the sparse-mask kernel finishes the rows
    (201088, 0.0005, 1.2, 0.95),   # a hundred allowed ids
    (201088, 0.079, 0.8, 0.9),     # close to what the sort buffer holds; a penalty below one lifts masked history ids
    (201088, 0.0816, 1.2, 0.9),    # around the capacity: some rows fit, some are left to the dense kernels
    (201088, 0.5, 1.2, 0.95),      # dense: every row declined
    (70001, 0.05, 1.3, 0.999),     # the nucleus takes nearly every allowed id
    (70001, 0.02, 1.0, 0.3),       # no penalty: no history bitmap
    (4099, 0.3, 1.1, 0.95),
])
def test_nucleus_rows_under_sparse_and_dense_masks(ctx, orc, vocab, frac, penalty, p):
    """Rows in nucleus mode with a grammar mask of any density, min-length EOS masking, a history with ids that
    are masked, ids that are allowed, repeats and out-of-range ids; a few allowed logits are -inf, NaN or
    lowest().  Kept ids, probability bits and tokens equal the oracle's."""
    say("nucleus under mask", vocab, frac, penalty, p)
    rng = np.random.default_rng(int(vocab * 1000 + frac * 1e6))
    rows = 6
    x = (rng.standard_normal((rows, vocab)) * 3).astype(np.float32)
    mask = make_mask(rng, rows, vocab, frac)
    allowed = np.unpackbits(mask.view(np.uint8), axis=1, bitorder="little")[:, :vocab].astype(bool)
    for r in range(rows):
        ids = np.flatnonzero(allowed[r])
        if len(ids) > 8:  # special values among the allowed logits
            x[r, ids[1]] = -np.inf
            x[r, ids[3]] = np.nan if r % 2 else LOWEST
            x[r, ids[5]] = x[r, ids[6]]  # a tie
    hist = rng.integers(0, vocab, (rows, 200)).astype(np.int32)
    hist[:, 7] = hist[:, 3]  # a repeat
    hist[:, 9] = -1
    for r in range(rows):
        ids = np.flatnonzero(allowed[r])
        hist[r, 0] = ids[0]                      # allowed ids in the history
        hist[r, 1] = ids[len(ids) // 2]
        hist[r, 2] = np.flatnonzero(~allowed[r])[0] if (~allowed[r]).any() else 0  # the first masked id is in the history
    eos = [int(np.flatnonzero(allowed[0])[0]), 2]
    u = rng.random(rows)
    xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(), history=torch.from_numpy(hist).cuda(),
                           repetition_penalty=penalty, eos_ids=eos, apply_min_length=True)
    cap = 20000
    proc = orc.apply_mask(x, mask)
    want = []
    for r in range(rows):
        row = proc[r].copy()
        row[eos] = LOWEST
        row = orc.apply_repetition_penalty(row, hist[r][(hist[r] >= 0)], penalty)
        want.append(orc.sampled_categorical(row, 0, p, 0.9))
    # without a promise about the mask, with the true bound on the allowed ids per row, and with a promise
    # that the rows break (they are still sampled correctly, by the exact path)
    for promise in (0, int(allowed.sum(axis=1).max()), 3):
        xf.c.mask_allowed_max = promise
        tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=p, temperature=0.9,
                                     xf=xf, kept_capacity=cap)
        tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
        for r in range(rows):
            idx, probs = want[r]
            n = min(len(idx), cap)
            assert kc[r] == len(idx), (promise, r, kc[r], len(idx))
            assert np.array_equal(ki[r, :n], idx[:n]), (promise, r)
            assert np.array_equal(bits(kp[r, :n]), bits(probs[:n])), (promise, r)
            assert tok[r] == idx[orc.discrete_draw(probs, u[r])], (promise, r)


def exact_path_rows(name, rng, vocab):
    if name == "gaussian":
        return (rng.standard_normal((2, vocab)) * 3).astype(np.float32)
    if name == "constant":
        return np.full((2, vocab), 1.5, np.float32)
    if name == "rounded":  # thirteen distinct scores: every digit of the sort's first level overflows
        return np.round(rng.standard_normal((2, vocab)) * 2).astype(np.float32)
    if name == "peaked":  # nearly every score inside a sliver of the row's range
        x = (5.0 + rng.random((2, vocab)) * 1e-3).astype(np.float32)
        x[:, rng.integers(0, vocab, 6)] = [100.0, -100.0, 50.0, 7.0, 5.0005, -3.0]
        return x
    if name == "mostly_lowest":  # what a grammar mask leaves behind
        x = (rng.standard_normal((2, vocab)) * 3).astype(np.float32)
        x[rng.random((2, vocab)) < 0.95] = LOWEST
        return x
    if name == "specials":
        x = (rng.standard_normal((2, vocab)) * 3).astype(np.float32)
        x[0, rng.integers(0, vocab, 9)] = [np.inf, -np.inf, np.nan, -np.inf, np.inf, 0.0, -0.0, LOWEST, np.nan]
        x[1, rng.integers(0, vocab, 4)] = [-np.inf, -np.inf, LOWEST, LOWEST]
        return x
    raise KeyError(name)


@pytest.mark.parametrize("vocab", [65, 511, 513, 4100, 10239, 10241, 16384, 70001, 128256, 201088])
@pytest.mark.parametrize("name", ["gaussian", "constant", "rounded", "peaked", "mostly_lowest", "specials"])
def test_exact_path_orders_whole_rows(ctx, orc, name, vocab):
    """k above the candidate-list bound (8192) and sampling from the whole vocabulary (k = 0, p = 1) take the exact
    path, which sorts the entire row; the kept ids are that order, checked to the last element."""
    say("exact path", name, vocab)
    rng = np.random.default_rng(vocab + len(name))
    x = exact_path_rows(name, rng, vocab)
    u = rng.random(2)
    before = ctx.fallback_rows()
    sample_and_check(ctx, orc, x, u, vocab, 0.0, 0.9, cap=vocab)
    sample_and_check(ctx, orc, x, u, 0, 1.0, 1.1, cap=vocab)
    if vocab > 2048:
        sample_and_check(ctx, orc, x, u, 2049, 0.97, 1.0, cap=2049)
    # k <= 8192 goes through the candidate lists, which hand rows with ties or NaNs at their bound to the exact path too
    assert ctx.fallback_rows() - before >= (4 if vocab > 8192 else 2)


def test_exact_path_sixteen_bit_rows(ctx, orc):
    """fp16 rows hold a few thousand distinct scores: long runs of ties through the exact path's sort."""
    say("exact path fp16")
    rng = np.random.default_rng(16)
    x16 = (rng.standard_normal((2, 128256)) * 3).astype(np.float16)
    u = rng.random(2)
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x16).cuda(), torch.from_numpy(u).cuda(), k=0, p=1.0, temperature=1.0,
                                 kept_capacity=128256)
    x = x16.astype(np.float32)
    for r in range(2):
        idx, probs = orc.sampled_categorical(x[r], 0, 1.0, 1.0)
        assert kc[r].item() == len(idx)
        assert np.array_equal(ki[r, :len(idx)].cpu().numpy(), idx), r
        assert np.array_equal(bits(kp[r, :len(idx)].cpu().numpy()), bits(probs)), r
        assert tok[r].item() == idx[orc.discrete_draw(probs, u[r])], r


@pytest.mark.parametrize("rows,cap", [(1, 8), (9, 64), (70, 300), (5, 20000)])
def test_draw_in_order_follows_one_engine(ctx, orc, rows, cap):
    """mi355x_draw_in_order: rows take the prepared canonical doubles in the order one std::mt19937 would serve them:
    a row with a single kept token and a finished row consume none, every other row the next one."""
    say("draw_in_order", rows, cap)
    rng = np.random.default_rng(rows * 7 + cap)
    counts = rng.integers(1, cap + 1, rows).astype(np.int32)
    counts[rng.random(rows) < 0.3] = 1
    skip = (rng.random(rows) < 0.25).astype(np.int32)
    ids = rng.integers(0, 1 << 20, (rows, cap)).astype(np.int32)
    probs = rng.random((rows, cap)).astype(np.float32)
    for r in range(rows):
        probs[r, :counts[r]] /= probs[r, :counts[r]].sum(dtype=np.float32)
    pool = rng.random(rows)
    for use_skip in (True, False):
        tok, used = ctx.draw_in_order(torch.from_numpy(counts).cuda(), torch.from_numpy(ids).cuda(),
                                      torch.from_numpy(probs).cuda(), torch.from_numpy(pool).cuda(),
                                      torch.from_numpy(skip).cuda() if use_skip else None)
        tok = tok.cpu().numpy()
        d = 0
        for r in range(rows):
            if (use_skip and skip[r]) or counts[r] < 2:
                assert tok[r] == ids[r, 0], r
                continue
            assert tok[r] == ids[r, orc.discrete_draw(probs[r, :counts[r]], pool[d])], (r, d)
            d += 1
        assert used.item() == d
    # a kept-set size beyond the capacity of the lists breaks the contract: the call says so instead of counting
    broken = counts.copy()
    broken[rows // 2] = cap + 3
    _, used = ctx.draw_in_order(torch.from_numpy(broken).cuda(), torch.from_numpy(ids).cuda(),
                                torch.from_numpy(probs).cuda(), torch.from_numpy(pool).cuda(), None)
    assert used.item() == -1
