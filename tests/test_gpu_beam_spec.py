"""GPU parity for the remaining entry points, through the C ABI, against the CPU oracle on the same
seeded inputs: top-k scores, softmax / log-softmax (bit-exact: the sequential fp32 sum is emulated
exactly), beam top-2B selection + BeamSearchScorer + sequence reorder, KV-cache gather (bit-exact)
and speculative verification (bit-exact lengths and tokens)."""
import numpy as np
import pytest
import torch

import orc_lib
from gpu_common import pkg, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = pkg().SearchContext(64, 201088)
    yield c
    c.close()


def bits(a):
    return np.asarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("rows,vocab,k,dtype", [(3, 32064, 8, np.float32), (9, 151936, 50, np.float16),
                                                (2, 40, 5, np.float32), (2, 5000, 1, np.float32),
                                                (17, 128256, 64, np.float32)])
def test_topk_scores(ctx, orc, rows, vocab, k, dtype):
    say("topk_scores", rows, vocab, k, dtype.__name__)
    rng = np.random.default_rng(vocab + k)
    x = (rng.standard_normal((rows, vocab)) * 2).astype(dtype)
    tok, sc = ctx.topk_scores(torch.from_numpy(x).cuda(), k)
    tok, sc = tok.cpu().numpy(), sc.cpu().numpy()
    xf = orc.fp16_to_fp32(x) if dtype == np.float16 else x
    for r in range(rows):
        order = np.lexsort((np.arange(vocab), -xf[r].astype(np.float64)))[:k]  # score desc, index asc
        assert np.array_equal(tok[r], order)
        assert np.array_equal(sc[r], xf[r][order])


@pytest.mark.parametrize("rows", [1, 4, 32])
@pytest.mark.parametrize("vocab", [200, 2000, 20000, 200000])
def test_topk_scores_on_the_reference_grid(ctx, orc, rows, vocab):
    """The parity grid of the reference's own top-k tests (test/cuda/cuda_topk_tests.cpp:199-201: batch 1 / 4 / 32,
    vocabulary 200 ... 200000, k up to 256), extended past the large-k route's limit: every k goes through the one
    entry point (up to 64: the fused kernel, up to 2048: the candidate lists, beyond: the whole-row sort) and must
    give the ids and raw scores of a stable sort by (score descending, id ascending)."""
    say("topk_scores grid", rows, vocab)
    rng = np.random.default_rng(rows * 7 + vocab)
    x = (rng.standard_normal((rows, vocab)) * 2).astype(np.float32)
    x[0, : min(vocab, 300)] = np.round(x[0, : min(vocab, 300)])  # ties among the best
    xd = torch.from_numpy(x).cuda()
    order = [np.lexsort((np.arange(vocab), -x[r].astype(np.float64))) for r in range(rows)]
    ks = [1, 2, 5, 8, 16, 50, 64, 65, 100, 128, 200, 256, 512, 1000, 2048, 2049, 3000]
    for k in [k for k in ks if k <= vocab]:
        tok, sc = ctx.topk_scores(xd, k)
        tok, sc = tok.cpu().numpy(), sc.cpu().numpy()
        for r in range(rows):
            assert np.array_equal(tok[r], order[r][:k]), (k, r)
            assert np.array_equal(bits(sc[r]), bits(x[r][order[r][:k]])), (k, r)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_topk_scores_large_k_of_sixteen_bit_rows(ctx, orc, dtype):
    """k beyond 64 on fp16 / bf16 rows read as they are: long runs of equal values, ids in ascending order inside a run."""
    say("topk_scores large k", dtype)
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(3, 70001, generator=g) * 2).to(dtype)
    wide = x.float().numpy()
    xd = x.cuda()
    for k in (100, 700, 2048):
        tok, sc = ctx.topk_scores(xd, k)
        tok, sc = tok.cpu().numpy(), sc.cpu().numpy()
        for r in range(3):
            order = np.lexsort((np.arange(wide.shape[1]), -wide[r].astype(np.float64)))[:k]
            assert np.array_equal(tok[r], order), (k, r)
            assert np.array_equal(bits(sc[r]), bits(wide[r][order])), (k, r)


@pytest.mark.parametrize("rows,vocab,t", [(4, 1000, 1.0), (3, 151936, 1.0), (2, 32064, 0.7), (2, 7, 2.0), (5, 50257, 1.0)])
def test_softmax_bit_exact(ctx, orc, rows, vocab, t):
    say("softmax", rows, vocab, t)
    rng = np.random.default_rng(vocab)
    x = (rng.standard_normal((rows, vocab)) * 2).astype(np.float32)
    sm = ctx.softmax(torch.from_numpy(x.copy()).cuda(), t, log=False).cpu().numpy()
    lsm = ctx.softmax(torch.from_numpy(x.copy()).cuda(), t, log=True).cpu().numpy()
    for r in range(rows):
        assert np.array_equal(bits(sm[r]), bits(orc.softmax(x[r], t)))  # tolerance allowed: 1e-5 rel; achieved: 0
        assert np.array_equal(bits(lsm[r]), bits(orc.log_softmax(x[r], t)))


def test_log_softmax_extreme_rows(ctx, orc):
    """Sums that start subnormal, cross many binades, or hit exact ties in the running sum."""
    say("softmax extreme")
    rng = np.random.default_rng(1)
    v = 20000
    x = np.zeros((4, v), np.float32)
    x[0] = np.linspace(-100, 0, v)  # first terms underflow / subnormal
    x[1] = 0.0  # all ones: exact integer sums, ties to even past 2^24? (no) but every add exact
    x[2] = np.where(rng.random(v) < 0.5, 0.0, -16.635532).astype(np.float32)  # ~2^-24 against 1.0
    x[3] = rng.standard_normal(v) * 20
    got = ctx.softmax(torch.from_numpy(x.copy()).cuda(), 1.0, log=True).cpu().numpy()
    for r in range(4):
        assert np.array_equal(bits(got[r]), bits(orc.log_softmax(x[r], 1.0))), r


@pytest.mark.parametrize("batch,beams,vocab,dtype", [(3, 4, 50001, torch.float16), (2, 3, 900, torch.float32),
                                                     (2, 4, 33000, torch.bfloat16)])
def test_beam_search_step_is_select_plus_scorer_step(ctx, batch, beams, vocab, dtype):
    """mi355x_beam_search_step (BeamSearch_Cpu::SelectTop in one call) against mi355x_beam_select +
    mi355x_beam_scorer_step on a second scorer: same next scores, tokens, indices and sequences after every step."""
    say("beam_search_step", batch, beams, vocab)
    rng = np.random.default_rng(vocab)
    one = pkg().BeamScorer(ctx, batch, beams, 12, 0, [7], 0.8, False)
    two = pkg().BeamScorer(ctx, batch, beams, 12, 0, [7], 0.8, False)
    prompt = rng.integers(1, vocab, (batch, 2)).astype(np.int32)
    one.set_prompt(prompt)
    two.set_prompt(prompt)
    for step in range(8):
        x = torch.from_numpy((rng.standard_normal((batch * beams, vocab)) * 2).astype(np.float32)).to(dtype).cuda()
        if step % 3 == 1:
            x[:, 7] += 6.0  # EOS candidates
        one.search_step(x)
        sc, tok, idx = ctx.beam_select(x, batch, beams, two.next_scores)
        two.step(sc, tok, idx)
        assert torch.equal(one.next_scores.view(torch.int32), two.next_scores.view(torch.int32)), step
        assert torch.equal(one.next_tokens, two.next_tokens) and torch.equal(one.next_indices, two.next_indices), step
        assert torch.equal(one.sequences()[0], two.sequences()[0]), step
    one.close()
    two.close()


@pytest.mark.parametrize("batch,beams,vocab,early,dtype", [(70, 2, 20000, False, torch.float32),
                                                           (5, 4, 17000, True, torch.float16),
                                                           (8, 4, 151936, False, torch.float16),
                                                           (3, 3, 16384, False, torch.bfloat16)])
def test_search_step_finishes_entries_like_the_two_calls(ctx, batch, beams, vocab, early, dtype):
    """Rows long enough for the launch that finishes the selection to do the scorer step as well: entries collect
    hypotheses and become done at different steps (the "can it still improve" test reads other entries' candidates),
    and next scores, tokens, indices, sequences, the done state and every hypothesis equal those of
    mi355x_beam_select + mi355x_beam_scorer_step on a second scorer."""
    say("search_step done entries", batch, beams, vocab, early)
    rng = np.random.default_rng(batch * 131 + beams)
    big = pkg().SearchContext(batch * beams, vocab)
    one = pkg().BeamScorer(big, batch, beams, 14, 0, [7, 9], 1.3, early)
    two = pkg().BeamScorer(big, batch, beams, 14, 0, [7, 9], 1.3, early)
    prompt = rng.integers(10, vocab, (batch, 3)).astype(np.int32)
    one.set_prompt(prompt)
    two.set_prompt(prompt)
    base = torch.from_numpy((rng.standard_normal((batch * beams, vocab)) * 2).astype(np.float32))
    for step in range(11):
        x = base.roll(step * 37 + 1, 1).clone()
        rows = rng.random(batch * beams) < 0.4
        x[torch.from_numpy(rows), 7 if step % 2 else 9] += 9.0  # EOS candidates in some rows
        x = x.to(dtype).cuda()
        one.search_step(x)
        sc, tok, idx = big.beam_select(x, batch, beams, two.next_scores)
        two.step(sc, tok, idx)
        assert torch.equal(one.next_scores.view(torch.int32), two.next_scores.view(torch.int32)), step
        assert torch.equal(one.next_tokens, two.next_tokens) and torch.equal(one.next_indices, two.next_indices), step
        assert torch.equal(one.sequences()[0], two.sequences()[0]), step
        assert one.is_done() == two.is_done(), step
    finished = 0
    for b in range(batch):
        for i in range(beams):
            try:
                h1 = one.hypothesis(b, i)
            except RuntimeError:
                with pytest.raises(RuntimeError):
                    two.hypothesis(b, i)
                continue
            h2 = two.hypothesis(b, i)
            assert h1[0] == h2[0] and np.float32(h1[1]).view(np.int32) == np.float32(h2[1]).view(np.int32), (b, i)
            finished += 1
    assert finished > 0
    one.close()
    two.close()
    big.close()


def test_first_calls_of_a_new_context_on_a_side_stream(orc):
    """A context (and a scorer) used right after creation on a stream that does not wait for the null stream:
    the workspace's initial fills must be complete by then.  Long rows, so the exact sums read their "not
    written" pattern."""
    say("new context on a side stream")
    rng = np.random.default_rng(5)
    batch, beams, vocab = 3, 2, 40000
    x = (rng.standard_normal((batch * beams, vocab)) * 2).astype(np.float32)
    want = [orc.log_softmax(x[r], 1.0) for r in range(batch * beams)]
    xd = torch.from_numpy(x).cuda()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    for attempt in range(3):
        with torch.cuda.stream(side):
            c = pkg().SearchContext(batch * beams, vocab)
            got = c.softmax(xd.clone(), 1.0, log=True)
            scorer = pkg().BeamScorer(c, batch, beams, 8, 0, [1], 1.0, False)
            scorer.set_prompt(np.full((batch, 2), 5, np.int32))
            scorer.search_step(xd)
            osc, otok, oidx, _ = orc.beam_select_top(x, batch, beams, np.tile(np.array([0.0, -1e9], np.float32), batch))
            side.synchronize()
            got = got.cpu().numpy()
            for r in range(batch * beams):
                assert np.array_equal(bits(got[r]), bits(want[r])), (attempt, r)
            assert np.array_equal(scorer.next_tokens.cpu().numpy().reshape(batch, beams), otok[:, :beams]), attempt
            assert c.sum_waits_gave_up() == 0
            scorer.close()
            c.close()


def test_exact_sums_whose_waits_give_up(orc):
    """Failure handling of the exact sums' look-back, forced from the host: with a poll limit of 0 a segment's
    workgroup gives up on every earlier sum that has not arrived yet and its segment is added element by element.
    Log-softmax and beam selection must come out bit-identical, the context must count the event, and with the
    limit restored the same calls must be right again (and count nothing new)."""
    say("exact sums, poll limit 0")
    rng = np.random.default_rng(78)
    rows, vocab, batch, beams = 24, 151936, 6, 4
    c = pkg().SearchContext(rows, vocab)
    try:
        x = (rng.standard_normal((rows, vocab)) * 2).astype(np.float32)
        bs = (rng.standard_normal(rows) * 3).astype(np.float32)
        want = [orc.log_softmax(x[r], 1.0) for r in range(rows)]
        wsc, wtok, widx, _ = orc.beam_select_top(x, batch, beams, bs)
        xd, bd = torch.from_numpy(x).cuda(), torch.from_numpy(bs).cuda()

        def check():
            got = c.softmax(xd.clone(), 1.0, log=True).cpu().numpy()
            for r in range(rows):
                assert np.array_equal(bits(got[r]), bits(want[r])), r
            sc, tok, idx = c.beam_select(xd, batch, beams, bd)
            assert np.array_equal(tok.cpu().numpy(), wtok) and np.array_equal(idx.cpu().numpy(), widx)
            assert np.array_equal(bits(sc.cpu().numpy()), bits(wsc))

        check()
        assert c.sum_waits_gave_up() == 0
        c.set_poll_limit(0)
        check()
        gave_up = c.sum_waits_gave_up()
        assert gave_up > 0
        c.set_poll_limit(1 << 21)
        check()
        assert c.sum_waits_gave_up() == gave_up
        assert not c.wait_gave_up()  # the sampling paths' own flag is untouched
    finally:
        c.close()


@pytest.mark.parametrize("vocab", [3, 5000, 20000, 70000])
def test_softmax_rows_whose_maximum_is_a_signed_zero(ctx, orc, vocab):
    """The reference subtracts the row's own first maximal element, -0.0 included: a single -0.0 maximum above
    values whose exponentials vanish gives log-softmax +0.0, not -0.0; mixed zeros give -log(count)."""
    say("softmax signed zeros", vocab)
    x = np.full((6, vocab), -np.inf, np.float32)
    x[0, 0] = -0.0
    x[1, :] = -300.0
    x[1, vocab // 2] = -0.0
    x[2, 0], x[2, 1] = 0.0, -0.0
    x[3, 0], x[3, 1] = -0.0, 0.0
    x[4, :] = -0.0
    x[5, :] = -300.0
    x[5, vocab - 1] = 0.0
    for t in (1.0, 0.05):
        for log in (True, False):
            got = ctx.softmax(torch.from_numpy(x.copy()).cuda(), t, log=log).cpu().numpy()
            for r in range(6):
                want = orc.log_softmax(x[r], t) if log else orc.softmax(x[r], t)
                assert np.array_equal(bits(got[r]), bits(want)), (r, t, log)


@pytest.mark.parametrize("batch,beams,vocab,dtype", [(2, 3, 1000, np.float32), (8, 4, 151936, np.float16),
                                                     (1, 16, 5000, np.float32), (3, 2, 2, np.float32),
                                                     (2, 4, 3000, np.float16), (2, 4, 3001, "bf16"),
                                                     (8, 4, 151936, "bf16"), (1, 3, 40000, "bf16")])
def test_beam_select(ctx, orc, batch, beams, vocab, dtype):
    say("beam_select", batch, beams, vocab, getattr(dtype, "__name__", dtype))
    rng = np.random.default_rng(vocab + beams)
    bs = (rng.standard_normal(batch * beams) * 3).astype(np.float32)
    bs[1::beams] = -1e9
    if dtype == "bf16":  # rows of bfloat16 are read as they lie; the oracle sees the widened values
        x_dev = torch.from_numpy((rng.standard_normal((batch * beams, vocab)) * 2).astype(np.float32)).to(torch.bfloat16).cuda()
        xf = x_dev.float().cpu().numpy()
    else:
        x = (rng.standard_normal((batch * beams, vocab)) * 2).astype(dtype)
        x_dev = torch.from_numpy(x).cuda()
        xf = orc.fp16_to_fp32(x) if dtype == np.float16 else x
    sc, tok, idx = ctx.beam_select(x_dev, batch, beams, torch.from_numpy(bs).cuda())
    osc, otok, oidx, _ = orc.beam_select_top(xf, batch, beams, bs)
    assert np.array_equal(tok.cpu().numpy(), otok)
    assert np.array_equal(idx.cpu().numpy(), oidx)
    assert np.array_equal(bits(sc.cpu().numpy()), bits(osc))  # allowed 1e-5 relative; achieved bit-exact


def test_beam_select_constant_rows(ctx, orc):
    """All-equal logits: every candidate ties, selection must fall back to lowest flat index."""
    say("beam_select ties")
    batch, beams, vocab = 2, 3, 4000
    x = np.zeros((batch * beams, vocab), np.float16)
    x[4] = 1.0
    bs = np.zeros(batch * beams, np.float32)
    sc, tok, idx = ctx.beam_select(torch.from_numpy(x).cuda(), batch, beams, torch.from_numpy(bs).cuda())
    osc, otok, oidx, _ = orc.beam_select_top(orc.fp16_to_fp32(x), batch, beams, bs)
    assert np.array_equal(tok.cpu().numpy(), otok) and np.array_equal(idx.cpu().numpy(), oidx)


def _check_beam_select(ctx, orc, x, batch, beams, bs):
    if isinstance(x, torch.Tensor):  # bfloat16 rows: the oracle sees the widened values
        dev_x, xf = x.cuda(), x.float().numpy()
    else:
        dev_x = torch.from_numpy(x).cuda()
        xf = orc.fp16_to_fp32(x) if x.dtype == np.float16 else x
    sc, tok, idx = ctx.beam_select(dev_x, batch, beams, torch.from_numpy(bs).cuda())
    osc, otok, oidx, _ = orc.beam_select_top(xf, batch, beams, bs)
    assert np.array_equal(tok.cpu().numpy(), otok)
    assert np.array_equal(idx.cpu().numpy(), oidx)
    assert np.array_equal(bits(sc.cpu().numpy()), bits(osc))


@pytest.mark.parametrize("case", ["random_fp32", "beams16", "constant", "one_segment", "equal_finals_spread",
                                  "equal_finals_dense", "minus_inf", "ragged_fp16", "strided_fp32", "ragged_bf16",
                                  "coarse_bf16"])
def test_beam_select_long_rows_through_segment_lists(ctx, orc, case):
    """Rows of at least 16384 logits: every 4096-element segment lists its 2*beams largest logits and one
    workgroup per batch entry scores them.  The cases force the lists' limits: all candidates of an entry inside
    one segment, different logits that round to one final score (lowest flat index must win, with and without the
    lists being full), constant rows (list overflow), -inf fill, rows that end inside a vector, strided rows."""
    say("beam_select long rows", case)
    rng = np.random.default_rng(len(case))
    if case == "random_fp32":
        batch, beams, vocab = 3, 4, 50001
        x = (rng.standard_normal((batch * beams, vocab)) * 2).astype(np.float32)
    elif case == "beams16":
        batch, beams, vocab = 2, 16, 20000
        x = (rng.standard_normal((batch * beams, vocab)) * 2).astype(np.float16)
    elif case == "constant":
        batch, beams, vocab = 2, 3, 20000
        x = np.zeros((batch * beams, vocab), np.float16)
        x[4] = 1.0
    elif case == "one_segment":
        batch, beams, vocab = 2, 4, 40000
        x = rng.standard_normal((batch * beams, vocab)).astype(np.float32)
        for r in range(batch * beams):
            x[r, 3 * 4096 + rng.choice(4096, 12, replace=False)] += 10
    elif case in ("equal_finals_spread", "equal_finals_dense"):
        # logits within a few ulp of 1e-3 above a negative bulk: (x - max) - log(sum) rounds them all to one score
        batch, beams, vocab = 2, 2, 30000
        x = (-np.abs(rng.standard_normal((batch * beams, vocab))) - 1).astype(np.float32)
        top = np.float32(1e-3)
        ladder = [top]
        for _ in range(5):
            ladder.append(np.nextafter(ladder[-1], np.float32(1), dtype=np.float32))
        for r in range(batch * beams):
            if case == "equal_finals_spread":
                pos = np.concatenate([s * 4096 + rng.choice(4096, 2, replace=False) for s in range(7)])
            else:
                pos = 2 * 4096 + rng.choice(4096, 40, replace=False)
            x[r, pos] = rng.choice(ladder, pos.size)
    elif case == "minus_inf":
        batch, beams, vocab = 2, 2, 17000
        x = (rng.standard_normal((batch * beams, vocab)) * 2).astype(np.float32)
        x[:, rng.choice(vocab, 9000, replace=False)] = -np.inf
        x[1, :] = -np.inf
        x[1, 16999] = 0.5  # one number in the row
    elif case == "ragged_fp16":
        batch, beams, vocab = 2, 3, 16384 + 4099
        x = (rng.standard_normal((batch * beams, vocab)) * 2).astype(np.float16)  # odd row length: unaligned rows
    elif case == "ragged_bf16":
        batch, beams, vocab = 2, 3, 16384 + 4099
        x = torch.from_numpy((rng.standard_normal((batch * beams, vocab)) * 2).astype(np.float32)).to(torch.bfloat16)
    elif case == "coarse_bf16":
        # values near 8 carry three fraction bits in bfloat16: most of the row's best logits are equal
        batch, beams, vocab = 2, 4, 70000
        x = torch.from_numpy((8 + rng.random((batch * beams, vocab))).astype(np.float32)).to(torch.bfloat16)
    else:
        batch, beams, vocab = 2, 2, 24001
        full = (rng.standard_normal((batch * beams, vocab + 7)) * 2).astype(np.float32)
        bs = (rng.standard_normal(batch * beams) * 3).astype(np.float32)
        dev = torch.from_numpy(full).cuda()[:, :vocab]
        sc, tok, idx = ctx.beam_select(dev, batch, beams, torch.from_numpy(bs).cuda())
        osc, otok, oidx, _ = orc.beam_select_top(np.ascontiguousarray(full[:, :vocab]), batch, beams, bs)
        assert np.array_equal(tok.cpu().numpy(), otok) and np.array_equal(idx.cpu().numpy(), oidx)
        assert np.array_equal(bits(sc.cpu().numpy()), bits(osc))
        return
    bs = (rng.standard_normal(batch * beams) * 3).astype(np.float32)
    if case in ("constant", "equal_finals_spread", "equal_finals_dense"):
        bs[:] = 0.25  # equal running scores: ties run across the beams of an entry
    _check_beam_select(ctx, orc, x, batch, beams, bs)


def run_beam_search(ctx, orc, batch, beams, vocab, steps, eos, max_length, length_penalty, early_stopping, seed,
                    dtype=np.float16, eos_boost=0.0, fused=False):
    rng = np.random.default_rng(seed)
    prompt = rng.integers(0, vocab, (batch, 3)).astype(np.int32)
    dev = pkg().BeamScorer(ctx, batch, beams, max_length, 0, eos, length_penalty, early_stopping)
    dev.set_prompt(prompt)
    ref = orc_lib.BeamScorer(orc, batch, beams, max_length, 0, eos, length_penalty, early_stopping)
    seq = np.zeros((batch * beams, max_length), np.int32)
    seq[:, :3] = np.repeat(prompt, beams, axis=0)
    length = 3
    for step in range(steps):
        say("beam search step", step)
        x = (rng.standard_normal((batch * beams, vocab)) * 2).astype(dtype)
        for e in eos:
            x[:, e] += eos_boost
        xf = orc.fp16_to_fp32(x) if dtype == np.float16 else x
        # device
        if fused:  # selection and scorer step in one call: only the state after the step shows
            dev.search_step(torch.from_numpy(x).cuda())
        else:
            dsc, dtok, didx = ctx.beam_select(torch.from_numpy(x).cuda(), batch, beams, dev.next_scores)
            dev.step(dsc, dtok, didx)
        # oracle
        osc, otok, oidx, _ = orc.beam_select_top(xf, batch, beams, ref.next_scores)
        ref.process(seq, length, osc, otok, oidx)
        nxt = np.zeros_like(seq)
        orc.lib.orc_beam_append(seq.reshape(-1), nxt.reshape(-1), batch * beams, max_length, length,
                                ref.next_indices, ref.next_tokens)
        seq, length = nxt, length + 1
        if not fused:
            assert np.array_equal(dtok.cpu().numpy(), otok) and np.array_equal(didx.cpu().numpy(), oidx)
            assert np.array_equal(bits(dsc.cpu().numpy()), bits(osc))
        assert np.array_equal(dev.next_tokens.cpu().numpy(), ref.next_tokens)
        assert np.array_equal(dev.next_indices.cpu().numpy(), ref.next_indices)
        assert np.array_equal(bits(dev.next_scores.cpu().numpy()), bits(ref.next_scores))
        dseq, dlen = dev.sequences()
        assert dlen == length and np.array_equal(dseq.cpu().numpy(), seq[:, :length])
        assert dev.is_done() == (ref.is_done() or length == max_length)
        if dev.is_done():
            break
    finished_early = sum(ref.hyp_count(b) for b in range(batch))  # hypotheses that ended with an EOS along the way
    ref.finalize(seq, length)
    for b in range(batch):
        for i in range(ref.hyp_count(b)):
            want_t, want_s = ref.hyp(b, i)
            got_t, got_s = dev.hypothesis(b, i)
            assert got_t == list(want_t) and np.float32(got_s) == np.float32(want_s), (b, i)
    dev.close()
    return length - 3, finished_early


@pytest.mark.parametrize("batch,beams,vocab", [(2, 8, 131072), (2, 8, 131073), (1, 16, 16384), (40, 4, 16385)])
def test_beam_search_at_the_edges_of_the_segment_route(orc, batch, beams, vocab):
    """Whole searches through mi355x_beam_search_step where the long-row route changes: beams x segments x 2 beams
    exactly at the finishing kernel's capacity and one segment over (which takes the row-wise kernels), sixteen beams
    at the shortest long row, forty batch entries whose rows end one logit into a segment."""
    say("beam search edges", batch, beams, vocab)
    c = pkg().SearchContext(batch * beams, vocab)
    try:
        for early in (False, True):
            run_beam_search(c, orc, batch, beams, vocab, 5, [3, vocab - 1], 10, 1.1, early, 1000 + batch + beams,
                            dtype=np.float16 if beams == 8 else np.float32, eos_boost=5.0, fused=True)
    finally:
        c.close()


def test_config3_beam_search_steps(ctx, orc):
    """Benchmark configuration 3 shape (batch 8, beams 4, vocab 151936 fp16, length_penalty 1.0), 6 of the 64
    steps: selection, scorer state, beam-reordered sequences and final hypotheses match the oracle."""
    run_beam_search(ctx, orc, 8, 4, 151936, 6, [151935], 80, 1.0, True, 3)


@pytest.mark.parametrize("early,lp", [(True, 1.0), (False, 1.0), (False, 0.6), (True, 2.0)])
def test_beam_search_with_eos_hypotheses(ctx, orc, early, lp):
    """Small vocabulary with a boosted EOS so hypotheses finish, batches become done and get padded."""
    run_beam_search(ctx, orc, 3, 3, 50, 14, [7, 9], 20, lp, early, 11 + int(early), dtype=np.float32, eos_boost=2.5)


@pytest.mark.parametrize("name", sorted(__import__("beam_scorer_cases").CASES))
def test_device_scorer_matches_handworked_case(ctx, name):
    """mi355x_beam_scorer_* against literal expectations worked out by hand from the reference source
    (tests/beam_scorer_cases.py): EOS hypotheses, eviction, ties, CanImprove with its window offset, early
    stopping, padding of done entries, Finalize.  No oracle involved."""
    from beam_scorer_cases import CASES
    from test_beam_scorer_handworked import check_hyps
    case = CASES[name]
    say("hand-worked scorer case", name)
    batch, beams, ml = case["batch"], case["beams"], case["max_length"]
    dev = pkg().BeamScorer(ctx, batch, beams, ml, case["pad"], case["eos"], case["length_penalty"],
                           case["early_stopping"])
    dev.set_prompt(np.asarray(case["prompt"], np.int32))
    init = np.tile(np.array([0.0] + [-1e9] * (beams - 1), np.float32), batch)
    assert np.array_equal(dev.next_scores.cpu().numpy(), init)
    length = len(case["prompt"][0])
    for si, step in enumerate(case["steps"]):
        cs = torch.tensor([[c[0] for c in row] for row in step["cands"]], dtype=torch.float32).cuda()
        ct = torch.tensor([[c[1] for c in row] for row in step["cands"]], dtype=torch.int32).cuda()
        ci = torch.tensor([[c[2] for c in row] for row in step["cands"]], dtype=torch.int32).cuda()
        dev.step(cs, ct, ci)
        length += 1
        got_s, got_t, got_i = (dev.next_scores.cpu().numpy(), dev.next_tokens.cpu().numpy(),
                               dev.next_indices.cpu().numpy())
        for r, (ws, wt, wi) in enumerate(step["next"]):
            assert got_s[r] == np.float32(ws) and got_t[r] == wt and got_i[r] == wi, (si, r, got_s, got_t, got_i)
        dseq, dlen = dev.sequences()
        assert dlen == length and dseq.cpu().numpy().tolist() == step["sequences"], si
        assert dev.is_done() == (step["all_done"] or length == ml), si
    for b in range(batch):
        got = []
        for i in range(len(case["final"][b])):
            got.append(dev.hypothesis(b, i))
        check_hyps(("final", b), got, case["final"][b])
        with pytest.raises(RuntimeError, match="out of bounds"):
            dev.hypothesis(b, len(case["final"][b]))
    dev.close()


def test_kv_gather_bit_exact(ctx, orc):
    say("kv_gather")
    rng = np.random.default_rng(5)
    rows, shape = 8, (4, 96, 128)  # fp16 blocks of 96 KiB: exercises a partial last tile
    present = [torch.from_numpy(rng.integers(0, 1 << 16, (rows,) + shape).astype(np.uint16).view(np.float16)).cuda()
               for _ in range(6)]
    past = [torch.zeros_like(p) for p in present]
    idx = np.array([3, 3, 0, 7, 1, 1, 6, 2], np.int32)
    ctx.kv_gather(present, past, torch.from_numpy(idx).cuda())
    for p, q in zip(present, past):
        want = orc.kv_gather(p.cpu().numpy().view(np.uint16), idx)
        assert np.array_equal(q.cpu().numpy().view(np.uint16), want)


def test_config3_kv_gather_full_block_size(ctx):
    """Config-3 block (4 heads x 2048 x 128 fp16 = 2 MiB) on 2 of the 56 tensors, checked with torch."""
    say("kv_gather 2MiB blocks")
    g = torch.Generator(device="cuda").manual_seed(0)
    present = [torch.randint(-30000, 30000, (32, 4, 2048, 128), generator=g, device="cuda", dtype=torch.int16)
               .view(torch.float16) for _ in range(2)]
    past = [torch.zeros_like(p) for p in present]
    idx = torch.randint(0, 32, (32,), generator=g, device="cuda", dtype=torch.int32)
    ctx.kv_gather(present, past, idx)
    for p, q in zip(present, past):
        assert torch.equal(q.view(torch.int16), p.view(torch.int16)[idx.long()])


def softmax64(x):
    z = x - x.max(-1, keepdims=True)
    e = np.exp(z)
    return (e / e.sum(-1, keepdims=True)).astype(np.float32)


@pytest.mark.parametrize("batch,K,vocab", [(16, 8, 32064), (4, 3, 500), (5, 1, 2), (6, 8, 32001), (6, 6, 32003),
                                             (6, 8, 4099)])  # (the last three: rows on every offset of a 16-byte line)
def test_spec_verify(ctx, orc, batch, K, vocab):
    """Benchmark configuration 4 (first case): target/draft probabilities from N(0,2^2) logits, draft = target
    logits + N(0,0.5^2); accept tests and residual / bonus resampling with shared uniforms."""
    say("spec_verify", batch, K, vocab)
    rng = np.random.default_rng(vocab + K)
    lt = rng.standard_normal((batch, K + 1, vocab)) * 2
    p = softmax64(lt)
    q = softmax64(lt + rng.standard_normal((batch, K + 1, vocab)) * 0.5)
    if batch > 2:
        q[1] = p[1]  # identical distributions: always accepted -> bonus row
        q[2, 0] = 0.0  # draft probability 0 -> accept probability 1
    draft = np.stack([[rng.choice(vocab, p=q[b, i].astype(np.float64) / q[b, i].astype(np.float64).sum())
                       if q[b, i].sum() > 0 else 0 for i in range(K)] for b in range(batch)]).astype(np.int32)
    uf = rng.random((batch, K)).astype(np.float32)
    ud = rng.random(batch)
    acc, tok = ctx.spec_verify(torch.from_numpy(p).cuda(), torch.from_numpy(q).cuda(), torch.from_numpy(draft).cuda(),
                               torch.from_numpy(uf).cuda(), torch.from_numpy(ud).cuda())
    oacc, otok = orc.spec_verify_dense(p, q, draft, uf, ud)
    assert np.array_equal(acc.cpu().numpy(), oacc)
    assert np.array_equal(tok.cpu().numpy(), otok)
    assert len(set(oacc.tolist())) > 1 or batch < 4


def test_cast_matches_cpu_path(ctx, orc):
    """DeviceInterface::Cast, every supported pair, against the oracle's CPU conversions: all 65536
    fp16 / bf16 patterns, random and special fp32 values, int32 extremes."""
    say("cast")
    h = torch.arange(65536, dtype=torch.int32).to(torch.int16).cuda()
    got = ctx.cast(h.view(torch.float16), torch.float32).cpu().numpy()
    assert np.array_equal(bits(got), bits(orc.cast(np.arange(65536, dtype=np.uint16), 0, np.float32)))
    got = ctx.cast(h.view(torch.bfloat16), torch.float32).cpu().numpy()
    assert np.array_equal(bits(got), bits(orc.cast(np.arange(65536, dtype=np.uint16), 1, np.float32)))
    rng = np.random.default_rng(8)
    x = np.concatenate([(rng.standard_normal(100000) * 10 ** rng.uniform(-9, 6, 100000)).astype(np.float32),
                        np.array([0.0, -0.0, 65504.0, 65520.0, 1e9, -1e9, 1.0 + 2.0 ** -11, 6e-8, 3e-8, np.inf, -np.inf],
                                 np.float32),
                        rng.integers(0, 2 ** 32, 100000, dtype=np.uint64).astype(np.uint32).view(np.float32)])
    got = ctx.cast(torch.from_numpy(x).cuda(), torch.float16).view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got, orc.cast(x, 2, np.uint16))
    got = ctx.cast(torch.from_numpy(x).cuda(), torch.bfloat16).view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got, orc.cast(x, 3, np.uint16))
    i = np.array([0, -1, 5, 2 ** 31 - 1, -2 ** 31], np.int32)
    assert np.array_equal(ctx.cast(torch.from_numpy(i).cuda(), torch.int64).cpu().numpy(), i.astype(np.int64))
    with pytest.raises(RuntimeError, match="same"):
        ctx.cast(torch.zeros(4, device="cuda"), torch.float32)
    with pytest.raises(RuntimeError, match="not implemented"):
        ctx.cast(torch.zeros(4, device="cuda", dtype=torch.int64), torch.int32)


@pytest.mark.parametrize("dtype,kind", [(torch.float16, 0), (torch.bfloat16, 1), (torch.float32, None)])
def test_logits_handoff_slices_and_widens(ctx, orc, dtype, kind):
    """Logits::Get (src/models/logits.cpp:33-82): the logits of each row's last real token, widened to
    fp32 with the CPU path's conversion, from a [rows, seq_len, vocab] model output."""
    say("logits handoff", dtype)
    rows, seq_len, vocab = 5, 7, 4099
    g = torch.Generator(device="cuda").manual_seed(2)
    raw = (torch.randn(rows, seq_len, vocab, generator=g, device="cuda") * 4).to(dtype)
    tok = [6, 0, 3, 6, 2]
    for index in (None, tok):
        got = ctx.logits_handoff(raw, index).cpu().numpy()
        picked = torch.stack([raw[r, seq_len - 1 if index is None else index[r]] for r in range(rows)])
        if kind is None:
            want = picked.cpu().numpy()
        else:
            want = orc.cast(picked.view(torch.int16).cpu().numpy().view(np.uint16), kind, np.float32)
        assert np.array_equal(bits(got), bits(want))
    with pytest.raises(RuntimeError, match="outside"):
        ctx.logits_handoff(raw, [0, 0, 0, 0, 7])
