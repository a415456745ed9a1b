"""Randomised differential tests of the remaining entry points (softmax / log-softmax, argmax with
fused logits processing, top-k scores, beam selection, whole beam searches, speculative
verification, KV gather) through the C ABI against the CPU oracle.  Shapes are drawn around the
kernels' internal edges (64-lane waves, 4096-element sum segments, the 16384-logit switch to the
multi-workgroup sum, 32768-logit chunks); values include ties, -inf, lowest() and constant rows.
Integer results and fp32 results must be bit-identical (NaNs compare equal to NaNs).
MI355X_RANDOM_CASES scales the number of seeds per test (default 300 -> 40 .. 100 per test);
MI355X_RANDOM_FIRST is the first seed (default 0)."""
import os

import numpy as np
import pytest
import torch

import orc_lib
from gpu_common import LOWEST, make_mask, pkg, say
from test_gpu_beam_spec import run_beam_search

pytestmark = pytest.mark.gpu

CASES = int(os.environ.get("MI355X_RANDOM_CASES", "300"))
FIRST = int(os.environ.get("MI355X_RANDOM_FIRST", "0"))
EDGES = [1, 2, 3, 63, 64, 65, 255, 256, 257, 1023, 1025, 4095, 4096, 4097, 8191, 8193, 16383, 16384, 16385, 20480,
         32767, 32768, 32769, 65535, 65537, 98304, 131073, 151936, 201088]


@pytest.fixture(scope="module")
def ctx():
    c = pkg().SearchContext(64, 201088)
    yield c
    c.close()


def same_bits(a, b):
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    nan = np.isnan(a) & np.isnan(b)
    return np.array_equal(np.where(nan, 0, a.view(np.uint32)), np.where(nan, 0, b.view(np.uint32)))


def random_logits(rng, rows, vocab, seed):
    scale = float(rng.choice([0.05, 1.0, 3.0, 30.0, 300.0]))
    x = (rng.standard_normal((rows, vocab)) * scale).astype(np.float32)
    if seed % 3 == 0:
        x = (np.round(x * 2) / 2).astype(np.float32)
    if seed % 5 == 0:
        x[0, :] = -2.5
    if seed % 7 == 0:
        x[rows - 1, rng.random(vocab) < 0.7] = -np.inf
    if seed % 11 == 0:
        x[rows // 2, rng.random(vocab) < 0.9] = LOWEST
    if seed % 13 == 0:
        x[0, :] = -np.inf
    return x


@pytest.mark.parametrize("seed", range(FIRST, FIRST + max(CASES // 3, 1)))
def test_softmax_randomised(ctx, orc, seed):
    rng = np.random.default_rng(2000 + seed)
    vocab = int(rng.choice(EDGES)) if seed % 2 else int(rng.integers(1, 70000))
    rows = int(rng.integers(1, 5))
    t = float(rng.choice([1.0, 0.7, 2.0, 0.05]))
    x = random_logits(rng, rows, vocab, seed)
    say("softmax random", seed, rows, vocab, t)
    sm = ctx.softmax(torch.from_numpy(x.copy()).cuda(), t, log=False).cpu().numpy()
    lsm = ctx.softmax(torch.from_numpy(x.copy()).cuda(), t, log=True).cpu().numpy()
    for r in range(rows):
        assert same_bits(sm[r], orc.softmax(x[r], t)), r
        assert same_bits(lsm[r], orc.log_softmax(x[r], t)), r


@pytest.mark.parametrize("seed", range(FIRST, FIRST + max(CASES // 3, 1)))
def test_argmax_and_topk_scores_randomised(ctx, orc, seed):
    rng = np.random.default_rng(3000 + seed)
    vocab = int(rng.choice(EDGES)) if seed % 2 else int(rng.integers(1, 140000))
    rows = int(rng.integers(1, 9))
    x = random_logits(rng, rows, vocab, seed)
    say("argmax random", seed, rows, vocab)
    xf, proc = None, x
    if seed % 4 in (1, 2):
        mask = make_mask(rng, rows, vocab, float(rng.choice([0.02, 0.5, 0.98])))
        hist = rng.integers(-1, vocab + 1, (rows, int(rng.integers(1, 300)))).astype(np.int32)
        pen = float(rng.choice([1.0, 1.3, 0.8]))
        eos = [int(rng.integers(0, vocab)), vocab + 3]
        xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(), history=torch.from_numpy(hist).cuda(),
                               repetition_penalty=pen, eos_ids=eos, apply_min_length=bool(seed % 8 == 1))
        proc = orc.apply_mask(x, mask)
        proc = np.stack([orc.apply_repetition_penalty(orc.apply_min_length(proc[r], 0, 1 if seed % 8 == 1 else 0, eos),
                                                       hist[r], pen) for r in range(rows)])
    use_half = seed % 6 == 5 and xf is None
    if use_half:
        xh = np.clip(x, -60000, 60000).astype(np.float16)
        x = xh
        proc = orc.fp16_to_fp32(xh)
    tok = ctx.argmax(torch.from_numpy(x).cuda(), xf=xf).cpu().numpy()
    assert np.array_equal(tok, orc.argmax_batch(proc))
    if xf is None:
        k = int(rng.choice([1, 2, 7, 50, 64])) if vocab >= 64 else int(rng.integers(1, vocab + 1))
        ttok, tsc = ctx.topk_scores(torch.from_numpy(x).cuda(), k)
        ttok, tsc = ttok.cpu().numpy(), tsc.cpu().numpy()
        for r in range(rows):
            order = np.lexsort((np.arange(vocab), -proc[r].astype(np.float64)))[:k]
            assert np.array_equal(ttok[r], order), r
            assert same_bits(tsc[r], proc[r][order]), r


@pytest.mark.parametrize("seed", range(FIRST, FIRST + max(CASES // 3, 1)))
def test_beam_select_randomised(ctx, orc, seed):
    rng = np.random.default_rng(4000 + seed)
    beams = int(rng.choice([1, 2, 3, 4, 5, 8, 16]))
    batch = int(rng.integers(1, max(64 // beams, 1) // 4 + 2))
    batch = min(batch, 64 // beams)
    vocab = int(rng.choice([v for v in EDGES if v >= 2 * beams] + [2 * beams])) if seed % 2 else int(
        rng.integers(2 * beams, 60000))
    x = random_logits(rng, batch * beams, vocab, seed)
    x = np.where(np.isinf(x), LOWEST, x).astype(np.float32)  # the scorer's inputs are finite in the reference's use
    dtype = np.float16 if seed % 4 == 3 else np.float32
    if dtype == np.float16:
        x = np.clip(x, -60000, 60000).astype(np.float16)
    bs = (rng.standard_normal(batch * beams) * 3).astype(np.float32)
    if seed % 3 == 1:
        bs[:] = 0.0
    if seed % 5 == 2 and beams > 1:
        bs[1::beams] = -1e9
    say("beam_select random", seed, batch, beams, vocab, dtype.__name__)
    sc, tok, idx = ctx.beam_select(torch.from_numpy(x).cuda(), batch, beams, torch.from_numpy(bs).cuda())
    xf = orc.fp16_to_fp32(x) if dtype == np.float16 else x
    osc, otok, oidx, _ = orc.beam_select_top(xf, batch, beams, bs)
    assert np.array_equal(tok.cpu().numpy(), otok)
    assert np.array_equal(idx.cpu().numpy(), oidx)
    assert same_bits(sc.cpu().numpy(), osc)


@pytest.mark.parametrize("seed", range(FIRST, FIRST + max(CASES // 8, 1)))
def test_beam_search_randomised(ctx, orc, seed):
    rng = np.random.default_rng(5000 + seed)
    beams = int(rng.choice([2, 3, 4, 6]))
    batch = int(rng.integers(1, 5))
    vocab = int(rng.choice([2 * beams + 1, 50, 300, 20000, 33001]))
    n_eos = int(rng.integers(1, 3))
    eos = sorted(set(int(v) for v in rng.integers(0, vocab, n_eos)))
    steps = int(rng.integers(2, 12))
    max_length = 3 + steps + int(rng.integers(0, 3))
    lp = float(rng.choice([1.0, 0.6, 2.0, 0.0]))
    say("beam search random", seed, batch, beams, vocab, eos, steps, max_length, lp)
    run_beam_search(ctx, orc, batch, beams, vocab, steps, eos, max_length, lp, bool(seed % 2), 6000 + seed,
                    dtype=np.float32 if seed % 3 else np.float16, eos_boost=float(rng.choice([0.0, 2.5, 6.0])),
                    fused=bool((seed // 2) % 2))


def random_distributions(rng, shape, vocab, sparse):
    z = rng.standard_normal(shape + (vocab,)) * float(rng.choice([0.5, 2.0, 6.0]))
    if sparse:
        z = np.where(rng.random(z.shape) < 0.6, -np.inf, z)
        z[..., 0] = np.where(np.isinf(z).all(-1), 0.0, z[..., 0])
    z = z - z.max(-1, keepdims=True)
    e = np.exp(z)
    return (e / e.sum(-1, keepdims=True)).astype(np.float32)


@pytest.mark.parametrize("seed", range(FIRST, FIRST + max(CASES // 4, 1)))
def test_spec_verify_randomised(ctx, orc, seed):
    rng = np.random.default_rng(7000 + seed)
    batch = int(rng.integers(1, 17))
    K = int(rng.integers(1, 9))
    vocab = int(rng.choice([2, 3, 64, 65, 500, 2047, 2049, 4097, 32064])) if seed % 2 else int(rng.integers(2, 9000))
    if batch * (K + 1) * vocab > 6_000_000:
        batch = max(1, 6_000_000 // ((K + 1) * vocab))
    p = random_distributions(rng, (batch, K + 1), vocab, sparse=seed % 3 == 0)
    if seed % 4 == 0:
        q = random_distributions(rng, (batch, K + 1), vocab, sparse=seed % 3 == 1)
    else:
        q = p.copy()
        noise = rng.random(q.shape) < 0.05
        q = np.where(noise, q * 0.5, q).astype(np.float32)
    if seed % 5 == 0:
        q[0] = p[0]
    draft = np.zeros((batch, K), np.int32)
    for b in range(batch):
        for i in range(K):
            w = q[b, i].astype(np.float64)
            draft[b, i] = rng.choice(vocab, p=w / w.sum()) if seed % 7 else rng.integers(0, vocab)
    uf = rng.random((batch, K)).astype(np.float32)
    ud = rng.random(batch)
    say("spec_verify random", seed, batch, K, vocab)
    acc, tok = ctx.spec_verify(torch.from_numpy(p).cuda(), torch.from_numpy(q).cuda(), torch.from_numpy(draft).cuda(),
                               torch.from_numpy(uf).cuda(), torch.from_numpy(ud).cuda())
    oacc, otok = orc.spec_verify_dense(p, q, draft, uf, ud)
    assert np.array_equal(acc.cpu().numpy(), oacc)
    assert np.array_equal(tok.cpu().numpy(), otok)


@pytest.mark.parametrize("seed", range(FIRST, FIRST + max(CASES // 10, 1)))
def test_kv_gather_randomised(ctx, orc, seed):
    rng = np.random.default_rng(8000 + seed)
    rows = int(rng.integers(1, 33))
    heads, seq, dim = int(rng.integers(1, 5)), int(rng.integers(1, 200)), int(rng.choice([1, 3, 8, 64, 128]))
    elem = [torch.float16, torch.float32, torch.int8][seed % 3]
    n = int(rng.integers(1, 9))
    say("kv_gather random", seed, rows, heads, seq, dim, elem, n)
    present = []
    for _ in range(n):
        raw = torch.from_numpy(rng.integers(-128, 128, (rows, heads, seq, dim * elem.itemsize)).astype(np.int8))
        present.append(raw.cuda().view(elem))
    past = [torch.zeros_like(p) for p in present]
    idx = rng.integers(0, rows, rows).astype(np.int32)
    ctx.kv_gather(present, past, torch.from_numpy(idx).cuda())
    for p, q in zip(present, past):
        assert torch.equal(q.view(torch.int8).cpu(), p.view(torch.int8).cpu()[torch.from_numpy(idx).long()])


def pack_rows(rows_per_seq, cap):
    """[(ids, probs), ...] per sequence -> count [b, n], ids [b, n, cap], probs [b, n, cap] (padded)."""
    b, n = len(rows_per_seq), len(rows_per_seq[0])
    cnt = np.zeros((b, n), np.int32)
    ids = np.full((b, n, cap), -7, np.int32)
    pr = np.zeros((b, n, cap), np.float32)
    for s, rows in enumerate(rows_per_seq):
        for r, (ix, p) in enumerate(rows):
            cnt[s, r] = len(ix)
            ids[s, r, :len(ix)] = ix
            pr[s, r, :len(ix)] = p
    return tuple(torch.from_numpy(t).cuda() for t in (cnt, ids, pr))


def random_round(rng, orc, vocab, K, big):
    def rows(n):
        out = []
        for _ in range(n):
            x = (rng.standard_normal(vocab) * 2).astype(np.float32)
            k = int(rng.choice([0, 1, 2, 5, 50])) if big else int(rng.choice([1, 2, 5, 50]))
            p = float(rng.choice([0.0, 0.6, 0.95])) if k else float(rng.choice([0.5, 0.9]))
            out.append(orc.sampled_categorical(x, k, p, float(rng.choice([0.7, 1.0]))))
        return out
    target, draft = rows(K + 1), rows(K)
    for i in range(K):
        if rng.random() < 0.6:
            draft[i] = (target[i][0].copy(), target[i][1].copy())
            if len(draft[i][0]) > 2 and rng.random() < 0.5:
                draft[i] = (draft[i][0][::-1].copy(), draft[i][1].copy())
    proposal = np.array([d[0][rng.integers(0, len(d[0]))] for d in draft], np.int32)
    for i in range(K):
        if rng.random() < 0.1:
            proposal[i] = rng.integers(0, vocab)
    return proposal, target, draft


@pytest.mark.parametrize("seed", range(FIRST, FIRST + max(CASES // 4, 1)))
def test_spec_verify_sparse_randomised(ctx, orc, seed):
    """The three modes of mi355x_spec_verify_sparse on kept sets (top-k sized, and nucleus sized for every
    fourth seed) against orc_spec_verify_sparse / orc_verify_deterministic: accepted length, final token
    and the number of engine outputs the reference would have consumed."""
    rng = np.random.default_rng(9000 + seed)
    batch = int(rng.integers(1, 7))
    K = int(rng.integers(1, 9))
    big = seed % 4 == 0
    vocab = int(rng.choice([3, 60, 500, 5000])) if not big else 3000
    say("spec_verify_sparse random", seed, batch, K, vocab, big)
    rounds = [random_round(rng, orc, vocab, K, big) for _ in range(batch)]
    cap_t = max(len(r[0]) for _, t, _ in rounds for r in t)
    cap_d = max(len(r[0]) for _, _, d in rounds for r in d)
    target = pack_rows([t for _, t, _ in rounds], cap_t + int(rng.integers(0, 3)))
    draft = pack_rows([d for _, _, d in rounds], cap_d)
    proposal = torch.from_numpy(np.stack([p for p, _, _ in rounds])).cuda()
    au = rng.random((batch, K)).astype(np.float32)
    su = rng.random((batch, K + 1))
    acc, tok, used = ctx.spec_verify_sparse(target, draft, proposal, torch.from_numpy(au).cuda(),
                                            torch.from_numpy(su).cuda(), mode=0)
    for s, (prop, t, d) in enumerate(rounds):
        assert (acc[s].item(), tok[s].item(), used[s].item()) == orc.spec_verify_sparse(prop, t, d, au[s], su[s]), s
    # deterministic proposals: make them likely to match by proposing the oracle's own samples now and then
    acc, tok, used = ctx.spec_verify_sparse(target, None, proposal, None, torch.from_numpy(su).cuda(), mode=1)
    for s, (prop, t, _) in enumerate(rounds):
        want = orc.verify_deterministic(prop, t, su[s])
        assert (acc[s].item(), tok[s].item(), used[s].item()) == (want["accepted"], want["final_token"],
                                                                   2 * want["draws_used"]), s
    # greedy targets
    acc, tok, used = ctx.spec_verify_sparse(target, None, proposal, None, None, mode=2)
    for s, (prop, t, _) in enumerate(rounds):
        n = 0
        while n < K and t[n][0][0] == prop[n]:
            n += 1
        assert (acc[s].item(), tok[s].item(), used[s].item()) == (n, int(t[n][0][0]), 0), s


def test_spec_verify_sparse_end_to_end_with_sampler_outputs(ctx, orc):
    """The verify rows' kept sets come straight from mi355x_sample (device buffers, no host round trip) and
    the proposal is built so that the first positions are accepted; a truncated kept set is reported as -1."""
    say("spec_verify_sparse end to end")
    rng = np.random.default_rng(77)
    batch, K, vocab, cap = 3, 4, 32064, 64
    x = (rng.standard_normal((batch * (K + 1), vocab)) * 3).astype(np.float32)
    u = rng.random(batch * (K + 1))
    _, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=50, p=0.9, temperature=0.8,
                               kept_capacity=cap)
    target = (kc.view(batch, K + 1), ki.view(batch, K + 1, cap), kp.view(batch, K + 1, cap))
    rows = [[orc.sampled_categorical(x[s * (K + 1) + r], 50, 0.9, 0.8) for r in range(K + 1)] for s in range(batch)]
    draft_rows = [[(t[0][:8].copy(), np.full(min(8, len(t[0])), 1.0 / min(8, len(t[0])), np.float32)) for t in seq[:K]]
                  for seq in rows]
    proposal = np.array([[seq[i][0][0] for i in range(K)] for seq in rows], np.int32)  # the targets' best tokens
    proposal[1, 2] = 5  # an id the draft holds and the target row does not: certain reject
    draft_rows[1][2][0][0] = 5
    draft = pack_rows(draft_rows, 8)
    au = rng.random((batch, K)).astype(np.float32)
    su = rng.random((batch, K + 1))
    acc, tok, used = ctx.spec_verify_sparse(target, draft, torch.from_numpy(proposal).cuda(),
                                            torch.from_numpy(au).cuda(), torch.from_numpy(su).cuda(), mode=0)
    for s in range(batch):
        assert (acc[s].item(), tok[s].item(), used[s].item()) == orc.spec_verify_sparse(proposal[s], rows[s], draft_rows[s],
                                                                                        au[s], su[s]), s
    assert acc[1].item() <= 2
    kc2 = kc.clone()
    kc2[K + 2] = cap + 1  # sequence 1, row 1 claims more entries than the buffers hold
    acc, tok, used = ctx.spec_verify_sparse((kc2.view(batch, K + 1), target[1], target[2]), draft,
                                            torch.from_numpy(proposal).cuda(), torch.from_numpy(au).cuda(),
                                            torch.from_numpy(su).cuda(), mode=0)
    assert acc[1].item() == -1 and tok[1].item() == -1 and acc[0].item() >= 0
