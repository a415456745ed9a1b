"""Every benchmark configuration at its FULL size, one step each, through the C ABI against the CPU oracle
(configuration 2 and the selection phase of 3 are covered at full size in test_gpu_sampling.py /
test_gpu_beam_spec.py; here: all 256 rows of configuration 5, a heterogeneous batch of more than 64 rows
at a 128K vocabulary, exact sums over more segments than the GPU runs at once, and the 56-tensor KV gather of
configuration 3), and configurations 1 and 3 as whole runs of all their steps, where every step's state feeds
the next."""
import numpy as np
import pytest
import torch

from gpu_common import make_mask, pkg, say

pytestmark = pytest.mark.gpu


def bits(a):
    return np.asarray(a, np.float32).view(np.uint32)


def test_config5_all_256_rows(orc):
    """256 x 201088 fp32 ~N(0, 3^2), 5 % grammar mask, repetition penalty 1.2 over 1024 ids per row, top-p
    0.95 at T=1: token, kept count, kept ids and probability bits of every row."""
    say("config5 full batch")
    rng = np.random.default_rng(55)
    rows, vocab = 256, 201088
    ctx = pkg().SearchContext(rows, vocab)
    x = rng.standard_normal((rows, vocab), dtype=np.float32) * np.float32(3)
    mask = make_mask(rng, rows, vocab, 0.05)
    hist = rng.integers(0, vocab, (rows, 1024)).astype(np.int32)
    u = rng.random(rows)
    xf = pkg().LogitsXform(mask=torch.from_numpy(mask.view(np.int32)).cuda(),
                           history=torch.from_numpy(hist).cuda(), repetition_penalty=1.2)
    before = ctx.fallback_rows()
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), k=0, p=0.95,
                                 temperature=1.0, xf=xf, kept_capacity=12288)
    tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    assert ctx.fallback_rows() == before, "a row left the fast path"
    proc = orc.apply_mask(x, mask)
    for r in range(rows):
        row = orc.apply_repetition_penalty(proc[r], hist[r], 1.2)
        idx, probs = orc.sampled_categorical(row, 0, 0.95, 1.0)
        n = len(idx)
        assert kc[r] == n and 1000 < n <= 12288, (r, kc[r], n)
        assert np.array_equal(ki[r, :n], idx), r
        assert np.array_equal(bits(kp[r, :n]), bits(probs)), r
        assert tok[r] == idx[orc.discrete_draw(probs, u[r])], r
    ctx.close()


def test_heterogeneous_batch_of_96_rows_at_128k_vocab(orc):
    """More than 64 rows (the per-row parameters travel through the context's device table) of 128256
    logits with every selection mode mixed: greedy, top-k <= 64 with and without top-p, 64 < k <= 512,
    k above that (exact path), nucleus."""
    say("heterogeneous 96 x 128256")
    rng = np.random.default_rng(96)
    rows, vocab = 96, 128256
    ctx = pkg().SearchContext(rows, vocab)
    x = rng.standard_normal((rows, vocab), dtype=np.float32) * np.float32(3)
    x[np.arange(rows)[:, None], rng.integers(0, vocab, (rows, 8))] += 10.0
    u = rng.random(rows)
    menu = [(1, 0.0, 1.0), (50, 0.9, 0.7), (40, 0.0, 1.3), (64, 0.95, 0.8), (0, 0.9, 1.0), (0, 0.5, 0.6),
            (100, 0.9, 1.0), (512, 0.0, 0.9), (2, 1.0, 1.0), (7, 0.3, 2.0), (600, 0.9, 1.0), (0, 0.0, 1.0)]
    per_row = [menu[(r * 5 + r // 12) % len(menu)] for r in range(rows)]
    cap = 1024
    tok, kc, ki, kp = ctx.sample(torch.from_numpy(x).cuda(), torch.from_numpy(u).cuda(), per_row=per_row,
                                 kept_capacity=cap)
    tok, kc, ki, kp = tok.cpu().numpy(), kc.cpu().numpy(), ki.cpu().numpy(), kp.cpu().numpy()
    assert len(set(per_row)) == len(menu)
    for r, (k, p, t) in enumerate(per_row):
        idx, probs = orc.sampled_categorical(x[r], k, p, t)
        n = min(len(idx), cap)
        assert kc[r] == len(idx), (r, per_row[r])
        assert np.array_equal(ki[r, :n], idx[:n]), (r, per_row[r])
        assert np.array_equal(bits(kp[r, :n]), bits(probs[:n])), (r, per_row[r])
        assert tok[r] == idx[orc.discrete_draw(probs, u[r])], (r, per_row[r])
    ctx.close()


def test_exact_sums_of_more_segments_than_the_gpu_runs_at_once(orc):
    """Log-softmax of 256 rows x 151936: 9728 segment workgroups in one launch, several times what the GPU holds
    at once, each waiting for the sums of its row's earlier segments that the same launch publishes.  The rows repeat
    six distinct ones (softmax-like, constant, sparse with -inf, tiny and huge spreads), so six oracle rows pin all
    256; a second call on the same context checks the state the first one left behind."""
    say("softmax 256 x 151936")
    rng = np.random.default_rng(77)
    rows, vocab = 256, 151936
    ctx = pkg().SearchContext(rows, vocab)
    base = np.empty((6, vocab), np.float32)
    base[0] = rng.standard_normal(vocab) * 2
    base[1] = -1.25
    base[2] = np.where(rng.random(vocab) < 0.8, -np.inf, rng.standard_normal(vocab) * 4).astype(np.float32)
    base[3] = rng.standard_normal(vocab) * 1e-4
    base[4] = rng.standard_normal(vocab) * 40
    base[5] = np.linspace(-30, 0, vocab)
    want = [orc.log_softmax(base[i], 1.0) for i in range(6)]
    pick = rng.integers(0, 6, rows)
    x = torch.from_numpy(base[pick]).cuda()
    for call in range(2):
        got = ctx.softmax(x.clone(), 1.0, log=True).cpu().numpy()
        for r in range(rows):
            assert np.array_equal(bits(got[r]), bits(want[pick[r]])), (call, r, int(pick[r]))
    ctx.close()


def test_config3_kv_gather_all_56_tensors():
    """The whole KV reorder of one configuration-3 step: 28 layers x (key, value) tensors
    [32, 4, 2048, 128] fp16 (64 MiB each, 3.76 GB read and written), every byte compared with torch indexing."""
    say("kv_gather 56 tensors of 64 MiB")
    ctx = pkg().SearchContext(32, 1024)
    g = torch.Generator(device="cuda").manual_seed(3)
    present = [torch.randint(-32768, 32767, (32, 4, 2048, 128), generator=g, device="cuda", dtype=torch.int16)
               .view(torch.float16) for _ in range(56)]
    past = [torch.zeros_like(p) for p in present]
    idx = torch.tensor([b * 4 + int(j) for b in range(8) for j in torch.randint(0, 4, (4,), generator=torch.Generator().manual_seed(b))],
                       dtype=torch.int32, device="cuda")  # beams of an entry continue beams of the same entry
    ctx.kv_gather(present, past, idx)
    torch.cuda.synchronize()
    for t, (p, q) in enumerate(zip(present, past)):
        assert torch.equal(q.view(torch.int16), p.view(torch.int16)[idx.long()]), t
    ctx.close()


def test_config1_whole_run_of_256_steps_with_growing_history(orc):
    """Benchmark configuration 1 as a whole generation, not step by step: batch 1, vocab 32064, greedy with
    repetition penalty 1.1 over everything generated so far (a 256-token prompt, then 256 steps), EOS check, pad and
    append on the device.  The state a step leaves (the sequence, which is the next step's history; the EOS flag)
    feeds the next one on both sides; the sequences must agree token for token to the end, where a boosted EOS ends
    the run."""
    say("config1 whole run")
    rng = np.random.default_rng(101)
    vocab, prompt_len, steps, eos, pad = 32064, 256, 256, 17, 0
    max_length = prompt_len + steps
    ctx = pkg().SearchContext(1, vocab)
    prompt = rng.integers(0, vocab, prompt_len).astype(np.int32)
    prompt[prompt == eos] = eos + 1
    seq = np.zeros(max_length, np.int32)
    seq[:prompt_len] = prompt
    d_seq = torch.zeros((1, max_length), dtype=torch.int32, device="cuda")
    d_seq[0, :prompt_len] = torch.from_numpy(prompt).cuda()
    d_seen = torch.zeros(1, dtype=torch.int32, device="cuda")
    d_done = torch.zeros(1, dtype=torch.int32, device="cuda")
    length, ended_at = prompt_len, None
    for step in range(steps):
        x = (rng.standard_normal((1, vocab)) * 2).astype(np.float32)
        x[0, rng.integers(0, vocab)] += 8
        if step % 3 == 0:  # a token already generated gets the spike: the penalty decides whether it still wins
            x[0, seq[rng.integers(0, length)]] += 9
        if step == steps - 6:
            x[0, eos] += 40
        xf = pkg().LogitsXform(history=d_seq[:, :length].contiguous(), repetition_penalty=1.1)
        tok = ctx.argmax(torch.from_numpy(x).cuda(), xf=xf)
        ctx.greedy_tail(tok, d_seen, [eos], pad, d_seq, length, d_done)
        want = orc.argmax(orc.apply_repetition_penalty(x[0], seq[:length], 1.1))
        assert tok.item() == want, step
        if want == eos:
            ended_at = step
            assert d_done.item() == 1 and d_seen.item() == 1
            break
        assert d_done.item() == 0
        seq[length] = want
        length += 1
        if step % 32 == 31:
            assert np.array_equal(d_seq[0, :length].cpu().numpy(), seq[:length]), step
    assert ended_at == steps - 6
    assert np.array_equal(d_seq[0, :length].cpu().numpy(), seq[:length])
    ctx.close()


def test_config3_whole_beam_search_of_64_steps(orc):
    """Benchmark configuration 3 as a whole search: batch 8, beams 4, vocab 151936 fp16, length penalty 1.0, all 64
    steps through the fused per-step call, with an EOS boosted just enough that hypotheses finish along the way
    while the search runs its full length.  After every step the scorer's state and the beam-reordered sequences
    equal the oracle's; at the end the hypotheses do."""
    from test_gpu_beam_spec import run_beam_search
    say("config3 whole search")
    ctx = pkg().SearchContext(32, 151936)
    steps, finished_early = run_beam_search(ctx, orc, 8, 4, 151936, 64, [151935], 80, 1.0, False, 33, eos_boost=3.0,
                                            fused=True)
    ctx.close()
    assert steps == 64 and finished_early >= 4, (steps, finished_early)
