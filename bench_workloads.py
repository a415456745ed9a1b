"""Timing of the non-headline configurations (greedy, beam search + KV gather, speculative
verification, constrained nucleus sampling) for bench.py --workload c1|c3|c4|c5.  Same protocol as
the headline run: seeded synthetic inputs resident in HBM, untimed warm-up, HIP events on the launch
stream around exactly K steps, a parity gate against the CPU oracle before any number is returned,
and the oracle timed on one host core as the CPU baseline."""
import os
import time

import numpy as np
import torch

HBM_PEAK_GBS = 8000.0
# HBM bytes per step from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of these same commands, scaled by a
# known-size copy; counters cannot be read from inside the process, so these are offline profile constants.
# c3: KV gather 6.22 GB + selection kernels 0.04 GB; c5: the one sparse-mask kernel; topp: stream (fetch + write) and
# finish kernel.  None where no counter run exists.
MEASURED_TRAFFIC = {"c3": 6_222_000_000 + 42_000_000, "c5": 203_900_000, "topp": 33_000_000 + 5_300_000 + 9_200_000}
TRAFFIC_SOURCE = {"c3": "offline profile constant: profiles/beam_step_kernels_config3.md",
                  "c5": "offline profile constant: profiles/nucleus_sparse_kernel_config5.md",
                  "topp": "offline profile constant: profiles/nucleus_stream_and_finish_kernels_top_p_and_large_k.md"}

def _timed(fn_step, K, W, graph=True):
    """Runs W warm-up steps, then K steps between two events; with graph=True the K steps are
    captured once and replayed (first replay untimed)."""
    for i in range(W):
        fn_step(i)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    R = 1
    with torch.cuda.stream(side):
        if graph:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                for i in range(W, W + K):
                    fn_step(i)
            g.replay()
            side.synchronize()
            R = max(8, -(-1024 // K))  # replays inside the timed region, as in the headline run
            start.record(side)
            for _ in range(R):
                g.replay()
            end.record(side)
        else:
            start.record(side)
            for i in range(W, W + K):
                fn_step(i)
            end.record(side)
        side.synchronize()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / R


def _line(args, metric, unit, value, ms_total, K, W, dtype, workload, extra, algo_bytes, cpu):
    ms = ms_total / K
    achieved = algo_bytes / (ms * 1e-3) / 1e9
    return {
        "metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": ms, "step_latency_us": ms * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": dict({"workload": workload}, **extra),
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC.get(args.workload),
                     "traffic_source": TRAFFIC_SOURCE.get(args.workload),
                     "algorithmic_bytes_per_step": algo_bytes},
        "cpu_baseline": cpu,
    }


def _cpu(value, unit, sample, ms_per_step):
    return {"value": value, "unit": unit, "cores": 1, "kind": "port", "sample": sample,
            "ms_per_step": ms_per_step, "host_cpus": os.cpu_count()}


def c1(args, pkg, orc, dev):
    """Greedy, batch 1 x vocab 32064, repetition penalty 1.1 over 512 history ids, 256 steps."""
    V, H = 32064, 512
    K = args.steps if args.steps != 128 else 256
    W = args.warmup
    g = torch.Generator(device=dev).manual_seed(11)
    pool = 64
    logits = torch.randn(pool, 1, V, generator=g, device=dev) * 2.0
    spikes = torch.randint(0, V, (pool,), generator=g, device=dev)
    logits[torch.arange(pool, device=dev), 0, spikes] += 8.0
    hist = torch.randint(0, V, (1, H), generator=g, device=dev, dtype=torch.int32)
    xf = pkg.LogitsXform(history=hist, repetition_penalty=1.1)
    ctx = pkg.SearchContext(1, V)
    out = torch.empty((K + W, 1), dtype=torch.int32, device=dev)
    ms = _timed(lambda i: ctx.argmax(logits[i % pool], xf=xf, out=out[i]), K, W)
    n = min(K, 64)
    hh = hist.cpu().numpy()[0]
    rows = [logits[(W + i) % pool, 0].cpu().numpy() for i in range(n)]
    t0 = time.perf_counter()
    want = []
    for r in rows:
        want.append(orc.argmax(orc.apply_repetition_penalty(r, hh, 1.1)))
    cpu_s = time.perf_counter() - t0
    got = out[W:W + n, 0].cpu().numpy()
    assert np.array_equal(got, np.array(want, np.int32)), "PARITY FAILURE (c1)"
    algo = V * 4 + H * 4 + 4
    return _line(args, "greedy tokens/sec + step latency, B=1 V=32064 with repetition penalty", "tokens/s",
                 K / (ms * 1e-3), ms, K, W, "f32",
                 "config 1: greedy argmax with fused repetition penalty 1.1 over 512 ids, batch 1 x vocab 32064, "
                 "%d steps replayed from a HIP graph (latency-bound: 130 KB per step)" % K,
                 {"parity": "%d steps bit-identical to the CPU oracle" % n}, algo,
                 _cpu(n / cpu_s, "tokens/s", "%d of the timed steps, penalty + argmax, one thread" % n, cpu_s / n * 1e3))


def c3(args, pkg, orc, orc_lib, dev):
    """Beam search, batch 8 x 4 beams, vocab 151936 fp16, plus the KV gather over 56 tensors of
    [32, 4, 2048, 128] fp16 per step."""
    B, NB, V, L2, MAXLEN = 8, 4, 151936, 56, 96
    BB = B * NB
    K = min(args.steps, 88) if args.steps != 128 else 64  # the sequences hold 96 tokens: prompt 3 + warm-up 4 + K
    W = min(args.warmup, 4)
    g = torch.Generator(device=dev).manual_seed(3)
    pool = 16
    logits = [(torch.randn(BB, V, generator=g, device=dev) * 2.0).half() for _ in range(pool)]
    ctx = pkg.SearchContext(BB, V)

    def new_scorer():
        s = pkg.BeamScorer(ctx, B, NB, MAXLEN, 0, [V - 1], 1.0, True)
        s.set_prompt(np.arange(B * 3, dtype=np.int32).reshape(B, 3))
        return s

    # ---- parity: 4 steps of selection + scorer against the oracle ---------------------------------
    scorer = new_scorer()
    ref = orc_lib.BeamScorer(orc, B, NB, MAXLEN, 0, [V - 1], 1.0, True)
    seq = np.zeros((BB, MAXLEN), np.int32)
    seq[:, :3] = np.repeat(np.arange(B * 3, dtype=np.int32).reshape(B, 3), NB, axis=0)
    length, cpu_s, n_cpu = 3, 0.0, 4
    for i in range(n_cpu):
        sc, tok, idx = ctx.beam_select(logits[i], B, NB, scorer.next_scores)
        scorer.step(sc, tok, idx)
        x32 = orc.fp16_to_fp32(logits[i].cpu().numpy())
        t0 = time.perf_counter()
        osc, otok, oidx, _ = orc.beam_select_top(x32, B, NB, ref.next_scores)
        ref.process(seq, length, osc, otok, oidx)
        nxt = np.zeros_like(seq)
        orc.lib.orc_beam_append(seq.reshape(-1), nxt.reshape(-1), BB, MAXLEN, length, ref.next_indices, ref.next_tokens)
        cpu_s += time.perf_counter() - t0
        seq, length = nxt, length + 1
        assert np.array_equal(tok.cpu().numpy(), otok) and np.array_equal(idx.cpu().numpy(), oidx), "PARITY FAILURE (c3 select)"
        assert np.array_equal(scorer.next_tokens.cpu().numpy(), ref.next_tokens), "PARITY FAILURE (c3 scorer)"
        assert np.array_equal(scorer.next_indices.cpu().numpy(), ref.next_indices), "PARITY FAILURE (c3 scorer)"
    scorer.close()

    # ---- phase 1: selection + scorer --------------------------------------------------------------
    scorer = new_scorer()

    def select_step(i):
        scorer.search_step(logits[i % pool])  # BeamSearch_Cpu::SelectTop in one call: selection + scorer step

    # launched eagerly, as a host loop does: the scorer's step takes the sequence length by value
    ms_sel = _timed(select_step, K, W, graph=False)
    beam_idx = scorer.next_indices.clone()
    # ---- phase 2: KV gather ------------------------------------------------------------------------
    shape = (BB, 4, 2048, 128)
    present = [torch.randint(-30000, 30000, shape, generator=g, device=dev, dtype=torch.int16).view(torch.float16)
               for _ in range(L2)]
    past = [torch.empty_like(p) for p in present]
    ms_kv = _timed(lambda i: ctx.kv_gather(present, past, beam_idx), K, W, graph=False)
    for t in (0, L2 - 1):
        assert torch.equal(past[t].view(torch.int16), present[t].view(torch.int16)[beam_idx.long()]), "PARITY FAILURE (c3 gather)"
    # CPU gather baseline on a bounded sample: 2 of the 56 tensors
    sample = [present[t].cpu().numpy().view(np.uint16) for t in range(2)]
    bi = beam_idx.cpu().numpy()
    t0 = time.perf_counter()
    for s in sample:
        orc.kv_gather(s, bi)
    cpu_kv = (time.perf_counter() - t0) * (L2 / 2)
    sel_bytes = BB * V * 2
    kv_bytes = 2 * L2 * int(np.prod(shape)) * 2
    ms = ms_sel + ms_kv
    out = _line(args, "beam-search steps/sec, B=8 beams=4 V=151936 fp16 incl. KV gather", "steps/s",
                K / (ms * 1e-3), ms, K, W, "f16",
                "config 3: log-softmax + top-8 per batch + BeamSearchScorer (%d steps) and KV gather of 56 tensors "
                "[32,4,2048,128] fp16 (%d steps), phases timed separately and summed" % (K, K),
                {"select_ms_per_step": ms_sel / K, "kv_gather_ms_per_step": ms_kv / K,
                 "select_GBps": sel_bytes / (ms_sel / K * 1e-3) / 1e9,
                 "kv_gather_GBps": kv_bytes / (ms_kv / K * 1e-3) / 1e9,
                 "kv_gather_frac_of_peak": kv_bytes / (ms_kv / K * 1e-3) / 1e9 / HBM_PEAK_GBS,
                 "parity": "%d selection+scorer steps identical to the CPU oracle; gathered tensors byte-identical to "
                           "an index_select" % n_cpu}, sel_bytes + kv_bytes,
                _cpu(1.0 / (cpu_s / n_cpu + cpu_kv), "steps/s",
                     "%d selection+scorer steps and the gather of 2 of 56 tensors (scaled x28), one thread" % n_cpu,
                     (cpu_s / n_cpu + cpu_kv) * 1e3))
    return out


def softmax64(x):
    z = x - x.max(-1, keepdims=True)
    e = np.exp(z)
    return (e / e.sum(-1, keepdims=True)).astype(np.float32)


def c4(args, pkg, orc, dev):
    """Speculative-decoding verification, batch 16, draft length 8, vocab 32064."""
    B, Kd, V = 16, 8, 32064
    K, W = args.steps, args.warmup
    rng = np.random.default_rng(4)
    pool = 8
    cases = []
    for _ in range(pool):
        lt = rng.standard_normal((B, Kd + 1, V)) * 2
        p = softmax64(lt)
        q = softmax64(lt + rng.standard_normal((B, Kd + 1, V)) * 0.5)
        cdf = np.cumsum(q[:, :Kd].astype(np.float64), -1)
        uu = rng.random((B, Kd, 1)) * cdf[..., -1:]
        draft = np.minimum((cdf < uu).sum(-1), V - 1).astype(np.int32)
        uf = rng.random((B, Kd)).astype(np.float32)
        ud = rng.random(B)
        cases.append((p, q, draft, uf, ud))
    devc = [tuple(torch.from_numpy(a).to(dev) for a in c) for c in cases]
    ctx = pkg.SearchContext(B, V)
    outs = {}

    def step(i):
        outs[i % pool] = ctx.spec_verify(*devc[i % pool])

    ms = _timed(step, K, W)
    t0 = time.perf_counter()
    want = [orc.spec_verify_dense(*c) for c in cases]
    cpu_s = time.perf_counter() - t0
    accepted = 0
    for j in range(pool):
        acc, tok = outs[j]
        assert np.array_equal(acc.cpu().numpy(), want[j][0]) and np.array_equal(tok.cpu().numpy(), want[j][1]), "PARITY FAILURE (c4)"
        accepted += int(want[j][0].sum())
    algo = B * (Kd * 16 + 2 * V * 4)
    return _line(args, "speculative verification rounds/sec, B=16 K=8 V=32064", "rounds/s",
                 B * K / (ms * 1e-3), ms, K, W, "f32",
                 "config 4: accept loop + residual/bonus resampling on dense [16,9,32064] fp32 target/draft "
                 "probabilities, %d steps replayed from a HIP graph (latency-bound)" % K,
                 {"mean_accepted_len": accepted / (pool * B),
                  "parity": "accepted lengths and tokens of %d distinct inputs identical to the CPU oracle" % pool}, algo,
                 _cpu(B * pool / cpu_s, "rounds/s", "%d inputs, orc_spec_verify_dense, one thread" % pool, cpu_s / pool * 1e3))


def c5(args, pkg, orc, dev):
    """Constrained nucleus sampling, batch 256 x vocab 201088, 5 % mask, penalty 1.2 over 1024 ids."""
    B, V, H = 256, 201088, 1024
    K = args.steps if args.steps != 128 else 32
    W = min(args.warmup, 4)
    words = (V - 1) // 32 + 1
    g = torch.Generator(device=dev).manual_seed(5)
    pool = 4
    logits = [torch.randn(B, V, generator=g, device=dev) * 3.0 for _ in range(pool)]
    bits = (torch.rand(B, words * 32, generator=g, device=dev) < 0.05)
    bits[:, 0] = True
    weights = (2 ** torch.arange(32, device=dev, dtype=torch.int64))
    mask = (bits.view(B, words, 32).long() * weights).sum(-1)
    mask = torch.where(mask >= 2 ** 31, mask - 2 ** 32, mask).int().contiguous()
    hist = torch.randint(0, V, (B, H), generator=g, device=dev, dtype=torch.int32)
    # the grammar engine builds the mask on the host and knows how many ids it allows; here the count is taken
    # from the synthetic mask once, outside the timed region
    allowed_max = int(bits.sum(dim=1).max().item())
    xf = pkg.LogitsXform(mask=mask, history=hist, repetition_penalty=1.2, mask_allowed_max=allowed_max)
    del bits
    u_host = np.random.default_rng(55).random((K + W, B))
    uniforms = torch.from_numpy(u_host).to(dev)
    tokens = torch.empty((K + W, B), dtype=torch.int32, device=dev)
    ctx = pkg.SearchContext(B, V)
    ms = _timed(lambda i: ctx.sample(logits[i % pool], uniforms[i], k=0, p=0.95, temperature=1.0, xf=xf, out=tokens[i]),
                K, W)
    rows_cpu = B  # every row of the checked step (about 1.3 s of oracle time)
    x = logits[W % pool][:rows_cpu].cpu().numpy()
    m = mask[:rows_cpu].cpu().numpy().view(np.uint32)
    hh = hist[:rows_cpu].cpu().numpy()
    t0 = time.perf_counter()
    x = orc.apply_mask(x, m)
    want = []
    for r in range(rows_cpu):
        want.append(orc.sample_row(orc.apply_repetition_penalty(x[r], hh[r], 1.2), 0, 0.95, 1.0, u_host[W, r]))
    cpu_s = time.perf_counter() - t0
    got = tokens[W, :rows_cpu].cpu().numpy()
    assert np.array_equal(got, np.array(want, np.int32)), "PARITY FAILURE (c5)"
    algo = B * V * 4 + B * words * 4 + B * H * 4
    return _line(args, "sampled tokens/sec + step latency, B=256 V=201088 masked top-p", "tokens/s",
                 B * K / (ms * 1e-3), ms, K, W, "f32",
                 "config 5: grammar mask (5%% allowed, at most %d ids per row, passed as mask_allowed_max) + repetition "
                 "penalty 1.2 over 1024 ids + nucleus p=0.95 T=1.0, batch 256 x vocab 201088, %d steps replayed from a "
                 "HIP graph over %d logits buffers" % (allowed_max, K, pool),
                 {"general_path_rows": ctx.fallback_rows(),
                  "parity": "%d rows of one step bit-identical to the CPU oracle" % rows_cpu}, algo,
                 _cpu(rows_cpu / cpu_s, "tokens/s", "the %d rows of one step, one thread" % rows_cpu,
                      cpu_s / rows_cpu * B * 1e3))


def topp(args, pkg, orc, dev, k=0, sigma=5.0):
    """The reference's other sampling modes on config 2's shape (batch 64 x vocab 128256 fp32): unmasked top-p
    (SampleTopP: k = 0, p = 0.9, T = 1.0) and, with k = 1024, top-k beyond the 64 ids the fused kernel ranks; with
    sigma = 2 the rows are so flat that a nucleus holds 56 000 tokens, several times what the finish kernel sorts at
    once.  Not a configuration of the headline metric: a workload to profile and to report next to it."""
    B, V = 64, 128256
    K = args.steps if args.steps != 128 else 32
    W = min(args.warmup, 4)
    g = torch.Generator(device=dev).manual_seed(9)
    pool = 8
    logits = [torch.randn(B, V, generator=g, device=dev) * sigma for _ in range(pool)]
    u_host = np.random.default_rng(99).random((K + W, B))
    uniforms = torch.from_numpy(u_host).to(dev)
    tokens = torch.empty((K + W, B), dtype=torch.int32, device=dev)
    ctx = pkg.SearchContext(B, V)
    ms = _timed(lambda i: ctx.sample(logits[i % pool], uniforms[i], k=k, p=0.9, temperature=1.0, out=tokens[i]), K, W)
    rows_cpu = 16 if sigma >= 5.0 else 8
    x = logits[W % pool][:rows_cpu].cpu().numpy()
    t0 = time.perf_counter()
    want = [orc.sample_row(x[r], k, 0.9, 1.0, u_host[W, r]) for r in range(rows_cpu)]
    cpu_s = time.perf_counter() - t0
    got = tokens[W, :rows_cpu].cpu().numpy()
    assert np.array_equal(got, np.array(want, np.int32)), "PARITY FAILURE (top-p / large k)"
    what = "unmasked top-p, p=0.9 T=1.0" if k == 0 else "top-k k=%d with p=0.9 T=1.0" % k
    return _line(args, "sampled tokens/sec + step latency, B=64 V=128256 " + ("top-p" if k == 0 else "k=%d" % k) +
                 (" (wide nuclei)" if sigma < 5.0 else ""), "tokens/s",
                 B * K / (ms * 1e-3), ms, K, W, "f32",
                 "%s, batch 64 x vocab 128256 fp32 (logits N(0, %g^2)), %d steps replayed from a HIP graph over %d logits "
                 "buffers" % (what, sigma, K, pool),
                 {"general_path_rows": ctx.fallback_rows(),
                  "parity": "%d rows of one step bit-identical to the CPU oracle" % rows_cpu}, B * V * 4,
                 _cpu(rows_cpu / cpu_s, "tokens/s", "%d rows of one step, one thread" % rows_cpu, cpu_s / rows_cpu * B * 1e3))


def variant(args, pkg, orc, dev, name):
    """Two workloads beside the configurations: `odd_vocab`, config 2's parameters on 64 x 50257 rows (GPT-2's
    vocabulary: rows 50257 fp32 elements apart start on every 4-byte offset of a 16-byte line), and `mixed_modes`,
    64 x 128256 rows whose per-row parameters put them in four selection modes (k = 50 with p = 0.9, top-p only,
    greedy, k = 200), whose kernels run side by side."""
    B = 64
    V = 50257 if name == "odd_vocab" else 128256
    K = args.steps if args.steps != 128 else 32
    W = min(args.warmup, 4)
    g = torch.Generator(device=dev).manual_seed(13)
    pool = 8
    logits = [torch.randn(B, V, generator=g, device=dev) * 5.0 for _ in range(pool)]
    u_host = np.random.default_rng(77).random((K + W, B))
    uniforms = torch.from_numpy(u_host).to(dev)
    tokens = torch.empty((K + W, B), dtype=torch.int32, device=dev)
    ctx = pkg.SearchContext(B, V)
    menu = [(50, 0.9, 0.7), (0, 0.9, 1.0), (1, 0.0, 1.0), (200, 0.95, 1.0)]
    params = [menu[0]] * B if name == "odd_vocab" else [menu[r % 4] for r in range(B)]
    if name == "odd_vocab":
        step = lambda i: ctx.sample(logits[i % pool], uniforms[i], k=50, p=0.9, temperature=0.7, out=tokens[i])
    else:
        step = lambda i: ctx.sample(logits[i % pool], uniforms[i], per_row=params, out=tokens[i])
    ms = _timed(step, K, W)
    rows_cpu = 16
    x = logits[W % pool][:rows_cpu].cpu().numpy()
    t0 = time.perf_counter()
    want = [orc.sample_row(x[r], *params[r], u_host[W, r]) for r in range(rows_cpu)]
    cpu_s = time.perf_counter() - t0
    got = tokens[W, :rows_cpu].cpu().numpy()
    assert np.array_equal(got, np.array(want, np.int32)), "PARITY FAILURE (%s)" % name
    what = ("top-k/top-p sampling (T=0.7 k=50 p=0.9), batch 64 x vocab 50257 fp32: rows off 16-byte boundaries"
            if name == "odd_vocab" else
            "rows in four selection modes (k=50 p=0.9 T=0.7 / top-p 0.9 / greedy / k=200 p=0.95), batch 64 x vocab 128256 fp32")
    return _line(args, "sampled tokens/sec + step latency, " + ("B=64 V=50257 top-k/p" if name == "odd_vocab" else "B=64 V=128256 mixed modes"),
                 "tokens/s", B * K / (ms * 1e-3), ms, K, W, "f32",
                 "%s, %d steps replayed from a HIP graph over %d logits buffers" % (what, K, pool),
                 {"general_path_rows": ctx.fallback_rows(),
                  "parity": "%d rows of one step bit-identical to the CPU oracle" % rows_cpu}, B * V * 4,
                 _cpu(rows_cpu / cpu_s, "tokens/s", "%d rows of one step, one thread" % rows_cpu, cpu_s / rows_cpu * B * 1e3))


def run(args, pkg, orc, orc_lib, dev):
    if args.workload in ("odd_vocab", "mixed_modes"):
        return variant(args, pkg, orc, dev, args.workload)
    if args.workload == "topp":
        return topp(args, pkg, orc, dev)
    if args.workload == "largek":
        return topp(args, pkg, orc, dev, k=1024)
    if args.workload == "topp_wide":
        return topp(args, pkg, orc, dev, sigma=2.0)
    if args.workload == "c1":
        return c1(args, pkg, orc, dev)
    if args.workload == "c3":
        return c3(args, pkg, orc, orc_lib, dev)
    if args.workload == "c4":
        return c4(args, pkg, orc, dev)
    return c5(args, pkg, orc, dev)
