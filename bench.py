#!/usr/bin/env python3
"""Headline benchmark: top-k/top-p sampling step, batch 64 x vocab 128256 (Benchmark configuration 2).

A step is one pass of the sampling hot path (mi355x_sample: fused selection + softmax + nucleus cut +
categorical draw) over one batch of seeded synthetic fp32 logits resident in HBM.  The K timed steps
are recorded once into a HIP graph (one kernel launch per step, each on its own logits buffer from a
pool larger than twice the 256 MB Infinity Cache) and replayed between two HIP events on the launch
stream.  Before any number is printed, token ids of the checked steps are compared with the CPU
oracle on identical logits and uniforms and, where the reference's own headers were compiled into
oracle/_ref, with the reference's ComputeSampledCategorical + SampleCategoricalToken driven by
std::mt19937 engines of the same seeds; that reference build (else the oracle), timed on one host
core, is the cpu_baseline.  Prints ONE JSON line."""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

ROWS, VOCAB, TOP_K, TOP_P, TEMP = 64, 128256, 50, 0.9, 0.7
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the dominant kernel (fetch 33.26 MB + write 0.20 MB), a constant taken from the
# rocprofv3 --pmc summary named below: counters cannot be read from inside this process.
MEASURED_TRAFFIC_BYTES = 33_460_000
TRAFFIC_SOURCE = "offline profile constant: profiles/sample_fused_kernel_config2_pmc.md"


def replays_for(K):
    """Replays of a K-step graph inside one timed region: at least 8, and at least 1024 steps in all."""
    return max(8, -(-1024 // K))


def time_fp16_steps(torch, np, orc, ctx, side, logits, uniforms, u_host, W, K, pool, n_cpu):
    """The same K steps on fp16 copies of the logits, read directly by the sampling kernel (no widening pass):
    graph replay between two events as for the fp32 run; the tokens of the first n_cpu steps must equal the CPU
    oracle's on the rows widened as the reference's CPU path widens them.  Returns milliseconds for the K steps."""
    half = [x.half() for x in logits]
    tok16 = torch.empty((K + W, ROWS), dtype=torch.int32, device=uniforms.device)

    def step16(i):
        ctx.sample(half[i % pool], uniforms[i], k=TOP_K, p=TOP_P, temperature=TEMP, out=tok16[i])

    with torch.cuda.stream(side):
        for i in range(W):
            step16(i)
        side.synchronize()
        g16 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g16, stream=side):
            for i in range(W, W + K):
                step16(i)
        g16.replay()
        side.synchronize()
        R = replays_for(K)
        s16, e16 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s16.record(side)
        for _ in range(R):
            g16.replay()
        e16.record(side)
        side.synchronize()
    torch.cuda.synchronize()
    n = min(n_cpu, 4)
    for i in range(n):
        wide = orc.fp16_to_fp32(half[(W + i) % pool].cpu().numpy())
        want = orc.sample_batch(wide, TOP_K, TOP_P, TEMP, u_host[W + i])
        if not np.array_equal(tok16[W + i].cpu().numpy(), want):
            sys.exit("PARITY FAILURE: tokens sampled from fp16 logits differ from the CPU oracle on the widened rows")
    return s16.elapsed_time(e16) / R, n


def time_batches_in_flight(torch, pkg, ctx, side, n_streams, logits, uniforms, tokens, pool, W, K):
    """Times the K steps issued round-robin over n_streams streams / contexts in one HIP graph and checks
    that the tokens equal those of the sequential run already in `tokens`.  Returns milliseconds."""
    seq_tokens = tokens[W:W + K].clone()
    tokens[W:W + K].zero_()
    ctxs = [ctx] + [pkg.SearchContext(ROWS, VOCAB) for _ in range(n_streams - 1)]
    streams = [side] + [torch.cuda.Stream() for _ in range(n_streams - 1)]
    for s, c in zip(streams[1:], ctxs[1:]):
        with torch.cuda.stream(s):
            c.sample(logits[0], uniforms[0], k=TOP_K, p=TOP_P, temperature=TEMP, out=tokens[0])
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        graph3 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph3, stream=side):
            for s in streams[1:]:
                s.wait_stream(side)
            for i in range(W, W + K):
                with torch.cuda.stream(streams[i % n_streams]):
                    ctxs[i % n_streams].sample(logits[i % pool], uniforms[i], k=TOP_K, p=TOP_P, temperature=TEMP,
                                               out=tokens[i])
            for s in streams[1:]:
                side.wait_stream(s)
        graph3.replay()
        side.synchronize()
        R = replays_for(K)
        start3, end3 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start3.record(side)
        for _ in range(R):
            graph3.replay()
        end3.record(side)
        side.synchronize()
    torch.cuda.synchronize()
    if not torch.equal(tokens[W:W + K], seq_tokens):
        sys.exit("PARITY FAILURE: tokens differ between the sequential run and the run with several batches in flight")
    overlapped_ms = start3.elapsed_time(end3) / R
    for c in ctxs[1:]:
        c.close()
    return overlapped_ms


def hbm_copy_probe(torch, dev):
    """GB/s (read + write) of a plain device-to-device copy of 1 GiB, ten times between two events: what this
    GPU's HBM sustains for the simplest streaming kernel, reported next to the nominal 8 TB/s."""
    n = 1 << 28
    src = torch.ones(n, dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        dst.copy_(src)
    e1.record()
    torch.cuda.synchronize()
    return 2 * n * 4 * 10 / (e0.elapsed_time(e1) * 1e-3) / 1e9


def step_latencies(torch, np, step, tokens, side, W, K, prepare=None):
    """Distribution of the step latency, outside the timed region: every one of the K steps launched eagerly
    between its own pair of HIP events on the launch stream (GPU time of one step), and the host-clock time
    from the call of a single step to its token ids being on the host (launch + kernel + copy back)."""
    n = min(K, 128)
    with torch.cuda.stream(side):
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for j, (e0, e1) in enumerate(pairs):
            e0.record(side)
            step(W + j)
            e1.record(side)
        side.synchronize()
        per_step = np.array([e0.elapsed_time(e1) for e0, e1 in pairs]) * 1e3
        host = []
        for j in range(min(n, 64)):
            t0 = time.perf_counter()
            step(W + j)
            tokens[W + j].cpu()
            host.append((time.perf_counter() - t0) * 1e6)
        # The same with the kernel storing its tokens in pinned host memory itself: the host fills the buffer with -1
        # and watches it, no copy and no synchronisation follow the launch.
        pinned = torch.full((tokens.shape[1],), -1, dtype=torch.int32).pin_memory()
        view = pinned.numpy()
        direct, returned = [], []
        for j in range(min(n, 64)):
            view[:] = -1
            t0 = time.perf_counter()
            step(W + j, pinned)
            returned.append((time.perf_counter() - t0) * 1e6)
            while (view < 0).any():
                if time.perf_counter() - t0 > 5.0:
                    sys.exit("tokens never arrived in pinned host memory")
            direct.append((time.perf_counter() - t0) * 1e6)
            side.synchronize()
            if not np.array_equal(view, tokens[W + j].cpu().numpy()):
                sys.exit("PARITY FAILURE: tokens written to pinned host memory differ from the tokens in device memory")
        # And with the call marshalled beforehand, as a serving loop with fixed buffers issues it (the Python
        # binding's per-call tensor lookups are gone; the foreign call, the launch and the kernel remain).
        prepared_t, prepared_ret = [], []
        if prepare is not None:
            calls = [prepare(W + j, pinned, side) for j in range(min(n, 64))]
            for j, call in enumerate(calls):
                view[:] = -1
                t0 = time.perf_counter()
                call()
                prepared_ret.append((time.perf_counter() - t0) * 1e6)
                while (view < 0).any():
                    if time.perf_counter() - t0 > 5.0:
                        sys.exit("tokens never arrived in pinned host memory")
                prepared_t.append((time.perf_counter() - t0) * 1e6)
                side.synchronize()
                if not np.array_equal(view, tokens[W + j].cpu().numpy()):
                    sys.exit("PARITY FAILURE: tokens of a prepared call differ from the tokens in device memory")
    torch.cuda.synchronize()
    return {"note": "informational: single eager launches, each between its own HIP events; host clock from the "
                    "call to the token ids on the host, first with a copy back from device memory, then with the "
                    "kernel writing them to pinned host memory (same tokens required); of_which_host_call = the "
                    "Python binding's call until it returns, before anything runs on the GPU",
            "gpu_us_mean": float(per_step.mean()), "gpu_us_p50": float(np.percentile(per_step, 50)),
            "gpu_us_p95": float(np.percentile(per_step, 95)),
            "launch_to_result_us_p50": float(np.percentile(direct, 50)),
            "launch_to_result_us_p95": float(np.percentile(direct, 95)),
            "of_which_host_call_us_p50": float(np.percentile(returned, 50)),
            "launch_to_result_via_copy_us_p50": float(np.percentile(host, 50)),
            "launch_to_result_via_copy_us_p95": float(np.percentile(host, 95)),
            "prepared_call": None if not prepared_t else {
                "note": "the same step with its arguments marshalled once beforehand (SearchContext.prepared_sample)",
                "launch_to_result_us_p50": float(np.percentile(prepared_t, 50)),
                "launch_to_result_us_p95": float(np.percentile(prepared_t, 95)),
                "of_which_host_call_us_p50": float(np.percentile(prepared_ret, 50))}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--pool", type=int, default=32, help="distinct logits buffers cycled through")
    ap.add_argument("--cpu-steps", type=int, default=24, help="steps replayed on the CPU oracle")
    ap.add_argument("--traffic", type=str, default=None, help="JSON {fetch_bytes, write_bytes} from rocprofv3 --pmc")
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3", "c4", "c5", "topp", "largek", "topp_wide", "odd_vocab", "mixed_modes"],
                    help="c2 (default) is the headline configuration; the others time the remaining "
                         "configurations with the same JSON shape")
    ap.add_argument("--other-configs", type=int, default=1,
                    help="c2 only: 1 (default) also runs configurations 1, 3, 4 and 5 after the headline measurement and "
                         "reports them under config.other_configs; 0 skips them")
    ap.add_argument("--batches-in-flight", type=int, default=3,
                    help="c2 only: after the timed sequential run, also time the same steps spread over this many "
                         "streams and contexts (informational field of the JSON line; 0 skips it, which keeps a "
                         "profiler's per-kernel statistics to the sequential launches)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (rows shard across GPUs "
                 "without communication). Run with --gpus 1.")

    import numpy as np
    import torch
    import __graft_entry__ as ge
    import orc_lib

    pkg = ge.ensure_built()
    orc = orc_lib.Oracle()
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.workload != "c2":
        import bench_workloads
        print(json.dumps(bench_workloads.run(args, pkg, orc, orc_lib, dev)))
        return
    K, W = args.steps, args.warmup
    pool = max(2, min(args.pool, K + W))

    # ---- seeded synthetic inputs: N(0, 3^2) logits + 8 peaks per row at +10 -------------------------
    gen = torch.Generator(device=dev).manual_seed(1234)
    logits = []
    for _ in range(pool):
        x = torch.randn(ROWS, VOCAB, generator=gen, device=dev, dtype=torch.float32) * 3.0
        peaks = torch.randint(0, VOCAB, (ROWS, 8), generator=gen, device=dev)
        x.scatter_add_(1, peaks, torch.full((ROWS, 8), 10.0, device=dev))
        logits.append(x)
    rng = np.random.default_rng(99)
    u_host = rng.random((K + W, ROWS))
    # Where the reference's own headers were compiled (oracle/_ref), the draws of the checked steps are
    # the ones its std::mt19937 engines produce from known seeds, so that the reference's tokens can be
    # compared with the GPU's one to one.
    ref = orc_lib.Reference.load()
    n_cpu = max(1, min(args.cpu_steps, K))
    seeds = None
    if ref is not None:
        seeds = np.arange(n_cpu * ROWS, dtype=np.uint32).reshape(n_cpu, ROWS) * np.uint32(2654435761) + np.uint32(12345)
        two = (np.array([0, 1], np.int32), np.array([0.5, 0.5], np.float32))
        for i in range(n_cpu):
            for r in range(ROWS):
                u_host[W + i, r] = ref.sample_categorical(two[0], two[1], int(seeds[i, r]))[1]
    uniforms = torch.from_numpy(u_host).to(dev)
    tokens = torch.empty((K + W, ROWS), dtype=torch.int32, device=dev)
    ctx = pkg.SearchContext(ROWS, VOCAB)

    def step(i, out=None):
        ctx.sample(logits[i % pool], uniforms[i], k=TOP_K, p=TOP_P, temperature=TEMP, out=tokens[i] if out is None else out)

    for i in range(W):  # warm-up, untimed
        step(i)
    torch.cuda.synchronize()

    # ---- parity gate: GPU tokens == CPU oracle tokens on identical inputs ---------------------------
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for i in range(W, W + K):
                step(i)
        graph.replay()  # first replay untimed (graph upload)
        side.synchronize()
        # The K-step graph is replayed R times between the two events and the time divided by R: what one replay
        # pays for being launched is spread over R * K steps, so the figure does not depend on K.
        R = replays_for(K)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(side)
        for _ in range(R):
            graph.replay()
        end.record(side)
        side.synchronize()
    torch.cuda.synchronize()
    gpu_ms = start.elapsed_time(end) / R
    got = tokens[W:W + n_cpu].cpu().numpy()
    cpu_in = [logits[(W + i) % pool].cpu().numpy() for i in range(n_cpu)]
    t0 = time.perf_counter()
    want = np.stack([orc.sample_batch(cpu_in[i], TOP_K, TOP_P, TEMP, u_host[W + i]) for i in range(n_cpu)])
    cpu_s = time.perf_counter() - t0
    if not np.array_equal(got, want):
        bad = int((got != want).sum())
        sys.exit(f"PARITY FAILURE: {bad} of {got.size} sampled tokens differ from the CPU oracle")
    fallback = ctx.fallback_rows()
    def prepare(i, out, stream):
        return ctx.prepared_sample(logits[i % pool], uniforms[i], out, k=TOP_K, p=TOP_P, temperature=TEMP, stream=stream)

    latency = step_latencies(torch, np, step, tokens, side, W, K, prepare)
    # ---- CPU baseline: the reference's own functions where they were built, else the oracle ---------
    baseline = {"value": ROWS * n_cpu / cpu_s, "unit": "tokens/s", "cores": 1, "kind": "port",
                "sample": "%d of the %d timed steps (same logits and uniforms), oracle/search_oracle.cpp "
                          "orc_sample_batch, one thread as in the reference's serial row loop" % (n_cpu, K),
                "ms_per_step": cpu_s / n_cpu * 1e3, "host_cpus": os.cpu_count()}
    parity = "token ids of %d steps bit-identical to the CPU oracle" % n_cpu
    if ref is not None:
        t0 = time.perf_counter()
        ref_tok = np.empty((n_cpu, ROWS), np.int32)
        for i in range(n_cpu):
            for r in range(ROWS):
                idx, probs = ref.sampled_categorical(cpu_in[i][r], TOP_K, TOP_P, TEMP)
                ref_tok[i, r] = ref.sample_categorical(idx, probs, int(seeds[i, r]))[0]
        ref_s = time.perf_counter() - t0
        if not np.array_equal(got, ref_tok):
            bad = int((got != ref_tok).sum())
            sys.exit(f"PARITY FAILURE: {bad} of {got.size} sampled tokens differ from the reference's own functions")
        baseline = {"value": ROWS * n_cpu / ref_s, "unit": "tokens/s", "cores": 1, "kind": "reference",
                    "sample": "%d of the %d timed steps (same logits; draws from std::mt19937 engines with the same "
                              "seeds): the reference's ComputeSampledCategorical + SampleCategoricalToken compiled "
                              "from its own headers (oracle/_ref), one thread as in its serial row loop" % (n_cpu, K),
                    "ms_per_step": ref_s / n_cpu * 1e3, "host_cpus": os.cpu_count(),
                    "oracle_port_ms_per_step": cpu_s / n_cpu * 1e3}
        parity += " and to the reference's own functions"

    # ---- informational: the same K steps with three independent batches in flight ------------------
    # A generation loop is sequential (a step's tokens feed the next step's logits), which is what
    # `value` measures.  An engine that serves several independent batches can keep one sampling step
    # per batch in flight; the steps then overlap each other's latency-bound tails.  Three contexts on
    # three streams inside one HIP graph, same inputs, tokens required to be identical.
    n_streams = args.batches_in_flight
    overlapped_ms = None
    if n_streams >= 2:
        overlapped_ms = time_batches_in_flight(torch, pkg, ctx, side, n_streams, logits, uniforms, tokens, pool, W, K)

    fp16_ms, fp16_checked = time_fp16_steps(torch, np, orc, ctx, side, logits, uniforms, u_host, W, K, pool, n_cpu)
    copy_gbps = hbm_copy_probe(torch, dev)
    ctx.close()
    del logits, uniforms, tokens
    torch.cuda.empty_cache()
    # ---- the other four configurations, each with its own parity gate (informational, not `value`) ---------
    other = {}
    if args.other_configs:
        import bench_workloads
        for name in ("c1", "c3", "c4", "c5", "topp", "largek", "topp_wide", "odd_vocab", "mixed_modes"):
            sub = argparse.Namespace(**vars(args))
            sub.workload = name
            line = bench_workloads.run(sub, pkg, orc, orc_lib, dev)
            other[name] = {"us_per_step": line["ms_per_step"] * 1e3, "steps": line["steps"],
                           "value": line["value"], "unit": line["unit"],
                           "roofline_frac": line["roofline"]["frac"] if name in ("c3", "c5") else None,
                           "parity": line["config"]["parity"]}
            for key in ("select_ms_per_step", "kv_gather_ms_per_step", "kv_gather_frac_of_peak"):
                if key in line["config"]:
                    other[name][key] = line["config"][key]
            torch.cuda.empty_cache()
    ms_per_step = gpu_ms / K
    algo_bytes = ROWS * VOCAB * 4 + ROWS * 8 + ROWS * 4  # logits once + uniforms + tokens
    achieved = algo_bytes / (ms_per_step * 1e-3) / 1e9
    # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel of known
    # size (profiles/sample_fused_kernel_config2_pmc.md); counters cannot be read from inside this process.
    traffic = MEASURED_TRAFFIC_BYTES
    if args.traffic:
        t = json.loads(args.traffic)
        traffic = t.get("fetch_bytes", 0) + t.get("write_bytes", 0)
    out = {
        "metric": "sampled tokens/sec + step latency, B=64 V=128256 top-k/p; % HBM roofline",
        "value": ROWS * K / (gpu_ms * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": ms_per_step,
        "step_latency_us": ms_per_step * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "config 2: top-k/top-p sampling, batch 64 x vocab 128256 fp32, T=0.7 k=50 p=0.9, "
                               "one fused kernel per step, %d steps replayed from a HIP graph over a pool of %d "
                               "logits buffers" % (K, pool),
                   "rows": ROWS, "vocab": VOCAB, "top_k": TOP_K, "top_p": TOP_P, "temperature": TEMP,
                   "parity": parity,
                   "timed_region": "%d replays of the %d-step graph between two HIP events; ms_per_step = time / "
                                   "(%d * %d)" % (replays_for(K), K, replays_for(K), K),
                   "other_configs": other,
                   "general_path_rows": fallback,
                   "single_step_latency": latency,
                   "fp16_logits": {
                       "note": "informational, not `value`: the same steps with fp16 logits read directly by the "
                               "kernel (tokens of %d steps identical to the CPU oracle on the widened rows)" % fp16_checked,
                       "us_per_step": fp16_ms / K * 1e3, "tokens_per_s": ROWS * K / (fp16_ms * 1e-3),
                       "roofline_frac": (ROWS * VOCAB * 2) / (fp16_ms / K * 1e-3) / 1e9 / HBM_PEAK_GBS},
                   "independent_batches_in_flight": None if overlapped_ms is None else {
                       "note": "informational, not `value`: the same steps issued round-robin on %d streams / "
                               "contexts in one HIP graph (tokens identical)" % n_streams,
                       "streams": n_streams, "us_per_step": overlapped_ms / K * 1e3,
                       "tokens_per_s": ROWS * K / (overlapped_ms * 1e-3),
                       "roofline_frac": algo_bytes / (overlapped_ms / K * 1e-3) / 1e9 / HBM_PEAK_GBS}},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "traffic_source": "rocprofv3 --pmc passed with --traffic" if args.traffic else TRAFFIC_SOURCE,
                     "kernel": "sample_fused_kernel", "algorithmic_bytes_per_launch": algo_bytes,
                     "measured_copy_GBps": copy_gbps},
        "cpu_baseline": baseline,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
