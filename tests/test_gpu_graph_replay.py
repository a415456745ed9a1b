"""The entry points a serving loop would capture (sampling, argmax, softmax, beam selection) recorded into one HIP
graph and replayed several times, with eager calls of the same context and synchronisations between the replays:
every replay must reproduce the eager results bit for bit (workspace that must start clean is cleaned by the kernels
themselves, nothing is allocated or cleared by the host per call)."""
import numpy as np
import pytest
import torch

from gpu_common import pkg, say

pytestmark = pytest.mark.gpu


def test_graph_replays_match_eager_calls(orc):
    say("graph replay")
    rows, vocab, batch, beams = 16, 40000, 2, 4
    ctx = pkg().SearchContext(rows, vocab)
    g = torch.Generator(device="cuda").manual_seed(7)
    inputs = [torch.randn(rows, vocab, generator=g, device="cuda") * 3 for _ in range(3)]
    uniforms = torch.rand(3, rows, generator=g, device="cuda", dtype=torch.float64)
    bs = torch.randn(batch * beams, generator=g, device="cuda")

    def run(out):
        for i, x in enumerate(inputs):
            ctx.sample(x, uniforms[i], k=50, p=0.9, temperature=0.7, out=out["topk"][i])
            ctx.sample(x, uniforms[i], k=0, p=0.8, temperature=1.0, out=out["nucleus"][i])
            ctx.argmax(x, out=out["argmax"][i])
            sc, tok, idx = ctx.beam_select(x[:batch * beams], batch, beams, bs)
            out["beam"][i].copy_(torch.cat([sc.view(torch.int32), tok, idx], 1))
            y = x[:4].clone()
            ctx.softmax(y, 1.0, log=True)
            out["lsm"][i].copy_(y)

    def outputs():
        return {"topk": torch.zeros(3, rows, dtype=torch.int32, device="cuda"),
                "nucleus": torch.zeros(3, rows, dtype=torch.int32, device="cuda"),
                "argmax": torch.zeros(3, rows, dtype=torch.int32, device="cuda"),
                "beam": torch.zeros(3, batch, 6 * beams, dtype=torch.int32, device="cuda"),
                "lsm": torch.zeros(3, 4, vocab, device="cuda")}

    eager = outputs()
    run(eager)
    torch.cuda.synchronize()
    want = orc.sample_batch(inputs[0].cpu().numpy(), 50, 0.9, 0.7, uniforms[0].cpu().numpy())
    assert np.array_equal(eager["topk"][0].cpu().numpy(), want)

    captured = outputs()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            run(captured)
    torch.cuda.synchronize()
    for replay in range(4):
        for t in captured.values():
            t.zero_()
        with torch.cuda.stream(side):
            graph.replay()
        side.synchronize()
        for name in eager:
            assert torch.equal(captured[name].view(torch.int32), eager[name].view(torch.int32)), (replay, name)
        # the program's own eager work between replays, on the same context
        again = outputs()
        run(again)
        torch.cuda.synchronize()
        for name in eager:
            assert torch.equal(again[name].view(torch.int32), eager[name].view(torch.int32)), (replay, name, "eager")
    ctx.close()


def test_host_tables_are_staged_for_graph_capture(orc):
    """Calls that take a table from a host array -- per-row parameters of more than 64 rows, the KV gather's pointer
    tables -- copy it into pinned memory of the context when they are called, so their graph nodes do not read the
    caller's array again: a 96-row heterogeneous batch and a KV gather captured into one graph, the host arrays
    overwritten afterwards, four replays with eager calls between them."""
    say("graph replay of staged host tables")
    rows, vocab = 96, 50000
    ctx = pkg().SearchContext(rows, vocab)
    g = torch.Generator(device="cuda").manual_seed(11)
    x = torch.randn(rows, vocab, generator=g, device="cuda") * 3
    u = torch.rand(rows, generator=g, device="cuda", dtype=torch.float64)
    rng = np.random.default_rng(3)
    params = [(int(rng.choice([0, 1, 5, 50, 64, 100])), float(rng.choice([0.0, 0.5, 0.9, 1.0])), float(rng.choice([0.7, 1.0, 1.5])))
              for _ in range(rows)]
    layers = [torch.randint(-30000, 30000, (8, 2, 16, 64), generator=g, device="cuda", dtype=torch.int16) for _ in range(6)]
    past = [torch.zeros_like(t) for t in layers]
    beam_idx = torch.tensor([3, 3, 0, 1, 7, 6, 6, 2], dtype=torch.int32, device="cuda")
    xh, uh = x.cpu().numpy(), u.cpu().numpy()
    want = np.array([orc.sample_row(xh[r], *params[r], uh[r]) for r in range(rows)], np.int32)
    eager = ctx.sample(x, u, per_row=params)
    torch.cuda.synchronize()
    assert np.array_equal(eager.cpu().numpy(), want)

    out = torch.zeros(rows, dtype=torch.int32, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            ctx.sample(x, u, per_row=params, out=out)
            ctx.kv_gather(layers, past, beam_idx)
    torch.cuda.synchronize()
    for replay in range(4):
        out.zero_()
        for t in past:
            t.zero_()
        with torch.cuda.stream(side):
            graph.replay()
        side.synchronize()
        assert np.array_equal(out.cpu().numpy(), want), replay
        for t, src in zip(past, layers):
            assert torch.equal(t, src[beam_idx.long()]), replay
        # eager calls with other tables between the replays: they use other staging slots
        other = [(50, 0.9, 0.7)] * rows
        got = ctx.sample(x, u, per_row=other)
        ctx.kv_gather(layers[:3], past[:3], torch.flip(beam_idx, [0]))
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), orc.sample_batch(xh, 50, 0.9, 0.7, uh)), replay
    ctx.close()


def test_rows_in_several_modes_run_side_by_side(orc):
    """A call whose rows are in several modes (top-k up to 64, nucleus, 64 < k) runs each mode's kernels on a stream
    of the context's own, forked from the caller's stream and joined to it before the call returns.  Two such calls
    in a row on a stream that is not the default one, with different inputs, then both captured into one graph and
    replayed with eager calls of the same kind between the replays: tokens and kept sets equal the oracle's."""
    say("modes side by side")
    rows, vocab = 40, 70001
    ctx = pkg().SearchContext(rows, vocab)
    g = torch.Generator(device="cuda").manual_seed(29)
    xs = [torch.randn(rows, vocab, generator=g, device="cuda") * 4 for _ in range(2)]
    us = [torch.rand(rows, generator=g, device="cuda", dtype=torch.float64) for _ in range(2)]
    menu = [(50, 0.9, 0.7), (0, 0.9, 1.0), (1, 0.0, 1.0), (200, 0.95, 1.0), (0, 0.5, 0.8), (64, 0.0, 1.2), (1000, 0.9, 1.0)]
    params = [menu[(r * 5 + r // 7) % len(menu)] for r in range(rows)]
    want = []
    for x, u in zip(xs, us):
        xh, uh = x.cpu().numpy(), u.cpu().numpy()
        want.append(np.array([orc.sample_row(xh[r], *params[r], uh[r]) for r in range(rows)], np.int32))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    outs = [torch.zeros(rows, dtype=torch.int32, device="cuda") for _ in range(2)]
    with torch.cuda.stream(side):
        for i in range(2):
            ctx.sample(xs[i], us[i], per_row=params, out=outs[i])
    side.synchronize()
    for i in range(2):
        assert np.array_equal(outs[i].cpu().numpy(), want[i]), i
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for i in range(2):
                ctx.sample(xs[i], us[i], per_row=params, out=outs[i])
    torch.cuda.synchronize()
    for replay in range(3):
        for o in outs:
            o.zero_()
        with torch.cuda.stream(side):
            graph.replay()
        side.synchronize()
        for i in range(2):
            assert np.array_equal(outs[i].cpu().numpy(), want[i]), (replay, i)
        tok, kc, ki, kp = ctx.sample(xs[replay % 2], us[replay % 2], per_row=params, kept_capacity=1024)
        torch.cuda.synchronize()
        assert np.array_equal(tok.cpu().numpy(), want[replay % 2]), replay
        xh = xs[replay % 2].cpu().numpy()
        for r in range(0, rows, 9):
            idx, probs = orc.sampled_categorical(xh[r], *params[r])
            n = min(len(idx), 1024)
            assert kc[r].item() == len(idx) and np.array_equal(ki[r, :n].cpu().numpy(), idx[:n]), (replay, r)
    assert ctx.fallback_rows() == 0
    ctx.close()


def test_scorer_steps_refuse_a_capturing_stream():
    """The scorer's steps carry host-side state (sequence length, which of two buffers holds the sequences):
    recording one into a graph would replay the same step, so they decline on a capturing stream."""
    say("scorer step under capture")
    batch, beams, vocab = 2, 2, 5000
    ctx = pkg().SearchContext(batch * beams, vocab)
    scorer = pkg().BeamScorer(ctx, batch, beams, 16, 0, [vocab - 1], 1.0, True)
    scorer.set_prompt(np.zeros((batch, 2), np.int32))
    x = torch.randn(batch * beams, vocab, device="cuda")
    scorer.search_step(x)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    refused = False
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            try:
                scorer.search_step(x)
            except RuntimeError as e:
                refused = "replay" in str(e)
            ctx.argmax(x)  # the capture itself stays usable
    torch.cuda.synchronize()
    assert refused
    scorer.search_step(x)  # and the scorer carries on eagerly
    torch.cuda.synchronize()
    scorer.close()
    ctx.close()
