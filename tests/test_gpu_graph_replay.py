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
