"""mi355x_argmax_static (no context, no allocation: partial results in a static device array) against
mi355x_argmax on the same inputs, through the C ABI: two calls in a row, the second smaller."""
import numpy as np
import pytest
import torch

from gpu_common import pkg, say

pytestmark = pytest.mark.gpu


def test_static_argmax_matches_context_argmax_twice(orc):
    p = pkg()
    ctx = p.SearchContext(64, 151936)
    g = torch.Generator(device="cuda").manual_seed(7)
    # both shapes take the chunked kernel, the one that uses the scratch (rows x chunks >= 256)
    for rows, vocab, dtype in ((64, 151936, torch.float16), (40, 70001, torch.float16), (33, 100003, torch.float32),
                               (36, 66000, torch.bfloat16)):
        say("argmax_static", rows, vocab, dtype)
        x = (torch.randn(rows, vocab, generator=g, device="cuda") * 3).to(dtype)
        x[3, vocab - 1] = 40.0  # a winner in the last, partial chunk
        x[5, :] = 1.0           # all equal: lowest index
        want = ctx.argmax(x)
        out = torch.full((rows,), -1, dtype=torch.int32, device="cuda")  # allocated by the caller, before the call
        got = p.argmax_static(x, out)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert got[3].item() == vocab - 1 and got[5].item() == 0
        # and against the CPU oracle on the rows as the reference's CPU path widens them
        assert np.array_equal(got.cpu().numpy(), orc.argmax_batch(x.float().cpu().numpy()))
    # with fused logits processing (penalty over a history, min-length EOS masking)
    rows, vocab = 40, 70001
    x = torch.randn(rows, vocab, generator=g, device="cuda") * 3
    hist = torch.randint(0, vocab, (rows, 100), generator=g, device="cuda", dtype=torch.int32)
    hist[:, 0] = x.argmax(dim=1).int()  # the winners get penalised
    xf = p.LogitsXform(history=hist, repetition_penalty=1.7, eos_ids=[2, 9], apply_min_length=True)
    out = torch.empty(rows, dtype=torch.int32, device="cuda")
    assert torch.equal(p.argmax_static(x, out, xf), ctx.argmax(x, xf))
    # limits are reported, not overrun
    big = torch.zeros(4097, 8, device="cuda")
    with pytest.raises(RuntimeError, match="4096"):
        p.argmax_static(big, torch.empty(4097, dtype=torch.int32, device="cuda"))
    xf = p.LogitsXform(history=hist, no_repeat_ngram_size=2)
    with pytest.raises(RuntimeError, match="context"):
        p.argmax_static(x, out, xf)
    ctx.close()


def test_static_argmax_in_a_captured_graph(orc):
    """Two mi355x_argmax_static calls recorded into one HIP graph (the address of the static array is known by
    then: a context exists on the device) and replayed twice on new logits, with an eager call between the
    replays; every result against the CPU oracle."""
    p = pkg()
    ctx = p.SearchContext(8, 1000)  # resolves the array's address on this device
    say("argmax_static under capture")
    g = torch.Generator(device="cuda").manual_seed(9)
    a = torch.empty(48, 90001, device="cuda")
    b = torch.empty(20, 70001, device="cuda", dtype=torch.float16)
    out_a = torch.empty(48, dtype=torch.int32, device="cuda")
    out_b = torch.empty(20, dtype=torch.int32, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            p.argmax_static(a, out_a)
            p.argmax_static(b, out_b)
    torch.cuda.synchronize()
    for replay in range(2):
        a.copy_(torch.randn(a.shape, generator=g, device="cuda") * 3)
        b.copy_((torch.randn(b.shape, generator=g, device="cuda") * 3).half())
        out_a.fill_(-1)
        out_b.fill_(-1)
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            graph.replay()
        side.synchronize()
        assert np.array_equal(out_a.cpu().numpy(), orc.argmax_batch(a.cpu().numpy())), replay
        assert np.array_equal(out_b.cpu().numpy(), orc.argmax_batch(b.float().cpu().numpy())), replay
        eager = p.argmax_static(a[:5], torch.empty(5, dtype=torch.int32, device="cuda"))
        torch.cuda.synchronize()
        assert np.array_equal(eager.cpu().numpy(), orc.argmax_batch(a[:5].cpu().numpy()))
    ctx.close()
