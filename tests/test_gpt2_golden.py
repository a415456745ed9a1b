"""The reference's own greedy and beam-search golden tests (ModelTests.GreedySearchGptFp32 and
ModelTests.BeamSearchGptFp32, test/model_tests.cpp:57-130) replayed without ONNX Runtime: the logits the tiny GPT-2
of those tests produces along the expected trajectory are a committed fixture
(tests/golden/gpt2_search_vectors.npz, written by tests/golden/make_gpt2_search_vectors.py), and the token
sequences the reference expects must come out of the oracle (CPU) and of the HIP kernels through the C ABI (GPU).

This is what pins ArgMax, BeamSearch_Cpu::SelectTop (src/search.cpp:101-176), BeamSearchScorer::Process / Finalize
(src/beam_search_scorer.cpp:84-196) and the beam append (src/search.cpp:354-381) to the reference's results: those
translation units cannot be compiled here.  Every replay checks at each step that the token rows it would feed the
model are the rows the stored logits were computed for, so a wrong beam choice cannot hide behind later logits."""
import os

import numpy as np
import pytest

import orc_lib
from gpu_common import pkg, say

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gpt2_search_vectors.npz")


@pytest.fixture(scope="module")
def vec():
    return dict(np.load(FIXTURE))


def oracle_beam(orc, vec, beams=None, length_penalty=1.0, early_stopping=True, check_inputs=True, select=None):
    pad, eos, nb = (int(x) for x in vec["options"])
    beams = beams or nb
    prompt, expected, logits = vec["beam_prompt"], vec["beam_expected"], vec["beam_logits"]
    batch, max_length = prompt.shape[0], expected.shape[1]
    ref = orc_lib.BeamScorer(orc, batch, beams, max_length, pad, [eos], length_penalty, early_stopping)
    seq = np.zeros((batch * beams, max_length), np.int32)
    seq[:, :prompt.shape[1]] = np.repeat(prompt, beams, axis=0)
    length = prompt.shape[1]
    for step in range(len(logits)):
        if check_inputs:
            assert np.array_equal(seq, vec["beam_inputs"][step]), step
        sc, tok, idx, _ = (select or orc.beam_select_top)(logits[step], batch, beams, ref.next_scores)
        ref.process(seq, length, sc, tok, idx)
        nxt = np.zeros_like(seq)
        orc.lib.orc_beam_append(seq.reshape(-1), nxt.reshape(-1), batch * beams, max_length, length,
                                ref.next_indices, ref.next_tokens)
        seq, length = nxt, length + 1
    assert length == max_length or ref.is_done()
    ref.finalize(seq, length)
    return np.stack([np.pad(ref.hyp(b, 0)[0], (0, max_length))[:max_length] for b in range(batch)])


def test_oracle_greedy_reproduces_reference_golden(orc, vec):
    prompt, expected, logits = vec["greedy_prompt"], vec["greedy_expected"], vec["greedy_logits"]
    seq = prompt.copy()
    for step in range(len(logits)):
        assert np.array_equal(seq, expected[:, :seq.shape[1]])
        seq = np.concatenate([seq, orc.argmax_batch(logits[step])[:, None]], 1)
    assert np.array_equal(seq, expected)


def test_oracle_beam_search_reproduces_reference_golden(orc, vec):
    assert np.array_equal(oracle_beam(orc, vec), vec["beam_expected"])


def test_beam_golden_is_sensitive_to_plausible_mistakes(orc, vec):
    """The fixture only pins something if wrong searches fail it: each variant below is one plausible slip.  (Dropping
    the log-softmax is NOT among them: this model's rows have nearly equal normalisers and the expected tokens survive
    it; LogSoftMax is pinned against the reference's own softmax.h build instead.)"""
    expected = vec["beam_expected"]

    def no_beam_scores(x, batch, beams, bs):  # running scores dropped
        return orc.beam_select_top(x, batch, beams, np.zeros_like(bs))

    def ascending_candidates(x, batch, beams, bs):  # candidates handed over worst-first
        sc, tok, idx, _ = orc.beam_select_top(x, batch, beams, bs)
        return sc[:, ::-1].copy(), tok[:, ::-1].copy(), idx[:, ::-1].copy(), None

    def lowest_id_among_beams(x, batch, beams, bs):  # beam index and token swapped when the flat index is split
        sc, tok, idx, _ = orc.beam_select_top(x, batch, beams, bs)
        return sc, tok, (tok % beams).astype(np.int32), None

    for wrong in (no_beam_scores, ascending_candidates, lowest_id_among_beams):
        assert not np.array_equal(oracle_beam(orc, vec, check_inputs=False, select=wrong), expected), wrong.__name__


@pytest.mark.gpu
def test_gpu_greedy_reproduces_reference_golden(vec):
    import torch
    ctx = pkg().SearchContext(16, 1000)
    prompt, expected, logits = vec["greedy_prompt"], vec["greedy_expected"], vec["greedy_logits"]
    pad, eos, _ = (int(x) for x in vec["options"])
    batch, max_length = expected.shape
    seq = torch.zeros((batch, max_length), dtype=torch.int32, device="cuda")
    seq[:, :prompt.shape[1]] = torch.from_numpy(prompt).cuda()
    seen = torch.zeros(batch, dtype=torch.int32, device="cuda")
    done = torch.zeros(1, dtype=torch.int32, device="cuda")
    length = prompt.shape[1]
    for step in range(len(logits)):
        say("gpt2 greedy golden step", step)
        assert np.array_equal(seq.cpu().numpy()[:, :length], expected[:, :length])
        tok = ctx.argmax(torch.from_numpy(logits[step]).cuda())
        ctx.greedy_tail(tok, seen, [eos], pad, seq, length, done)
        length += 1
    assert np.array_equal(seq.cpu().numpy(), expected)
    ctx.close()


@pytest.mark.gpu
def test_gpu_beam_search_reproduces_reference_golden(vec):
    import torch
    ctx = pkg().SearchContext(16, 1000)
    pad, eos, beams = (int(x) for x in vec["options"])
    prompt, expected, logits = vec["beam_prompt"], vec["beam_expected"], vec["beam_logits"]
    batch, max_length = prompt.shape[0], expected.shape[1]
    dev = pkg().BeamScorer(ctx, batch, beams, max_length, pad, [eos], 1.0, True)
    dev.set_prompt(prompt)
    for step in range(len(logits)):
        say("gpt2 beam golden step", step)
        dseq, dlen = dev.sequences()
        assert dlen == prompt.shape[1] + step
        assert np.array_equal(dseq.cpu().numpy(), vec["beam_inputs"][step][:, :dlen]), step
        sc, tok, idx = ctx.beam_select(torch.from_numpy(logits[step]).cuda(), batch, beams, dev.next_scores)
        dev.step(sc, tok, idx)
    assert dev.is_done()
    for b in range(batch):
        got, _ = dev.hypothesis(b, 0)
        assert got == expected[b].tolist(), b
    dev.close()
    ctx.close()
