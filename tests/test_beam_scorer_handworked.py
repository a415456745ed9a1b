"""The oracle's BeamSearchScorer against hand-worked literal cases (tests/beam_scorer_cases.py), and proof
that the cases notice plausible mistakes: the oracle's source is patched one mistake at a time, compiled to
a temporary library, and every such variant must fail at least one case."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

import orc_lib
from beam_scorer_cases import CASES

REL = 1e-6  # scores: fp32 division by pow(); the literals carry 7 significant digits


def close(got, want):
    return abs(got - want) <= REL * max(1.0, abs(want)) if want != 0.0 else got == 0.0


def check_hyps(label, got, want):
    assert len(got) == len(want), (label, got, want)
    for (gt, gs), (ws, wt) in zip(got, want):
        assert list(gt) == list(wt), (label, got, want)
        assert close(gs, ws), (label, got, want)
    scores = [s for _, s in got]
    assert scores == sorted(scores, reverse=True), (label, "hypotheses not sorted", scores)


def run_case_on_oracle(orc, case):
    """Drives Process + append per step and Finalize at the end, checking every literal of the case."""
    batch, beams, ml = case["batch"], case["beams"], case["max_length"]
    sc = orc_lib.BeamScorer(orc, batch, beams, ml, case["pad"], case["eos"], case["length_penalty"],
                            case["early_stopping"])
    # BeamSearchScorer's constructor: 0, -1e9, -1e9, ... per entry (src/beam_search_scorer.cpp:76-81)
    init = np.tile(np.array([0.0] + [-1e9] * (beams - 1), np.float32), batch)
    assert np.array_equal(sc.next_scores, init)
    prompt = np.asarray(case["prompt"], np.int32)
    length = prompt.shape[1]
    seq = np.zeros((batch * beams, ml), np.int32)
    seq[:, :length] = np.repeat(prompt, beams, axis=0)
    was_done = [False] * batch
    for si, step in enumerate(case["steps"]):
        cs = np.array([[c[0] for c in row] for row in step["cands"]], np.float32)
        ct = np.array([[c[1] for c in row] for row in step["cands"]], np.int32)
        ci = np.array([[c[2] for c in row] for row in step["cands"]], np.int32)
        assert cs.shape == (batch, 2 * beams)
        sc.process(seq, length, cs, ct, ci)
        want = step["next"]
        got_s, got_t, got_i = sc.next_scores, sc.next_tokens, sc.next_indices
        for r, (ws, wt, wi) in enumerate(want):
            assert got_s[r] == np.float32(ws) and got_t[r] == wt and got_i[r] == wi, (si, r, got_s, got_t, got_i)
        for b in range(batch):
            n = sc.hyp_count(b)
            assert n <= beams
            check_hyps((si, b), [sc.hyp(b, i) for i in range(n)], step["hyps"][b])
            assert sc.batch_done(b) == step["done"][b], (si, b)
            assert sc.batch_done(b) or not was_done[b], "done is monotone"
            was_done[b] = sc.batch_done(b)
        assert sc.is_done() == step["all_done"], si
        nxt = np.zeros_like(seq)
        orc.lib.orc_beam_append(seq.reshape(-1), nxt.reshape(-1), batch * beams, ml, length, got_i, got_t)
        seq, length = nxt, length + 1
        assert seq[:, :length].tolist() == step["sequences"], (si, seq[:, :length].tolist())
    sc.finalize(seq, length)
    for b in range(batch):
        check_hyps(("final", b), [sc.hyp(b, i) for i in range(sc.hyp_count(b))], case["final"][b])


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_scorer_matches_handworked_case(orc, name):
    run_case_on_oracle(orc, CASES[name])


# One plausible mistake per entry: (text in oracle/search_oracle.cpp, replacement).
MUTATIONS = {
    "window_at_own_candidates": ("const float* w = cand_scores + batch * nb;", "const float* w = cand_scores + batch * top_k;"),
    "full_list_accepts_equal": ("if (score <= beams[--index].score) return;", "if (score < beams[--index].score) return;"),
    "insertion_passes_equal": ("index > 0 && score > beams[index - 1].score", "index > 0 && score >= beams[index - 1].score"),
    "no_length_penalty": ("const float score = sum_logprobs / std::pow(static_cast<float>(length), length_penalty);",
                          "const float score = sum_logprobs;"),
    "penalty_is_plain_length": ("const float score = sum_logprobs / std::pow(static_cast<float>(length), length_penalty);",
                                "const float score = sum_logprobs / static_cast<float>(length);"),
    "can_improve_on_equal": ("return beams.back().score < current;", "return beams.back().score <= current;"),
    "can_improve_against_best": ("return beams.back().score < current;", "return beams.front().score < current;"),
    "low_rank_eos_is_added": ("if (j >= nb) continue;", "if (j >= top_k) continue;"),
    "done_window_uses_next_length": ("if (hyp.CanImprove(best, sequence_length)) continue;",
                                     "if (hyp.CanImprove(best, sequence_length + 1)) continue;"),
    "always_early_stopping": ("if (!s.early_stopping) {", "if (false) {"),
    "never_early_stopping": ("if (!s.early_stopping) {", "if (true) {"),
    "padding_keeps_own_row": ("s.next_indices[batch * nb + j] = 0;", "s.next_indices[batch * nb + j] = batch * nb + j;"),
    "padding_score_kept": ("s.next_scores[batch * nb + j] = 0.0f;", ""),
    "hypothesis_includes_eos_position": (
        "hyp.Add(sequences + static_cast<size_t>(batch_beam_idx) * s.max_length, sequence_length, score);",
        "hyp.Add(sequences + static_cast<size_t>(batch_beam_idx) * s.max_length, sequence_length + 1, score);"),
    "relative_next_indices": ("s.next_indices[batch * nb + beam_idx] = batch_beam_idx;",
                              "s.next_indices[batch * nb + beam_idx] = bidx;"),
    "finalize_includes_done_entries": ("if (hyp.done) continue;\n    for (int j = 0; j < s.beams; ++j) {",
                                       "for (int j = 0; j < s.beams; ++j) {"),
}


@pytest.mark.parametrize("name", sorted(MUTATIONS))
def test_handworked_cases_notice_a_mistake(tmp_path, name):
    """A scorer with this one change must disagree with at least one hand-worked case."""
    old, new = MUTATIONS[name]
    src = open(os.path.join(orc_lib.ORACLE_DIR, "search_oracle.cpp")).read()
    assert src.count(old) == 1, "the oracle no longer contains exactly one: " + old
    cpp, so = tmp_path / "mutant.cpp", tmp_path / "libmutant.so"
    cpp.write_text(src.replace(old, new))
    subprocess.check_call(["g++", "-O0", "-std=c++20", "-fPIC", "-fno-fast-math", "-ffp-contract=off", "-shared",
                           str(cpp), "-o", str(so)])
    mutant = orc_lib.Oracle(str(so))
    failed = []
    for case_name in sorted(CASES):
        try:
            run_case_on_oracle(mutant, CASES[case_name])
        except AssertionError:
            failed.append(case_name)
    assert failed, "no hand-worked case notices: " + name
