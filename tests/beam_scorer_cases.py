"""Hand-worked BeamSearchScorer cases with literal expected values.

Every expected number below was derived by hand from the reference source
(src/beam_search_scorer.cpp:19-44 BeamHypotheses::Add / CanImprove, :84-171 Process, :173-196 Finalize,
src/search.cpp:354-381 AppendNextTokensToSequences), not produced by any code of this repository.  The
derivation is written next to each step.  Facts of the reference that the cases rely on:

  * A hypothesis is the beam's sequence BEFORE the EOS token is appended (`sequences.GetSequence`), so its
    length is the current sequence length S, and its score is sum_logprobs / pow(S, length_penalty).
  * Only EOS candidates of rank j < num_beams are added; EOS candidates of rank >= num_beams are skipped.
  * Add: when the list is full, a score <= the worst one is dropped; otherwise the new entry starts at the
    last position and moves up while its score is strictly greater than the entry above (equal scores keep
    insertion order).
  * The done decision of a batch entry needs a full list; with early_stopping it is then immediate, without
    it the entry is done unless CanImprove(max of next_scores[batch*num_beams .. +2*num_beams], S).  The
    window starts at batch*num_beams although each entry owns 2*num_beams candidates (:161): for batch
    entry b > 0 it covers candidates of earlier entries.
  * A done entry emits (score 0, pad token, index 0); the append then copies global row 0's sequence.
  * Candidate beam indices are relative to the batch entry; next_indices are global (batch*num_beams + i).

Layout of a case: `cands[b]` lists the 2*num_beams (score, token, beam) candidates of batch entry b in rank
order; `next` is the expected (score, token, global index) of every beam row after Process; `hyps[b]` is
the expected hypothesis list [(score, tokens)] best first after Process (oracle only: the device API
finalises when hypotheses are read); `done[b]` the entry's done flag; `all_done` BeamSearchScorer::IsDone;
`sequences` every row after the append.  `final[b]` is the list after Finalize."""

PAD = 11
EOS = 9

CASES = {}

# ---------------------------------------------------------------------------------------------------------
# 1 entry, 2 beams, length_penalty 1, no early stopping: rank skip, eviction, equal-to-worst rejection,
# CanImprove true and false, padding after done.
CASES["evict_equal_reject_done_pad"] = dict(
    batch=1, beams=2, max_length=10, pad=PAD, eos=[EOS], length_penalty=1.0, early_stopping=False,
    prompt=[[5, 6]],
    steps=[
        # S=2.  j0 EOS rank 0 -> Add([5,6], -1.0): -1.0 / 2^1 = -0.5.  j1 -> beam row 0.  j2 EOS rank 2 >= 2:
        # skipped, nothing added.  j3 -> beam row 1.  One hypothesis < 2: no done check.
        dict(cands=[[(-1.0, EOS, 0), (-1.5, 3, 0), (-2.0, EOS, 1), (-2.5, 4, 1)]],
             next=[(-1.5, 3, 0), (-2.5, 4, 1)],
             hyps=[[(-0.5, [5, 6])]], done=[False], all_done=False,
             sequences=[[5, 6, 3], [5, 6, 4]]),
        # S=3.  j0 -> row 0.  j1 EOS rank 1 < 2 -> Add(row 1 = [5,6,4], -2.25): -2.25/3 = -0.75, appended
        # below -0.5.  j2 -> row 1, beams full, stop (j3 never read).  List full; window = all four
        # candidates, max -1.2; CanImprove: -1.2/3 = -0.4 > worst -0.75 -> true -> not done.
        dict(cands=[[(-1.2, 7, 0), (-2.25, EOS, 1), (-3.0, 8, 1), (-3.5, 2, 0)]],
             next=[(-1.2, 7, 0), (-3.0, 8, 1)],
             hyps=[[(-0.5, [5, 6]), (-0.75, [5, 6, 4])]], done=[False], all_done=False,
             sequences=[[5, 6, 3, 7], [5, 6, 4, 8]]),
        # S=4.  j0 EOS -> Add(row 0 = [5,6,3,7], -2.4): -2.4/4 = -0.6; list full, -0.6 <= -0.75 is false, so it
        # replaces the worst; not > -0.5, stays second.  j1 EOS rank 1 -> Add(row 1 = [5,6,4,8], -2.4) = -0.6:
        # full and -0.6 <= worst -0.6 -> dropped (a `<` here would have replaced [5,6,3,7] by [5,6,4,8]).
        # j2, j3 -> rows.  Window max -2.4 -> -0.6; worst -0.6 < -0.6 false -> cannot improve -> done.
        # (With S+1 = 5 as the length it would be -0.48 > -0.6 and the entry would stay open.)
        dict(cands=[[(-2.4, EOS, 0), (-2.4, EOS, 1), (-2.6, 1, 0), (-2.8, 2, 1)]],
             next=[(-2.6, 1, 0), (-2.8, 2, 1)],
             hyps=[[(-0.5, [5, 6]), (-0.6, [5, 6, 3, 7])]], done=[True], all_done=True,
             sequences=[[5, 6, 3, 7, 1], [5, 6, 4, 8, 2]]),
        # S=5.  The entry is done: (0, pad, 0) for both rows whatever the candidates say (here EOS with a high
        # score); both rows copy row 0 and append pad.
        dict(cands=[[(-0.1, EOS, 0), (-0.2, 3, 1), (-0.3, 4, 0), (-0.4, 5, 1)]],
             next=[(0.0, PAD, 0), (0.0, PAD, 0)],
             hyps=[[(-0.5, [5, 6]), (-0.6, [5, 6, 3, 7])]], done=[True], all_done=True,
             sequences=[[5, 6, 3, 7, 1, PAD], [5, 6, 3, 7, 1, PAD]]),
    ],
    # Finalize skips done entries.
    final=[[(-0.5, [5, 6]), (-0.6, [5, 6, 3, 7])]],
)


# ---------------------------------------------------------------------------------------------------------
# The same three steps under early_stopping on/off and length_penalty 2: a later, longer hypothesis moves to
# the front; early stopping ends the entry although a candidate could still improve on the worst.
def _front_insert(early):
    done3 = early
    steps = [
        # S=3, no EOS: rows take j0, j1 (both continue beam 0).
        dict(cands=[[(-1.0, 20, 0), (-2.0, 21, 0), (-3.0, 22, 1), (-4.0, 23, 1)]],
             next=[(-1.0, 20, 0), (-2.0, 21, 0)],
             hyps=[[]], done=[False], all_done=False,
             sequences=[[1, 2, 3, 20], [1, 2, 3, 21]]),
        # S=4.  j0 EOS (id 9) -> Add(row 1 = [1,2,3,21], -8.0): -8/4^2 = -0.5.  j1 -> row 0.  j2 EOS (id 10,
        # second EOS id) rank 2 >= 2: skipped.  j3 -> row 1.  One hypothesis: no check.
        dict(cands=[[(-8.0, 9, 1), (-9.0, 30, 0), (-9.5, 10, 0), (-10.0, 31, 1)]],
             next=[(-9.0, 30, 0), (-10.0, 31, 1)],
             hyps=[[(-0.5, [1, 2, 3, 21])]], done=[False], all_done=False,
             sequences=[[1, 2, 3, 20, 30], [1, 2, 3, 21, 31]]),
        # S=5.  j0 -> row 0.  j1 EOS (id 10) rank 1 -> Add(row 1 = [1,2,3,21,31], -6.25): -6.25/5^2 = -0.25 >
        # -0.5: moves to the front.  j2 -> row 1.  List full.  early_stopping: done at once.  Otherwise window
        # max -5.0 -> -5/25 = -0.2 > worst -0.5 -> can improve -> open.
        dict(cands=[[(-5.0, 32, 0), (-6.25, 10, 1), (-7.5, 33, 1), (-8.0, 34, 0)]],
             next=[(-5.0, 32, 0), (-7.5, 33, 1)],
             hyps=[[(-0.25, [1, 2, 3, 21, 31]), (-0.5, [1, 2, 3, 21])]], done=[done3], all_done=done3,
             sequences=[[1, 2, 3, 20, 30, 32], [1, 2, 3, 21, 31, 33]]),
    ]
    if early:
        # S=6: padded.
        steps.append(dict(cands=[[(-1.0, 40, 0), (-2.0, 41, 1), (-3.0, 42, 0), (-4.0, 43, 1)]],
                          next=[(0.0, PAD, 0), (0.0, PAD, 0)],
                          hyps=[[(-0.25, [1, 2, 3, 21, 31]), (-0.5, [1, 2, 3, 21])]], done=[True], all_done=True,
                          sequences=[[1, 2, 3, 20, 30, 32, PAD], [1, 2, 3, 20, 30, 32, PAD]]))
        final = [[(-0.25, [1, 2, 3, 21, 31]), (-0.5, [1, 2, 3, 21])]]
    else:
        # S=6.  j0 EOS -> Add(row 0 = [1,2,3,20,30,32], -4.5): -4.5/36 = -0.125 -> front, (-0.5) evicted.
        # j1, j2 -> rows.  Window max -4.5 -> -0.125; worst -0.25 < -0.125 -> can improve -> open.
        steps.append(dict(cands=[[(-4.5, 9, 0), (-9.0, 40, 1), (-9.5, 41, 0), (-10.0, 42, 1)]],
                          next=[(-9.0, 40, 1), (-9.5, 41, 0)],
                          hyps=[[(-0.125, [1, 2, 3, 20, 30, 32]), (-0.25, [1, 2, 3, 21, 31])]],
                          done=[False], all_done=False,
                          sequences=[[1, 2, 3, 21, 31, 33, 40], [1, 2, 3, 20, 30, 32, 41]]))
        # Finalize at S=7 adds both rows with their beam scores: -9.0/49 = -0.18367 between the two: the list
        # becomes (-0.125, -0.18367), -0.25 evicted; then -9.5/49 = -0.19388 <= worst -0.18367: dropped.
        final = [[(-0.125, [1, 2, 3, 20, 30, 32]), (-0.1836735, [1, 2, 3, 21, 31, 33, 40])]]
    return dict(batch=1, beams=2, max_length=12, pad=PAD, eos=[9, 10], length_penalty=2.0, early_stopping=early,
                prompt=[[1, 2, 3]], steps=steps, final=final)


CASES["front_insert_early_stopping"] = _front_insert(True)
CASES["front_insert_can_improve"] = _front_insert(False)

# ---------------------------------------------------------------------------------------------------------
# 3 entries x 2 beams: the done window of entry b starts at candidate b*2, not b*4.  Entry 1's window holds
# entry 0's ranks 2-3 and its own ranks 0-1; entry 2's window is exactly entry 1's four candidates.  Both
# decisions below differ from what a window over the entry's own candidates would give.
CASES["done_window_offset_quirk"] = dict(
    batch=3, beams=2, max_length=12, pad=PAD, eos=[EOS], length_penalty=1.0, early_stopping=False,
    prompt=[[1, 2], [3, 4], [5, 6]],
    steps=[
        # S=2.
        # entry 0: no EOS -> rows 0,1 continue beam 0.  No hypotheses.
        # entry 1: j0, j1 EOS -> Add([3,4], -3.0) = -1.5, Add([3,4], -4.0) = -2.0; j2, j3 -> rows 2,3 (global
        #   indices 2+0, 2+1).  Full.  Window = flat candidates 2..5 = {-2.0, -2.5 (entry 0), -3.0, -4.0}: max
        #   -2.0 -> -1.0 > worst -2.0 -> open.  (Own candidates: -3.0 -> -1.5 > -2.0: open as well.)
        # entry 2: j0, j1 EOS -> Add([5,6], -0.5) = -0.25, Add([5,6], -1.0) = -0.5; j2, j3 -> rows 4,5.  Full.
        #   Window = flat candidates 4..7 = entry 1's {-3,-4,-5,-6}: max -3.0 -> -1.5; worst -0.5 < -1.5 is
        #   false -> DONE.  (Own candidates: max -0.5 -> -0.25 > -0.5 -> would stay open.)
        dict(cands=[[(-1.0, 20, 0), (-1.5, 21, 0), (-2.0, 22, 1), (-2.5, 23, 1)],
                    [(-3.0, EOS, 0), (-4.0, EOS, 1), (-5.0, 24, 0), (-6.0, 25, 1)],
                    [(-0.5, EOS, 0), (-1.0, EOS, 1), (-1.5, 27, 0), (-2.0, 28, 1)]],
             next=[(-1.0, 20, 0), (-1.5, 21, 0), (-5.0, 24, 2), (-6.0, 25, 3), (-1.5, 27, 4), (-2.0, 28, 5)],
             hyps=[[], [(-1.5, [3, 4]), (-2.0, [3, 4])], [(-0.25, [5, 6]), (-0.5, [5, 6])]],
             done=[False, False, True], all_done=False,
             sequences=[[1, 2, 20], [1, 2, 21], [3, 4, 24], [3, 4, 25], [5, 6, 27], [5, 6, 28]]),
        # S=3.
        # entry 0: no EOS -> rows 0 (beam 0), 1 (beam 1).
        # entry 1: no EOS -> rows 2, 3.  List still full.  Window = {-1.8, -2.1 (entry 0's ranks 2-3), -9.0,
        #   -9.3}: max -1.8 -> -0.6 > worst -2.0 -> open.  (Own candidates: -9.0/3 = -3.0 < -2.0 -> would be done.)
        # entry 2: done -> (0, pad, 0) twice; its rows copy global row 0.
        dict(cands=[[(-1.2, 30, 0), (-1.5, 31, 1), (-1.8, 32, 0), (-2.1, 33, 1)],
                    [(-9.0, 34, 0), (-9.3, 35, 1), (-9.6, 36, 0), (-9.9, 37, 1)],
                    [(-0.1, EOS, 0), (-0.2, 38, 1), (-0.3, 39, 0), (-0.4, 40, 1)]],
             next=[(-1.2, 30, 0), (-1.5, 31, 1), (-9.0, 34, 2), (-9.3, 35, 3), (0.0, PAD, 0), (0.0, PAD, 0)],
             hyps=[[], [(-1.5, [3, 4]), (-2.0, [3, 4])], [(-0.25, [5, 6]), (-0.5, [5, 6])]],
             done=[False, False, True], all_done=False,
             sequences=[[1, 2, 20, 30], [1, 2, 21, 31], [3, 4, 24, 34], [3, 4, 25, 35],
                        [1, 2, 20, PAD], [1, 2, 20, PAD]]),
        # S=4.
        # entry 0: rows 0, 1.
        # entry 1: j0 EOS -> Add(row 2 = [3,4,24,34], -10.0) = -2.5 <= worst -2.0 -> dropped.  j1 -> row 2
        #   (beam 1 -> global 3), j2 -> row 3 (beam 0 -> global 2); j3 (EOS) never read.  Window = {-9.0, -9.5
        #   (entry 0), -10.0, -10.4}: max -9.0 -> -2.25; worst -2.0 < -2.25 false -> done.
        # entry 2: padded.
        dict(cands=[[(-1.25, 40, 0), (-2.5, 41, 1), (-9.0, 42, 0), (-9.5, 43, 1)],
                    [(-10.0, EOS, 0), (-10.4, 38, 1), (-10.8, 39, 0), (-11.2, EOS, 1)],
                    [(-0.1, 44, 0), (-0.2, 45, 1), (-0.3, 46, 0), (-0.4, 47, 1)]],
             next=[(-1.25, 40, 0), (-2.5, 41, 1), (-10.4, 38, 3), (-10.8, 39, 2), (0.0, PAD, 0), (0.0, PAD, 0)],
             hyps=[[], [(-1.5, [3, 4]), (-2.0, [3, 4])], [(-0.25, [5, 6]), (-0.5, [5, 6])]],
             done=[False, True, True], all_done=False,
             sequences=[[1, 2, 20, 30, 40], [1, 2, 21, 31, 41], [3, 4, 25, 35, 38], [3, 4, 24, 34, 39],
                        [1, 2, 20, 30, PAD], [1, 2, 20, 30, PAD]]),
    ],
    # Finalize at S=5: entry 0 is open -> Add(row 0, -1.25) = -0.25, Add(row 1, -2.5) = -0.5; done entries untouched.
    final=[[(-0.25, [1, 2, 20, 30, 40]), (-0.5, [1, 2, 21, 31, 41])],
           [(-1.5, [3, 4]), (-2.0, [3, 4])],
           [(-0.25, [5, 6]), (-0.5, [5, 6])]],
)


# ---------------------------------------------------------------------------------------------------------
# One event sequence under three length penalties: hypothesis A (length 2, sum -1.0) and B (length 4, sum
# -1.6).  pow(len, lp) decides their order and the done decision.
#   lp 0.6: A = -1/2^0.6 = -1/1.5157166 = -0.6597540;  B = -1.6/4^0.6 = -1.6/2.2973967 = -0.6964405 -> [A, B];
#           CanImprove: current = B's own score, worst = B -> not strictly better -> done.
#   lp 1.0: A = -0.5, B = -0.4 -> [B, A]; current -0.4 > worst -0.5 -> open.
#   lp 2.0: A = -0.25, B = -0.1 -> [B, A]; current -0.1 > worst -0.25 -> open.
# (Without any penalty the scores would be -1.0 and -1.6.)
def _penalty_case(lp, a, b, b_first, done):
    seq_a, seq_b = [7, 8], [7, 8, 20, 24]
    after = [(b, seq_b), (a, seq_a)] if b_first else [(a, seq_a), (b, seq_b)]
    # Finalize (only when still open) at S=5 with beam scores -1.7 and -1.8:
    #   lp 1.0: -1.7/5 = -0.34 -> front of [-0.4, -0.5] -> [-0.34, -0.4]; -1.8/5 = -0.36 -> between -> [-0.34, -0.36].
    #   lp 2.0: -1.7/25 = -0.068 -> front of [-0.1, -0.25] -> [-0.068, -0.1]; -1.8/25 = -0.072 -> [-0.068, -0.072].
    row0, row1 = [7, 8, 21, 23, 27], [7, 8, 20, 24, 28]
    if done:
        final = after
    elif lp == 1.0:
        final = [(-0.34, row0), (-0.36, row1)]
    else:
        final = [(-0.068, row0), (-0.072, row1)]
    return dict(
        batch=1, beams=2, max_length=8, pad=PAD, eos=[EOS], length_penalty=lp, early_stopping=False,
        prompt=[[7, 8]],
        steps=[
            # S=2: j0 EOS -> A.  j1, j2 -> rows.
            dict(cands=[[(-1.0, EOS, 0), (-1.25, 20, 0), (-1.5, 21, 1), (-1.75, 22, 1)]],
                 next=[(-1.25, 20, 0), (-1.5, 21, 1)],
                 hyps=[[(a, seq_a)]], done=[False], all_done=False,
                 sequences=[[7, 8, 20], [7, 8, 21]]),
            # S=3: no EOS; the rows swap parents.
            dict(cands=[[(-1.3, 23, 1), (-1.4, 24, 0), (-1.9, 25, 0), (-2.0, 26, 1)]],
                 next=[(-1.3, 23, 1), (-1.4, 24, 0)],
                 hyps=[[(a, seq_a)]], done=[False], all_done=False,
                 sequences=[[7, 8, 21, 23], [7, 8, 20, 24]]),
            # S=4: j0 EOS on beam 1 -> B = Add([7,8,20,24], -1.6).  j1, j2 -> rows.  Full -> done check.
            dict(cands=[[(-1.6, EOS, 1), (-1.7, 27, 0), (-1.8, 28, 1), (-1.9, 29, 0)]],
                 next=[(-1.7, 27, 0), (-1.8, 28, 1)],
                 hyps=[after], done=[done], all_done=done,
                 sequences=[row0, row1]),
        ],
        final=[final])


CASES["length_penalty_0.6"] = _penalty_case(0.6, -0.6597540, -0.6964405, False, True)
CASES["length_penalty_1.0"] = _penalty_case(1.0, -0.5, -0.4, True, False)
CASES["length_penalty_2.0"] = _penalty_case(2.0, -0.25, -0.1, True, False)

# ---------------------------------------------------------------------------------------------------------
# 1 entry x 3 beams: the insertion loop moving an entry past two others, into the middle, and Finalize
# feeding the open beams through Add.
CASES["three_beams_rotate_and_finalize"] = dict(
    batch=1, beams=3, max_length=10, pad=PAD, eos=[EOS], length_penalty=1.0, early_stopping=False,
    prompt=[[1, 2]],
    steps=[
        # S=2.  j0, j1 EOS -> Add([1,2], -2.0) = -1.0, Add([1,2], -3.0) = -1.5.  j2 -> row 0.  j3 EOS rank 3 >= 3:
        # skipped.  j4, j5 -> rows 1, 2.  Two hypotheses < 3: no check.
        dict(cands=[[(-2.0, EOS, 0), (-3.0, EOS, 1), (-4.0, 20, 0), (-5.0, EOS, 2), (-6.0, 21, 1), (-7.0, 22, 2)]],
             next=[(-4.0, 20, 0), (-6.0, 21, 1), (-7.0, 22, 2)],
             hyps=[[(-1.0, [1, 2]), (-1.5, [1, 2])]], done=[False], all_done=False,
             sequences=[[1, 2, 20], [1, 2, 21], [1, 2, 22]]),
        # S=3.  j0 EOS -> Add(row 2 = [1,2,22], -1.5) = -0.5: third slot, then past -1.5 and past -1.0 to the front.
        # j1 EOS rank 1 -> Add(row 0 = [1,2,20], -3.75) = -1.25: full, not <= -1.5 -> replaces the worst; not > -1.0.
        # j2, j3 -> rows 0, 1.  j4 EOS rank 4 >= 3: skipped.  j5 -> row 2.  Window max -1.5 -> -0.5 > worst -1.25: open.
        dict(cands=[[(-1.5, EOS, 2), (-3.75, EOS, 0), (-4.0, 23, 1), (-4.5, 24, 0), (-5.0, EOS, 1), (-5.5, 25, 2)]],
             next=[(-4.0, 23, 1), (-4.5, 24, 0), (-5.5, 25, 2)],
             hyps=[[(-0.5, [1, 2, 22]), (-1.0, [1, 2]), (-1.25, [1, 2, 20])]], done=[False], all_done=False,
             sequences=[[1, 2, 21, 23], [1, 2, 20, 24], [1, 2, 22, 25]]),
        # S=4.  j0 -> row 0.  j1 EOS rank 1 -> Add(row 1 = [1,2,20,24], -3.0) = -0.75: replaces -1.25 at the end,
        # passes -1.0, stops below -0.5.  j2, j3 -> rows 1, 2.  Window max -2.8 -> -0.7 > worst -1.0: open.
        dict(cands=[[(-2.8, 26, 0), (-3.0, EOS, 1), (-3.2, 27, 2), (-3.4, 28, 1), (-5.0, 29, 0), (-5.2, 30, 2)]],
             next=[(-2.8, 26, 0), (-3.2, 27, 2), (-3.4, 28, 1)],
             hyps=[[(-0.5, [1, 2, 22]), (-0.75, [1, 2, 20, 24]), (-1.0, [1, 2])]], done=[False], all_done=False,
             sequences=[[1, 2, 21, 23, 26], [1, 2, 22, 25, 27], [1, 2, 20, 24, 28]]),
    ],
    # Finalize at S=5: Add(row 0, -2.8) = -0.56 -> replaces -1.0, passes -0.75 -> [-0.5, -0.56, -0.75];
    # Add(row 1, -3.2) = -0.64 -> replaces -0.75, not > -0.56 -> [-0.5, -0.56, -0.64]; Add(row 2, -3.4) = -0.68 <=
    # -0.64 -> dropped.
    final=[[(-0.5, [1, 2, 22]), (-0.56, [1, 2, 21, 23, 26]), (-0.64, [1, 2, 22, 25, 27])]],
)

# ---------------------------------------------------------------------------------------------------------
# Equal scores keep insertion order (the insertion loop compares with strict `>`).
CASES["equal_scores_keep_insertion_order"] = dict(
    batch=1, beams=3, max_length=6, pad=PAD, eos=[EOS], length_penalty=1.0, early_stopping=False,
    prompt=[[1]],
    steps=[
        # S=1, no EOS: three different continuations of beam 0.
        dict(cands=[[(-0.1, 20, 0), (-0.2, 21, 0), (-0.3, 22, 0), (-0.4, 23, 0), (-0.5, 24, 0), (-0.6, 25, 0)]],
             next=[(-0.1, 20, 0), (-0.2, 21, 0), (-0.3, 22, 0)],
             hyps=[[]], done=[False], all_done=False,
             sequences=[[1, 20], [1, 21], [1, 22]]),
        # S=2.  j0 EOS on beam 2 -> Add([1,22], -1.0) = -0.5.  j1 EOS on beam 0 -> Add([1,20], -1.0) = -0.5: equal,
        # stays behind.  j2..j4 -> rows.  Two hypotheses < 3: no check.
        dict(cands=[[(-1.0, EOS, 2), (-1.0, EOS, 0), (-1.5, 30, 1), (-1.6, 31, 0), (-1.7, 32, 2), (-1.8, 33, 1)]],
             next=[(-1.5, 30, 1), (-1.6, 31, 0), (-1.7, 32, 2)],
             hyps=[[(-0.5, [1, 22]), (-0.5, [1, 20])]], done=[False], all_done=False,
             sequences=[[1, 21, 30], [1, 20, 31], [1, 22, 32]]),
    ],
    # Finalize at S=3: Add(row 0, -1.5) = -0.5: third slot, equal to the entry above -> stays third.
    # Add(row 1, -1.6) = -0.5333 <= worst -0.5 -> dropped; Add(row 2, -1.7) dropped.
    final=[[(-0.5, [1, 22]), (-0.5, [1, 20]), (-0.5, [1, 21, 30])]],
)
