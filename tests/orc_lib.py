"""ctypes bindings to the CPU oracle (oracle/libsearch_oracle.so) and to the wrapper around the
reference's stand-alone headers (oracle/_ref/libref_headers.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")


def _ensure_built():
    so = os.path.join(ORACLE_DIR, "libsearch_oracle.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", ORACLE_DIR], stdout=subprocess.DEVNULL)
    return so


def _i32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32))


def _csr(rows):
    """(ids, probs) rows -> offsets, concatenated ids, concatenated probs."""
    off = np.zeros(len(rows) + 1, np.int32)
    for i, (ix, _) in enumerate(rows):
        off[i + 1] = off[i] + len(ix)
    idx = np.concatenate([np.asarray(r[0], np.int32) for r in rows] + [np.zeros(1, np.int32)])
    probs = np.concatenate([np.asarray(r[1], np.float32) for r in rows] + [np.zeros(1, np.float32)])
    return off, np.ascontiguousarray(idx, np.int32), np.ascontiguousarray(probs, np.float32)


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


class Oracle:
    def __init__(self, path=None):
        """`path`: a differently built copy of the oracle library (the mutation tests load patched ones)."""
        L = self.lib = C.CDLL(path or _ensure_built())
        L.orc_argmax.restype = C.c_int32
        L.orc_argmax.argtypes = [f32p, C.c_int]
        L.orc_apply_min_length.argtypes = [f32p, C.c_int, C.c_int, C.c_int, i32p, C.c_int]
        L.orc_apply_repetition_penalty.argtypes = [f32p, C.c_int, i32p, C.c_int, C.c_float]
        L.orc_apply_no_repeat_ngram.argtypes = [f32p, C.c_int, i32p, C.c_int, C.c_int]
        L.orc_apply_mask.argtypes = [f32p, C.c_int, C.c_int, u32p]
        L.orc_sampled_categorical.restype = C.c_int
        L.orc_sampled_categorical.argtypes = [f32p, C.c_int, C.c_int, C.c_float, C.c_float, i32p, i32p, f32p]
        L.orc_discrete_draw.restype = C.c_int
        L.orc_discrete_draw.argtypes = [f32p, C.c_int, C.c_double]
        L.orc_sample_batch.argtypes = [f32p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, f64p, i32p]
        L.orc_argmax_batch.argtypes = [f32p, C.c_int, C.c_int, i32p]
        for n in ("orc_softmax", "orc_log_softmax"):
            getattr(L, n).argtypes = [f32p, C.c_int, C.c_float]
        for n in ("orc_softmax_plain", "orc_log_softmax_plain"):
            getattr(L, n).argtypes = [f32p, C.c_int]
        L.orc_fp16_to_fp32_array.argtypes = [u16p, f32p, C.c_size_t]
        L.orc_beam_select_top.argtypes = [f32p, C.c_int, C.c_int, C.c_int, f32p, f32p, i32p, i32p]
        L.orc_beam_scorer_create.restype = C.c_void_p
        L.orc_beam_scorer_create.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, i32p, C.c_int, C.c_float, C.c_int]
        L.orc_beam_scorer_destroy.argtypes = [C.c_void_p]
        L.orc_beam_scorer_process.argtypes = [C.c_void_p, i32p, C.c_int, f32p, i32p, i32p]
        L.orc_beam_scorer_finalize.argtypes = [C.c_void_p, i32p, C.c_int]
        L.orc_beam_scorer_is_done.restype = C.c_int
        L.orc_beam_scorer_is_done.argtypes = [C.c_void_p]
        L.orc_beam_scorer_next_scores.restype = C.POINTER(C.c_float)
        L.orc_beam_scorer_next_scores.argtypes = [C.c_void_p]
        L.orc_beam_scorer_next_tokens.restype = C.POINTER(C.c_int32)
        L.orc_beam_scorer_next_tokens.argtypes = [C.c_void_p]
        L.orc_beam_scorer_next_indices.restype = C.POINTER(C.c_int32)
        L.orc_beam_scorer_next_indices.argtypes = [C.c_void_p]
        L.orc_beam_scorer_batch_done.restype = C.c_int
        L.orc_beam_scorer_batch_done.argtypes = [C.c_void_p, C.c_int]
        L.orc_beam_scorer_hyp_count.restype = C.c_int
        L.orc_beam_scorer_hyp_count.argtypes = [C.c_void_p, C.c_int]
        L.orc_beam_scorer_hyp.restype = C.c_int
        L.orc_beam_scorer_hyp.argtypes = [C.c_void_p, C.c_int, C.c_int, i32p, C.c_int, C.POINTER(C.c_float)]
        L.orc_beam_append.argtypes = [i32p, i32p, C.c_int, C.c_int, C.c_int, i32p, i32p]
        L.orc_kv_gather.argtypes = [C.c_void_p, C.c_void_p, i32p, C.c_int, C.c_size_t]
        L.orc_accept_prob.restype = C.c_float
        L.orc_accept_prob.argtypes = [C.c_float, C.c_float]
        L.orc_build_correction.argtypes = [f32p, f32p, f32p, C.c_int]
        L.orc_sparse_prob.restype = C.c_float
        L.orc_sparse_prob.argtypes = [i32p, f32p, C.c_int, C.c_int32]
        L.orc_sample_correction.restype = C.c_int32
        L.orc_sample_correction.argtypes = [i32p, f32p, C.c_int, i32p, f32p, C.c_int, C.c_double]
        L.orc_spec_verify_dense.argtypes = [f32p, f32p, i32p, f32p, f64p, C.c_int, C.c_int, C.c_int, i32p, i32p]
        L.orc_target_selection.restype = C.c_int
        L.orc_target_selection.argtypes = [f32p, C.c_int, C.c_int, i32p, C.c_int, C.c_int, C.c_int, C.c_float,
                                           C.c_float, C.c_float, C.c_int, C.c_int, i32p, C.c_int,
                                           C.POINTER(C.c_int32), i32p, f32p]
        L.orc_spec_verify_sparse.argtypes = [i32p, C.c_int, i32p, i32p, f32p, i32p, i32p, f32p, f32p, f64p,
                                             C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
        L.orc_verify_deterministic.restype = C.c_int
        L.orc_verify_deterministic.argtypes = [i32p, C.c_int, i32p, i32p, f32p, f64p, C.POINTER(C.c_int32),
                                               C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]

    # ---- convenience wrappers (numpy in / numpy out) ----
    def argmax(self, row):
        row = _f32(row)
        return int(self.lib.orc_argmax(row, row.size))

    def argmax_batch(self, logits):
        logits = _f32(logits)
        out = np.empty(logits.shape[0], np.int32)
        self.lib.orc_argmax_batch(logits, logits.shape[0], logits.shape[1], out)
        return out

    def apply_min_length(self, row, cur, min_len, eos):
        row = _f32(row).copy()
        eos = _i32(eos)
        self.lib.orc_apply_min_length(row, row.size, cur, min_len, eos, eos.size)
        return row

    def apply_repetition_penalty(self, row, prefix, pen):
        row = _f32(row).copy()
        prefix = _i32(prefix)
        self.lib.orc_apply_repetition_penalty(row, row.size, prefix, prefix.size, pen)
        return row

    def apply_no_repeat_ngram(self, row, prefix, n):
        row = _f32(row).copy()
        prefix = _i32(prefix)
        self.lib.orc_apply_no_repeat_ngram(row, row.size, prefix, prefix.size, n)
        return row

    def apply_mask(self, logits, mask):
        logits = _f32(logits).copy()
        rows, vocab = logits.shape
        mask = np.ascontiguousarray(mask, dtype=np.uint32)
        assert mask.shape == (rows, (vocab - 1) // 32 + 1)
        self.lib.orc_apply_mask(logits, rows, vocab, mask)
        return logits

    def sampled_categorical(self, scores, k, p, t):
        scores = _f32(scores)
        v = scores.size
        scratch = np.empty(v, np.int32)
        idx = np.empty(v, np.int32)
        probs = np.empty(v, np.float32)
        n = self.lib.orc_sampled_categorical(scores, v, k, p, t, scratch, idx, probs)
        return idx[:n].copy(), probs[:n].copy()

    def discrete_draw(self, w, u):
        w = _f32(w)
        return int(self.lib.orc_discrete_draw(w, w.size, u))

    def sample_row(self, scores, k, p, t, u):
        idx, probs = self.sampled_categorical(scores, k, p, t)
        return int(idx[self.discrete_draw(probs, u)])

    def sample_batch(self, logits, k, p, t, u):
        logits = _f32(logits)
        u = np.ascontiguousarray(u, dtype=np.float64)
        out = np.empty(logits.shape[0], np.int32)
        self.lib.orc_sample_batch(logits, logits.shape[0], logits.shape[1], k, p, t, u, out)
        return out

    def softmax(self, s, t=1.0):
        s = _f32(s).copy()
        self.lib.orc_softmax(s, s.size, t)
        return s

    def log_softmax(self, s, t=1.0):
        s = _f32(s).copy()
        self.lib.orc_log_softmax(s, s.size, t)
        return s

    def softmax_plain(self, s):
        s = _f32(s).copy()
        self.lib.orc_softmax_plain(s, s.size)
        return s

    def log_softmax_plain(self, s):
        s = _f32(s).copy()
        self.lib.orc_log_softmax_plain(s, s.size)
        return s

    def cast(self, src, kind, out_dtype):
        """kind: 0 fp16->fp32, 1 bf16->fp32, 2 fp32->fp16, 3 fp32->bf16, 4 int32->int64 (bit patterns in,
        bit patterns out for the 16-bit types)."""
        src = np.ascontiguousarray(src)
        out = np.empty(src.shape, out_dtype)
        self.lib.orc_cast.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.lib.orc_cast.restype = None
        self.lib.orc_cast(src.ctypes.data, out.ctypes.data, src.size, kind)
        return out

    def fp16_to_fp32(self, h):
        h = np.ascontiguousarray(h).view(np.uint16)
        out = np.empty(h.shape, np.float32)
        self.lib.orc_fp16_to_fp32_array(h.reshape(-1), out.reshape(-1), h.size)
        return out

    def beam_select_top(self, scores, batch, beams, beam_scores):
        scores = _f32(scores).copy()
        vocab = scores.shape[-1]
        k = 2 * beams
        os_ = np.empty((batch, k), np.float32)
        ot = np.empty((batch, k), np.int32)
        oi = np.empty((batch, k), np.int32)
        self.lib.orc_beam_select_top(scores.reshape(-1), batch, beams, vocab, _f32(beam_scores), os_.reshape(-1),
                                     ot.reshape(-1), oi.reshape(-1))
        return os_, ot, oi, scores

    def kv_gather(self, present, idx):
        present = np.ascontiguousarray(present)
        idx = _i32(idx)
        past = np.empty((idx.size,) + present.shape[1:], present.dtype)
        block = present[0].nbytes
        self.lib.orc_kv_gather(present.ctypes.data, past.ctypes.data, idx, idx.size, block)
        return past

    def accept_prob(self, pt, pd):
        return float(self.lib.orc_accept_prob(pt, pd))

    def build_correction(self, pt, pd):
        pt, pd = _f32(pt), _f32(pd)
        out = np.empty_like(pt)
        self.lib.orc_build_correction(pt, pd, out, pt.size)
        return out

    def sample_correction(self, t_idx, t_probs, d_idx, d_probs, u):
        t_idx, d_idx = _i32(t_idx), _i32(d_idx)
        t_probs, d_probs = _f32(t_probs), _f32(d_probs)
        return int(self.lib.orc_sample_correction(t_idx, t_probs, t_idx.size, d_idx, d_probs, d_idx.size, u))

    def spec_verify_dense(self, p, q, draft, uf, ud):
        p, q = _f32(p), _f32(q)
        b, k1, v = p.shape
        draft = _i32(draft)
        uf = _f32(uf)
        ud = np.ascontiguousarray(ud, np.float64)
        acc = np.empty(b, np.int32)
        tok = np.empty(b, np.int32)
        self.lib.orc_spec_verify_dense(p.reshape(-1), q.reshape(-1), draft.reshape(-1), uf.reshape(-1), ud, b, k1 - 1,
                                       v, acc, tok)
        return acc, tok

    def spec_verify_sparse(self, proposal, target_rows, draft_rows, accept_u, sample_u):
        """One sequence's round: K+1 target rows and K draft rows of (ids, probs), K accept uniforms and the
        K+1 candidate categorical draws.  Returns (accepted, final token, engine draws consumed)."""
        proposal = _i32(proposal)
        k = proposal.size
        assert len(target_rows) == k + 1 and len(draft_rows) == k
        toff, tidx, tprob = _csr(target_rows)
        doff, didx, dprob = _csr(draft_rows)
        acc, tok, used = C.c_int32(), C.c_int32(), C.c_int32()
        self.lib.orc_spec_verify_sparse(proposal, k, toff, tidx, tprob, doff, didx, dprob, _f32(accept_u),
                                        np.ascontiguousarray(sample_u, np.float64), C.byref(acc), C.byref(tok),
                                        C.byref(used))
        return acc.value, tok.value, used.value

    def target_selection(self, logits, cur_len, prefix, greedy, k, p, t, rep_pen=1.0, min_len=0, ngram=0, eos=()):
        logits = _f32(logits)
        prefix = _i32(prefix)
        eos = _i32(eos)
        v = logits.size
        idx = np.empty(v, np.int32)
        probs = np.empty(v, np.float32)
        g = C.c_int32(-1)
        n = self.lib.orc_target_selection(logits, v, cur_len, prefix, prefix.size, int(greedy), k, p, t, rep_pen,
                                          min_len, ngram, eos, eos.size, C.byref(g), idx, probs)
        return g.value, idx[:n].copy(), probs[:n].copy()

    def verify_deterministic(self, proposal, selections, draws):
        proposal = _i32(proposal)
        off = np.zeros(len(selections) + 1, np.int32)
        for i, (ix, _) in enumerate(selections):
            off[i + 1] = off[i] + len(ix)
        sidx = _i32(np.concatenate([np.asarray(s[0]) for s in selections]))
        sprob = _f32(np.concatenate([np.asarray(s[1]) for s in selections]))
        draws = np.ascontiguousarray(np.asarray(draws, np.float64))
        if draws.size == 0:
            draws = np.zeros(1, np.float64)
        ft, ev, ub, nd = C.c_int32(), C.c_int(), C.c_int(), C.c_int()
        acc = self.lib.orc_verify_deterministic(proposal, proposal.size, off, sidx, sprob, draws, C.byref(ft),
                                                C.byref(ev), C.byref(ub), C.byref(nd))
        return dict(accepted=acc, evaluated=ev.value, final_token=ft.value, used_bonus=bool(ub.value),
                    draws_used=nd.value)


class BeamScorer:
    """Handle around the oracle's BeamSearchScorer restatement."""

    def __init__(self, orc, batch, beams, max_length, pad, eos, length_penalty=1.0, early_stopping=True):
        self.L = orc.lib
        eos = _i32(eos)
        self.batch, self.beams, self.max_length = batch, beams, max_length
        self.h = self.L.orc_beam_scorer_create(batch, beams, max_length, pad, eos, eos.size, length_penalty,
                                               int(early_stopping))

    def __del__(self):
        if getattr(self, "h", None):
            self.L.orc_beam_scorer_destroy(self.h)
            self.h = None

    def process(self, sequences, seq_len, scores, tokens, indices):
        self.L.orc_beam_scorer_process(self.h, _i32(sequences).reshape(-1), seq_len, _f32(scores).reshape(-1),
                                       _i32(tokens).reshape(-1), _i32(indices).reshape(-1))

    def finalize(self, sequences, seq_len):
        self.L.orc_beam_scorer_finalize(self.h, _i32(sequences).reshape(-1), seq_len)

    def _arr(self, p, dt):
        n = self.batch * self.beams
        return np.ctypeslib.as_array(p, shape=(n,)).astype(dt).copy()

    @property
    def next_scores(self):
        return self._arr(self.L.orc_beam_scorer_next_scores(self.h), np.float32)

    @property
    def next_tokens(self):
        return self._arr(self.L.orc_beam_scorer_next_tokens(self.h), np.int32)

    @property
    def next_indices(self):
        return self._arr(self.L.orc_beam_scorer_next_indices(self.h), np.int32)

    def is_done(self):
        return bool(self.L.orc_beam_scorer_is_done(self.h))

    def batch_done(self, b):
        return bool(self.L.orc_beam_scorer_batch_done(self.h, b))

    def hyp_count(self, b):
        return self.L.orc_beam_scorer_hyp_count(self.h, b)

    def hyp(self, b, i):
        out = np.empty(self.max_length, np.int32)
        sc = C.c_float()
        n = self.L.orc_beam_scorer_hyp(self.h, b, i, out, out.size, C.byref(sc))
        return out[:n].copy(), sc.value


class Reference:
    """The unmodified reference headers behind a C wrapper (only where oracle/_ref was built)."""

    @staticmethod
    def load():
        so = os.path.join(ORACLE_DIR, "_ref", "libref_headers.so")
        if not os.path.exists(so):
            return None
        return Reference(so)

    def __init__(self, so):
        L = self.lib = C.CDLL(so)
        L.ref_sampled_categorical.restype = C.c_int
        L.ref_sampled_categorical.argtypes = [f32p, C.c_int, C.c_int, C.c_float, C.c_float, i32p, f32p]
        L.ref_sample_categorical.restype = C.c_int32
        L.ref_sample_categorical.argtypes = [i32p, f32p, C.c_int, C.c_uint32, C.POINTER(C.c_double), C.POINTER(C.c_int)]
        L.ref_uniform_float.restype = C.c_float
        L.ref_uniform_float.argtypes = [C.c_uint32]
        L.ref_softmax.argtypes = [f32p, C.c_int, C.c_float]
        L.ref_log_softmax.argtypes = [f32p, C.c_int, C.c_float]
        L.ref_apply_min_length.argtypes = [f32p, C.c_int, C.c_int, C.c_int, i32p, C.c_int]
        L.ref_apply_repetition_penalty.argtypes = [f32p, C.c_int, i32p, C.c_int, C.c_float]
        L.ref_apply_no_repeat_ngram.argtypes = [f32p, C.c_int, i32p, C.c_int, C.c_int]
        L.ref_accept_prob.restype = C.c_float
        L.ref_accept_prob.argtypes = [C.c_float, C.c_float]
        L.ref_build_correction.argtypes = [f32p, f32p, f32p, C.c_int]
        L.ref_sample_correction.restype = C.c_int32
        L.ref_sample_correction.argtypes = [i32p, f32p, C.c_int, i32p, f32p, C.c_int, C.c_uint32, C.POINTER(C.c_double)]
        L.ref_target_selection.restype = C.c_int
        L.ref_target_selection.argtypes = [f32p, C.c_int, C.c_int, i32p, C.c_int, C.c_int, C.c_int, C.c_float,
                                           C.c_float, C.c_float, C.c_int, C.c_int, i32p, C.c_int,
                                           C.POINTER(C.c_int32), i32p, f32p]
        L.ref_spec_round_sparse.argtypes = [i32p, C.c_int, i32p, i32p, f32p, i32p, i32p, f32p, C.c_uint32, f32p, f64p,
                                            C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
        L.ref_verify_deterministic.restype = C.c_int
        L.ref_verify_deterministic.argtypes = [i32p, C.c_int, i32p, i32p, f32p, C.c_uint32, C.POINTER(C.c_int32),
                                               C.POINTER(C.c_int), C.POINTER(C.c_int), f64p, C.POINTER(C.c_int)]

    def sampled_categorical(self, scores, k, p, t):
        scores = _f32(scores)
        v = scores.size
        idx = np.empty(v, np.int32)
        probs = np.empty(v, np.float32)
        n = self.lib.ref_sampled_categorical(scores, v, k, p, t, idx, probs)
        return idx[:n].copy(), probs[:n].copy()

    def sample_categorical(self, idx, probs, seed):
        idx, probs = _i32(idx), _f32(probs)
        u = C.c_double()
        d = C.c_int()
        tok = self.lib.ref_sample_categorical(idx, probs, idx.size, seed, C.byref(u), C.byref(d))
        return int(tok), u.value, d.value

    def softmax(self, s, t):
        s = _f32(s).copy()
        self.lib.ref_softmax(s, s.size, t)
        return s

    def log_softmax(self, s, t):
        s = _f32(s).copy()
        self.lib.ref_log_softmax(s, s.size, t)
        return s

    def apply_min_length(self, row, cur, min_len, eos):
        row = _f32(row).copy()
        eos = _i32(eos)
        self.lib.ref_apply_min_length(row, row.size, cur, min_len, eos, eos.size)
        return row

    def apply_repetition_penalty(self, row, prefix, pen):
        row = _f32(row).copy()
        prefix = _i32(prefix)
        self.lib.ref_apply_repetition_penalty(row, row.size, prefix, prefix.size, pen)
        return row

    def apply_no_repeat_ngram(self, row, prefix, n):
        row = _f32(row).copy()
        prefix = _i32(prefix)
        self.lib.ref_apply_no_repeat_ngram(row, row.size, prefix, prefix.size, n)
        return row

    def accept_prob(self, pt, pd):
        return float(self.lib.ref_accept_prob(pt, pd))

    def build_correction(self, pt, pd):
        pt, pd = _f32(pt), _f32(pd)
        out = np.empty_like(pt)
        self.lib.ref_build_correction(pt, pd, out, pt.size)
        return out

    def sample_correction(self, t_idx, t_probs, d_idx, d_probs, seed):
        t_idx, d_idx = _i32(t_idx), _i32(d_idx)
        t_probs, d_probs = _f32(t_probs), _f32(d_probs)
        u = C.c_double()
        tok = self.lib.ref_sample_correction(t_idx, t_probs, t_idx.size, d_idx, d_probs, d_idx.size, seed, C.byref(u))
        return int(tok), u.value

    def target_selection(self, logits, cur_len, prefix, greedy, k, p, t, rep_pen=1.0, min_len=0, ngram=0, eos=()):
        logits = _f32(logits)
        prefix = _i32(prefix)
        eos = _i32(eos)
        v = logits.size
        idx = np.empty(v, np.int32)
        probs = np.empty(v, np.float32)
        g = C.c_int32(-1)
        n = self.lib.ref_target_selection(logits, v, cur_len, prefix, prefix.size, int(greedy), k, p, t, rep_pen,
                                          min_len, ngram, eos, eos.size, C.byref(g), idx, probs)
        return g.value, idx[:n].copy(), probs[:n].copy()

    def spec_round_sparse(self, proposal, target_rows, draft_rows, seed):
        """The reference's accept loop with std::mt19937{seed}: returns (accepted, final token, engine draws
        consumed, accept uniforms [K], candidate categorical draws [K+1])."""
        proposal = _i32(proposal)
        k = proposal.size
        toff, tidx, tprob = _csr(target_rows)
        doff, didx, dprob = _csr(draft_rows)
        au = np.zeros(max(k, 1), np.float32)
        su = np.zeros(k + 1, np.float64)
        acc, tok, used = C.c_int32(), C.c_int32(), C.c_int32()
        self.lib.ref_spec_round_sparse(proposal, k, toff, tidx, tprob, doff, didx, dprob, seed, au, su, C.byref(acc),
                                       C.byref(tok), C.byref(used))
        return acc.value, tok.value, used.value, au[:k].copy(), su

    def verify_deterministic(self, proposal, selections, seed):
        proposal = _i32(proposal)
        off = np.zeros(len(selections) + 1, np.int32)
        for i, (ix, _) in enumerate(selections):
            off[i + 1] = off[i] + len(ix)
        sidx = _i32(np.concatenate([np.asarray(s[0]) for s in selections]))
        sprob = _f32(np.concatenate([np.asarray(s[1]) for s in selections]))
        draws = np.zeros(proposal.size + 2, np.float64)
        ft, ev, ub, nd = C.c_int32(), C.c_int(), C.c_int(), C.c_int()
        acc = self.lib.ref_verify_deterministic(proposal, proposal.size, off, sidx, sprob, seed, C.byref(ft),
                                                C.byref(ev), C.byref(ub), draws, C.byref(nd))
        return dict(accepted=acc, evaluated=ev.value, final_token=ft.value, used_bonus=bool(ub.value),
                    draws=draws[:nd.value].copy())
