"""ctypes binding of include/mi355x_search.h for Python callers (tests, bench).  Device memory is
supplied by the caller as torch CUDA tensors; this module only passes pointers.  There is no CPU
fallback: if the shared library is missing, loading fails."""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
MI355X_F32 = 1
MI355X_F16 = 10
MAX_EOS = 16


def library_path():
    return os.path.join(_HERE, "libmi355x_search.so")


class LogitsXformC(C.Structure):
    _fields_ = [("mask", C.c_void_p), ("history", C.c_void_p), ("history_stride", C.c_int32),
                ("history_len", C.c_int32), ("repetition_penalty", C.c_float), ("apply_min_length", C.c_int32),
                ("n_eos", C.c_int32), ("eos_ids", C.c_int32 * MAX_EOS), ("history_lens", C.c_void_p),
                ("min_length", C.c_int32), ("no_repeat_ngram_size", C.c_int32), ("mask_allowed_max", C.c_int32)]


class SampleParams(C.Structure):
    _fields_ = [("k", C.c_int32), ("p", C.c_float), ("temperature", C.c_float)]


_lib = None


def load_library():
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with __graft_entry__.build() (hipcc, gfx950); "
                           "there is no CPU fallback")
    L = C.CDLL(path)
    vp, i32, i64, f32 = C.c_void_p, C.c_int, C.c_int64, C.c_float
    L.mi355x_search_create.argtypes = [i32, i32, i32, C.POINTER(vp)]
    L.mi355x_search_destroy.argtypes = [vp]
    L.mi355x_search_destroy.restype = None
    L.mi355x_search_last_error.restype = C.c_char_p
    L.mi355x_search_workspace_bytes.argtypes = [vp]
    L.mi355x_search_workspace_bytes.restype = C.c_size_t
    L.mi355x_process_logits.argtypes = [vp, vp, vp, i64, i32, i32, C.POINTER(LogitsXformC)]
    L.mi355x_argmax.argtypes = [vp, vp, vp, i32, i64, i32, i32, C.POINTER(LogitsXformC), vp]
    L.mi355x_argmax_static.argtypes = [vp, vp, i32, i64, i32, i32, C.POINTER(LogitsXformC), vp]
    L.mi355x_sample.argtypes = [vp, vp, vp, i64, i32, i32, C.POINTER(LogitsXformC), SampleParams,
                                C.POINTER(SampleParams), vp, vp, vp, vp, vp, i32]
    L.mi355x_sample_typed.argtypes = [vp, vp, vp, i32, i64, i32, i32, C.POINTER(LogitsXformC), SampleParams,
                                      C.POINTER(SampleParams), vp, vp, vp, vp, vp, i32]
    L.mi355x_sample_scattered.argtypes = [vp, vp, C.POINTER(vp), i32, i32, i32, C.POINTER(LogitsXformC), SampleParams,
                                          C.POINTER(SampleParams), vp, vp, vp, vp, vp, i32]
    L.mi355x_search_fallback_rows.argtypes = [vp, vp, C.POINTER(C.c_uint)]
    L.mi355x_search_wait_gave_up.argtypes = [vp, vp, C.POINTER(C.c_int)]
    L.mi355x_search_set_poll_limit.argtypes = [vp, C.c_int]
    L.mi355x_search_sum_waits_gave_up.argtypes = [vp, vp, C.POINTER(C.c_uint)]
    for name, args in {
        "mi355x_topk_scores": [vp, vp, vp, i32, i64, i32, i32, i32, vp, vp],
        "mi355x_softmax": [vp, vp, vp, i64, i32, i32, f32, i32],
        "mi355x_beam_select": [vp, vp, vp, i32, i64, i32, i32, i32, vp, vp, vp, vp],
        "mi355x_beam_scorer_create": [vp, i32, i32, i32, i32, C.POINTER(C.c_int32), i32, f32, i32, C.POINTER(vp)],
        "mi355x_beam_scorer_set_prompt": [vp, vp, C.POINTER(C.c_int32), i32],
        "mi355x_draw_in_order": [vp, vp, vp, vp, vp, i32, i32, vp, vp, vp, vp],
        "mi355x_beam_scorer_step": [vp, vp, vp, vp, vp],
        "mi355x_beam_search_step": [vp, vp, vp, i32, i64, i32],
        "mi355x_beam_scorer_is_done": [vp, vp, C.POINTER(C.c_int)],
        "mi355x_beam_scorer_hypothesis": [vp, vp, i32, i32, C.POINTER(C.c_int32), i32, C.POINTER(C.c_int),
                                          C.POINTER(C.c_float)],
        "mi355x_kv_gather": [vp, vp, C.POINTER(vp), C.POINTER(vp), i32, vp, i32, C.c_size_t],
        "mi355x_spec_verify": [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, vp],
        "mi355x_spec_verify_sparse": [vp, vp, vp, vp, vp, i32, vp, vp, vp, i32, vp, vp, vp, i32, i32, i32, vp, vp, vp],
        "mi355x_greedy_tail": [vp, vp, vp, vp, i32, C.POINTER(C.c_int32), i32, i32, vp, i32, i32, vp],
        "mi355x_cast": [vp, vp, vp, i32, vp, i32, C.c_size_t],
        "mi355x_logits_handoff": [vp, vp, vp, i32, i32, i32, i32, C.POINTER(C.c_int32), vp, i64],
    }.items():
        if hasattr(L, name):
            getattr(L, name).argtypes = args
    if hasattr(L, "mi355x_beam_scorer_destroy"):
        L.mi355x_beam_scorer_destroy.argtypes = [vp]
        L.mi355x_beam_scorer_destroy.restype = None
        for n in ("next_scores", "next_tokens", "next_indices"):
            f = getattr(L, "mi355x_beam_scorer_" + n)
            f.argtypes = [vp]
            f.restype = vp
        L.mi355x_beam_scorer_sequences.argtypes = [vp, C.POINTER(C.c_int)]
        L.mi355x_beam_scorer_sequences.restype = vp
    _lib = L
    return L


class LogitsXform:
    """Python-side description of the fused logits processing (mask / min length / repetition penalty /
    no-repeat n-grams).  Holds references to the tensors so they outlive the asynchronous call.
    shared_history=True lets every row read the one history row given (stride 0), with history_lens
    telling how much of it each row sees: the verify rows of speculative decoding."""

    def __init__(self, mask=None, history=None, history_len=None, repetition_penalty=1.0, eos_ids=(),
                 apply_min_length=False, history_lens=None, min_length=0, no_repeat_ngram_size=0,
                 shared_history=False, mask_allowed_max=0):
        self.mask, self.history, self.history_lens = mask, history, history_lens
        c = self.c = LogitsXformC()
        c.mask = mask.data_ptr() if mask is not None else None
        if mask is not None:
            assert mask.dtype == torch.int32 and mask.is_cuda and mask.is_contiguous()
        if history is not None:
            assert history.dtype == torch.int32 and history.is_cuda and history.is_contiguous() and history.dim() == 2
            c.history = history.data_ptr()
            c.history_stride = 0 if shared_history else history.shape[1]
            c.history_len = history.shape[1] if history_len is None else history_len
        if history_lens is not None:
            assert history_lens.dtype == torch.int32 and history_lens.is_cuda and history_lens.is_contiguous()
            c.history_lens = history_lens.data_ptr()
        c.repetition_penalty = repetition_penalty
        c.apply_min_length = int(apply_min_length)
        c.min_length = min_length
        c.no_repeat_ngram_size = no_repeat_ngram_size
        c.mask_allowed_max = mask_allowed_max
        c.n_eos = len(eos_ids)
        for i, e in enumerate(eos_ids):
            c.eos_ids[i] = e


_DTYPE_CODES = {torch.float32: 1, torch.int32: 6, torch.int64: 7, torch.float16: 10, torch.bfloat16: 16}


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def argmax_static(logits, out, xf=None):
    """mi355x_argmax_static: argmax of every row into the caller's `out` ([rows] int32 on the same device), on the
    current stream of the current device; needs no context and allocates nothing."""
    L = load_library()
    assert logits.is_cuda and logits.dim() == 2 and logits.stride(1) == 1
    assert out.is_cuda and out.dtype == torch.int32 and out.numel() >= logits.shape[0] and out.is_contiguous()
    dtype = _DTYPE_CODES[logits.dtype]
    rc = L.mi355x_argmax_static(_stream(), logits.data_ptr(), dtype, logits.stride(0), logits.shape[0], logits.shape[1],
                                C.byref(xf.c) if xf else None, out.data_ptr())
    if rc != 0:
        raise RuntimeError(f"mi355x_search error {rc}: {L.mi355x_search_last_error().decode()}")
    return out


class SearchContext:
    """Owns a mi355x_search_ctx.  All tensor arguments must be CUDA tensors on the context's device."""

    def __init__(self, max_rows, max_vocab, device=0):
        self.L = load_library()
        torch.cuda.init()
        h = C.c_void_p()
        self._check(self.L.mi355x_search_create(device, max_rows, max_vocab, C.byref(h)))
        self.h = h
        self.device = torch.device("cuda", device)

    def close(self):
        if getattr(self, "h", None):
            self.L.mi355x_search_destroy(self.h)
            self.h = None

    __del__ = close

    def _check(self, rc):
        if rc != 0:
            raise RuntimeError(f"mi355x_search error {rc}: {self.L.mi355x_search_last_error().decode()}")

    def workspace_bytes(self):
        return self.L.mi355x_search_workspace_bytes(self.h)

    def fallback_rows(self):
        n = C.c_uint()
        self._check(self.L.mi355x_search_fallback_rows(self.h, _stream(), C.byref(n)))
        return n.value

    def wait_gave_up(self):
        g = C.c_int()
        self._check(self.L.mi355x_search_wait_gave_up(self.h, _stream(), C.byref(g)))
        return bool(g.value)

    def sum_waits_gave_up(self):
        n = C.c_uint()
        self._check(self.L.mi355x_search_sum_waits_gave_up(self.h, _stream(), C.byref(n)))
        return n.value

    def set_poll_limit(self, polls):
        self._check(self.L.mi355x_search_set_poll_limit(self.h, int(polls)))

    @staticmethod
    def _rows(logits):
        assert logits.is_cuda and logits.dim() == 2 and logits.stride(1) == 1
        return logits.shape[0], logits.shape[1], logits.stride(0)

    def process_logits(self, logits, xf):
        rows, vocab, stride = self._rows(logits)
        assert logits.dtype == torch.float32
        self._check(self.L.mi355x_process_logits(self.h, _stream(), logits.data_ptr(), stride, rows, vocab,
                                                 C.byref(xf.c)))
        return logits

    def argmax(self, logits, xf=None, out=None):
        rows, vocab, stride = self._rows(logits)
        dtype = _DTYPE_CODES[logits.dtype]
        if out is None:
            out = torch.empty(rows, dtype=torch.int32, device=logits.device)
        self._check(self.L.mi355x_argmax(self.h, _stream(), logits.data_ptr(), dtype, stride, rows, vocab,
                                         C.byref(xf.c) if xf else None, out.data_ptr()))
        return out

    def sample(self, logits, uniforms, k=0, p=0.0, temperature=1.0, per_row=None, xf=None, out=None,
               kept_capacity=0):
        """logits: a [rows, vocab] tensor, or a list of rows (1-D tensors of one dtype and length, anywhere in
        device memory), which goes through mi355x_sample_scattered."""
        scattered = isinstance(logits, (list, tuple))
        if scattered:
            row_list, logits = logits, logits[0].unsqueeze(0)
            assert all(r.is_cuda and r.dim() == 1 and r.stride(0) == 1 and r.dtype == logits.dtype and
                       r.numel() == logits.shape[1] for r in row_list)
            rows, vocab, stride = len(row_list), logits.shape[1], logits.shape[1]
        else:
            rows, vocab, stride = self._rows(logits)
        assert uniforms.dtype == torch.float64 and uniforms.numel() >= rows
        if out is None:
            out = torch.empty(rows, dtype=torch.int32, device=logits.device)
        pr = None
        if per_row is not None:
            pr = (SampleParams * rows)(*[SampleParams(int(a), float(b), float(c)) for a, b, c in per_row])
        kc = ki = kp = None
        if kept_capacity:
            kc = torch.empty(rows, dtype=torch.int32, device=logits.device)
            ki = torch.full((rows, kept_capacity), -1, dtype=torch.int32, device=logits.device)
            kp = torch.zeros((rows, kept_capacity), dtype=torch.float32, device=logits.device)
        args = (stride, rows, vocab, C.byref(xf.c) if xf else None, SampleParams(int(k), float(p), float(temperature)),
                pr, uniforms.data_ptr(), out.data_ptr(), kc.data_ptr() if kept_capacity else None,
                ki.data_ptr() if kept_capacity else None, kp.data_ptr() if kept_capacity else None, kept_capacity)
        if scattered:
            ptrs = (C.c_void_p * rows)(*[r.data_ptr() for r in row_list])
            self._check(self.L.mi355x_sample_scattered(self.h, _stream(), ptrs, _DTYPE_CODES[logits.dtype], *args[1:]))
        elif logits.dtype == torch.float32:
            self._check(self.L.mi355x_sample(self.h, _stream(), logits.data_ptr(), *args))
        else:  # fp16 / bf16 rows are read as they are
            self._check(self.L.mi355x_sample_typed(self.h, _stream(), logits.data_ptr(), _DTYPE_CODES[logits.dtype], *args))
        if kept_capacity:
            return out, kc, ki, kp
        return out

    def prepared_sample(self, logits, uniforms, out, k=0, p=0.0, temperature=1.0, xf=None, stream=None):
        """Marshals one mi355x_sample call once and returns a function that issues it: what a serving loop with fixed
        buffers does (the tensors, `xf` and the stream -- default: the stream current now -- must stay alive and
        where they are; the function takes no arguments and raises on an error code).  `out` may be pinned host
        memory.  The per-call cost is the foreign call alone, none of the tensor lookups of `sample`.  As with every
        call, one context serves one stream at a time: calls prepared for different streams must not overlap."""
        rows, vocab, stride = self._rows(logits)
        assert uniforms.dtype == torch.float64 and uniforms.numel() >= rows and out.dtype == torch.int32 and out.numel() >= rows
        handle = C.c_void_p(stream.cuda_stream) if stream is not None else _stream()
        typed = logits.dtype != torch.float32
        fn = self.L.mi355x_sample_typed if typed else self.L.mi355x_sample
        head = (self.h, handle, C.c_void_p(logits.data_ptr())) + ((C.c_int32(_DTYPE_CODES[logits.dtype]),) if typed else ())
        args = head + (C.c_int64(stride), C.c_int32(rows), C.c_int32(vocab), C.byref(xf.c) if xf else None,
                       SampleParams(int(k), float(p), float(temperature)), None, C.c_void_p(uniforms.data_ptr()),
                       C.c_void_p(out.data_ptr()), None, None, None, C.c_int32(0))
        keep = (logits, uniforms, out, xf, stream)
        check = self._check

        def issue(_args=args, _fn=fn, _keep=keep):
            rc = _fn(*_args)
            if rc != 0:
                check(rc)
        return issue



_hip_lib = None


def _hip():
    """The HIP runtime torch already loaded (device-to-device copies of library-owned buffers)."""
    global _hip_lib
    if _hip_lib is None:
        _hip_lib = C.CDLL("libamdhip64.so")
        _hip_lib.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        _hip_lib.hipMemcpy.restype = C.c_int
    return _hip_lib


def _dtype_code(t):
    return _DTYPE_CODES[t.dtype]


def _topk_scores(self, logits, k):
    rows, vocab, stride = self._rows(logits)
    tok = torch.empty((rows, k), dtype=torch.int32, device=logits.device)
    sc = torch.empty((rows, k), dtype=torch.float32, device=logits.device)
    self._check(self.L.mi355x_topk_scores(self.h, _stream(), logits.data_ptr(), _dtype_code(logits), stride, rows,
                                          vocab, k, tok.data_ptr(), sc.data_ptr()))
    return tok, sc


def _softmax(self, scores, temperature=1.0, log=False):
    rows, vocab, stride = self._rows(scores)
    assert scores.dtype == torch.float32
    self._check(self.L.mi355x_softmax(self.h, _stream(), scores.data_ptr(), stride, rows, vocab, temperature, int(log)))
    return scores


def _beam_select(self, logits, batch, beams, beam_scores):
    rows, vocab, stride = self._rows(logits)
    assert rows == batch * beams and beam_scores.dtype == torch.float32 and beam_scores.numel() == rows
    k = 2 * beams
    sc = torch.empty((batch, k), dtype=torch.float32, device=logits.device)
    tok = torch.empty((batch, k), dtype=torch.int32, device=logits.device)
    idx = torch.empty((batch, k), dtype=torch.int32, device=logits.device)
    self._check(self.L.mi355x_beam_select(self.h, _stream(), logits.data_ptr(), _dtype_code(logits), stride, batch,
                                          beams, vocab, beam_scores.data_ptr(), sc.data_ptr(), tok.data_ptr(),
                                          idx.data_ptr()))
    return sc, tok, idx


def _kv_gather(self, present, past, beam_indices):
    """present/past: lists of equally shaped contiguous CUDA tensors [rows, ...]; past[t][j] = present[t][idx[j]]."""
    n = len(present)
    assert n == len(past) and beam_indices.dtype == torch.int32
    block = present[0][0].numel() * present[0].element_size()
    for a, b in zip(present, past):
        assert a.is_contiguous() and b.is_contiguous() and a[0].numel() * a.element_size() == block
    pp = (C.c_void_p * n)(*[t.data_ptr() for t in present])
    qq = (C.c_void_p * n)(*[t.data_ptr() for t in past])
    self._check(self.L.mi355x_kv_gather(self.h, _stream(), pp, qq, n, beam_indices.data_ptr(), beam_indices.numel(),
                                        block))
    return past


def _spec_verify(self, p_target, p_draft, draft_tokens, accept_u, sample_u):
    b, k1, v = p_target.shape
    for t in (p_target, p_draft, draft_tokens, accept_u, sample_u):
        assert t.is_cuda and t.is_contiguous()
    assert p_target.dtype == torch.float32 and accept_u.dtype == torch.float32 and sample_u.dtype == torch.float64
    acc = torch.empty(b, dtype=torch.int32, device=p_target.device)
    tok = torch.empty(b, dtype=torch.int32, device=p_target.device)
    self._check(self.L.mi355x_spec_verify(self.h, _stream(), p_target.data_ptr(), p_draft.data_ptr(),
                                          draft_tokens.data_ptr(), accept_u.data_ptr(), sample_u.data_ptr(), b, k1 - 1,
                                          v, acc.data_ptr(), tok.data_ptr()))
    return acc, tok


def _spec_verify_sparse(self, target, draft, proposal, accept_u, sample_u, mode=0):
    """target = (count [b, K+1], ids [b, K+1, cap], probs [b, K+1, cap]) as mi355x_sample returns them;
    draft likewise with K rows (None unless mode 0).  Returns (accepted_len, final_token, engine_draws)."""
    tc, ti, tp = target
    b, k = proposal.shape
    assert tuple(tc.shape) == (b, k + 1) and tuple(ti.shape[:2]) == (b, k + 1)
    ptr = lambda t: t.data_ptr() if t is not None else None
    for t in (tc, ti, tp, proposal, accept_u, sample_u) + (tuple(draft) if draft is not None else ()):
        assert t is None or (t.is_cuda and t.is_contiguous())
    dc, di, dp = draft if draft is not None else (None, None, None)
    acc = torch.empty(b, dtype=torch.int32, device=proposal.device)
    tok = torch.empty(b, dtype=torch.int32, device=proposal.device)
    used = torch.empty(b, dtype=torch.int32, device=proposal.device)
    self._check(self.L.mi355x_spec_verify_sparse(self.h, _stream(), ptr(tc), ptr(ti), ptr(tp), ti.shape[2], ptr(dc), ptr(di),
                                                 ptr(dp), di.shape[2] if di is not None else 0, ptr(proposal),
                                                 ptr(accept_u), ptr(sample_u), b, k, mode, acc.data_ptr(), tok.data_ptr(),
                                                 used.data_ptr()))
    return acc, tok, used


def _greedy_tail(self, next_tokens, eos_seen, eos_ids, pad, sequences, current_length, done, allow_host=False):
    """EOS padding / marking, append at column current_length, all-rows-finished flag; all in place.
    allow_host: next_tokens and done may be pinned host tensors, which the kernel reads and writes in place."""
    for t in (next_tokens, eos_seen, sequences, done):
        assert t.is_contiguous() and t.dtype == torch.int32
        assert t.is_cuda or (allow_host and t.is_pinned())
    eos = (C.c_int32 * max(len(eos_ids), 1))(*eos_ids)
    self._check(self.L.mi355x_greedy_tail(self.h, _stream(), next_tokens.data_ptr(), eos_seen.data_ptr(),
                                          next_tokens.numel(), eos, len(eos_ids), pad, sequences.data_ptr(),
                                          sequences.shape[1], current_length, done.data_ptr()))




def _draw_in_order(self, kept_count, kept_ids, kept_probs, uniform_pool, skip_rows=None):
    """SampleCategoricalToken for a batch served by one engine, rows in order: returns (tokens [rows], draws used)."""
    rows, cap = kept_ids.shape
    assert kept_count.dtype == torch.int32 and kept_ids.dtype == torch.int32 and kept_probs.dtype == torch.float32
    assert uniform_pool.dtype == torch.float64 and uniform_pool.numel() >= rows
    for t in (kept_count, kept_ids, kept_probs, uniform_pool):
        assert t.is_cuda and t.is_contiguous()
    out = torch.empty(rows, dtype=torch.int32, device=self.device)
    used = torch.zeros(1, dtype=torch.int32, device=self.device)
    self._check(self.L.mi355x_draw_in_order(self.h, _stream(), kept_count.data_ptr(), kept_ids.data_ptr(),
                                            kept_probs.data_ptr(), cap, rows,
                                            skip_rows.data_ptr() if skip_rows is not None else None,
                                            uniform_pool.data_ptr(), out.data_ptr(), used.data_ptr()))
    return out, used


def _cast(self, src, dtype):
    """DeviceInterface::Cast: returns a new tensor of `dtype` with the reference CPU path's conversion."""
    assert src.is_cuda and src.is_contiguous()
    out = torch.empty(src.shape, dtype=dtype, device=src.device)
    self._check(self.L.mi355x_cast(self.h, _stream(), src.data_ptr(), _DTYPE_CODES[src.dtype], out.data_ptr(),
                                   _DTYPE_CODES[dtype], src.numel()))
    return out


def _logits_handoff(self, raw, token_index=None, out=None):
    """Logits::Get: raw [rows, seq_len, vocab] (fp32 / fp16 / bf16) -> fp32 [rows, vocab] of each row's
    token_index (a host sequence; the last token when None)."""
    assert raw.is_cuda and raw.is_contiguous() and raw.dim() == 3
    rows, seq_len, vocab = raw.shape
    if out is None:
        out = torch.empty((rows, vocab), dtype=torch.float32, device=raw.device)
    ti = None
    if token_index is not None:
        ti = (C.c_int32 * rows)(*[int(t) for t in token_index])
    self._check(self.L.mi355x_logits_handoff(self.h, _stream(), raw.data_ptr(), _DTYPE_CODES[raw.dtype], rows, seq_len,
                                             vocab, ti, out.data_ptr(), out.stride(0)))
    return out


SearchContext.cast = _cast
SearchContext.logits_handoff = _logits_handoff
SearchContext.topk_scores = _topk_scores
SearchContext.softmax = _softmax
SearchContext.draw_in_order = _draw_in_order
SearchContext.beam_select = _beam_select
SearchContext.spec_verify_sparse = _spec_verify_sparse
SearchContext.greedy_tail = _greedy_tail
SearchContext.kv_gather = _kv_gather
SearchContext.spec_verify = _spec_verify


class BeamScorer:
    """Device-resident BeamSearchScorer + Sequences (mi355x_beam_scorer)."""

    def __init__(self, ctx, batch, beams, max_length, pad, eos, length_penalty=1.0, early_stopping=True):
        self.ctx, self.L = ctx, ctx.L
        self.batch, self.beams, self.max_length = batch, beams, max_length
        e = (C.c_int32 * max(1, len(eos)))(*eos)
        h = C.c_void_p()
        ctx._check(self.L.mi355x_beam_scorer_create(ctx.h, batch, beams, max_length, pad, e, len(eos),
                                                    length_penalty, int(early_stopping), C.byref(h)))
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            self.L.mi355x_beam_scorer_destroy(self.h)
            self.h = None

    __del__ = close

    def set_prompt(self, tokens):
        import numpy as np
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        assert t.shape[0] == self.batch
        self.ctx._check(self.L.mi355x_beam_scorer_set_prompt(self.h, _stream(), t.ctypes.data_as(C.POINTER(C.c_int32)),
                                                             t.shape[1]))

    def step(self, cand_scores, cand_tokens, cand_indices):
        self.ctx._check(self.L.mi355x_beam_scorer_step(self.h, _stream(), cand_scores.data_ptr(),
                                                       cand_tokens.data_ptr(), cand_indices.data_ptr()))

    def search_step(self, logits):
        """Selection and scorer step in one call (BeamSearch_Cpu::SelectTop): logits [batch*beams, vocab] fp32, fp16 or bf16."""
        assert logits.dim() == 2 and logits.stride(1) == 1 and logits.shape[0] == self.batch * self.beams
        self.ctx._check(self.L.mi355x_beam_search_step(self.h, _stream(), logits.data_ptr(), _DTYPE_CODES[logits.dtype],
                                                       logits.stride(0), logits.shape[1]))

    def _copy(self, ptr, dtype, count):
        out = torch.empty(count, dtype=dtype, device=self.ctx.device)
        torch.cuda.current_stream().synchronize()
        rc = _hip().hipMemcpy(C.c_void_p(out.data_ptr()), C.c_void_p(ptr), C.c_size_t(count * out.element_size()), 3)
        assert rc == 0, f"hipMemcpy failed: {rc}"
        return out

    @property
    def next_scores(self):
        return self._copy(self.L.mi355x_beam_scorer_next_scores(self.h), torch.float32, self.batch * self.beams)

    @property
    def next_tokens(self):
        return self._copy(self.L.mi355x_beam_scorer_next_tokens(self.h), torch.int32, self.batch * self.beams)

    @property
    def next_indices(self):
        return self._copy(self.L.mi355x_beam_scorer_next_indices(self.h), torch.int32, self.batch * self.beams)

    def next_scores_ptr(self):
        return self.L.mi355x_beam_scorer_next_scores(self.h)

    def sequences(self):
        n = C.c_int()
        p = self.L.mi355x_beam_scorer_sequences(self.h, C.byref(n))
        full = self._copy(p, torch.int32, self.batch * self.beams * self.max_length)
        return full.view(self.batch * self.beams, self.max_length)[:, :n.value], n.value

    def is_done(self):
        d = C.c_int()
        self.ctx._check(self.L.mi355x_beam_scorer_is_done(self.h, _stream(), C.byref(d)))
        return bool(d.value)

    def hypothesis(self, batch, index):
        buf = (C.c_int32 * self.max_length)()
        n = C.c_int()
        sc = C.c_float()
        self.ctx._check(self.L.mi355x_beam_scorer_hypothesis(self.h, _stream(), batch, index, buf, self.max_length,
                                                             C.byref(n), C.byref(sc)))
        return list(buf[:n.value]), sc.value
