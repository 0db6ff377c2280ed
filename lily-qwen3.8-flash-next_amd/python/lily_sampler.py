"""Host-side mirror of the reference's sampler interface over liblily_sampler_hip.so.

Names, argument meaning and error behaviour follow src/kernels/sample.rs,
src/kernels/spec.rs and src/kernels/elementwise.rs of the reference: every draw is
enqueued on the sampler's HIP stream, results land in device tensors, failures raise
`SamplerError` with the message the reference's `ensure!` would carry.  PyTorch is
used only to own device memory and the stream; all compute goes through the C ABI.
There is no fallback: if the library is missing, importing this module raises.
"""
import ctypes as C
import os
import weakref

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
# LILY_SAMPLER_LIBRARY names another build of the library (build.py --strict-handover leaves
# liblily_sampler_hip_strict.so beside the default one).
LIB_PATH = os.environ.get("LILY_SAMPLER_LIBRARY") or os.path.join(os.path.dirname(HERE), "liblily_sampler_hip.so")

SAMPLE_K_CAP = 1024
CTRL_STRIDE = 4
SLOT_ACCEPTED = 0
SLOT_KEEP = 1
NO_TOKEN = 0xFFFFFFFF
F32, BF16 = 0, 1


class SamplerError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"[{code}] {message}")
        self.code = code


class SamplingParams(C.Structure):
    """src/kernels/sample.rs:21-31."""

    _fields_ = [
        ("temperature", C.c_float),
        ("top_k", C.c_uint32),
        ("top_p", C.c_float),
        ("min_p", C.c_float),
        ("presence_penalty", C.c_float),
        ("frequency_penalty", C.c_float),
        ("repetition_penalty", C.c_float),
        ("reserved", C.c_uint32),
        ("seed", C.c_uint64),
    ]

    @classmethod
    def greedy(cls, **over):
        p = cls()
        _lib.lily_params_greedy(C.byref(p))
        for k, v in over.items():
            setattr(p, k, v)
        return p

    def is_greedy(self):
        return bool(_lib.lily_params_is_greedy(C.byref(self)))

    def uses_penalties(self):
        return bool(_lib.lily_params_uses_penalties(C.byref(self)))

    def validate(self):
        _check(_lib.lily_params_validate(C.byref(self)))

    def effective(self):
        t, k = C.c_float(), C.c_uint32()
        _lib.lily_params_effective(C.byref(self), C.byref(t), C.byref(k))
        return t.value, k.value


class _Bias(C.Structure):
    _fields_ = [("id", C.c_uint32), ("delta", C.c_float)]


class DraftDist(C.Structure):
    """src/kernels/sample.rs:193-197: one slot's device arrays."""

    _fields_ = [("ids_dev", C.c_void_p), ("probs_dev", C.c_void_p), ("count_dev", C.c_void_p)]


class _Rows(C.Structure):
    _fields_ = [
        ("rows", C.c_uint32), ("vocab", C.c_uint32), ("dtype", C.c_uint32),
        ("reserved", C.c_uint32),
        ("logits_dev", C.c_void_p), ("row_stride", C.c_uint64),
        ("params", C.POINTER(SamplingParams)), ("steps", C.POINTER(C.c_uint32)),
        ("scratch", C.POINTER(C.c_void_p)),
        ("allow_dev", C.c_void_p), ("allow_stride", C.c_uint64),
        ("bias_dev", C.c_void_p), ("bias_offsets", C.POINTER(C.c_uint32)),
        ("forced", C.POINTER(C.c_uint32)), ("uniforms", C.POINTER(C.c_float)),
        ("out_ids_dev", C.c_void_p), ("out_logprobs_dev", C.c_void_p),
        ("dbg_ids_dev", C.c_void_p), ("dbg_probs_dev", C.c_void_p),
        ("dbg_counts_dev", C.c_void_p),
    ]


class _LmHead(C.Structure):
    _fields_ = [("hidden_dev", C.c_void_p), ("hidden_stride", C.c_uint64),
                ("weight_dev", C.c_void_p), ("weight_stride", C.c_uint64),
                ("d", C.c_uint32), ("weight_bits", C.c_uint32),
                ("tile_max_dev", C.c_void_p), ("tile_sum_dev", C.c_void_p),
                ("scales_dev", C.c_void_p), ("biases_dev", C.c_void_p),
                ("group_size", C.c_uint32), ("logits_f32", C.c_uint32)]


class QuantWeights:
    """The reference's affine weights (src/weights.rs:27-36): codes int32 [out, in * bits / 32]
    (u32 words, the lowest code first), scales and biases bf16 [out, in / group_size]."""

    def __init__(self, codes, scales, biases, group_size, bits):
        self.codes, self.scales, self.biases = codes, scales, biases
        self.group_size, self.bits = int(group_size), int(bits)

    @property
    def in_features(self):
        return self.codes.shape[1] * (32 // self.bits)


LOGIT_TILE_COLS = 128


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with "
            "`python lily-qwen3.8-flash-next_amd/build.py` (there is no CPU fallback)")
    L = C.CDLL(LIB_PATH)
    L.lily_last_error.restype = C.c_char_p
    L.lily_uniform_for.restype = C.c_float
    L.lily_uniform_for.argtypes = [C.c_uint64, C.c_uint32]
    L.lily_draft_step.restype = C.c_uint32
    L.lily_draft_step.argtypes = [C.c_uint32]
    for n in ("lily_slot_pos", "lily_slot_block", "lily_slot_count", "lily_ctrl_words"):
        getattr(L, n).restype = C.c_uint32
        getattr(L, n).argtypes = [C.c_uint32]
    L.lily_sampler_slices_for.restype = C.c_uint32
    L.lily_sampler_slices_for.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int]
    L.lily_scratch_vocab.restype = C.c_uint32
    L.lily_scratch_vocab.argtypes = [C.c_void_p]
    vp, u32, u64 = C.c_void_p, C.c_uint32, C.c_uint64
    P = C.POINTER(SamplingParams)
    sigs = {
        "lily_sampler_create": [C.c_int, vp, C.POINTER(vp)],
        "lily_sampler_synchronize": [vp],
        "lily_sampler_set_phase_trace": [vp, vp, u64],
        "lily_sampler_set_path_stats": [vp, vp],
        "lily_probe_read": [vp, vp, C.c_uint32, C.c_uint64, C.c_uint64, vp],
        "lily_scratch_create": [vp, u32, C.POINTER(vp)],
        "lily_scratch_reset_counts": [vp],
        "lily_scratch_uncount": [vp, u32],
        "lily_scratch_uncount_after": [vp, vp, u32, vp, u32],
        "lily_scratch_copy_counts_from": [vp, vp],
        "lily_scratch_add_history": [vp, vp, u32],
        "lily_scratch_write_counts": [vp, vp],
        "lily_scratch_read_counts": [vp, vp],
        "lily_draft_dists_create": [vp, u32, C.POINTER(vp)],
        "lily_draft_dists_slot": [vp, u32, C.POINTER(DraftDist)],
        "lily_sample_f32": [vp, vp, u32, vp, P, u32, vp],
        "lily_sample_draft_f32": [vp, vp, u32, vp, P, u32, vp, C.POINTER(DraftDist)],
        "lily_token_slots_create": [vp, u32, u32, C.POINTER(vp)],
        "lily_token_slots_publish": [vp, u32],
        "lily_token_slots_poll": [vp, u32, vp, C.POINTER(C.c_int)],
        "lily_token_slots_wait_polled": [vp, u32, vp, u64],
        "lily_scratch_move_counts": [vp, vp],
        "lily_sample_f32_at": [vp, vp, u32, u64, u32, vp, vp, P, u32, vp, vp],
        "lily_sample_draft_f32_at": [vp, vp, u32, u64, u32, vp, vp, P, u32, vp, vp, C.POINTER(DraftDist)],
        "lily_sample_spec_f32": [vp, vp, u32, vp, P, u32, C.POINTER(DraftDist), vp, vp],
        "lily_argmax_f32": [vp, vp, u32, vp],
        "lily_sample_f32_static": [vp, vp, u32, vp, P, u32, vp],
        "lily_spec_accept": [vp, vp, vp, u32, vp, u32, u32, u32, u32],
        "lily_copy_row_u32": [vp, vp, u32, u32, vp, vp],
        "lily_spec_verify": [vp, vp, C.c_int, u32, u64, u32, vp, P, u32, vp, vp, vp, vp, u32, u32,
                             u32, u32, C.POINTER(C.c_float)],
        "lily_sample_spec_f32_uniforms": [vp, vp, u32, vp, P, u32, C.POINTER(DraftDist), vp, vp,
                                          C.c_float, C.c_float],
        "lily_sample_rows": [vp, C.POINTER(_Rows)],
        "lily_plan_create": [vp, u32, C.POINTER(vp)],
        "lily_plan_set": [vp, C.POINTER(_Rows)],
        "lily_plan_run": [vp, u32],
        "lily_params_validate": [P],
        "lily_lm_head_bf16": [vp, C.POINTER(_LmHead), u32, u32, C.POINTER(C.c_float), vp, u64],
        "lily_sample_rows_tiled": [vp, C.POINTER(_Rows), vp, vp],
        "lily_lm_head_sample_rows": [vp, C.POINTER(_LmHead), C.POINTER(_Rows)],
    }
    L.lily_insertions_create.restype = C.c_int
    L.lily_insertions_create.argtypes = [u32, C.POINTER(vp)]
    L.lily_insertions_push.restype = C.c_int
    L.lily_insertions_push.argtypes = [vp, u32, C.c_int, u32, C.POINTER(u32), u32, vp]
    L.lily_insertions_next.restype = u32
    L.lily_insertions_next.argtypes = [vp, C.POINTER(u32)]
    L.lily_insertions_pending.restype = u32
    L.lily_insertions_pending.argtypes = [vp, u32]
    L.lily_insertions_clear.restype = None
    L.lily_insertions_clear.argtypes = [vp, u32]
    L.lily_insertions_destroy.restype = None
    L.lily_insertions_destroy.argtypes = [vp]
    L.lily_lm_head_tiles.restype = C.c_uint32
    L.lily_lm_head_tiles.argtypes = [C.c_uint32]
    L.lily_lm_head_library_calls.restype = C.c_uint64
    L.lily_lm_head_library_calls.argtypes = [vp]
    for name, args in sigs.items():
        getattr(L, name).restype = C.c_int
        getattr(L, name).argtypes = args
    for name in ("lily_sampler_destroy", "lily_scratch_destroy", "lily_draft_dists_destroy",
                 "lily_plan_destroy", "lily_token_slots_destroy"):
        getattr(L, name).restype = None
        getattr(L, name).argtypes = [vp]
    L.lily_token_slots_device.restype = vp
    L.lily_token_slots_device.argtypes = [vp, u32]
    return L


_lib = _load()


def _check(rc):
    if rc != 0:
        raise SamplerError(rc, _lib.lily_last_error().decode())


def _ptr(t, dtype=None):
    if t is None:
        return None
    if not t.is_cuda:
        raise SamplerError(-1, "tensor must live on the GPU")
    if dtype is not None and t.dtype != dtype:
        raise SamplerError(-1, f"tensor must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise SamplerError(-1, "tensor must be contiguous")
    return C.c_void_p(t.data_ptr())


def sample_f32_static(stream, logits, scratch, params, step, out):
    """lily_sample_f32_static: the draw that needs no sampler object and allocates nothing,
    enqueued on `stream` (a torch.cuda.Stream) of the current device."""
    _check(_lib.lily_sample_f32_static(C.c_void_p(stream.cuda_stream), _ptr(logits, torch.float32),
                                       logits.numel(), scratch._h if scratch else None,
                                       C.byref(params), step, _ptr(out, torch.int32)))


def uniform_for(seed, step):
    """src/kernels/sample.rs:435-441."""
    return float(_lib.lily_uniform_for(seed, step))


def draft_step(step):
    """src/kernels/sample.rs:220-222."""
    return int(_lib.lily_draft_step(step))


def draft_params(p):
    """src/kernels/sample.rs:227-234."""
    out = SamplingParams()
    _lib.lily_draft_params(C.byref(p), C.byref(out))
    return out


def slot_pos(i):
    return int(_lib.lily_slot_pos(i))


def slot_block(i):
    return int(_lib.lily_slot_block(i))


def slot_count(i):
    return int(_lib.lily_slot_count(i))


def ctrl_words(chain):
    return int(_lib.lily_ctrl_words(chain))


class Sampler:
    """The context a draw is encoded on: one device, one HIP stream."""

    def __init__(self, device=0, stream=None):
        torch.cuda.init()
        self.device = device
        # Default: torch's current stream, so draws are ordered with the tensor work around them.
        self.stream = stream if stream is not None else torch.cuda.current_stream(device)
        h = C.c_void_p()
        _check(_lib.lily_sampler_create(device, C.c_void_p(self.stream.cuda_stream), C.byref(h)))
        self._h = h
        self._children = weakref.WeakSet()  # scratches, dists, plans: closed before the sampler

    def close(self):
        if self._h:
            for child in list(self._children):
                child.close()
            _lib.lily_sampler_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_phase_trace(self, trace):
        """trace: device int64 tensor (or None); see lily_sampler_set_phase_trace."""
        self._trace = trace
        _check(_lib.lily_sampler_set_phase_trace(
            self._h, _ptr(trace, torch.int64) if trace is not None else None,
            trace.numel() if trace is not None else 0))

    def set_path_stats(self, stats):
        """stats: device int32 tensor of 4 counters (or None); see lily_sampler_set_path_stats."""
        self._stats = stats
        _check(_lib.lily_sampler_set_path_stats(
            self._h, _ptr(stats, torch.int32) if stats is not None else None))

    def probe_read(self, rows_tensor, out):
        """One read-only launch over a 2-D contiguous device tensor, a workgroup per row; out:
        int32[rows], cleared by the caller.  See lily_probe_read."""
        assert rows_tensor.dim() == 2 and rows_tensor.is_contiguous()
        row_bytes = rows_tensor.shape[1] * rows_tensor.element_size()
        _check(_lib.lily_probe_read(self._h, C.c_void_p(rows_tensor.data_ptr()), rows_tensor.shape[0],
                                    row_bytes // 16 * 16, row_bytes, _ptr(out, torch.int32)))

    def slices_for(self, rows, k, vocab, bf16=False):
        return int(_lib.lily_sampler_slices_for(self._h, rows, k, vocab, 1 if bf16 else 0))

    def synchronize(self):
        """ComputePass::commit_wait."""
        _check(_lib.lily_sampler_synchronize(self._h))

    # -- single-row draws, src/kernels/sample.rs:373-432
    def sample_f32(self, logits, scratch, params, step, out):
        _check(_lib.lily_sample_f32(self._h, _ptr(logits, torch.float32), logits.numel(),
                                    scratch._h if scratch else None, C.byref(params), step,
                                    _ptr(out, torch.int32)))

    def sample_draft_f32(self, logits, scratch, params, step, out, dist):
        _check(_lib.lily_sample_draft_f32(self._h, _ptr(logits, torch.float32), logits.numel(),
                                          scratch._h if scratch else None, C.byref(params), step,
                                          _ptr(out, torch.int32), C.byref(dist)))

    def sample_f32_at(self, logits_rows, row_dev, scratch, params, step_base, step_dev, out):
        """lily_sample_f32_at: logits_rows [rows, V] f32; row_dev / step_dev: int32 device tensors
        (or views) holding the row index and the step offset, or None."""
        rows, vocab = logits_rows.shape
        _check(_lib.lily_sample_f32_at(
            self._h, _ptr(logits_rows, torch.float32), vocab, logits_rows.stride(0), rows,
            _ptr(row_dev, torch.int32) if row_dev is not None else None,
            scratch._h if scratch else None, C.byref(params), step_base,
            _ptr(step_dev, torch.int32) if step_dev is not None else None, _ptr(out, torch.int32)))

    def sample_draft_f32_at(self, logits_rows, row_dev, scratch, params, step_base, step_dev, out, dist):
        rows, vocab = logits_rows.shape
        _check(_lib.lily_sample_draft_f32_at(
            self._h, _ptr(logits_rows, torch.float32), vocab, logits_rows.stride(0), rows,
            _ptr(row_dev, torch.int32) if row_dev is not None else None,
            scratch._h if scratch else None, C.byref(params), step_base,
            _ptr(step_dev, torch.int32) if step_dev is not None else None, _ptr(out, torch.int32),
            C.byref(dist)))

    def sample_spec_f32(self, logits, scratch, params, step, dist, draft, out, uniforms=None):
        """uniforms: None (seeded draws) or (u1, u2) for the accept test and the residual draw."""
        if uniforms is not None:
            _check(_lib.lily_sample_spec_f32_uniforms(
                self._h, _ptr(logits, torch.float32), logits.numel(),
                scratch._h if scratch else None, C.byref(params), step, C.byref(dist),
                _ptr(draft, torch.int32), _ptr(out, torch.int32), float(uniforms[0]),
                float(uniforms[1])))
            return
        _check(_lib.lily_sample_spec_f32(self._h, _ptr(logits, torch.float32), logits.numel(),
                                         scratch._h if scratch else None, C.byref(params), step,
                                         C.byref(dist), _ptr(draft, torch.int32),
                                         _ptr(out, torch.int32)))

    def argmax_f32(self, x, out):
        """src/kernels/elementwise.rs:297-308."""
        _check(_lib.lily_argmax_f32(self._h, _ptr(x, torch.float32), x.numel(),
                                    _ptr(out, torch.int32)))

    # -- speculative control, src/kernels/spec.rs:52-127
    def spec_accept(self, draws, ids, ctrl, pos0, ratio, chain):
        if draws.numel() != ids.numel():
            raise SamplerError(-1, "draws and ids must both hold the verified rows")
        _check(_lib.lily_spec_accept(self._h, _ptr(draws, torch.int32), _ptr(ids, torch.int32),
                                     draws.numel(), _ptr(ctrl, torch.int32), ctrl.numel(), pos0,
                                     ratio, chain))

    def copy_row(self, src, row, dst):
        rows = src.shape[0]
        words = src.numel() // rows
        if dst.numel() != words:
            raise SamplerError(-1, f"dst must hold one row ({words} words)")
        _check(_lib.lily_copy_row_u32(self._h, _ptr(src, torch.int32), rows, words,
                                      _ptr(row, torch.int32), _ptr(dst, torch.int32)))

    def spec_verify(self, logits, scratch, params, step0, dists, ids, verify_tokens, ctrl=None,
                    pos0=0, ratio=1, chain=0, uniforms=None):
        """uniforms: None or [m][2] host values (u1, u2) per row replacing the seeded draws."""
        m, vocab = logits.shape
        dtype = BF16 if logits.dtype == torch.bfloat16 else F32
        uarr = None
        if uniforms is not None:
            flat = [float(u) for pair in uniforms for u in pair]
            if len(flat) != 2 * m:
                raise SamplerError(-1, "uniforms must hold (u1, u2) per verify row")
            uarr = (C.c_float * (2 * m))(*flat)
        _check(_lib.lily_spec_verify(
            self._h, _ptr(logits), dtype, vocab, logits.stride(0) if m > 1 else vocab, m,
            scratch._h if scratch else None, C.byref(params), step0,
            dists._h if dists else None, _ptr(ids, torch.int32), _ptr(verify_tokens, torch.int32),
            _ptr(ctrl, torch.int32) if ctrl is not None else None,
            ctrl.numel() if ctrl is not None else 0, pos0, ratio, chain, uarr))

    # -- batched rows, src/qwen4exp/batch.rs:583-593
    def _rows(self, logits, params, steps, out_ids, scratch=None, allow=None, bias=None,
              forced=None, uniforms=None, out_logprobs=None, dbg_ids=None, dbg_probs=None,
              dbg_counts=None):
        """Builds the lily_rows descriptor; returns (descriptor, keepalive)."""
        rows, vocab = logits.shape
        keep = [logits, out_ids]
        r = _Rows()
        r.rows, r.vocab = rows, vocab
        r.dtype = BF16 if logits.dtype == torch.bfloat16 else F32
        if logits.dtype not in (torch.float32, torch.bfloat16) or logits.stride(1) != 1:
            raise SamplerError(-1, "logits must be F32 or BF16 [rows, V], rows contiguous")
        r.logits_dev = logits.data_ptr()
        r.row_stride = logits.stride(0) if rows > 1 else vocab  # a [1, V] view may carry any stride
        parr = (SamplingParams * rows)(*params)
        sarr = (C.c_uint32 * rows)(*[int(s) for s in steps])
        keep += [parr, sarr]
        r.params, r.steps = parr, sarr
        if scratch is not None:
            harr = (C.c_void_p * rows)(*[(s._h if s is not None else None) for s in scratch])
            keep.append(harr)
            r.scratch = harr
        if allow is not None:
            keep.append(allow)
            r.allow_dev = allow.data_ptr()
            r.allow_stride = allow.stride(0) if allow.dim() == 2 else 0
        if bias is not None:
            # bias: list (per row) of [(id, delta), ...]
            flat, offs = [], [0]
            for lst in bias:
                flat += [(int(i), float(d)) for i, d in lst]
                offs.append(len(flat))
            if flat:
                ids = torch.tensor([i for i, _ in flat], dtype=torch.int64)
                dl = torch.tensor([d for _, d in flat], dtype=torch.float32)
                packed = torch.empty(len(flat), 2, dtype=torch.int32)
                packed[:, 0] = ids.to(torch.int32)
                packed[:, 1] = dl.view(torch.int32)
                dev = packed.to(logits.device)
                oarr = (C.c_uint32 * (rows + 1))(*offs)
                keep += [dev, oarr]
                r.bias_dev = dev.data_ptr()
                r.bias_offsets = oarr
        if forced is not None:
            farr = (C.c_uint32 * rows)(*[NO_TOKEN if f is None else int(f) for f in forced])
            keep.append(farr)
            r.forced = farr
        if uniforms is not None:
            uarr = (C.c_float * rows)(*[float("nan") if u is None else float(u) for u in uniforms])
            keep.append(uarr)
            r.uniforms = uarr
        r.out_ids_dev = _ptr(out_ids, torch.int32)
        for name, t, dt in (("out_logprobs_dev", out_logprobs, torch.float32),
                            ("dbg_ids_dev", dbg_ids, torch.int32),
                            ("dbg_probs_dev", dbg_probs, torch.float32),
                            ("dbg_counts_dev", dbg_counts, torch.int32)):
            if t is not None:
                keep.append(t)
                setattr(r, name, _ptr(t, dt))
        return r, keep

    def sample_rows(self, logits, params, steps, out_ids, **kw):
        r, keep = self._rows(logits, params, steps, out_ids, **kw)
        _check(_lib.lily_sample_rows(self._h, C.byref(r)))
        return keep

    def plan(self, logits, params, steps, out_ids, **kw):
        return Plan(self, logits, params, steps, out_ids, **kw)

    # -- the logits' producer and the draws from its summaries,
    #    src/qwen4exp/batch.rs:573-593, src/qwen4exp/model.rs:4157-4169
    @staticmethod
    def _head(hidden, weight, tile_max, tile_sum, logits):
        """weight: a bf16 tensor [V, d] or a QuantWeights; logits: bf16 or f32 [rows, V]."""
        if hidden.dtype != torch.bfloat16 or hidden.dim() != 2 or hidden.stride(1) != 1:
            raise SamplerError(-1, "hidden must be BF16 [rows, d], rows contiguous")
        if logits.dtype not in (torch.bfloat16, torch.float32) or logits.stride(1) != 1:
            raise SamplerError(-1, "logits must be BF16 or F32 [rows, V], rows contiguous")
        h = _LmHead()
        h.hidden_dev, h.hidden_stride = hidden.data_ptr(), hidden.stride(0)
        h.d = hidden.shape[1]
        if isinstance(weight, QuantWeights):
            if weight.codes.dtype != torch.int32 or weight.codes.stride(1) != 1 or weight.in_features != h.d:
                raise SamplerError(-1, "codes must be int32 [V, d * bits / 32], rows contiguous")
            for t in (weight.scales, weight.biases):
                if t.dtype != torch.bfloat16 or not t.is_contiguous() or t.shape != (weight.codes.shape[0], h.d // weight.group_size):
                    raise SamplerError(-1, "scales and biases must be BF16 [V, d / group_size], contiguous")
            h.weight_dev, h.weight_stride = weight.codes.data_ptr(), weight.codes.stride(0)
            h.weight_bits, h.group_size = weight.bits, weight.group_size
            h.scales_dev, h.biases_dev = weight.scales.data_ptr(), weight.biases.data_ptr()
        else:
            if weight.dtype != torch.bfloat16 or weight.dim() != 2 or weight.stride(1) != 1:
                raise SamplerError(-1, "weight must be BF16 [V, d], rows contiguous")
            if hidden.shape[1] != weight.shape[1]:
                raise SamplerError(-1, "hidden and weight differ in d")
            h.weight_dev, h.weight_stride = weight.data_ptr(), weight.stride(0)
        h.logits_f32 = 1 if logits.dtype == torch.float32 else 0
        h.tile_max_dev = _ptr(tile_max, torch.float32)
        h.tile_sum_dev = _ptr(tile_sum, torch.float32)
        return h

    def lm_head_library_calls(self):
        """lily_lm_head_library_calls: producer calls of this sampler that went through the
        platform's GEMM library."""
        return int(_lib.lily_lm_head_library_calls(self._h))

    def lm_head(self, hidden, weight, temperatures, logits, tile_max, tile_sum):
        """lily_lm_head_bf16: logits[rows, V] (bf16 or f32) = hidden @ weight.T with the summaries;
        weight a bf16 tensor or a QuantWeights."""
        rows, vocab = logits.shape
        h = self._head(hidden, weight, tile_max, tile_sum, logits)
        tarr = None if temperatures is None else (C.c_float * rows)(*[float(t) for t in temperatures])
        _check(_lib.lily_lm_head_bf16(self._h, C.byref(h), rows, vocab, tarr, logits.data_ptr(),
                                      logits.stride(0) if rows > 1 else vocab))

    def sample_rows_tiled(self, logits, tile_max, tile_sum, params, steps, out_ids, **kw):
        r, keep = self._rows(logits, params, steps, out_ids, **kw)
        _check(_lib.lily_sample_rows_tiled(self._h, C.byref(r), _ptr(tile_max, torch.float32),
                                           _ptr(tile_sum, torch.float32)))
        return keep

    def lm_head_sample_rows(self, hidden, weight, logits, tile_max, tile_sum, params, steps, out_ids, **kw):
        r, keep = self._rows(logits, params, steps, out_ids, **kw)
        h = self._head(hidden, weight, tile_max, tile_sum, logits)
        _check(_lib.lily_lm_head_sample_rows(self._h, C.byref(h), C.byref(r)))
        return keep


class Plan:
    """A resident batch: packed and uploaded once, one launch per run."""

    def __init__(self, sampler, logits, params, steps, out_ids, **kw):
        self._s = sampler
        h = C.c_void_p()
        _check(_lib.lily_plan_create(sampler._h, logits.shape[0], C.byref(h)))
        self._h = h
        sampler._children.add(self)
        r, self._keep = sampler._rows(logits, params, steps, out_ids, **kw)
        _check(_lib.lily_plan_set(self._h, C.byref(r)))

    def run(self, step_delta=0):
        _check(_lib.lily_plan_run(self._h, step_delta))

    def close(self):
        if self._h:
            # The library object points at its sampler: once that is gone (a garbage collection
            # that finalised the sampler first) the handle is only dropped.
            if self._s._h:
                _lib.lily_plan_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class SamplerScratch:
    """src/kernels/sample.rs:116-179."""

    def __init__(self, sampler, vocab):
        self._s = sampler
        h = C.c_void_p()
        _check(_lib.lily_scratch_create(sampler._h, vocab, C.byref(h)))
        self._h = h
        sampler._children.add(self)

    def close(self):
        if self._h:
            # The library object points at its sampler: once that is gone (a garbage collection
            # that finalised the sampler first) the handle is only dropped.
            if self._s._h:
                _lib.lily_scratch_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def vocab(self):
        return int(_lib.lily_scratch_vocab(self._h))

    def uncount(self, token):
        _check(_lib.lily_scratch_uncount(self._h, token))

    def uncount_after(self, draws, accepted, accepted_cap=0xFFFFFFFF):
        """Un-counts draws[a + 1:], a = min(accepted[0], accepted_cap), read on the device
        (`draws`, `accepted`: int32 device tensors)."""
        _check(_lib.lily_scratch_uncount_after(self._h, draws.data_ptr(), draws.numel(),
                                               accepted.data_ptr(), accepted_cap))

    def reset_counts(self):
        _check(_lib.lily_scratch_reset_counts(self._h))

    def move_counts_to(self, other):
        """move_sampler_counts (src/qwen4exp/batch.rs:138-162): `other` takes these counts."""
        _check(_lib.lily_scratch_move_counts(self._h, other._h))

    def copy_counts_from(self, other):
        _check(_lib.lily_scratch_copy_counts_from(self._h, other._h))

    def add_history(self, ids):
        _check(_lib.lily_scratch_add_history(self._h, _ptr(ids, torch.int32), ids.numel()))

    def write_counts(self, counts):
        """`scratch.counts.write_bytes(...)` of the reference's tests; counts: CPU int32 [V]."""
        c = counts.contiguous()
        if c.is_cuda or c.dtype != torch.int32 or c.numel() != self.vocab():
            raise SamplerError(-1, "counts must be a CPU int32 [V] tensor")
        _check(_lib.lily_scratch_write_counts(self._h, C.c_void_p(c.data_ptr())))

    def read_counts(self):
        out = torch.empty(self.vocab(), dtype=torch.int32)
        _check(_lib.lily_scratch_read_counts(self._h, C.c_void_p(out.data_ptr())))
        return out


class _DeviceWords:
    """Device memory owned by the library, as something torch can wrap without copying."""

    def __init__(self, ptr, n):
        self.__cuda_array_interface__ = {"shape": (n,), "typestr": "<i4", "data": (int(ptr), False),
                                         "version": 2}


def _device_view(ptr, n, device):
    return torch.as_tensor(_DeviceWords(ptr, n), device=torch.device("cuda", device))


class TokenSlots:
    """The decode loop's ping-pong output slots with polled completion (src/generate.rs:776-891):
    `slots` device arrays of `words` int32 each, a pinned host mirror, an event per slot."""

    def __init__(self, sampler, slots=2, words=1):
        self._s = sampler
        self.slots, self.words = slots, words
        h = C.c_void_p()
        _check(_lib.lily_token_slots_create(sampler._h, slots, words, C.byref(h)))
        self._h = h
        sampler._children.add(self)
        self._views = []
        for i in range(slots):
            ptr = _lib.lily_token_slots_device(self._h, i)
            self._views.append(_device_view(ptr, words, sampler.device))

    def device(self, i):
        """Slot i as an int32 device tensor over the library's memory (valid until close())."""
        return self._views[i]

    def publish(self, i):
        _check(_lib.lily_token_slots_publish(self._h, i))

    def poll(self, i):
        """None while the slot's step is still running, else its words as a list."""
        out = (C.c_uint32 * self.words)()
        ready = C.c_int(0)
        _check(_lib.lily_token_slots_poll(self._h, i, out, C.byref(ready)))
        return list(out) if ready.value else None

    def wait_polled(self, i, max_polls=0):
        out = (C.c_uint32 * self.words)()
        _check(_lib.lily_token_slots_wait_polled(self._h, i, out, max_polls))
        return list(out)

    def close(self):
        if self._h:
            self._views = []
            if self._s._h:
                _lib.lily_token_slots_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


INSERT_AFTER, INSERT_BEFORE, INSERT_REPLACE = 0, 1, 2


class Insertions:
    """lily_insertions_*: the thinking control's Action::{After, Before, Replace}
    (src/thinking.rs:485-608) as the forced tokens of the steps that follow."""

    def __init__(self, rows):
        self._h = C.c_void_p()
        self.rows = rows
        _check(_lib.lily_insertions_create(rows, C.byref(self._h)))

    def push(self, row, kind, drawn, ids, scratch=None):
        arr = (C.c_uint32 * max(1, len(ids)))(*[int(i) for i in ids])
        _check(_lib.lily_insertions_push(self._h, row, kind, int(drawn), arr, len(ids),
                                         scratch._h if scratch is not None else None))

    def next(self):
        """(forced list for lily_rows: None = the row draws, number of forced rows)."""
        out = (C.c_uint32 * self.rows)()
        n = _lib.lily_insertions_next(self._h, out)
        return [None if v == NO_TOKEN else int(v) for v in out], int(n)

    def pending(self, row):
        return int(_lib.lily_insertions_pending(self._h, row))

    def clear(self, row):
        _lib.lily_insertions_clear(self._h, row)

    def close(self):
        if self._h:
            _lib.lily_insertions_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class DraftDists:
    """src/kernels/sample.rs:186-215."""

    def __init__(self, sampler, slots):
        self._s = sampler
        h = C.c_void_p()
        _check(_lib.lily_draft_dists_create(sampler._h, slots, C.byref(h)))
        self._h = h
        sampler._children.add(self)

    def close(self):
        if self._h:
            # The library object points at its sampler: once that is gone (a garbage collection
            # that finalised the sampler first) the handle is only dropped.
            if self._s._h:
                _lib.lily_draft_dists_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def slot(self, i):
        d = DraftDist()
        _check(_lib.lily_draft_dists_slot(self._h, i, C.byref(d)))
        return d

    def write(self, i, ids, probs):
        """Overwrites slot i with a hand-made distribution (numpy uint32 ids, float32 probs);
        synchronises.  For tests of cases no real draft head produces."""
        d = self.slot(i)
        self._s.synchronize()
        k = len(ids)
        if k > SAMPLE_K_CAP or len(probs) != k:
            raise SamplerError(-6, "a slot holds at most 1024 (id, prob) pairs")
        t_ids = torch.tensor([int(x) for x in ids], dtype=torch.int64).to(torch.int32)
        t_pr = torch.tensor([float(x) for x in probs], dtype=torch.float32)
        t_n = torch.tensor([k], dtype=torch.int32)
        if k:
            _hip_copy_to_device(d.ids_dev, t_ids, 4 * k)
            _hip_copy_to_device(d.probs_dev, t_pr, 4 * k)
        _hip_copy_to_device(d.count_dev, t_n, 4)

    def read(self, i):
        """(ids, probs) of slot i on the host; synchronises."""
        d = self.slot(i)
        self._s.synchronize()
        n = torch.empty(1, dtype=torch.int32)
        _hip_copy(n, d.count_dev, 4)
        k = int(n[0])
        ids = torch.empty(k, dtype=torch.int32)
        probs = torch.empty(k, dtype=torch.float32)
        if k:
            _hip_copy(ids, d.ids_dev, 4 * k)
            _hip_copy(probs, d.probs_dev, 4 * k)
        return ids, probs


_hip = None


def _hip_memcpy(dst, src, nbytes, kind):
    global _hip
    if _hip is None:
        _hip = C.CDLL("libamdhip64.so.7")  # the SONAME torch already loaded
        _hip.hipMemcpy.restype = C.c_int
        _hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    rc = _hip.hipMemcpy(C.c_void_p(dst), C.c_void_p(src), nbytes, kind)
    if rc != 0:
        raise SamplerError(-4, f"hipMemcpy failed with {rc}")


def _hip_copy(dst_cpu, src_dev, nbytes):
    """Device -> host copy of raw library-owned memory (tests read the draft export)."""
    _hip_memcpy(dst_cpu.data_ptr(), src_dev, nbytes, 2)


def _hip_copy_to_device(dst_dev, src_cpu, nbytes):
    """Host -> device copy into raw library-owned memory (tests write a draft export)."""
    _hip_memcpy(dst_dev, src_cpu.data_ptr(), nbytes, 1)
