"""ctypes loader of the CPU checker (oracle/sampler_oracle.cpp).

Test infrastructure only: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liblily_oracle.so")

F32, BF16 = 0, 1
EXP_LILY, EXP_LIBM = 0, 1
SORT_PARTIAL, SORT_FULL = 0, 1
K_CAP = 1024


class Params(C.Structure):
    """Field for field src/kernels/sample.rs:21-31 (top_k as u32)."""

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


def greedy():
    """SamplingParams::greedy(), src/kernels/sample.rs:34-45."""
    return Params(0.0, 1, 1.0, 0.0, 0.0, 0.0, 1.0, 0, 0)


def params(**kw):
    p = greedy()
    for k, v in kw.items():
        setattr(p, k, v)
    return p


class Bias(C.Structure):
    _fields_ = [("id", C.c_uint32), ("delta", C.c_float)]


class Ext(C.Structure):
    _fields_ = [
        ("allow", C.c_void_p),
        ("bias", C.c_void_p),
        ("n_bias", C.c_uint32),
        ("has_uniform", C.c_uint32),
        ("uniform", C.c_float),
        ("has_forced", C.c_uint32),
        ("forced", C.c_uint32),
        ("exp_mode", C.c_uint32),
        ("sort_mode", C.c_uint32),
        ("want_logprob", C.c_uint32),
    ]


class Result(C.Structure):
    _fields_ = [
        ("chosen", C.c_uint32),
        ("n_cand", C.c_uint32),
        ("n_kept", C.c_uint32),
        ("top", C.c_float),
        ("total", C.c_float),
        ("mass", C.c_float),
        ("target", C.c_float),
        ("uniform", C.c_float),
        ("gap", C.c_float),
        ("reserved", C.c_uint32),
        ("logprob", C.c_double),
    ]


def build():
    subprocess.run(["make", "-C", HERE, "-s"], check=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        L.lo_uniform_for.restype = C.c_float
        L.lo_uniform_for.argtypes = [C.c_uint64, C.c_uint32]
        L.lo_expf.restype = C.c_float
        L.lo_expf.argtypes = [C.c_float]
        L.lo_draft_step.restype = C.c_uint32
        L.lo_draft_step.argtypes = [C.c_uint32]
        for name in ("lo_is_greedy", "lo_uses_penalties", "lo_samples", "lo_validate"):
            getattr(L, name).restype = C.c_int
            getattr(L, name).argtypes = [C.POINTER(Params)]
        L.lo_effective.argtypes = [C.POINTER(Params), C.POINTER(C.c_float), C.POINTER(C.c_uint32)]
        L.lo_draft_params.argtypes = [C.POINTER(Params), C.POINTER(Params)]
        L.lo_argmax.restype = C.c_uint32
        L.lo_argmax.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        L.lo_adjust.argtypes = [C.c_void_p, C.c_int, C.c_size_t, C.c_void_p, C.POINTER(Params),
                                C.POINTER(Ext), C.c_void_p]
        L.lo_sample.restype = C.c_int
        L.lo_sample.argtypes = [C.c_void_p, C.c_int, C.c_size_t, C.c_void_p, C.POINTER(Params),
                                C.c_uint32, C.POINTER(Ext), C.POINTER(Result), C.c_void_p,
                                C.c_void_p, C.c_void_p, C.c_void_p]
        L.lo_kept.restype = C.c_uint32
        L.lo_kept.argtypes = [C.c_void_p, C.c_int, C.c_size_t, C.POINTER(Params), C.c_uint32,
                              C.c_void_p, C.c_void_p]
        L.lo_spec.restype = C.c_uint32
        L.lo_spec.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p, C.c_void_p,
                              C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint32, C.c_uint32,
                              C.c_float, C.c_float, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32),
                              C.POINTER(C.c_float)]
        L.lo_spec_accept.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32,
                                     C.c_uint32, C.c_uint32, C.c_void_p]
        L.lo_host_accept.restype = C.c_uint32
        L.lo_host_accept.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32]
        L.lo_uncount.argtypes = [C.c_void_p, C.c_size_t, C.c_uint32]
        L.lo_sample_rows.restype = C.c_int
        L.lo_sample_rows.argtypes = [C.c_void_p, C.c_int, C.c_size_t, C.c_size_t, C.c_uint32,
                                     C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32,
                                     C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _dtype_of(logits):
    if logits.dtype == np.float32:
        return F32
    if logits.dtype == np.uint16:
        return BF16
    raise TypeError("logits must be float32 or uint16 (bf16 bits)")


def uniform_for(seed, step):
    return float(lib().lo_uniform_for(seed, step))


def expf(x):
    return float(lib().lo_expf(C.c_float(x)))


def effective(p):
    t, k = C.c_float(), C.c_uint32()
    lib().lo_effective(C.byref(p), C.byref(t), C.byref(k))
    return t.value, k.value


def draft_params(p):
    out = Params()
    lib().lo_draft_params(C.byref(p), C.byref(out))
    return out


def argmax(x):
    x = np.ascontiguousarray(x)
    return int(lib().lo_argmax(_ptr(x), _dtype_of(x), x.size))


def make_ext(allow=None, bias=None, uniform=None, forced=None, exp_mode=EXP_LILY,
             sort_mode=SORT_PARTIAL, want_logprob=False):
    """Returns (Ext, keepalive) - keepalive holds the arrays Ext points into."""
    e = Ext()
    keep = []
    if allow is not None:
        allow = np.ascontiguousarray(allow, dtype=np.uint32)
        keep.append(allow)
        e.allow = allow.ctypes.data
    if bias is not None and len(bias):
        arr = (Bias * len(bias))(*[Bias(int(i), float(d)) for i, d in bias])
        keep.append(arr)
        e.bias = C.cast(arr, C.c_void_p)
        e.n_bias = len(bias)
    if uniform is not None:
        e.has_uniform, e.uniform = 1, float(uniform)
    if forced is not None:
        e.has_forced, e.forced = 1, int(forced)
    e.exp_mode, e.sort_mode, e.want_logprob = exp_mode, sort_mode, int(want_logprob)
    return e, keep


def adjust(logits, counts, p, **ext_kw):
    logits = np.ascontiguousarray(logits)
    e, keep = make_ext(**ext_kw)
    out = np.empty(logits.size, dtype=np.float32)
    lib().lo_adjust(_ptr(logits), _dtype_of(logits), logits.size, _ptr(counts), C.byref(p),
                    C.byref(e), _ptr(out))
    return out


class Draw:
    """One cpu_sample result with everything a parity test compares."""

    def __init__(self, res, cand_ids, cand_adj, cand_prob, cum):
        self.chosen = res.chosen
        self.n_cand = res.n_cand
        self.n_kept = res.n_kept
        self.top, self.total, self.mass = res.top, res.total, res.mass
        self.target, self.uniform, self.gap = res.target, res.uniform, res.gap
        self.logprob = res.logprob
        self.cand_ids = cand_ids[: res.n_cand].copy()
        self.cand_adj = cand_adj[: res.n_cand].copy()
        self.cand_prob = cand_prob[: res.n_cand].copy()
        self.kept_ids = cand_ids[: res.n_kept].copy()
        self.kept_cum = cum[: res.n_kept].copy()
        # Probabilities normalised over the kept mass (what a draft exports).
        self.kept_q = (cand_prob[: res.n_kept] / np.float32(res.mass)).astype(np.float32)


def sample(logits, counts, p, step, **ext_kw):
    """cpu_sample; `counts` (uint32 [V] or None) is bumped in place under penalties."""
    logits = np.ascontiguousarray(logits)
    e, keep = make_ext(**ext_kw)
    res = Result()
    ids = np.zeros(K_CAP, dtype=np.uint32)
    adj = np.zeros(K_CAP, dtype=np.float32)
    prob = np.zeros(K_CAP, dtype=np.float32)
    cum = np.zeros(K_CAP, dtype=np.float32)
    rc = lib().lo_sample(_ptr(logits), _dtype_of(logits), logits.size, _ptr(counts), C.byref(p),
                         step, C.byref(e), C.byref(res), _ptr(ids), _ptr(adj), _ptr(prob),
                         _ptr(cum))
    if rc != 0:
        raise ValueError("oracle lo_sample failed")
    return Draw(res, ids, adj, prob, cum)


def kept(logits, p, exp_mode=EXP_LILY):
    """cpu_kept: [(id, q)] normalised over the kept mass."""
    logits = np.ascontiguousarray(logits)
    ids = np.zeros(K_CAP, dtype=np.uint32)
    probs = np.zeros(K_CAP, dtype=np.float32)
    n = lib().lo_kept(_ptr(logits), _dtype_of(logits), logits.size, C.byref(p), exp_mode,
                      _ptr(ids), _ptr(probs))
    return ids[:n].copy(), probs[:n].copy()


def spec(p_ids, p_probs, q_ids, q_probs, d, seed, step, u1=None, u2=None):
    """cpu_spec -> (token, accepted, zero_residual, gap)."""
    p_ids = np.ascontiguousarray(p_ids, dtype=np.uint32)
    p_probs = np.ascontiguousarray(p_probs, dtype=np.float32)
    q_ids = np.ascontiguousarray(q_ids, dtype=np.uint32)
    q_probs = np.ascontiguousarray(q_probs, dtype=np.float32)
    acc, zr, gap = C.c_uint32(), C.c_uint32(), C.c_float()
    has_u = 0 if u1 is None else 1
    tok = lib().lo_spec(_ptr(p_ids), _ptr(p_probs), p_ids.size, _ptr(q_ids), _ptr(q_probs),
                        q_ids.size, d, seed, step, has_u, float(u1 or 0.0), float(u2 or 0.0),
                        C.byref(acc), C.byref(zr), C.byref(gap))
    return int(tok), bool(acc.value), bool(zr.value), gap.value


def spec_accept(draws, ids, pos0, ratio, chain, stride=4):
    draws = np.ascontiguousarray(draws, dtype=np.uint32)
    ids = np.ascontiguousarray(ids, dtype=np.uint32)
    ctrl = np.zeros((2 + 3 * chain) * stride, dtype=np.uint32)
    lib().lo_spec_accept(_ptr(draws), _ptr(ids), draws.size, pos0, ratio, chain, stride,
                         _ptr(ctrl))
    return ctrl


def sample_rows(logits2d, counts2d, params_list, steps, exts=None, threads=1,
                want_logprob=False):
    """Independent rows on `threads` host threads -> (ids, logprobs)."""
    logits2d = np.ascontiguousarray(logits2d)
    rows, v = logits2d.shape
    parr = (Params * rows)(*params_list)
    steps = np.ascontiguousarray(steps, dtype=np.uint32)
    keep = []
    if exts is None:
        e, k = make_ext(want_logprob=want_logprob)
        exts = [e] * rows
    earr = (Ext * rows)(*exts)
    ids = np.zeros(rows, dtype=np.uint32)
    lps = np.zeros(rows, dtype=np.float64)
    lib().lo_sample_rows(_ptr(logits2d), _dtype_of(logits2d), v, v, rows, _ptr(counts2d),
                         C.cast(parr, C.c_void_p), _ptr(steps), C.cast(earr, C.c_void_p),
                         threads, _ptr(ids), _ptr(lps))
    del keep
    return ids, lps
