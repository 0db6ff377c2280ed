"""The C-ABI library exists in-tree, loads, and exports every symbol include/lily_sampler.h
declares.  No compute calls (no GPU needed)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "lily-qwen3.8-flash-next_amd", "liblily_sampler_hip.so")
HEADER = os.path.join(ROOT, "include", "lily_sampler.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lily_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_reference_surface():
    names = declared_symbols()
    for need in ("lily_sample_f32", "lily_sample_draft_f32", "lily_sample_spec_f32",
                 "lily_argmax_f32", "lily_spec_accept", "lily_copy_row_u32", "lily_uniform_for",
                 "lily_draft_step", "lily_draft_params", "lily_scratch_uncount",
                 "lily_scratch_reset_counts", "lily_scratch_copy_counts_from",
                 "lily_draft_dists_slot", "lily_sample_rows", "lily_spec_verify"):
        assert need in names


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB), "build with: python lily-qwen3.8-flash-next_amd/build.py"
    lib = ctypes.CDLL(LIB)
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing


def test_pure_host_helpers_need_no_gpu():
    lib = ctypes.CDLL(LIB)
    lib.lily_uniform_for.restype = ctypes.c_float
    lib.lily_uniform_for.argtypes = [ctypes.c_uint64, ctypes.c_uint32]
    assert lib.lily_uniform_for(0, 1) == 0xE220A8 / 16777216.0
    lib.lily_ctrl_words.restype = ctypes.c_uint32
    assert lib.lily_ctrl_words(3) == (2 + 9) * 4
    lib.lily_draft_step.restype = ctypes.c_uint32
    assert lib.lily_draft_step(5) == 5 | 0x40000000


class _Params(ctypes.Structure):
    _fields_ = [("temperature", ctypes.c_float), ("top_k", ctypes.c_uint32), ("top_p", ctypes.c_float),
                ("min_p", ctypes.c_float), ("presence_penalty", ctypes.c_float),
                ("frequency_penalty", ctypes.c_float), ("repetition_penalty", ctypes.c_float),
                ("reserved", ctypes.c_uint32), ("seed", ctypes.c_uint64)]


class _Fields(ctypes.Structure):
    _fields_ = [("has", ctypes.c_uint32), ("temperature", ctypes.c_float), ("top_p", ctypes.c_float),
                ("min_p", ctypes.c_float), ("top_k", ctypes.c_int64), ("seed", ctypes.c_int64),
                ("presence_penalty", ctypes.c_float), ("frequency_penalty", ctypes.c_float),
                ("repetition_penalty", ctypes.c_float), ("reserved", ctypes.c_uint32)]


HAS = dict(temperature=1, top_p=2, top_k=4, min_p=8, seed=16, presence_penalty=32,
           frequency_penalty=64, repetition_penalty=128)


def test_request_fields_resolve_over_the_defaults():
    """resolve_sampling (src/serve/api.rs:798-834): fields over defaults, negative top_k = off,
    a missing seed replaced by fresh entropy, the result validated."""
    lib = ctypes.CDLL(LIB)
    lib.lily_params_resolve.restype = ctypes.c_int
    lib.lily_params_resolve.argtypes = [ctypes.POINTER(_Fields), ctypes.POINTER(_Params), ctypes.c_uint64,
                                        ctypes.POINTER(_Params)]
    lib.lily_last_error.restype = ctypes.c_char_p
    defaults = _Params(0.6, 20, 0.95, 0.0, 0.0, 0.0, 1.05, 0, 99)

    def resolve(fresh=4242, **given):
        f = _Fields()
        for k, v in given.items():
            f.has |= HAS[k]
            setattr(f, k, v)
        out = _Params()
        rc = lib.lily_params_resolve(ctypes.byref(f), ctypes.byref(defaults), fresh, ctypes.byref(out))
        return rc, out

    rc, p = resolve()
    assert rc == 0
    assert (p.temperature, p.top_k, p.top_p, p.repetition_penalty) == (defaults.temperature, 20,
                                                                      defaults.top_p, defaults.repetition_penalty)
    assert p.seed == 4242                      # no seed in the request: the fresh one, not the defaults'
    rc, p = resolve(temperature=0.0, top_k=-1, seed=-1, presence_penalty=1.5, min_p=0.1)
    assert rc == 0
    assert p.temperature == 0.0 and p.top_k == 0 and p.seed == 0xFFFFFFFFFFFFFFFF
    assert p.presence_penalty == 1.5 and abs(p.min_p - 0.1) < 1e-7 and p.top_p == defaults.top_p
    rc, p = resolve(top_k=5_000_000_000)
    assert rc == 0 and p.top_k == 0xFFFFFFFF   # beyond u32: still "more than the cap"
    for bad in (dict(top_p=0.0), dict(top_p=1.5), dict(min_p=-0.1), dict(temperature=-1.0),
                dict(repetition_penalty=0.0), dict(frequency_penalty=float("inf"))):
        rc, p = resolve(**bad)
        assert rc == -2 and lib.lily_last_error(), bad     # LILY_ERR_PARAMS with the rule's text
