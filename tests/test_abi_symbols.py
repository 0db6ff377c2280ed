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
