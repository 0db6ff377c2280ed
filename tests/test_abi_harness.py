"""The public header as another host sees it: it compiles as C and as C++ on its own, and a C++
program written against it alone (tests/abi_harness/harness.cpp, built with the library) gets the
oracle's draws through lily_sample_f32, lily_sample_rows and a plan."""
import os
import shutil
import subprocess

import numpy as np
import pytest

import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lily_sampler.h")
HARNESS = os.path.join(ROOT, "tests", "abi_harness", "harness.bin")


def _need_harness():
    if not os.path.exists(HARNESS):
        pytest.fail(f"{HARNESS} is missing: python lily-qwen3.8-flash-next_amd/build.py builds it")


@pytest.mark.parametrize("cc,lang,std", [("gcc", "c", "-std=c99"), ("g++", "c++", "-std=c++11")])
def test_header_compiles_on_its_own(cc, lang, std):
    if shutil.which(cc) is None:
        pytest.skip(f"{cc} not found")
    res = subprocess.run([cc, std, "-pedantic", "-Wall", "-Werror", "-fsyntax-only", "-x", lang, HEADER],
                         capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


def test_host_helpers_from_cpp_without_a_gpu():
    _need_harness()
    res = subprocess.run([HARNESS, "cpu"], capture_output=True, text=True, timeout=60)
    assert res.returncode == 0, res.stderr
    words = res.stdout.split()
    assert words[:2] == ["cpu", "ok"], res.stdout
    assert np.float32(float(words[3])) == np.float32(O.uniform_for(1234, 7))
    assert int(words[5]) == (5 | 0x40000000)
    # the structs as a C++ compiler lays them out against the ctypes mirror's
    import ctypes

    import lily_sampler as LS
    sizes = [int(w) for w in words[words.index("sizes") + 1:]]
    assert sizes == [ctypes.sizeof(LS.SamplingParams), ctypes.sizeof(LS._Rows), ctypes.sizeof(LS._LmHead),
                     ctypes.sizeof(LS.DraftDist)], sizes


def _logits(vocab, seed):
    """harness.cpp's logit_of, in wrapping 32-bit arithmetic."""
    i = np.arange(vocab, dtype=np.uint64)
    h = ((i + 1) * 2654435761 + seed * 40503) & 0xFFFFFFFF
    h ^= h >> 15
    h = (h * 2246822519) & 0xFFFFFFFF
    h ^= h >> 13
    return ((h >> 8).astype(np.float32) * np.float32(16.0 / 16777216.0) - np.float32(8.0)).astype(np.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("vocab,seed", [(50_021, 3), (151_936, 11)])
def test_draws_from_cpp_match_the_oracle(vocab, seed):
    _need_harness()
    res = subprocess.run([HARNESS, "gpu", str(vocab), str(seed)], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr + res.stdout
    line = [l for l in res.stdout.splitlines() if l.startswith("ids ")][0]
    got = [int(w) for w in line.split()[1:]]
    x = [_logits(vocab, seed), _logits(vocab, seed + 1)]
    hist = (np.arange(512, dtype=np.uint64) * 7919 + seed) % vocab
    counts = [np.bincount(hist.astype(np.int64), minlength=vocab).astype(np.uint32) for _ in range(2)]
    kw = dict(temperature=0.9, top_k=50, top_p=0.95, repetition_penalty=1.2, presence_penalty=0.1,
              frequency_penalty=0.05)
    p = [O.params(seed=77, **kw), O.params(seed=78, **kw)]
    want = []
    for step in (0, 1):                        # lily_sample_f32, row 0
        d = O.sample(x[0], counts[0], p[0], step)
        counts[0][d.chosen] += 1
        want.append(int(d.chosen))
    for step in (2, 3):                        # lily_sample_rows, then the plan with step_delta 1
        for r in range(2):
            d = O.sample(x[r], counts[r], p[r], step)
            counts[r][d.chosen] += 1
            want.append(int(d.chosen))
    assert got == want


@pytest.mark.gpu
def test_a_batch_of_the_producer_from_cpp_by_either_way():
    """A program that has loaded no copy of the platform's GEMM library: the producer opens the
    system's by its name for a batch of 300 rows, and what it stores equals what this library's
    own kernel stores to one bf16 step (the order of the f32 additions differs), the summaries
    likewise (a tile's largest value is one of those values; its sum moves with them: at T 0.8 a
    bf16 step of a value near 4 moves its term by 4 %)."""
    _need_harness()
    res = subprocess.run([HARNESS, "head", "300", "512", "5000"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr + res.stdout
    words = [l for l in res.stdout.splitlines() if l.startswith("head ")][0].split()
    got = dict(zip(words[1::2], words[2::2]))
    assert int(got["library_calls"]) == 1, res.stdout
    assert float(got["maxdiff"]) <= 2.0 ** -7
    assert float(got["maxdiff_max"]) <= 2.0 ** -7
    assert float(got["maxdiff_sum"]) <= 0.1
