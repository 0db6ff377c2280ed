"""The streaming scan keeps its block requests in flight only while hipcc's waits allow it.

hipcc places one `s_waitcnt vmcnt(N)` before each use of a loaded register, N being the
fewest loads any path can have issued after the awaited one.  A load that may be skipped on
some path to the use (a bounds check around it, a request behind `if (b + 2 < nblocks)`)
makes N zero, every block's wait then drains the wave's loads and the 1024-row launch runs
8 % slower with identical results - nothing else would notice.  This compiles the one kernel
of that launch to assembly (`-DLILY_ONE_VARIANT`, seconds) and checks the waits of its scan
loop: most of them must leave at least a block's four loads in flight.
"""
import collections
import os
import re
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "lily-qwen3.8-flash-next_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
KERNEL = "_ZN4lily12k_rows_tableILi1ELi2ELb1EEEvNS_9LaunchCfgE"  # <bf16, streaming, row sum>


@pytest.mark.skipif(shutil.which(HIPCC) is None, reason="hipcc not found")
def test_scan_loop_waits_leave_requests_in_flight():
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k.s")
        cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only",
               "-DLILY_ONE_VARIANT", "-I", os.path.join(ROOT, "include"), "-S",
               os.path.join(CSRC, "sampler_kernels.hip"), "-o", out]
        res = subprocess.run(cmd, capture_output=True, text=True)
        assert res.returncode == 0, res.stderr[-2000:]
        lines = open(out).read().split("\n")
    start = next(i for i, l in enumerate(lines) if l.startswith(KERNEL + ":"))
    end = next(i for i, l in enumerate(lines) if l.startswith("\t.size\t" + KERNEL))
    body = lines[start:end]
    heads = [i for i, l in enumerate(body) if "=>This" in l and "Loop Header: Depth=1" in l]
    heads.append(len(body))
    # the scan loop is by far the largest outermost loop of the kernel
    lo, hi = max(zip(heads, heads[1:]), key=lambda p: p[1] - p[0])
    loop = "\n".join(body[lo:hi])
    assert loop.count("global_load_dwordx4") >= 12, "not the scan loop"
    waits = collections.Counter(int(n) for n in re.findall(r"s_waitcnt vmcnt\((\d+)\)", loop))
    ahead = sum(c for n, c in waits.items() if n >= 4)
    drained = sum(c for n, c in waits.items() if n < 4)
    # three blocks per trip, four chunks each, several uses per chunk; the drains that remain
    # sit in rarely taken branches (a saturated count's reload, buckets beyond 256 ids)
    assert ahead >= 60 and drained <= 20, dict(waits)
