"""Builds liblily_sampler_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python lily-qwen3.8-flash-next_amd/build.py
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "liblily_sampler_hip.so")
SOURCES = ["sampler_kernels.hip", "sampler_api.cpp"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # Token ids depend on exact f32 arithmetic: no contraction into FMAs, IEEE division
    # (hipcc's default), denormals kept (hipcc's default).
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", LIB]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if verbose or res.returncode != 0:
        sys.stderr.write(err + "\n")
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
