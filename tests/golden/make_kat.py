"""Writes tests/golden/kat.json: the literal known answers the parity tests pin the
oracle (and, on the GPU, the HIP path) against.

Nothing here runs or imports the reference.  Each entry is a literal taken from a
test function of the reference (cited per entry, paths relative to the reference
checkout) or a published vector of a textbook routine.  Run from the repo root:
    python tests/golden/make_kat.py
"""
import json
import os

kat = {
    # SplitMix64 (Steele, Lea, Flood 2014; Vigna's splitmix64.c): the first outputs
    # for seed 0 and seed 1234567.  uniform_for(seed, j) is the top 24 bits of the
    # j-th output (src/kernels/sample.rs:435-441 adds step * golden to the seed).
    "splitmix64": {
        "0": ["0xe220a8397b1dcdaf", "0x6e789e6aa1b965f4", "0x06c45d188009454f",
              "0xf88bb8a8724c81ec"],
        "1234567": ["6457827717110365317", "3203168211198807973", "9817491932198370423"],
    },
    # tests/unit/kernels/sample.rs:74-83
    "greedy_ties": {"v": 5000, "set": {"1234": 7.5, "4321": 7.5}, "expect": 1234},
    # tests/unit/kernels/elementwise.rs:57-64 (values elsewhere below 8.0)
    "argmax_ties": {"v": 4097, "set": {"513": 9.5, "3501": 9.5}, "expect": 513},
    # tests/unit/kernels/sample.rs:142-172
    "penalties": {
        "v": 3000, "set": {"10": 5.0, "20": 4.0}, "counts": {"10": 3},
        "presence": 0.5, "frequency": 0.5, "repetition": 1.5,
        "expect_id": 20, "adjusted_10": 5.0 / 1.5 - 0.5 - 1.5, "adjusted_10_tol": 1e-5,
        "adjusted_20": 4.0, "counts_after": {"20": 1, "10": 3},
    },
    # tests/unit/kernels/sample.rs:177-197
    "counts_move": {"v": 3000, "counts": {"7": 2, "2999": 5}, "stale": 9},
    # tests/unit/kernels/spec.rs:17-42
    "spec_accept": {
        "pos0": 13, "ratio": 4, "chain": 3, "stride": 4,
        "cases": [
            {"draws": [5, 6, 7, 8], "ids": [1, 5, 6, 7], "a": 3},
            {"draws": [5, 6, 9, 8], "ids": [1, 5, 6, 7], "a": 2},
            {"draws": [5, 0, 7, 8], "ids": [1, 5, 6, 7], "a": 1},
            {"draws": [4, 6, 7, 8], "ids": [1, 5, 6, 7], "a": 0},
            {"draws": [5], "ids": [1], "a": 0},
        ],
    },
    # src/kernels/sample.rs:47-95: (params) -> (is_greedy, uses_penalties, effective T, k)
    "effective": [
        {"temperature": 0.0, "top_k": 1, "greedy": True, "T": 1.0, "k": 1},
        {"temperature": 0.0, "top_k": 40, "greedy": True, "T": 1.0, "k": 1},
        {"temperature": 0.8, "top_k": 1, "greedy": True, "T": 1.0, "k": 1},
        {"temperature": 0.8, "top_k": 0, "greedy": False, "T": 0.8, "k": 1024},
        {"temperature": 0.8, "top_k": 40, "greedy": False, "T": 0.8, "k": 40},
        {"temperature": 1.3, "top_k": 5000, "greedy": False, "T": 1.3, "k": 1024},
    ],
    # src/kernels/sample.rs:57-79: field overrides on greedy() -> failing rule (0 = valid)
    "validate": [
        [{}, 0],
        [{"temperature": -0.1}, 1], [{"temperature": "inf"}, 1], [{"temperature": "nan"}, 1],
        [{"top_p": 0.0}, 2], [{"top_p": 1.5}, 2], [{"top_p": 1.0}, 0], [{"top_p": "nan"}, 2],
        [{"min_p": -0.1}, 3], [{"min_p": 1.1}, 3], [{"min_p": 1.0}, 0],
        [{"repetition_penalty": 0.0}, 4], [{"repetition_penalty": "inf"}, 4],
        [{"presence_penalty": "inf"}, 5], [{"frequency_penalty": "nan"}, 5],
        [{"presence_penalty": -2.0, "frequency_penalty": 2.0}, 0],
    ],
}

out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kat.json")
with open(out, "w") as f:
    json.dump(kat, f, indent=1)
print("wrote", out)
