"""INTEGRATION.md's Rust `extern "C"` block declares every function of include/lily_sampler.h, and
every LILY_* constant its examples use is declared in it."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_functions():
    text = open(os.path.join(ROOT, "include", "lily_sampler.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(lily_[a-z0-9_]+)\s*\(", text))


def _rust_blocks():
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    return re.findall(r"```rust\n(.*?)```", text, flags=re.S)


def test_every_function_of_the_header_is_declared_in_the_rust_block():
    declared = set()
    for block in _rust_blocks():
        declared |= set(re.findall(r"pub fn (lily_[a-z0-9_]+)\s*\(", block))
    missing = sorted(_header_functions() - declared)
    assert not missing, missing
    unknown = sorted(declared - _header_functions())
    assert not unknown, unknown


def test_constants_used_in_the_rust_examples_are_declared():
    blocks = _rust_blocks()
    declared = set()
    for block in blocks:
        declared |= set(re.findall(r"pub const (LILY_[A-Z0-9_]+)\s*:", block))
    used = set()
    for block in blocks:
        used |= set(re.findall(r"\b(LILY_[A-Z0-9_]+)\b", block))
    header = open(os.path.join(ROOT, "include", "lily_sampler.h")).read()
    missing = sorted(used - declared)
    assert not missing, missing
    for name in declared:
        assert re.search(r"\b" + name + r"\b", header), name
