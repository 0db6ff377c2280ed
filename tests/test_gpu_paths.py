"""Every selection path of the HIP kernels against the oracle on awkward inputs.

The library picks its path itself (single-pass select for k <= 64, two-pass above,
exhaustive select when a slice overflows or the slack check fails).  LILY_SAMPLER_PATH
(1 = exhaustive only, 2 = two-pass only) and LILY_SAMPLER_SLICES (workgroups per row)
are read when a sampler is created; the tests use them to drive each path over rows
with heavy ties, unaligned row starts, masks with few allowed ids, ascending order
(the worst case of a running threshold), constant rows and -inf entries.
"""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import lily_sampler as LS
import lily_workloads as W
import oracle as O
from gpu_util import check_row_against_oracle, dev, o_params, run_rows


def make_sampler(path, slices):
    old = {k: os.environ.get(k) for k in ("LILY_SAMPLER_PATH", "LILY_SAMPLER_SLICES")}
    os.environ["LILY_SAMPLER_PATH"] = str(path)
    os.environ["LILY_SAMPLER_SLICES"] = str(slices)
    try:
        return LS.Sampler(0)
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


@pytest.fixture(scope="module", params=[(0, 0), (0, 1), (0, 3), (0, 64), (1, 0), (2, 1), (2, 5)],
                ids=lambda p: f"path{p[0]}-slices{p[1]}")
def sampler(request):
    s = make_sampler(*request.param)
    yield s
    s.close()


def _rows_of_kinds(rng, rows, vocab, bf16):
    x = np.empty((rows, vocab), np.float32)
    for r in range(rows):
        kind = r % 8
        if kind == 0:
            x[r] = rng.normal(0, 3, vocab)
        elif kind == 1:
            x[r] = rng.integers(-12, 13, vocab) / 4.0          # heavy ties
        elif kind == 2:
            x[r] = np.sort(rng.normal(0, 2, vocab))             # ascending: worst case
        elif kind == 3:
            x[r] = np.sort(rng.normal(0, 2, vocab))[::-1]       # descending
        elif kind == 4:
            x[r] = 1.5                                          # constant
        elif kind == 5:
            x[r] = rng.normal(0, 2, vocab)
            x[r, rng.random(vocab) < 0.7] = -np.inf             # mostly -inf
        elif kind == 6:
            x[r] = rng.standard_t(3, vocab) * 4
        else:
            x[r] = rng.normal(0, 1e-3, vocab)                   # tiny spread
    if bf16:
        return W.to_bf16_bits(x)
    return x


@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
@pytest.mark.parametrize("vocab", [48, 700, 5003, 40_961])
def test_plain_draws_every_row_kind(sampler, vocab, bf16):
    rng = np.random.default_rng(vocab + bf16)
    rows = 16
    x = _rows_of_kinds(rng, rows, vocab, bf16)
    ks = [1, 5, 20, 64, 65, 200, 1024, 0]
    for trial, k in enumerate(ks):
        kw = [dict(temperature=0.9, top_k=k, top_p=0.95, min_p=0.001, seed=50 + r) for r in range(rows)]
        r = run_rows(sampler, x, kw, [trial] * rows, logprobs=True)
        for i in range(rows):
            d = O.sample(x[i], None, o_params(**kw[i]), trial, want_logprob=True)
            check_row_against_oracle(r, i, d)
            if np.isfinite(d.logprob):
                assert abs(r.logprobs[i] - d.logprob) <= 1e-5 * max(1.0, abs(d.logprob)), (k, i)


def test_masks_bias_penalties_together(sampler):
    rng = np.random.default_rng(9)
    rows, vocab = 12, 30_011
    x = W.to_bf16_bits(rng.normal(0, 2, (rows, vocab)).astype(np.float32))
    masks = np.stack([W.allow_mask(rng, vocab, frac=f) for f in
                      (0.02, 0.5, 0.0005, 0.02, 0.9, 0.02, 0.001, 0.3, 0.02, 0.02, 0.6, 0.02)])
    masks[6] = 0
    masks[6, 5] = 1 << 7            # a single allowed id (167)
    bias = [[(int(i), float(d)) for i, d in zip(rng.integers(0, vocab, 40),
                                                 rng.choice([-5.0, 5.0, 30.0], 40))]
            for _ in range(rows)]
    bias[3] = bias[3] + [bias[3][0], bias[3][0]]   # duplicates accumulate in order
    hist = rng.integers(0, vocab, (rows, 3000)).astype(np.int32)
    hist[:, :200] = hist[:, 200:201]               # one id 200 times
    scratch = []
    counts = []
    for r in range(rows):
        sc = LS.SamplerScratch(sampler, vocab)
        sc.add_history(torch.from_numpy(hist[r]).to(dev()))
        scratch.append(sc)
        counts.append(np.bincount(hist[r], minlength=vocab).astype(np.uint32))
    for trial, k in enumerate((20, 64, 300, 0, 1)):
        kw = [dict(temperature=0.7 if k != 1 else 0.0, top_k=k, top_p=0.9, seed=70 + r,
                   repetition_penalty=1.2, presence_penalty=0.5, frequency_penalty=0.05)
              for r in range(rows)]
        r = run_rows(sampler, x, kw, [trial] * rows, scratch=scratch, allow=masks, bias=bias,
                     logprobs=True)
        for i in range(rows):
            d = O.sample(x[i], counts[i], o_params(**kw[i]), trial, allow=masks[i], bias=bias[i],
                         want_logprob=True)
            check_row_against_oracle(r, i, d)
            assert (masks[i][r.ids[i] >> 5] >> (r.ids[i] & 31)) & 1
            if np.isfinite(d.logprob):
                assert abs(r.logprobs[i] - d.logprob) <= 1e-5 * max(1.0, abs(d.logprob)), (k, i)
        for i in range(rows):
            assert np.array_equal(scratch[i].read_counts().numpy().view(np.uint32), counts[i])
    for sc in scratch:
        sc.close()


def test_unaligned_rows_of_a_matrix(sampler):
    """Rows of a [rows, V] matrix with odd V start at every 16-byte phase."""
    rng = np.random.default_rng(12)
    for vocab, bf16 in ((6007, False), (6007, True), (4099, True), (1021, False)):
        rows = 9
        x = rng.normal(0, 3, (rows, vocab)).astype(np.float32)
        xs = W.to_bf16_bits(x) if bf16 else x
        kw = [dict(temperature=0.8, top_k=40, top_p=0.9, min_p=0.02, seed=r) for r in range(rows)]
        r = run_rows(sampler, xs, kw, [3] * rows)
        g = run_rows(sampler, xs, [dict()] * rows, [0] * rows)
        for i in range(rows):
            check_row_against_oracle(r, i, O.sample(xs[i], None, o_params(**kw[i]), 3))
            assert g.ids[i] == O.argmax(xs[i])


def test_argmax_float_semantics(sampler):
    x = np.zeros((4, 3000), np.float32)
    x[0, 5] = -0.0
    x[1, :] = -np.inf
    x[2, :] = -1.0
    x[2, 100] = -0.0
    x[2, 2000] = 0.0
    x[3, :] = -np.inf
    x[3, 2999] = -3.0e38
    g = run_rows(sampler, x, [dict()] * 4, [0] * 4)
    assert list(g.ids) == [0, 0, 100, 2999]
    for i in range(4):
        assert g.ids[i] == O.argmax(x[i])
