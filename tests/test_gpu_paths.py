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


def _logprobs_against_oracle(sampler, x, kw, hist, bias=None, step=3):
    rows, vocab = x.shape
    scratch, counts = [], []
    for r in range(rows):
        sc = LS.SamplerScratch(sampler, vocab)
        sc.add_history(torch.from_numpy(hist[r]).to(dev()))
        scratch.append(sc)
        counts.append(np.bincount(hist[r], minlength=vocab).astype(np.uint32))
    r = run_rows(sampler, x, kw, [step] * rows, scratch=scratch, bias=bias, logprobs=True)
    for i in range(rows):
        d = O.sample(x[i], counts[i], o_params(**kw[i]), step, bias=None if bias is None else bias[i],
                     want_logprob=True)
        check_row_against_oracle(r, i, d)
        assert abs(r.logprobs[i] - d.logprob) <= 1e-5 * max(1.0, abs(d.logprob)), (i, r.logprobs[i], d.logprob)
    for sc in scratch:
        sc.close()


def test_logprob_under_penalties_of_both_signs(sampler):
    """Penalties that raise by one term and lower by another (presence < 0 with frequency > 0,
    repetition on either side of 1) over a history that names every id of a short row some fifty
    times: the frequency term takes 5 off every value, so the largest raw value says little about
    the largest true one, which the cut of the row's sum hangs from - it must hang from what the
    penalties can make of that value at the least."""
    rng = np.random.default_rng(216)
    rows, vocab = 9, 97
    x = np.sort(rng.normal(0, 3, (rows, vocab)), axis=1).astype(np.float32)
    x[1::2] = rng.normal(0, 3, (rows // 2, vocab)).astype(np.float32)
    hist = rng.integers(0, vocab, (rows, 5000)).astype(np.int32)
    kw = [dict(temperature=(0.5, 1.0, 1.7)[r % 3], top_k=(64, 7, 20)[r % 3], top_p=(1.0, 0.9)[r % 2], min_p=0.02,
               seed=1000 + r, repetition_penalty=(1.2, 0.8)[r % 2], presence_penalty=-0.5, frequency_penalty=0.1)
          for r in range(rows)]
    _logprobs_against_oracle(sampler, x, kw, hist)
    xb = W.to_bf16_bits(x)
    _logprobs_against_oracle(sampler, xb, kw, hist)


def test_logprob_with_a_bias_list_under_penalties_that_may_raise(sampler):
    """A flat row half of whose ids are named by the history, penalties that raise them above
    all others, and a bias list: the chunks that hold a named id are evaluated value by value,
    and the id of the bias list, which is dealt with apart, must not have a raw term taken off
    the row's sum that was never put there - one term in a thousand, 1.7e-3 of the
    log-probability."""
    rng = np.random.default_rng(78)
    rows, vocab = 24, 1000
    x = rng.normal(0, 0.02, (rows, vocab)).astype(np.float32)
    hist = rng.integers(0, vocab, (rows, 500)).astype(np.int32)
    bias = [[(int(rng.integers(0, vocab)), float(rng.choice([-5.0, 3.0, 0.25])))] for _ in range(rows)]
    bias[3] = bias[3] + [(int(hist[3][0]), 0.5), (int(hist[3][1]), -0.5)]   # named by both lists
    kw = [dict(temperature=(1.0, 0.5, 1.7)[r % 3], top_k=(64, 20, 7, 1 + r)[r % 4], top_p=(1.0, 0.9)[r % 2],
               min_p=0.0, seed=2000 + r, repetition_penalty=0.8, presence_penalty=-0.5, frequency_penalty=0.1)
          for r in range(rows)]
    _logprobs_against_oracle(sampler, x, kw, hist, bias=bias)
    big = rng.normal(0, 0.02, (5, 70_001)).astype(np.float32)
    hist5 = rng.integers(0, 70_001, (5, 5000)).astype(np.int32)
    bias5 = [[(int(i), float(d)) for i, d in zip(rng.integers(0, 70_001, 8), rng.choice([-5.0, 3.0, 20.0], 8))]
             for _ in range(5)]
    _logprobs_against_oracle(sampler, big, [dict(kw[r], top_k=(20, 64)[r % 2]) for r in range(5)], hist5, bias=bias5)


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
