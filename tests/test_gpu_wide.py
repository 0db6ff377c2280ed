"""Rows that draw among many candidates (k > 64; a request without top_k gets the reference's cap
of 1024, src/kernels/sample.rs:17 and :326-331) through the two launches that spread such a
row over as many workgroups as a row of few candidates: a bound from the lanes' maxima, then
the values that reach it.

Ids, candidates, probabilities and kept counts bit-exact against the oracle, the
log-probability within 1e-5 (relative, floor 1), the counts of penalised ids as the oracle
leaves them.  Which way a launch went shows in the path statistics: a row drawn this way adds
one to its entry, a row drawn by the other kernels one per workgroup.
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

LOGPROB_RTOL = 1e-5


@pytest.fixture(scope="module")
def sampler():
    s = LS.Sampler(0)
    yield s
    s.close()


def _with_stats(sampler, fn):
    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    sampler.set_path_stats(stats)
    try:
        out = fn()
    finally:
        sampler.synchronize()
        sampler.set_path_stats(None)
    return out, stats.cpu().numpy()


def _check_logprob(got, want, what):
    if np.isfinite(want):
        assert abs(got - want) <= LOGPROB_RTOL * max(1.0, abs(want)), (what, got, want)
    else:
        assert got == -np.inf, what


@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
@pytest.mark.parametrize("use_plan", [False, True], ids=["inline", "plan"])
def test_plain_rows_of_many_candidates(sampler, bf16, use_plan):
    """Rows of every k above the streaming select's, heavy tails, a row with fewer finite
    values than k, a vocabulary that leaves partial chunks at both ends of the slices."""
    rng = np.random.default_rng(71 + bf16)
    rows, vocab = 5, 151_937 if not bf16 else 151_939
    x = (rng.standard_t(5, (rows, vocab)) * 2.5).astype(np.float32)
    x[2, rng.random(vocab) < 0.997] = -np.inf          # ~450 finite values: fewer than k
    x[4, rng.integers(0, vocab, 2000)] = -np.inf
    if bf16:
        x = W.to_bf16_bits(x)
    assert sampler.slices_for(rows, 1024, vocab) > 1
    for trial, k in enumerate((0, 65, 200, 777)):
        kw = [dict(temperature=0.7 + 0.1 * r, top_k=k, top_p=0.95, min_p=0.01, seed=300 + r) for r in range(rows)]
        r, stats = _with_stats(sampler, lambda: run_rows(sampler, x, kw, [trial] * rows, logprobs=True,
                                                         use_plan=use_plan))
        assert stats[0] == 0 and stats[1] + stats[2] == rows, stats   # one count a row: the two launches
        for i in range(rows):
            d = O.sample(x[i], None, o_params(**kw[i]), trial, want_logprob=True)
            check_row_against_oracle(r, i, d)
            _check_logprob(r.logprobs[i], d.logprob, (k, i))


def test_prefix_sums_that_leave_their_binade_and_round_on_ties(sampler):
    """The left-to-right f32 sums of up to 1 024 weights are formed 64 at a time by integer
    additions while the running sum stays in one binade and no weight lies exactly half a last
    place above a multiple of it, and by the chain of real additions otherwise.  Rows that force
    either way: hundreds of ids at the row's largest value (weights of exactly 1: the sum walks
    through nine binades on integers), a flat row (the sum crosses a binade every few blocks and
    weights within a few binades of the sum tie often), a peaked row (one binade, no ties after
    the first block), and steps of one bf16 ulp (weights in a handful of exact ratios).  The
    kept counts and the probabilities are bit-exact against the oracle, so is every draw."""
    rng = np.random.default_rng(4242)
    vocab = 151_936
    x = np.empty((4, vocab), dtype=np.float32)
    x[0] = rng.normal(0, 1, vocab)
    x[0, rng.choice(vocab, 700, replace=False)] = 9.0
    x[1] = rng.normal(0, 0.05, vocab)
    x[2] = rng.normal(0, 1, vocab)
    x[2, 77] = 30.0
    x[3] = np.round(rng.normal(0, 3, vocab) * 8) / 8
    for trial, (t, top_p) in enumerate(((1.0, 0.999), (0.7, 0.9), (1.3, 0.97))):
        kw = [dict(temperature=t, top_k=0, top_p=top_p, seed=900 + r) for r in range(4)]
        r, stats = _with_stats(sampler, lambda: run_rows(sampler, x, kw, [trial] * 4, logprobs=True))
        assert stats[0] == 0 and stats[1] + stats[2] == 4, stats
        for i in range(4):
            d = O.sample(x[i], None, o_params(**kw[i]), trial, want_logprob=True)
            check_row_against_oracle(r, i, d)
            _check_logprob(r.logprobs[i], d.logprob, (trial, i))


def test_penalised_rows_over_decode_steps(sampler):
    """Lowering penalties (repetition >= 1, presence and frequency >= 0) on the ids that matter
    most: the lanes' maxima, the row's sum and the candidates are taken on penalised worth.
    Three steps, the counts moving with the draws; a last call with a penalty that may raise
    a value goes the other kernels' way and draws what the oracle draws as well."""
    rng = np.random.default_rng(72)
    rows, vocab = 4, 151_936
    x = rng.normal(0, 3, (rows, vocab)).astype(np.float32)
    kw = [dict(temperature=0.6, top_k=0, top_p=0.95, min_p=0.0, seed=77 + r, repetition_penalty=1.2,
               presence_penalty=0.4, frequency_penalty=0.3) for r in range(rows)]
    scratch, counts = [], []
    for r in range(rows):
        best = np.argsort(-x[r])[:400].astype(np.int32)
        hh = np.concatenate([rng.integers(0, vocab, 3000).astype(np.int32), np.repeat(best[:40], 5), best])
        sc = LS.SamplerScratch(sampler, vocab)
        sc.add_history(torch.from_numpy(hh).to(dev()))
        scratch.append(sc)
        counts.append(np.bincount(hh, minlength=vocab).astype(np.uint32))
    for step in range(3):
        r, stats = _with_stats(sampler, lambda: run_rows(sampler, x, kw, [step] * rows, scratch=scratch,
                                                         logprobs=True, use_plan=step == 1))
        assert stats[1] == rows and stats[2] == 0, stats
        for i in range(rows):
            d = O.sample(x[i], counts[i], o_params(**kw[i]), step, want_logprob=True)   # bumps the counts
            check_row_against_oracle(r, i, d)
            _check_logprob(r.logprobs[i], d.logprob, (step, i))
    kw[1] = dict(kw[1], repetition_penalty=0.8)
    r, stats = _with_stats(sampler, lambda: run_rows(sampler, x, kw, [3] * rows, scratch=scratch, logprobs=True))
    assert stats[1] > rows, stats
    for i in range(rows):
        d = O.sample(x[i], counts[i], o_params(**kw[i]), 3, want_logprob=True)
        check_row_against_oracle(r, i, d)
    for i in range(rows):
        assert np.array_equal(scratch[i].read_counts().numpy().view(np.uint32), counts[i]), i
        scratch[i].close()


def test_more_values_at_the_bound_than_the_list_holds(sampler):
    """A constant row, a row of a few distinct values and a row in ascending order: every lane's
    maximum ties or the bound lets most of the row through, the row's list overflows, and the
    workgroup that finishes the row takes the select that is right for any input."""
    rng = np.random.default_rng(73)
    rows, vocab = 4, 100_003
    x = rng.normal(0, 1, (rows, vocab)).astype(np.float32)
    x[0, :] = 0.25
    x[1] = rng.integers(-1, 2, vocab) / 4.0
    x[2] = np.linspace(-3, 3, vocab, dtype=np.float32)
    kw = [dict(temperature=1.1, top_k=0, top_p=0.99, min_p=0.0, seed=9 + r) for r in range(rows)]
    r, stats = _with_stats(sampler, lambda: run_rows(sampler, x, kw, [5] * rows, logprobs=True))
    assert stats[2] >= 2 and stats[1] + stats[2] == rows, stats
    for i in range(rows):
        d = O.sample(x[i], None, o_params(**kw[i]), 5, want_logprob=True)
        check_row_against_oracle(r, i, d)
        _check_logprob(r.logprobs[i], d.logprob, i)


def test_sixty_four_rows_and_the_way_of_the_other_kernels(sampler):
    """64 bf16 rows at k = 1024 (8 or 16 workgroups a row: the bound is then the median of the
    lanes' maxima); the same call on a sampler that has this way switched off draws the same."""
    c = W.config4(rows=64)
    x = c["logits"]
    rows, vocab = x.shape
    kw = c["params"]
    r, stats = _with_stats(sampler, lambda: run_rows(sampler, x, kw, [2] * rows, logprobs=True))
    assert stats[1] == rows and stats[2] == 0, stats
    old = os.environ.get("LILY_SAMPLER_WIDE")
    os.environ["LILY_SAMPLER_WIDE"] = "0"
    try:
        other = LS.Sampler(0)
    finally:
        if old is None:
            os.environ.pop("LILY_SAMPLER_WIDE", None)
        else:
            os.environ["LILY_SAMPLER_WIDE"] = old
    try:
        r2, stats2 = _with_stats(other, lambda: run_rows(other, x, kw, [2] * rows, logprobs=True))
    finally:
        other.close()
    assert stats2[1] > rows, stats2
    assert np.array_equal(r.ids, r2.ids) and np.array_equal(r.cand_ids, r2.cand_ids)
    assert np.all(np.abs(r.logprobs - r2.logprobs) <= LOGPROB_RTOL * np.maximum(1.0, np.abs(r2.logprobs)))   # (the rows' sums are grouped differently)
    for i in range(0, rows, 7):
        d = O.sample(x[i], None, o_params(**kw[i]), 2, want_logprob=True)
        check_row_against_oracle(r, i, d)
        _check_logprob(r.logprobs[i], d.logprob, i)


def test_random_launches_of_rows_of_many_candidates(sampler):
    """Forty seeded launches: 1 to 23 rows, vocabularies that leave partial chunks at the slices'
    ends, f32 and bf16, k from 65 to 1024, Gaussian, heavy-tailed and peaked rows, rows that are
    mostly -inf, lowering penalties over histories that hold the rows' best ids, with and
    without a log-probability, as a call and as a plan."""
    rng = np.random.default_rng(2024)
    went = 0
    for case in range(40):
        rows = int(rng.integers(1, 24))
        vocab = int(rng.choice([32_003, 50_021, 100_003, 151_936, 151_937, 151_939, 200_001]))
        bf16 = bool(rng.integers(0, 2))
        k = int(rng.choice([0, 65, 100, 300, 777, 1024]))
        pen, logprob, use_plan = (bool(rng.integers(0, 2)) for _ in range(3))
        kind = int(rng.integers(0, 3))
        if kind == 0:
            x = rng.normal(0, 3, (rows, vocab)).astype(np.float32)
        elif kind == 1:
            x = (rng.standard_t(3, (rows, vocab)) * 2).astype(np.float32)
        else:
            x = rng.normal(0, 0.5, (rows, vocab)).astype(np.float32)
            x[:, rng.integers(0, vocab, 50)] += 12.0
        if rng.integers(0, 4) == 0:
            x[rng.integers(0, rows), rng.random(vocab) < 0.99] = -np.inf
        xf = x
        if bf16:
            x = W.to_bf16_bits(x)
            xf = W.bf16_bits_to_f32(x)
        kw = []
        for r in range(rows):
            d = dict(temperature=float(rng.uniform(0.3, 1.5)), top_k=k, top_p=float(rng.choice([0.8, 0.95, 1.0])),
                     min_p=float(rng.choice([0.0, 0.01])), seed=int(rng.integers(0, 1 << 30)))
            if pen:
                d.update(repetition_penalty=float(rng.choice([1.0, 1.1, 1.5])),
                         presence_penalty=float(rng.choice([0.0, 0.5])),
                         frequency_penalty=float(rng.choice([0.0, 0.2])))
            kw.append(d)
        scratch = counts = None
        if pen:
            scratch, counts = [], []
            for r in range(rows):
                best = np.argsort(-xf[r])[:int(rng.integers(10, 600))].astype(np.int32)
                hh = np.concatenate([rng.integers(0, vocab, int(rng.integers(0, 5000))).astype(np.int32),
                                     np.repeat(best[:20], int(rng.integers(1, 6))), best])
                sc = LS.SamplerScratch(sampler, vocab)
                sc.add_history(torch.from_numpy(hh).to(dev()))
                scratch.append(sc)
                counts.append(np.bincount(hh, minlength=vocab).astype(np.uint32))
        step = int(rng.integers(0, 100))
        r, stats = _with_stats(sampler, lambda: run_rows(sampler, x, kw, [step] * rows, scratch=scratch,
                                                         logprobs=logprob, use_plan=use_plan))
        went += int(stats[1] + stats[2] == rows)
        for i in range(rows):
            d = O.sample(x[i], counts[i] if pen else None, o_params(**kw[i]), step, want_logprob=logprob)
            check_row_against_oracle(r, i, d)
            if logprob:
                _check_logprob(r.logprobs[i], d.logprob, (case, i))
        if pen:
            for i in range(rows):
                assert np.array_equal(scratch[i].read_counts().numpy().view(np.uint32), counts[i]), (case, i)
                scratch[i].close()
    assert went >= 30, went   # (a launch of one or two rows has too few slices for some k)
