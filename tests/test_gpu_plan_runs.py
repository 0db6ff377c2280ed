"""A resident plan run many times: the configuration the benchmark times.

Every run draws one token per row and counts it, so the scratches' lists grow from run to run:
first the unsorted tails, then - once the host's bound of a tail passes the sort threshold - a
sorting launch in front of the row kernel.  After every run the ids, the counts and the
log-probabilities must equal the oracle's, fed the counts accumulated so far.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import lily_sampler as LS
import lily_workloads as W
import oracle as O
from gpu_util import dev, ls_params, o_params, upload_logits

LOGPROB_RTOL = 1e-5


def _plan_case(sampler, x, hist, kw, runs, between=None, check_every=1):
    rows, vocab = x.shape
    sc, counts = [], []
    for h in hist:
        s_ = LS.SamplerScratch(sampler, vocab)
        s_.add_history(torch.from_numpy(np.ascontiguousarray(h)).to(dev()))
        sc.append(s_)
        counts.append(np.bincount(h, minlength=vocab).astype(np.uint32))
    logits = upload_logits(x)
    out = torch.full((rows,), -1, dtype=torch.int32, device=dev())
    lp = torch.zeros(rows, dtype=torch.float32, device=dev())
    params = [ls_params(**k) for k in kw]
    torch.cuda.synchronize()
    plan = sampler.plan(logits, params, [2] * rows, out, scratch=sc, out_logprobs=lp)
    for i in range(runs):
        if between is not None:
            between(i, sc, counts)
        plan.run(i)
        sampler.synchronize()
        ids, lps = out.cpu().numpy(), lp.cpu().numpy()
        for r in range(rows):
            if i % check_every == 0 or i == runs - 1:
                d = O.sample(x[r], counts[r], o_params(**kw[r]), 2 + i, want_logprob=True)
                assert ids[r] == d.chosen, (i, r, ids[r], d.chosen)
                assert abs(lps[r] - d.logprob) <= LOGPROB_RTOL * max(1.0, abs(d.logprob)), (i, r)
            else:
                counts[r][ids[r]] += 1  # trust the id between checks; the counts are compared below
        if i % check_every == 0 or i == runs - 1:
            for r in range(0, rows, max(1, rows // 4)):
                assert np.array_equal(sc[r].read_counts().numpy().view(np.uint32), counts[r]), (i, r)
    plan.close()
    for s_ in sc:
        s_.close()


@pytest.fixture(scope="module")
def sampler():
    s = LS.Sampler(0)
    yield s
    s.close()


def test_a_penalised_plan_with_logprobs_run_twelve_times(sampler):
    """The benchmark's shape at 40 rows: bf16, k 64, 2 048-id history, ids + log-probabilities."""
    c = W.config5(rows=40)
    _plan_case(sampler, c["logits"], c["history"], c["params"], 12)


def test_a_plan_run_past_the_sort_threshold(sampler):
    """300 runs of a 6-row plan over a small vocabulary: the tails pass 256 ids, the lists are
    sorted in front of run 256 or so, and nothing changes in the draws.  High temperature and a
    wide top-p so that most runs emit an id never counted before (the tails really grow)."""
    rng = np.random.default_rng(61)
    rows, vocab = 6, 24_001
    x = W.to_bf16_bits(rng.normal(0, 1.0, (rows, vocab)).astype(np.float32))
    hist = [rng.integers(0, vocab, 300).astype(np.int32) for _ in range(rows)]
    kw = [dict(temperature=1.5, top_k=64, top_p=1.0, seed=900 + r, repetition_penalty=1.3,
               presence_penalty=0.6, frequency_penalty=0.2) for r in range(rows)]
    _plan_case(sampler, x, hist, kw, 300, check_every=1)


def test_a_plan_whose_scratches_change_between_runs(sampler):
    """add_history, uncount and reset between the runs of one plan: the next run sees them."""
    rng = np.random.default_rng(67)
    rows, vocab = 4, 151_936
    x = rng.normal(0, 3, (rows, vocab)).astype(np.float32)
    hist = [rng.integers(0, vocab, 1000).astype(np.int32) for _ in range(rows)]
    kw = [dict(temperature=0.8, top_k=20, top_p=0.95, min_p=0.02, seed=70 + r, repetition_penalty=1.2,
               presence_penalty=0.5, frequency_penalty=0.3) for r in range(rows)]
    top = [np.argsort(-x[r])[:6].astype(np.int32) for r in range(rows)]

    def between(i, sc, counts):
        if i == 2:      # more history, with ids the draws look at
            for r in range(rows):
                extra = np.concatenate([top[r], rng.integers(0, vocab, 500).astype(np.int32)])
                sc[r].add_history(torch.from_numpy(extra).to(dev()))
                counts[r] += np.bincount(extra, minlength=vocab).astype(np.uint32)
        if i == 4:      # a rollback
            for r in range(rows):
                sc[r].uncount(int(top[r][0]))
                O.lib().lo_uncount(counts[r].ctypes.data, vocab, int(top[r][0]))
        if i == 6:      # a new request on row 1
            sc[1].reset_counts()
            counts[1][:] = 0

    _plan_case(sampler, x, hist, kw, 9, between=between)
