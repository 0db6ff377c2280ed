"""The hand-over between the workgroups that share a row (slices): partials are stored through
to memory, the workgroup that takes the row's ticket last reads them past its caches - behind a
release / acquire pair on the ticket, or in the relaxed form that large launches use (both forms
are run here whatever the launch's size, through LILY_SAMPLER_HANDOVER).  A
partial read too early, or found stale in a cache, would be the one the previous launch left
at the same place - so two plans over different logits run in turn, hundreds of times, and
every launch must draw what its own plan drew the first time (ids exactly, log-probabilities
within the 2e-6 by which replays differ), and that first draw is the oracle's."""
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import lily_sampler as LS
import lily_workloads as W
import oracle as O
from gpu_util import dev


@pytest.mark.parametrize("rows,vocab,k,bf16", [(4, 151_936, 20, False), (16, 151_936, 64, True),
                                               (64, 50_021, 40, False), (3, 151_936, 0, False),
                                               (48, 151_936, 0, True)],
                         ids=["4x38 slices", "16x32 bf16", "64x8", "k1024 two launches", "k1024 48 rows bf16"])
@pytest.mark.parametrize("form", ["strict", "relaxed"])
def test_plans_over_different_logits_in_turn(rows, vocab, k, bf16, form):
    old = os.environ.get("LILY_SAMPLER_HANDOVER")
    os.environ["LILY_SAMPLER_HANDOVER"] = form
    try:
        s = LS.Sampler(0)
    finally:
        if old is None:
            os.environ.pop("LILY_SAMPLER_HANDOVER", None)
        else:
            os.environ["LILY_SAMPLER_HANDOVER"] = old
    rng = np.random.default_rng(rows * 7 + k)
    plans, host_rows = [], []
    for which in range(2):
        x = rng.normal(0, 3, (rows, vocab)).astype(np.float32)
        if bf16:
            host_rows.append(W.to_bf16_bits(x))
            t = torch.from_numpy(host_rows[-1].view(np.int16)).to(dev()).view(torch.bfloat16)
        else:
            host_rows.append(x)
            t = torch.from_numpy(x).to(dev())
        out = torch.zeros(rows, dtype=torch.int32, device=dev())
        lp = torch.zeros(rows, dtype=torch.float32, device=dev())
        params = [LS.SamplingParams.greedy(temperature=0.7, top_k=k, top_p=0.95, seed=10 + r) for r in range(rows)]
        plans.append((s.plan(t, params, [7] * rows, out, out_logprobs=lp), out, lp, t))
    assert s.slices_for(rows, max(k, 1), vocab) > 1
    first = []
    for plan, out, lp, _ in plans:
        plan.run(3)
        s.synchronize()
        first.append((out.clone(), lp.clone()))
    assert not torch.equal(first[0][0], first[1][0]), "the two plans draw different tokens"
    # the draws every later launch is compared with are the oracle's (a sample of the rows)
    for x, (ids0, lp0) in zip(host_rows, first):
        got, got_lp = ids0.cpu().numpy(), lp0.cpu().numpy()
        for r in range(0, rows, max(1, rows // 6)):
            d = O.sample(x[r], None, O.params(temperature=0.7, top_k=k, top_p=0.95, seed=10 + r), 3 + 7,
                         want_logprob=True)
            assert got[r] == d.chosen, (r, got[r], d.chosen)
            assert abs(got_lp[r] - d.logprob) <= 1e-5 * max(1.0, abs(d.logprob)), (r, got_lp[r], d.logprob)
    wrong = torch.zeros(1, dtype=torch.int64, device=dev())
    for _ in range(300):
        for (plan, out, lp, _), (ids0, lp0) in zip(plans, first):
            plan.run(3)
            wrong += (out != ids0).sum() + ((lp - lp0).abs() > 1e-4).sum()
    s.synchronize()
    assert int(wrong.item()) == 0
    for plan, *_ in plans:
        plan.close()
    s.close()
