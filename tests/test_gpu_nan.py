"""NaN logits.  The reference has no rule for them (its CPU twin sorts with total_cmp, which puts
a positive NaN above +inf; its kernels compare with <, which a NaN never wins).  Here a NaN logit
is worth -inf in every select: never a candidate, no term of the row sum.  Each case runs a row
with NaNs planted among its best values and checks it against the oracle on the same row with
-inf in their place."""
import numpy as np
import pytest
import torch

import lily_sampler as LS
import lily_workloads as W
import oracle as O
from gpu_util import check_row_against_oracle, dev, o_params, run_rows

pytestmark = pytest.mark.gpu


def _plant(x, rng, n=12):
    """NaNs (both signs, quiet patterns) at the row's best ids, its first and last id and a few others."""
    bad = x.copy()
    ids = np.concatenate([np.argsort(x)[::-1][:n:2], [0, len(x) - 1], rng.integers(0, len(x), 5)])
    bits = bad.view(np.uint32)
    bits[ids[::2]] = 0x7FC00000
    bits[ids[1::2]] = 0xFFC00001
    clean = x.copy()
    clean[ids] = -np.inf
    return bad, clean


CASES = {
    "plain k50": dict(temperature=0.8, top_k=50, top_p=0.9),
    "penalties k64": dict(temperature=0.7, top_k=64, top_p=0.95, repetition_penalty=1.2,
                          presence_penalty=0.2, frequency_penalty=0.1),
    "k 1024": dict(temperature=1.0, top_k=0, top_p=0.9),
    "k 300 min_p": dict(temperature=1.3, top_k=300, top_p=1.0, min_p=0.001),
    "greedy": dict(),
    "greedy penalties": dict(repetition_penalty=1.3, presence_penalty=0.5),
}


@pytest.mark.parametrize("case", list(CASES))
@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
@pytest.mark.parametrize("slices", [0, 1], ids=["auto", "one-slice"])
def test_nan_logits_are_worth_minus_infinity(case, bf16, slices, monkeypatch):
    monkeypatch.setenv("LILY_SAMPLER_SLICES", str(slices))
    s = LS.Sampler(0)
    rng = np.random.default_rng(len(case) + 2 * bf16)
    vocab, rows = 151_936, 3
    kw = CASES[case]
    xs_bad, xs_clean = [], []
    for r in range(rows):
        x = rng.normal(0, 2, vocab).astype(np.float32)
        if r == 1:
            x[rng.integers(0, vocab)] = 40.0            # a dominant value next to the NaNs
        if bf16:
            x = (W.to_bf16_bits(x).astype(np.uint32) << 16).view(np.float32)
        b, c = _plant(x, rng)
        xs_bad.append(b)
        xs_clean.append(c)
    bad, clean = np.stack(xs_bad), np.stack(xs_clean)
    if bf16:
        up_bad = (bad.view(np.uint32) >> 16).astype(np.uint16)
        up_clean = (clean.view(np.uint32) >> 16).astype(np.uint16)
    else:
        up_bad, up_clean = bad, clean
    pen = "repetition_penalty" in kw
    hist = [rng.integers(0, vocab, 800) for _ in range(rows)]
    counts = [np.bincount(h, minlength=vocab).astype(np.uint32) for h in hist]
    sc = None
    if pen:
        sc = []
        for h in hist:
            t = LS.SamplerScratch(s, vocab)
            t.add_history(torch.from_numpy(np.ascontiguousarray(h, dtype=np.int32)).to(dev()))
            sc.append(t)
    params = [dict(seed=300 + r, **kw) for r in range(rows)]
    r = run_rows(s, up_bad, params, [4] * rows, scratch=sc, logprobs=True)
    for i in range(rows):
        d = O.sample(up_clean[i], counts[i] if pen else np.zeros(vocab, np.uint32), o_params(**params[i]), 4,
                     want_logprob=True)
        assert r.ids[i] == d.chosen, (case, i)
        if kw.get("temperature", 0.0) > 0.0:
            check_row_against_oracle(r, i, d)
        assert np.isfinite(r.logprobs[i]) or not np.isfinite(d.logprob), (case, i, r.logprobs[i])
        if np.isfinite(d.logprob):
            assert abs(r.logprobs[i] - d.logprob) <= 1e-5 * max(1.0, abs(d.logprob)), (case, i)
    if sc:
        for t in sc:
            t.close()
    s.close()
