"""Seeded random launches against the oracle: every combination the boundary accepts.

Each case draws a vocabulary size, a batch, a dtype, a value distribution (normal, heavy
ties, heavy tails, nearly flat, one late outlier far above the rest, ascending), per-row or
shared k / temperature / top-p / min-p, and independently an allow-mask of some density, a
bias list (up to 100 pairs, duplicates included), penalties of either sign over a history,
forced ids, explicit uniforms, the plan or the direct call, and one of three slices-per-row
settings.  Ids, candidates, probabilities, kept counts and scratch counts are compared bit for
bit, log-probabilities within 1e-5 (relative, floor 1).  (Temperatures stay at 0.5 and above:
below that, over the heavy-tailed rows and the rows with an outlier of 700, the oracle's own
rounding of l / T to f32 is what the 1e-5 would measure.)
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


def _sampler_with_slices(slices):
    old = os.environ.get("LILY_SAMPLER_SLICES")
    os.environ["LILY_SAMPLER_SLICES"] = str(slices)
    try:
        return LS.Sampler(0)
    finally:
        if old is None:
            os.environ.pop("LILY_SAMPLER_SLICES", None)
        else:
            os.environ["LILY_SAMPLER_SLICES"] = old


@pytest.fixture(scope="module")
def samplers():
    ss = [_sampler_with_slices(n) for n in (0, 1, 3)]
    yield ss
    for s in ss:
        s.close()


def _values(rng, kind, rows, vocab):
    if kind == 0:
        return rng.normal(0, 2, (rows, vocab))
    if kind == 1:
        return rng.integers(-8, 9, (rows, vocab)) / 4.0
    if kind == 2:
        return rng.standard_t(3, (rows, vocab)) * 4
    if kind == 3:
        return rng.normal(0, 0.02, (rows, vocab))
    if kind == 4:
        x = rng.normal(0, 1, (rows, vocab))
        x[:, -1 - int(rng.integers(0, 50))] = float(rng.choice([40.0, 300.0, 700.0]))
        return x
    return np.sort(rng.normal(0, 3, (rows, vocab)), axis=1)


@pytest.mark.parametrize("block", range(6))
def test_random_launches(samplers, block):
    _random_launches(samplers, range(block * 25, block * 25 + 25), 770_000, harsh=False)


@pytest.mark.parametrize("block", range(6))
def test_random_launches_with_wider_settings(samplers, block):
    """The same with batches of up to 130 rows, temperatures up to 2.5, repetition
    penalties of 0.5 to 2, presence penalties of -2 to 2, frequency penalties of -0.2 to 0.5
    (terms that raise beside terms that lower), min-p up to 0.3, and histories of 1 to 20 000
    ids of which half may repeat one id or all may come from the row's best 50."""
    _random_launches(samplers, range(block * 25, block * 25 + 25), 880_000, harsh=True)


def _random_launches(samplers, cases, seed_base, harsh):
    for case in cases:
        rng = np.random.default_rng(seed_base + case)
        s = samplers[int(rng.integers(0, 3))]
        use_plan = bool(rng.integers(0, 2))
        vocab = int(rng.choice([97, 1000, 4099, 30011, 70001, 151936]))
        rows = int(rng.choice([1, 2, 5, 9, 40, 130] if harsh else [1, 2, 5, 9, 40]))
        bf16 = bool(rng.integers(0, 2))
        x = _values(rng, int(rng.integers(0, 6)), rows, vocab).astype(np.float32)
        if rng.random() < 0.3:
            x[rng.random((rows, vocab)) < 0.5] = -np.inf
        if bf16:
            x = W.to_bf16_bits(x)
        masks = bias = forced = uniforms = sc = None
        counts, pen = [None] * rows, {}
        if rng.random() < 0.4:
            masks = np.stack([W.allow_mask(rng, vocab, frac=float(rng.choice([0.001, 0.02, 0.3, 0.9])))
                              for _ in range(rows)])
        if rng.random() < 0.4:
            nb = int(rng.choice([1, 8, 40, 100]))
            bias = [[(int(i), float(d)) for i, d in zip(rng.integers(0, vocab, nb),
                                                         rng.choice([-5.0, 3.0, 20.0], nb))]
                    for _ in range(rows)]
        if rng.random() < 0.5:
            pen = dict(repetition_penalty=float(rng.choice([0.5, 1.0, 1.05, 2.0] if harsh else [0.8, 1.2])),
                       presence_penalty=float(rng.choice([-2.0, 0.0, 0.3, 2.0] if harsh else [-0.5, 0.5])),
                       frequency_penalty=float(rng.choice([-0.2, 0.0, 0.05, 0.5] if harsh else [0.0, 0.1])))
            sc, counts = [], []
            length = int(rng.choice([1, 40, 2000, 20000] if harsh else [10, 500, 5000]))
            for r_ in range(rows):
                h = rng.integers(0, vocab, length).astype(np.int32)
                if harsh and rng.random() < 0.5:
                    h[: length // 2] = h[0]
                if harsh and rng.random() < 0.3:
                    xf = W.bf16_bits_to_f32(x[r_]) if bf16 else x[r_]
                    h[:] = np.argsort(-xf)[rng.integers(0, min(50, vocab), length)]
                t = LS.SamplerScratch(s, vocab)
                t.add_history(torch.from_numpy(h).to(dev()))
                sc.append(t)
                counts.append(np.bincount(h, minlength=vocab).astype(np.uint32))
        if rng.random() < 0.25:
            forced = [int(rng.integers(0, vocab)) if rng.random() < 0.5 else None for _ in range(rows)]
        if rng.random() < 0.3:
            uniforms = [float(rng.choice([0.0, 0.25, 0.999999])) if rng.random() < 0.7 else None
                        for _ in range(rows)]
        ks, temps = [1, 7, 20, 64, 65, 300, 1024, 0], ([0.5, 1.0, 2.5] if harsh else [0.5, 1.0, 1.7])
        mixed = rng.random() < 0.5
        k, temperature = int(rng.choice(ks)), float(rng.choice(temps))
        kw = []
        for r_ in range(rows):
            kw.append(dict(temperature=float(rng.choice([0.0] + temps)) if mixed else temperature,
                           top_k=int(rng.choice(ks)) if mixed else k,
                           top_p=float(rng.choice([0.5, 0.9, 1.0])),
                           min_p=float(rng.choice([0.0, 0.02, 0.3] if harsh else [0.0, 0.02])), seed=1000 + r_,
                           **pen))
        r = run_rows(s, x, kw, [case] * rows, scratch=sc, allow=masks, bias=bias, forced=forced,
                     uniforms=uniforms, logprobs=True, use_plan=use_plan)
        for i in range(rows):
            ext = dict(want_logprob=True)
            if masks is not None:
                ext["allow"] = masks[i]
            if bias is not None:
                ext["bias"] = bias[i]
            if forced is not None and forced[i] is not None:
                ext["forced"] = forced[i]
            if uniforms is not None and uniforms[i] is not None:
                ext["uniform"] = uniforms[i]
            d = O.sample(x[i], counts[i], o_params(**kw[i]), case, **ext)
            if forced is not None and forced[i] is not None:
                assert r.ids[i] == forced[i], (case, i)
            else:
                check_row_against_oracle(r, i, d)
            if np.isfinite(d.logprob):
                assert abs(r.logprobs[i] - d.logprob) <= 1e-5 * max(1.0, abs(d.logprob)), (case, i)
            elif not np.isnan(d.logprob):
                assert r.logprobs[i] == -np.inf, (case, i)
        if sc is not None:
            for i in range(rows):
                assert np.array_equal(sc[i].read_counts().numpy().view(np.uint32), counts[i]), (case, i)
            for t in sc:
                t.close()
