"""Rows outside the streaming select: k above 64 (the reference's default when top_k is 0
is 1024), allow-masks served by the sparse select, and forced rows that want a
log-probability.

Bit-exact ids, candidates, probabilities and kept counts against the oracle; the
log-probability within 1e-5 (relative, floor 1).  The 1024-candidate tail is the part under
test for flat rows: its prefix sums must be the reference's left-to-right f32 sums, or the
top-p cut and the pick move.
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


@pytest.fixture(scope="module")
def sampler():
    s = LS.Sampler(0)
    yield s
    s.close()


def _check_logprob(r, i, d, what):
    if np.isfinite(d.logprob):
        assert abs(r.logprobs[i] - d.logprob) <= 1e-5 * max(1.0, abs(d.logprob)), (what, i)
    else:
        assert r.logprobs[i] == -np.inf, (what, i)


@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
def test_all_1024_candidates_kept(sampler, bf16):
    """Flat rows with top_p 1 and min_p 0: every one of the 1024 candidates is kept, so the
    pick depends on all 1024 sequential prefix sums (several uniforms per row, among them
    draws at both ends)."""
    rng = np.random.default_rng(31 + bf16)
    rows, vocab = 6, 151_936
    x = rng.normal(0, 0.05, (rows, vocab)).astype(np.float32)
    x[1] = rng.integers(-2, 3, vocab) / 8.0          # heavy ties across the k-th place
    x[2, :] = 0.25                                    # constant: ids decide
    if bf16:
        x = W.to_bf16_bits(x)
    for trial, u in enumerate((None, 0.0, 0.999999, 0.5)):
        kw = [dict(temperature=1.3, top_k=0, top_p=1.0, min_p=0.0, seed=900 + r) for r in range(rows)]
        uniforms = None if u is None else [u] * rows
        r = run_rows(sampler, x, kw, [trial] * rows, uniforms=uniforms, logprobs=True)
        for i in range(rows):
            d = O.sample(x[i], None, o_params(**kw[i]), trial, want_logprob=True,
                         uniform=None if u is None else u)
            check_row_against_oracle(r, i, d)
            assert r.n_kept[i] == 1024
            _check_logprob(r, i, d, ("kept-all", trial))


def test_top_k_between_65_and_1024(sampler):
    """k just above the streaming select's limit, odd sizes, and k above the number of
    finite values."""
    rng = np.random.default_rng(32)
    rows, vocab = 8, 50_021
    x = rng.standard_t(4, (rows, vocab)).astype(np.float32) * 2
    x[3, rng.random(vocab) < 0.995] = -np.inf        # ~250 finite values < k
    for trial, k in enumerate((65, 100, 257, 513, 1000, 1023)):
        kw = [dict(temperature=0.9, top_k=k, top_p=0.97, min_p=1e-4, seed=40 + r) for r in range(rows)]
        r = run_rows(sampler, x, kw, [trial] * rows, logprobs=True)
        for i in range(rows):
            d = O.sample(x[i], None, o_params(**kw[i]), trial, want_logprob=True)
            check_row_against_oracle(r, i, d)
            _check_logprob(r, i, d, ("k", k))


def _sampler_with_slices(slices):
    """A sampler whose launches use `slices` workgroups per row (0 = its own choice)."""
    old = os.environ.get("LILY_SAMPLER_SLICES")
    os.environ["LILY_SAMPLER_SLICES"] = str(slices)
    try:
        return LS.Sampler(0)
    finally:
        if old is None:
            os.environ.pop("LILY_SAMPLER_SLICES", None)
        else:
            os.environ["LILY_SAMPLER_SLICES"] = old


@pytest.mark.parametrize("slices", [0, 1], ids=["auto-slices", "one-slice"])
def test_masks_of_every_density_report_their_select(slices):
    """Sparse masks are served from the mask's words (no row is streamed); masks that admit more
    ids than that select holds by the streaming select when k <= 64 (barred ids turn into -inf
    as their chunks arrive) and by the bitmap select otherwise; all agree with the oracle."""
    s = _sampler_with_slices(slices)
    rng = np.random.default_rng(33)
    vocab = 151_936
    fracs = (0.0, 0.0002, 0.02, 0.02, 0.05, 0.6)
    rows = len(fracs)
    x = W.to_bf16_bits(rng.normal(0, 2, (rows, vocab)).astype(np.float32))
    masks = np.stack([W.allow_mask(rng, vocab, frac=max(f, 1e-5)) for f in fracs])
    masks[0] = 0                                      # nothing allowed: id 0, log-probability -inf
    bias = [[(int(i), float(d)) for i, d in zip(rng.integers(0, vocab, 32),
                                                 rng.choice([-5.0, 5.0], 32))] for _ in range(rows)]
    hist = rng.integers(0, vocab, (rows, 2000)).astype(np.int32)
    sc = []
    counts = []
    for r_ in range(rows):
        t = LS.SamplerScratch(s, vocab)
        t.add_history(torch.from_numpy(hist[r_]).to(dev()))
        sc.append(t)
        counts.append(np.bincount(hist[r_], minlength=vocab).astype(np.uint32))
    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    for trial, k in enumerate((0, 300, 40)):
        kw = [dict(temperature=0.8, top_k=k, top_p=0.9, seed=60 + r_, repetition_penalty=1.1,
                   presence_penalty=0.3, frequency_penalty=0.1) for r_ in range(rows)]
        s.set_path_stats(stats)
        r = run_rows(s, x, kw, [trial] * rows, scratch=sc, allow=masks, bias=bias, logprobs=True)
        s.set_path_stats(None)
        st = stats.cpu().tolist()
            # rows whose mask leaves more ids than the sparse select holds are streamed when k
        # allows (barred ids become -inf as their chunks arrive); the others never are
        assert st[0] == 0 or k == 40, (k, st)
        if slices == 0:
            assert st[2] == 0, st                     # and with several slices never the exhaustive one
        for i in range(rows):
            d = O.sample(x[i], counts[i], o_params(**kw[i]), trial, allow=masks[i], bias=bias[i],
                         want_logprob=True)
            check_row_against_oracle(r, i, d)
            if fracs[i] > 0:
                assert (masks[i][r.ids[i] >> 5] >> (r.ids[i] & 31)) & 1
            _check_logprob(r, i, d, ("mask", fracs[i], k))
        stats.zero_()
    for t in sc:
        t.close()
    s.close()


@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
def test_forced_rows_with_a_log_probability(sampler, bf16):
    """A forced id consumes no draw; its log-probability is that of the full row
    (penalised, biased, masked), whichever select computed the row sum."""
    rng = np.random.default_rng(34 + bf16)
    rows, vocab = 8, 151_936
    x = rng.normal(0, 2, (rows, vocab)).astype(np.float32)
    if bf16:
        x = W.to_bf16_bits(x)
    hist = rng.integers(0, vocab, (rows, 1500)).astype(np.int32)
    forced = [int(hist[r, 0]) if r % 2 else int(rng.integers(0, vocab)) for r in range(rows)]
    forced[5] = None                                  # an ordinary row among them
    masks = np.stack([W.allow_mask(rng, vocab, frac=0.03) for _ in range(rows)])
    for variant in ("plain", "penalised", "masked"):
        for k in (20, 0):
            sc, counts = None, [None] * rows
            pen = dict()
            if variant == "penalised":
                pen = dict(repetition_penalty=1.2, presence_penalty=0.4, frequency_penalty=0.1)
                sc = []
                counts = []
                for r_ in range(rows):
                    t = LS.SamplerScratch(sampler, vocab)
                    t.add_history(torch.from_numpy(hist[r_]).to(dev()))
                    sc.append(t)
                    counts.append(np.bincount(hist[r_], minlength=vocab).astype(np.uint32))
            allow = masks if variant == "masked" else None
            kw = [dict(temperature=0.7, top_k=k, top_p=0.9, seed=80 + r_, **pen) for r_ in range(rows)]
            r = run_rows(sampler, x, kw, [3] * rows, scratch=sc, allow=allow, forced=forced,
                         logprobs=True)
            for i in range(rows):
                ext = dict(want_logprob=True)
                if allow is not None:
                    ext["allow"] = masks[i]
                d = O.sample(x[i], counts[i], o_params(**kw[i]), 3, forced=forced[i], **ext)
                if forced[i] is not None:
                    assert r.ids[i] == forced[i]
                else:
                    check_row_against_oracle(r, i, d)
                _check_logprob(r, i, d, (variant, k))
            if sc is not None:
                for i in range(rows):
                    assert np.array_equal(sc[i].read_counts().numpy().view(np.uint32), counts[i])
                for t in sc:
                    t.close()


@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
def test_log_probability_when_the_largest_value_arrives_late(bf16):
    """The row's largest values sit hundreds of units above everything the first block
    holds (one workgroup per row, as in large batches): the exponents of their terms must
    not be rounded to f32 relative to the first block's reference (that costs 1e-5 of the
    log-probability), and at temperature 0.5 they lie beyond 2^1000 times that reference,
    outside the range of the doubles the sum is kept in."""
    sampler = _sampler_with_slices(1)
    rng = np.random.default_rng(41 + bf16)
    rows, vocab = 6, 151_936
    x = rng.normal(0, 1, (rows, vocab)).astype(np.float32)
    for r_ in range(rows):
        at = vocab - 1 - 37 * r_
        x[r_, at] = 520.0 + 24.0 * r_                # the draw, with most of the mass
        x[r_, at - 5000] = 519.5 + 24.0 * r_         # a close second
    if bf16:
        x = W.to_bf16_bits(x)
    hist = rng.integers(0, vocab, (rows, 300)).astype(np.int32)
    for variant in ("plain", "penalised"):
        sc, counts, pen = None, [None] * rows, dict()
        if variant == "penalised":
            pen = dict(repetition_penalty=1.1, presence_penalty=0.2, frequency_penalty=0.1)
            sc, counts = [], []
            for r_ in range(rows):
                t = LS.SamplerScratch(sampler, vocab)
                t.add_history(torch.from_numpy(hist[r_]).to(dev()))
                sc.append(t)
                counts.append(np.bincount(hist[r_], minlength=vocab).astype(np.uint32))
        for k, temperature in ((20, 1.0), (300, 1.0), (20, 0.5)):
            kw = [dict(temperature=temperature, top_k=k, top_p=1.0, seed=7 + r_, **pen)
                  for r_ in range(rows)]
            r = run_rows(sampler, x, kw, [2] * rows, scratch=sc, logprobs=True)
            for i in range(rows):
                d = O.sample(x[i], counts[i], o_params(**kw[i]), 2, want_logprob=True)
                check_row_against_oracle(r, i, d)
                _check_logprob(r, i, d, ("late maximum", variant, k, temperature))
        if sc is not None:
            for t in sc:
                t.close()
    sampler.close()


def test_penalised_ids_in_the_partial_chunks_of_unaligned_rows(sampler):
    """Rows of odd length start at every 16-byte phase, so their first and last ids lie in
    partial chunks that no select streams.  With those ids penalised and k above 64 the row
    sum must still hold each of them once."""
    rng = np.random.default_rng(43)
    rows, vocab = 9, 4099
    for bf16 in (False, True):
        x = rng.normal(0, 0.02, (rows, vocab)).astype(np.float32)
        if bf16:
            x = W.to_bf16_bits(x)
        # the ids at both ends of the row and a tenth of the others
        hist = np.stack([np.concatenate([np.arange(12), np.arange(vocab - 12, vocab),
                                         rng.choice(np.arange(12, vocab - 12), 400, replace=False)])
                         for _ in range(rows)]).astype(np.int32)
        sc, counts = [], []
        for r_ in range(rows):
            t = LS.SamplerScratch(sampler, vocab)
            t.add_history(torch.from_numpy(hist[r_]).to(dev()))
            sc.append(t)
            counts.append(np.bincount(hist[r_], minlength=vocab).astype(np.uint32))
        for k in (300, 20):
            kw = [dict(temperature=1.0, top_k=k, top_p=1.0, seed=3 + r_, repetition_penalty=1.3,
                       presence_penalty=0.5, frequency_penalty=0.1) for r_ in range(rows)]
            r = run_rows(sampler, x, kw, [5] * rows, scratch=sc, logprobs=True)
            for i in range(rows):
                d = O.sample(x[i], counts[i], o_params(**kw[i]), 5, want_logprob=True)
                check_row_against_oracle(r, i, d)
                _check_logprob(r, i, d, ("edges", bf16, k))
        for t in sc:
            t.close()


@pytest.mark.parametrize("slices", [0, 1], ids=["auto-slices", "one-slice"])
def test_dense_masks_are_streamed(slices):
    """A mask that bars a few hundred ids - among them the row's best ones, as a list of
    banned tokens would - is served by the streaming select: the barred ids are replaced by
    -inf as their chunks arrive.  Penalties and a bias list on top; the row's largest raw
    value is barred, so the row sum must not be measured against it."""
    s = _sampler_with_slices(slices)
    rng = np.random.default_rng(51)
    rows, vocab = 7, 151_936
    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    for bf16 in (False, True):
        x = rng.normal(0, 2, (rows, vocab)).astype(np.float32)
        x[3, 70_000] = 400.0                              # far above everything, and barred
        masks = np.full((rows, (vocab + 31) // 32), 0xFFFFFFFF, np.uint32)
        masks[:, -1] = (1 << (vocab % 32)) - 1 if vocab % 32 else 0xFFFFFFFF
        for r_ in range(rows):
            barred = np.concatenate([np.argsort(x[r_])[::-1][:5 + 3 * r_],          # the best ones
                                     rng.choice(vocab, 300, replace=False),
                                     np.arange(0, 9), np.arange(vocab - 9, vocab)])   # both ends
            for id_ in barred:
                masks[r_, id_ >> 5] &= ~np.uint32(1 << (id_ & 31))
        xs = W.to_bf16_bits(x) if bf16 else x
        bias = [[(int(i), float(d)) for i, d in zip(rng.integers(0, vocab, 20),
                                                     rng.choice([-4.0, 6.0], 20))] for _ in range(rows)]
        hist = rng.integers(0, vocab, (rows, 1500)).astype(np.int32)
        sc, counts = [], []
        for r_ in range(rows):
            t = LS.SamplerScratch(s, vocab)
            t.add_history(torch.from_numpy(hist[r_]).to(dev()))
            sc.append(t)
            counts.append(np.bincount(hist[r_], minlength=vocab).astype(np.uint32))
        for trial, k in enumerate((64, 20)):
            kw = [dict(temperature=0.8, top_k=k, top_p=0.95, seed=90 + r_, repetition_penalty=1.15,
                       presence_penalty=0.3, frequency_penalty=0.1) for r_ in range(rows)]
            stats.zero_()
            s.set_path_stats(stats)
            r = run_rows(s, xs, kw, [trial] * rows, scratch=sc, allow=masks, bias=bias, logprobs=True)
            s.set_path_stats(None)
            st = stats.cpu().tolist()
            assert st[0] == rows * s.slices_for(rows, k, vocab, bf16=bf16) and st[1] == 0 and st[2] == 0, st
            for i in range(rows):
                d = O.sample(xs[i], counts[i], o_params(**kw[i]), trial, allow=masks[i], bias=bias[i],
                             want_logprob=True)
                check_row_against_oracle(r, i, d)
                assert (masks[i][r.ids[i] >> 5] >> (r.ids[i] & 31)) & 1
                _check_logprob(r, i, d, ("dense mask", bf16, k))
        for t in sc:
            t.close()
    s.close()


@pytest.mark.parametrize("use_plan", [False, True], ids=["direct", "plan"])
def test_mixed_batches_run_as_two_launches(sampler, use_plan):
    """A batch of mostly streamable rows with a few that need the other selects (k above
    64, a long bias list) is reordered and launched in two parts; every row still writes its
    own outputs and its own scratch, step after step."""
    rng = np.random.default_rng(61)
    rows, vocab = 150, 30_011
    x = W.to_bf16_bits(rng.normal(0, 2, (rows, vocab)).astype(np.float32))
    ks = rng.choice([20, 64, 300, 0, 1], rows, p=[0.5, 0.3, 0.08, 0.07, 0.05])
    bias = [[(int(i), float(d)) for i, d in zip(rng.integers(0, vocab, 100 if r_ % 17 == 0 else 5),
                                                 rng.choice([-3.0, 4.0], 100 if r_ % 17 == 0 else 5))]
            for r_ in range(rows)]
    hist = rng.integers(0, vocab, (rows, 400)).astype(np.int32)
    sc, counts = [], []
    for r_ in range(rows):
        t = LS.SamplerScratch(sampler, vocab)
        t.add_history(torch.from_numpy(hist[r_]).to(dev()))
        sc.append(t)
        counts.append(np.bincount(hist[r_], minlength=vocab).astype(np.uint32))
    kw = [dict(temperature=0.0 if ks[r_] == 1 else 0.9, top_k=int(ks[r_]), top_p=0.92, seed=300 + r_,
               repetition_penalty=1.1, presence_penalty=0.2, frequency_penalty=0.05)
          for r_ in range(rows)]
    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    for step in range(3):
        stats.zero_()
        sampler.set_path_stats(stats)
        r = run_rows(sampler, x, kw, [step] * rows, scratch=sc, bias=bias, logprobs=True,
                     use_plan=use_plan)
        sampler.set_path_stats(None)
        st = stats.cpu().tolist()
        assert st[0] > 0 and st[1] > 0 and st[2] == 0, st
        for i in range(rows):
            d = O.sample(x[i], counts[i], o_params(**kw[i]), step, bias=bias[i], want_logprob=True)
            check_row_against_oracle(r, i, d)
            _check_logprob(r, i, d, ("mixed", step, int(ks[i])))
        for i in range(0, rows, 11):
            assert np.array_equal(sc[i].read_counts().numpy().view(np.uint32), counts[i]), i
    for t in sc:
        t.close()
