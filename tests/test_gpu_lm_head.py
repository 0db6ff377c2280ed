"""The logits' producer (bf16 head on the matrix cores, with summaries) and the draws from its
summaries (src/qwen4exp/batch.rs:573-593, src/qwen4exp/model.rs:4157-4169).

Bar:
  * logits: each within one bf16 step of hidden @ weight.T computed in f64 from the same bf16
    inputs (the f32 accumulation of 512 products and the rounding to bf16 are what may differ);
  * summaries: tile_max bit-exact against the stored logits, tile_sum within 4e-6 relative of
    the f64 sum over the stored logits (128 terms whose exponents are formed in f32: 1e-6 each at
    the magnitudes of these logits);
  * draws: ids (and the candidate lists) bit-exact against the oracle ON THE STORED LOGITS,
    log-probabilities within 1e-5 * max(1, |logprob|) - the same bar as lily_sample_rows, whose
    results the tiled draws must equal.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import lily_sampler as LS
import lily_workloads as W
import oracle as O
from gpu_util import K_CAP, dev, ls_params, o_params

LOGPROB_RTOL = 1e-5
TILE = LS.LOGIT_TILE_COLS


@pytest.fixture(scope="module")
def sampler():
    s = LS.Sampler(0)
    yield s
    s.close()


def _bf16(x):
    return torch.from_numpy(W.to_bf16_bits(x).view(np.int16)).to(dev()).view(torch.bfloat16)


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _peaked_head(rng, rows, d, vocab, peaks=40, gain=6.0):
    """Hidden states and a head whose logits look like a language model's: a bulk from random
    weights and, per row, a few ids whose weight rows point along the row's hidden state."""
    hidden = rng.normal(0.0, 1.0, (rows, d)).astype(np.float32)
    weight = rng.normal(0.0, 2.0 / np.sqrt(d), (vocab, d)).astype(np.float32)
    for r in range(rows):
        ids = rng.choice(vocab, peaks, replace=False)
        scale = rng.uniform(0.3, 1.0, peaks).astype(np.float32) * gain / d
        weight[ids] += scale[:, None] * hidden[r][None, :]
    return hidden, weight


def _produce(sampler, hidden, weight, temps, rows, vocab, stride=None):
    stride = stride or vocab
    h, w = _bf16(hidden), _bf16(weight)
    buf = torch.full((rows, stride), 7.0, dtype=torch.bfloat16, device=dev())
    logits = buf[:, :vocab]
    tiles = (vocab + TILE - 1) // TILE
    tmax = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    tsum = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    sampler.lm_head(h, w, temps, logits, tmax, tsum)
    sampler.synchronize()
    return h, w, buf, logits, tmax, tsum


def _check_product(h, w, logits, tmax, tsum, temps):
    rows, vocab = logits.shape
    got = W.bf16_bits_to_f32(_bits(logits.contiguous()))
    ref = (h.double() @ w.double().T).cpu().numpy()
    # one bf16 step at the reference's magnitude (2^-8 relative is half a step), plus the f32
    # accumulation's error on sums that cancel
    tol = np.abs(ref) * 2.0 ** -7 + 1e-4
    assert np.all(np.abs(got - ref) <= tol), float(np.max(np.abs(got - ref) - tol))
    tiles = tmax.shape[1]
    pad = tiles * TILE - vocab
    g = np.pad(got, ((0, 0), (0, pad)), constant_values=-np.inf).reshape(rows, tiles, TILE)
    assert np.array_equal(tmax.cpu().numpy(), g.max(axis=2))
    for r in range(rows):
        t = temps[r] if temps is not None else 0.0
        if not t > 0.0:
            continue
        c2 = np.float32(1.4426950408889634 / t)
        top = (g[r].max(axis=1).astype(np.float32) * c2).astype(np.float64)
        want = np.exp2(g[r].astype(np.float64) * np.float64(c2) - top[:, None]).sum(axis=1)
        assert np.allclose(tsum[r].cpu().numpy(), want, rtol=4e-6, atol=0), r


@pytest.mark.parametrize("rows,d,vocab,slack", [(5, 256, 1000, 8), (130, 512, 4096 + 77, 8), (1, 64, 128, 8),
                                                (300, 128, 2000 + 3, 8), (37, 192, 777, 3),
                                                (65, 256, 1500, 8), (96, 320, 2048 + 5, 3), (128, 128, 3000, 8),
                                                (2049 + 130, 64, 300, 8)])
def test_producer_against_f64_product(sampler, rows, d, vocab, slack):
    """Every tile shape of the launcher: up to 32 rows, up to 64, 65 to 128 (three cases), more
    (256-row tiles), and more than 2 048 rows (more blocks of hidden rows than XCDs: the other
    branch of the tile numbering).  slack 8: rows of the logits start at multiples of 16 bytes;
    slack 3: they start at any even address (every value is stored by a 2-byte store)."""
    rng = np.random.default_rng(rows * 1000 + d)
    hidden, weight = _peaked_head(rng, rows, d, vocab, peaks=min(20, vocab // 8))
    temps = [0.0 if r % 5 == 4 else 0.5 + 0.1 * (r % 7) for r in range(rows)]
    stride = ((vocab + 7) // 8) * 8 + slack
    h, w, buf, logits, tmax, tsum = _produce(sampler, hidden, weight, temps, rows, vocab, stride)
    _check_product(h, w, logits, tmax, tsum, temps)
    # nothing behind a row's last column is written
    assert torch.all(buf[:, vocab:] == 7.0)


def _draw_all(sampler, fn, logits, params_kw, steps, scratch=None, **kw):
    rows = logits.shape[0]
    out = torch.full((rows,), -1, dtype=torch.int32, device=dev())
    lp = torch.full((rows,), 123.0, dtype=torch.float32, device=dev())
    dbg_ids = torch.full((rows, K_CAP), -1, dtype=torch.int32, device=dev())
    dbg_counts = torch.zeros((rows, 2), dtype=torch.int32, device=dev())
    keep = fn(out, lp, dbg_ids, dbg_counts)
    sampler.synchronize()
    del keep
    return (out.cpu().numpy().astype(np.int64), lp.cpu().numpy(), dbg_ids.cpu().numpy(),
            dbg_counts.cpu().numpy())


def _check_draws(stored, ids, lps, cand, counts, params_kw, steps, hist_counts=None, forced=None):
    for r, kw in enumerate(params_kw):
        if forced is not None and forced[r] is not None:
            assert ids[r] == forced[r], r
            continue
        p = o_params(**kw)
        if p.temperature == 0.0:
            assert ids[r] == O.argmax(stored[r]), r
            continue
        c = None if hist_counts is None or hist_counts[r] is None else hist_counts[r].copy()
        d = O.sample(stored[r], c, p, steps[r], want_logprob=True)
        n_fin = int(np.sum(d.cand_adj > -np.inf))
        assert counts[r, 0] == n_fin, (r, counts[r, 0], n_fin)
        assert np.array_equal(cand[r, :n_fin], d.cand_ids[:n_fin].astype(np.int64)), r
        assert counts[r, 1] == d.n_kept, r
        assert ids[r] == d.chosen, (r, ids[r], d.chosen)
        assert abs(lps[r] - d.logprob) <= LOGPROB_RTOL * max(1.0, abs(d.logprob)), (r, lps[r], d.logprob)


def _mixed_params(rows):
    out = []
    for r in range(rows):
        if r % 6 == 5:
            out.append(dict())   # greedy
        elif r % 6 == 4:
            out.append(dict(temperature=0.9, top_k=200, top_p=0.95, seed=900 + r))   # k beyond the summaries' reach
        else:
            out.append(dict(temperature=0.6 + 0.1 * (r % 4), top_k=(1, 20, 64, 40)[r % 4],
                            top_p=(1.0, 0.9, 0.95, 0.8)[r % 4], min_p=0.02 * (r % 3), seed=700 + r))
    return out


@pytest.mark.parametrize("rows,d,vocab", [(24, 256, 151_936), (9, 128, 5000), (3, 64, 333)])
def test_tiled_draws_equal_the_oracle_on_the_stored_logits(sampler, rows, d, vocab):
    rng = np.random.default_rng(vocab + rows)
    hidden, weight = _peaked_head(rng, rows, d, vocab, peaks=min(60, vocab // 6))
    params_kw = _mixed_params(rows)
    params = [ls_params(**kw) for kw in params_kw]
    temps = [p.effective()[0] for p in params]
    steps = [3 + r for r in range(rows)]
    h, w, buf, logits, tmax, tsum = _produce(sampler, hidden, weight, temps, rows, vocab,
                                             ((vocab + 7) // 8) * 8)
    stored = _bits(logits.contiguous())
    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    sampler.set_path_stats(stats)
    ids, lps, cand, counts = _draw_all(
        sampler, lambda out, lp, di, dc: sampler.sample_rows_tiled(
            logits, tmax, tsum, params, steps, out, out_logprobs=lp, dbg_ids=di, dbg_counts=dc),
        logits, params_kw, steps)
    sampler.set_path_stats(None)
    _check_draws(stored, ids, lps, cand, counts, params_kw, steps)
    if vocab > 100_000:   # (with fewer summaries than k every value is a candidate: too many)
        assert stats.cpu().numpy()[2] == 0, "no row fell back to the exhaustive select"
    # and the ordinary call on the same logits gives the same
    ids2, lps2, cand2, counts2 = _draw_all(
        sampler, lambda out, lp, di, dc: sampler.sample_rows(
            logits, params, steps, out, out_logprobs=lp, dbg_ids=di, dbg_counts=dc),
        logits, params_kw, steps)
    assert np.array_equal(ids, ids2)
    sampled = [r for r, kw in enumerate(params_kw) if kw]
    assert np.allclose(lps[sampled], lps2[sampled], rtol=LOGPROB_RTOL, atol=LOGPROB_RTOL)


def test_fused_call_with_rows_the_summaries_do_not_serve(sampler):
    """One call: product, then every row's draw - plain rows from the summaries, rows under
    penalties, masks, bias lists or a forced token by the selects that read the row."""
    rows, d, vocab = 40, 256, 20_000
    rng = np.random.default_rng(77)
    hidden, weight = _peaked_head(rng, rows, d, vocab)
    params_kw, hist, forced = [], [], []
    for r in range(rows):
        kw = dict(temperature=0.7 + 0.05 * (r % 5), top_k=(20, 64, 50)[r % 3], top_p=0.92, seed=100 + r)
        if r % 4 == 1:
            kw.update(repetition_penalty=1.1, presence_penalty=0.3, frequency_penalty=0.1)
        if r % 10 == 7:
            kw = dict()
        params_kw.append(kw)
        hist.append(rng.integers(0, vocab, 300).astype(np.int32) if r % 4 == 1 else None)
        forced.append(int(rng.integers(0, vocab)) if r % 8 == 6 else None)
    params = [ls_params(**kw) for kw in params_kw]
    steps = [11] * rows
    scratch, hist_counts = [], []
    for hh in hist:
        if hh is None:
            scratch.append(None)
            hist_counts.append(None)
        else:
            sc = LS.SamplerScratch(sampler, vocab)
            sc.add_history(torch.from_numpy(hh).to(dev()))
            scratch.append(sc)
            hist_counts.append(np.bincount(hh, minlength=vocab).astype(np.uint32))
    h, w = _bf16(hidden), _bf16(weight)
    logits = torch.zeros(rows, vocab, dtype=torch.bfloat16, device=dev())
    tiles = (vocab + TILE - 1) // TILE
    tmax = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    tsum = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    ids, lps, cand, counts = _draw_all(
        sampler, lambda out, lp, di, dc: sampler.lm_head_sample_rows(
            h, w, logits, tmax, tsum, params, steps, out, scratch=scratch, forced=forced,
            out_logprobs=lp, dbg_ids=di, dbg_counts=dc),
        logits, params_kw, steps)
    temps = [p.effective()[0] for p in params]
    _check_product(h, w, logits, tmax, tsum, temps)
    stored = _bits(logits)
    _check_draws(stored, ids, lps, cand, counts, params_kw, steps, hist_counts=hist_counts, forced=forced)
    # forced rows with a log-probability: that of the forced id under the row's own settings
    for r in range(rows):
        if forced[r] is not None and params_kw[r]:
            d = O.sample(stored[r], None if hist_counts[r] is None else hist_counts[r].copy(),
                         o_params(**params_kw[r]), steps[r], want_logprob=True, forced=forced[r])
            assert abs(lps[r] - d.logprob) <= LOGPROB_RTOL * max(1.0, abs(d.logprob)), r


def test_ties_by_the_thousand_take_the_exhaustive_select(sampler):
    """Constant logits: every value ties at the bound, the candidates overflow the buffer and the
    select that reads the whole row decides - ids still the oracle's."""
    rows, vocab = 3, 6000
    x = np.zeros((rows, vocab), dtype=np.float32)
    x[1, 4000:] = -1.0
    x[2, ::2] = 0.5
    bits = W.to_bf16_bits(x)
    logits = torch.from_numpy(bits.view(np.int16)).to(dev()).view(torch.bfloat16)
    tiles = (vocab + TILE - 1) // TILE
    g = np.pad(x, ((0, 0), (0, tiles * TILE - vocab)), constant_values=-np.inf).reshape(rows, tiles, TILE)
    params_kw = [dict(temperature=1.0, top_k=50, top_p=1.0, seed=5 + r) for r in range(rows)]
    c2 = np.float32(1.4426950408889634)
    tmax_np = g.max(axis=2).astype(np.float32)
    tsum_np = np.exp2(g.astype(np.float64) * c2 - (tmax_np * c2).astype(np.float64)[:, :, None]).sum(axis=2)
    tmax = torch.from_numpy(tmax_np).to(dev())
    tsum = torch.from_numpy(tsum_np.astype(np.float32)).to(dev())
    params = [ls_params(**kw) for kw in params_kw]
    steps = [0, 1, 2]
    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    sampler.set_path_stats(stats)
    ids, lps, cand, counts = _draw_all(
        sampler, lambda out, lp, di, dc: sampler.sample_rows_tiled(
            logits, tmax, tsum, params, steps, out, out_logprobs=lp, dbg_ids=di, dbg_counts=dc),
        logits, params_kw, steps)
    sampler.set_path_stats(None)
    _check_draws(bits, ids, lps, cand, counts, params_kw, steps)
    assert stats.cpu().numpy()[2] >= 1


def test_rejections(sampler):
    rows, d, vocab = 2, 64, 256
    h = torch.zeros(rows, d, dtype=torch.bfloat16, device=dev())
    w = torch.zeros(vocab, d, dtype=torch.bfloat16, device=dev())
    logits = torch.zeros(rows, vocab, dtype=torch.bfloat16, device=dev())
    tmax = torch.zeros(rows, 2, dtype=torch.float32, device=dev())
    tsum = torch.zeros(rows, 2, dtype=torch.float32, device=dev())
    with pytest.raises(LS.SamplerError):
        sampler.lm_head(h[:, :32], w[:, :32], None, logits, tmax, tsum)     # d not a multiple of 64
    f32 = torch.zeros(rows, vocab, dtype=torch.float32, device=dev())
    out = torch.zeros(rows, dtype=torch.int32, device=dev())
    with pytest.raises(LS.SamplerError):
        sampler.sample_rows_tiled(f32[:, 1:], tmax, tsum, [ls_params()] * rows, [0, 0], out)   # rows off 16-byte boundaries
    sampler.synchronize()


def test_rows_under_lowering_penalties_are_drawn_from_summaries(sampler):
    """Rows whose penalties can only lower a value (repetition >= 1, presence and frequency
    >= 0) are served from the summaries too: a wider set of tiles is read, listed ids are
    evaluated with their counts, and the tiles that matter to the row's sum are summed element
    by element.  Three decode steps on the same logits, the counts moving with the draws; rows
    whose penalties may raise a value go through the selects that read the row."""
    rows, d, vocab = 12, 256, 151_936
    rng = np.random.default_rng(404)
    hidden, weight = _peaked_head(rng, rows, d, vocab, peaks=60, gain=9.0)
    params_kw = []
    for r in range(rows):
        kw = dict(temperature=0.8, top_k=(64, 20, 5)[r % 3], top_p=0.9, seed=5000 + r,
                  repetition_penalty=1.1, presence_penalty=0.2, frequency_penalty=0.1)
        if r == 7:
            kw.update(repetition_penalty=0.9)        # may raise: not served from summaries
        if r == 9:
            kw.update(presence_penalty=-0.5)         # may raise
        params_kw.append(kw)
    params = [ls_params(**kw) for kw in params_kw]
    temps = [p.effective()[0] for p in params]
    h, w, buf, logits, tmax, tsum = _produce(sampler, hidden, weight, temps, rows, vocab)
    stored = _bits(logits.contiguous())
    stored_f = W.bf16_bits_to_f32(stored)
    # histories that hold the rows' best ids (what a model that repeats itself has emitted)
    scratch, hist_counts = [], []
    for r in range(rows):
        best = np.argsort(-stored_f[r])[:30].astype(np.int32)
        hh = np.concatenate([rng.integers(0, vocab, 2000).astype(np.int32), np.repeat(best[:10], 3), best])
        sc = LS.SamplerScratch(sampler, vocab)
        sc.add_history(torch.from_numpy(hh).to(dev()))
        scratch.append(sc)
        hist_counts.append(np.bincount(hh, minlength=vocab).astype(np.uint32))
    for step in range(3):
        steps = [step] * rows
        stats = torch.zeros(4, dtype=torch.int32, device=dev())
        sampler.set_path_stats(stats)
        ids, lps, cand, counts = _draw_all(
            sampler, lambda out, lp, di, dc: sampler.sample_rows_tiled(
                logits, tmax, tsum, params, steps, out, scratch=scratch, out_logprobs=lp, dbg_ids=di,
                dbg_counts=dc),
            logits, params_kw, steps)
        sampler.set_path_stats(None)
        assert stats.cpu().numpy()[2] == 0, "no row fell back to the exhaustive select"
        for r, kw in enumerate(params_kw):
            dd = O.sample(stored[r], hist_counts[r], o_params(**kw), step, want_logprob=True)   # bumps the counts
            n_fin = int(np.sum(dd.cand_adj > -np.inf))
            assert counts[r, 0] == n_fin, (step, r)
            assert np.array_equal(cand[r, :n_fin], dd.cand_ids[:n_fin].astype(np.int64)), (step, r)
            assert counts[r, 1] == dd.n_kept and ids[r] == dd.chosen, (step, r)
            assert abs(lps[r] - dd.logprob) <= LOGPROB_RTOL * max(1.0, abs(dd.logprob)), (step, r, lps[r], dd.logprob)
    for r in range(rows):
        assert np.array_equal(scratch[r].read_counts().numpy().view(np.uint32), hist_counts[r]), r
        scratch[r].close()


def _bias_lists(rng, stored_f, vocab):
    """Bias lists of the kinds that matter to a draw from summaries: the row's best ids barred
    (their tiles' summaries then overstate what the tiles hold), an id far down the row raised
    to the top (its tile's summary says nothing of it), many small shifts, pairs of one id that
    add up in list order, an id next to the row's best in the same tile, a full list of 64."""
    rows = stored_f.shape[0]
    out = []
    for r in range(rows):
        order = np.argsort(-stored_f[r])
        kind = r % 5
        if kind == 0:
            low = int(order[vocab // 2 + r])
            b = [(int(i), -100.0) for i in order[:3]] + [(low, 60.0)]
        elif kind == 1:
            ids = rng.integers(0, vocab, 40)
            b = [(int(i), float(d)) for i, d in zip(ids, rng.normal(0, 3.0, 40))]
            b += [b[0], b[0], (int(order[1]), 0.75), (int(order[1]), -0.25)]
        elif kind == 2:
            top = int(order[0])
            near = top + 1 if (top + 1) // TILE == top // TILE and top + 1 < vocab else top - 1
            b = [(int(i), -1.0e4) for i in order[:10]] + [(near, 25.0)]
        elif kind == 3:
            ids = np.concatenate([order[:20], rng.integers(0, vocab, 44)])
            b = [(int(i), float(d)) for i, d in zip(ids, rng.normal(0, 6.0, 64))]
        else:
            b = [(int(order[5]), float("-inf")), (int(order[40 + r]), 3.5)]
        out.append(b)
    return out


@pytest.mark.parametrize("f32", [False, True])
def test_rows_with_bias_lists_are_drawn_from_summaries(sampler, f32):
    """A bias list of up to 64 pairs (logit += delta before the mask and the penalties, pairs of
    one id adding up in list order) on rows drawn from the summaries: the tiles that hold a
    biased id are read whatever their summaries say, and the bound counts on as many tiles more
    as there are pairs.  Rows without penalties are all served by the kernel that reads
    summaries (one workgroup a row, where the ordinary launch cuts so few rows into slices);
    rows under lowering penalties with a history of their best ids likewise unless that kernel
    declines them; a greedy row and a forced row with a bias list go the ordinary way.  Ids,
    candidates, kept counts and log-probabilities are the oracle's on the stored logits."""
    rows, d, vocab = 15, 256, (151_936 if not f32 else 20_000)
    rng = np.random.default_rng(77 + int(f32))
    hidden, weight = _peaked_head(rng, rows, d, vocab, peaks=60, gain=9.0)
    params_kw = [dict(temperature=0.7 + 0.05 * (r % 3), top_k=(64, 20, 5, 1 + r)[r % 4], top_p=(0.9, 1.0)[r % 2],
                      min_p=0.01 * (r % 2), seed=900 + r) for r in range(rows)]
    params = [ls_params(**kw) for kw in params_kw]
    temps = [p.effective()[0] for p in params]
    h, w = _bf16(hidden), _bf16(weight)
    tiles = (vocab + TILE - 1) // TILE
    logits = torch.zeros(rows, vocab, dtype=torch.float32 if f32 else torch.bfloat16, device=dev())
    tmax = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    tsum = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    sampler.lm_head(h, w, temps, logits, tmax, tsum)
    sampler.synchronize()
    stored = logits.cpu().numpy() if f32 else _bits(logits.contiguous())
    stored_f = stored if f32 else W.bf16_bits_to_f32(stored)
    bias = _bias_lists(rng, stored_f, vocab)
    steps = [3 + r for r in range(rows)]

    def check(ids, lps, cand, counts, kws, hist=None, forced=None):
        for r, kw in enumerate(kws):
            if forced is not None and forced[r] is not None:
                assert ids[r] == forced[r], r
                continue
            c = None if hist is None else hist[r]
            dd = O.sample(stored[r], c, o_params(**kw), steps[r], bias=bias[r], want_logprob=True)
            if o_params(**kw).temperature == 0.0:
                assert ids[r] == dd.chosen, r
                continue
            n_fin = int(np.sum(dd.cand_adj > -np.inf))
            assert counts[r, 0] == n_fin, (r, counts[r, 0], n_fin)
            assert np.array_equal(cand[r, :n_fin], dd.cand_ids[:n_fin].astype(np.int64)), r
            assert counts[r, 1] == dd.n_kept and ids[r] == dd.chosen, (r, ids[r], dd.chosen)
            assert abs(lps[r] - dd.logprob) <= LOGPROB_RTOL * max(1.0, abs(dd.logprob)), (r, lps[r], dd.logprob)

    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    sampler.set_path_stats(stats)
    ids, lps, cand, counts = _draw_all(
        sampler, lambda out, lp, di, dc: sampler.sample_rows_tiled(
            logits, tmax, tsum, params, steps, out, bias=bias, out_logprobs=lp, dbg_ids=di, dbg_counts=dc),
        logits, params_kw, steps)
    sampler.set_path_stats(None)
    check(ids, lps, cand, counts, params_kw)
    st = stats.cpu().numpy()
    assert st[0] == rows and st[1] == 0 and st[2] == 0, st.tolist()
    # the same lists under lowering penalties, with histories that hold the rows' best ids
    pen_kw = [dict(kw, repetition_penalty=1.1, presence_penalty=0.2, frequency_penalty=0.1) for kw in params_kw]
    pen = [ls_params(**kw) for kw in pen_kw]
    scratch, hist = [], []
    for r in range(rows):
        best = np.argsort(-stored_f[r])[:30].astype(np.int32)
        hh = np.concatenate([rng.integers(0, vocab, 1500).astype(np.int32), np.repeat(best[:8], 3), best])
        sc = LS.SamplerScratch(sampler, vocab)
        sc.add_history(torch.from_numpy(hh).to(dev()))
        scratch.append(sc)
        hist.append(np.bincount(hh, minlength=vocab).astype(np.uint32))
    ids, lps, cand, counts = _draw_all(
        sampler, lambda out, lp, di, dc: sampler.sample_rows_tiled(
            logits, tmax, tsum, pen, steps, out, scratch=scratch, bias=bias, out_logprobs=lp, dbg_ids=di,
            dbg_counts=dc),
        logits, pen_kw, steps)
    check(ids, lps, cand, counts, pen_kw, hist=hist)
    for r in range(rows):
        assert np.array_equal(scratch[r].read_counts().numpy().view(np.uint32), hist[r]), r
        scratch[r].close()
    # a greedy row and a forced row with a bias list (served by the kernels that read the row)
    odd_kw = [dict() if r % 2 else kw for r, kw in enumerate(params_kw)]
    odd = [ls_params(**kw) for kw in odd_kw]
    forced = [int(np.argsort(-stored_f[r])[2]) if r % 4 == 0 else None for r in range(rows)]
    ids, lps, cand, counts = _draw_all(
        sampler, lambda out, lp, di, dc: sampler.sample_rows_tiled(
            logits, tmax, tsum, odd, steps, out, bias=bias, forced=forced, out_logprobs=lp, dbg_ids=di,
            dbg_counts=dc),
        logits, odd_kw, steps)
    check(ids, lps, cand, counts, odd_kw, forced=forced)


def _masks(rng, stored_f, vocab):
    """Allow-masks (packed u32, bit id & 31 of word id >> 5) of the kinds that matter to a draw
    from summaries: a handful of barred ids among the row's best (their tiles are allowed in
    part), a barred run of ids that holds the row's best tile and its neighbours (tiles that
    drop out altogether), everything allowed, one id in thirty barred at random (every tile
    allowed in part), and a sparse mask (a fiftieth of the ids, in runs)."""
    rows = stored_f.shape[0]
    words = (vocab + 31) // 32
    out = np.zeros((rows, words), dtype=np.uint32)
    kinds = []
    for r in range(rows):
        order = np.argsort(-stored_f[r])
        allowed = np.ones(vocab, dtype=bool)
        kind = r % 5
        if kind == 0:
            allowed[order[[0, 2, 3, 7, 11]]] = False
        elif kind == 1:
            t = int(order[0]) // TILE
            allowed[max(0, (t - 1) * TILE + 5):min(vocab, (t + 2) * TILE - 9)] = False
            allowed[order[1]] = False
        elif kind == 2:
            pass
        elif kind == 3:
            allowed[rng.random(vocab) < 1.0 / 30.0] = False
        else:
            out[r] = W.allow_mask(rng, vocab, frac=0.02)
            kinds.append(kind)
            continue
        bits = np.zeros(words * 32, dtype=bool)
        bits[:vocab] = allowed
        out[r] = np.packbits(bits.reshape(words, 32), axis=1, bitorder="little").view(np.uint32).reshape(words)
        kinds.append(kind)
    return out, kinds


@pytest.mark.parametrize("f32", [False, True])
def test_rows_with_allow_masks_are_drawn_from_summaries(sampler, f32):
    """An allow-mask on rows drawn from the summaries.  Tiles that the mask bars altogether drop
    out, tiles allowed in part are evaluated id by id; the bound is a guess that the row checks
    (k allowed values at or above it), and a row that fails the check, or has too many partly
    allowed tiles to sum, is drawn by the launch that follows.  Whichever way a row goes, ids,
    candidates, kept counts and log-probabilities are the oracle's on the stored logits; the
    rows with a handful of barred ids, a barred run and no barred id are all served by the kernel
    that reads summaries.  Then the same with bias lists and lowering penalties on top."""
    rows, d, vocab = 15, 256, (151_936 if not f32 else 20_000 + 24)
    rng = np.random.default_rng(131 + int(f32))
    hidden, weight = _peaked_head(rng, rows, d, vocab, peaks=60, gain=9.0)
    params_kw = [dict(temperature=0.7 + 0.05 * (r % 3), top_k=(64, 20, 5, 1 + r)[r % 4], top_p=(0.9, 1.0)[r % 2],
                      min_p=0.01 * (r % 2), seed=300 + r) for r in range(rows)]
    params = [ls_params(**kw) for kw in params_kw]
    temps = [p.effective()[0] for p in params]
    h, w = _bf16(hidden), _bf16(weight)
    tiles = (vocab + TILE - 1) // TILE
    logits = torch.zeros(rows, vocab, dtype=torch.float32 if f32 else torch.bfloat16, device=dev())
    tmax = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    tsum = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    sampler.lm_head(h, w, temps, logits, tmax, tsum)
    sampler.synchronize()
    stored = logits.cpu().numpy() if f32 else _bits(logits.contiguous())
    stored_f = stored if f32 else W.bf16_bits_to_f32(stored)
    masks, kinds = _masks(rng, stored_f, vocab)
    allow_t = torch.from_numpy(masks.view(np.int32)).to(dev())
    steps = [9 + r for r in range(rows)]

    def check(ids, lps, cand, counts, kws, which, hist=None, bias=None):
        for i, r in enumerate(which):
            kw = kws[r]
            c = None if hist is None else hist[r]
            dd = O.sample(stored[r], c, o_params(**kw), steps[r], allow=masks[r],
                          bias=None if bias is None else bias[r], want_logprob=True)
            n_fin = int(np.sum(dd.cand_adj > -np.inf))
            assert counts[i, 0] == n_fin, (r, counts[i, 0], n_fin)
            assert np.array_equal(cand[i, :n_fin], dd.cand_ids[:n_fin].astype(np.int64)), r
            assert counts[i, 1] == dd.n_kept and ids[i] == dd.chosen, (r, ids[i], dd.chosen)
            assert abs(lps[i] - dd.logprob) <= LOGPROB_RTOL * max(1.0, abs(dd.logprob)), (r, lps[i], dd.logprob)

    def run(which, pp, kws, **extra):
        sel = torch.tensor(which, device=dev())
        lg, tm, ts = logits[sel].contiguous(), tmax[sel].contiguous(), tsum[sel].contiguous()
        st = [steps[r] for r in which]
        for key in ("scratch", "bias"):
            if extra.get(key) is not None:
                extra[key] = [extra[key][r] for r in which]
        return _draw_all(
            sampler, lambda out, lp, di, dc: sampler.sample_rows_tiled(
                lg, tm, ts, [pp[r] for r in which], st, out, allow=allow_t[sel].contiguous(), out_logprobs=lp,
                dbg_ids=di, dbg_counts=dc, **extra),
            lg, [kws[r] for r in which], st)

    everyone = list(range(rows))
    check(*run(everyone, params, params_kw), params_kw, everyone)
    light = [r for r in everyone if kinds[r] in (0, 1, 2)]
    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    sampler.set_path_stats(stats)
    res = run(light, params, params_kw)
    sampler.set_path_stats(None)
    check(*res, params_kw, light)
    st = stats.cpu().numpy()
    assert st[0] == len(light) and st[1] == 0 and st[2] == 0, st.tolist()
    # bias lists and lowering penalties on top
    bias = _bias_lists(rng, stored_f, vocab)
    pen_kw = [dict(kw, repetition_penalty=1.1, presence_penalty=0.2, frequency_penalty=0.1) for kw in params_kw]
    pen = [ls_params(**kw) for kw in pen_kw]
    scratch, hist = [], []
    for r in range(rows):
        best = np.argsort(-stored_f[r])[:30].astype(np.int32)
        hh = np.concatenate([rng.integers(0, vocab, 1500).astype(np.int32), np.repeat(best[:8], 3), best])
        sc = LS.SamplerScratch(sampler, vocab)
        sc.add_history(torch.from_numpy(hh).to(dev()))
        scratch.append(sc)
        hist.append(np.bincount(hh, minlength=vocab).astype(np.uint32))
    check(*run(everyone, pen, pen_kw, scratch=scratch, bias=bias), pen_kw, everyone, hist=hist, bias=bias)
    for r in range(rows):
        assert np.array_equal(scratch[r].read_counts().numpy().view(np.uint32), hist[r]), r
        scratch[r].close()


def test_a_batch_of_penalised_rows_through_the_fused_call(sampler):
    """1 024 rows under config 5's draw settings (k 64, top-p 0.9, T 0.8, penalties that only
    lower, a 2 048-id history that holds the row's best ids, a log-probability) through the one
    call that runs the head and draws every row: ids, kept counts and log-probabilities against
    the oracle on the stored logits, the counts as the oracle leaves them.  Most rows are drawn
    from the summaries, the rest from their logits by the same call."""
    rows, d, vocab = 1024, 128, 40_000 + 72   # (rows of whole 16 bytes, a last tile of 8 columns)
    rng = np.random.default_rng(1024)
    hidden, weight = _peaked_head(rng, rows, d, vocab, peaks=50, gain=8.0)
    params_kw = [dict(temperature=0.8, top_k=64, top_p=0.9, seed=7000 + r, repetition_penalty=1.1,
                      presence_penalty=0.2, frequency_penalty=0.1) for r in range(rows)]
    params = [ls_params(**kw) for kw in params_kw]
    h, w = _bf16(hidden), _bf16(weight)
    tiles = (vocab + TILE - 1) // TILE
    logits = torch.zeros(rows, vocab, dtype=torch.bfloat16, device=dev())
    tmax = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    tsum = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    # the histories need the rows' best ids: a first pass of the producer alone
    sampler.lm_head(h, w, [0.8] * rows, logits, tmax, tsum)
    sampler.synchronize()
    stored = _bits(logits.contiguous())
    best = torch.topk(logits.float(), 12, dim=1).indices.cpu().numpy().astype(np.int32)
    scratch, hist_counts = [], []
    for r in range(rows):
        hh = np.concatenate([rng.integers(0, vocab, 2036).astype(np.int32), best[r]])
        sc = LS.SamplerScratch(sampler, vocab)
        sc.add_history(torch.from_numpy(hh).to(dev()))
        scratch.append(sc)
        hist_counts.append(np.bincount(hh, minlength=vocab).astype(np.uint32))
    steps = [2] * rows
    out = torch.full((rows,), -1, dtype=torch.int32, device=dev())
    lp = torch.zeros(rows, dtype=torch.float32, device=dev())
    dbg_counts = torch.zeros(rows, 2, dtype=torch.int32, device=dev())
    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    sampler.set_path_stats(stats)
    sampler.lm_head_sample_rows(h, w, logits, tmax, tsum, params, steps, out, scratch=scratch,
                                out_logprobs=lp, dbg_counts=dbg_counts)
    sampler.synchronize()
    sampler.set_path_stats(None)
    assert np.array_equal(_bits(logits.contiguous()), stored), "the same head, the same logits"
    assert stats.cpu().numpy()[2] == 0, "no row fell back to the exhaustive select"
    ids, lps, kept = out.cpu().numpy().astype(np.int64), lp.cpu().numpy(), dbg_counts.cpu().numpy()
    for r in range(rows):
        dd = O.sample(stored[r], hist_counts[r], o_params(**params_kw[r]), steps[r], want_logprob=True)
        assert ids[r] == dd.chosen and kept[r, 1] == dd.n_kept, (r, ids[r], dd.chosen, kept[r], dd.n_kept)
        assert abs(lps[r] - dd.logprob) <= LOGPROB_RTOL * max(1.0, abs(dd.logprob)), (r, lps[r], dd.logprob)
    for r in (0, 1, 511, 1023):
        assert np.array_equal(scratch[r].read_counts().numpy().view(np.uint32), hist_counts[r]), r
    for sc in scratch:
        sc.close()


def test_the_benchmarked_shape(sampler):
    """1 024 rows x 151 936 ids over d = 4 096, the shape bench.py times: a seeded subset of tiles
    against the f64 product of the same bf16 operands (logits within one bf16 step, tile_max
    exact on the stored logits, tile_sum within 4e-6), and the draws of 24 rows - through the one
    call that runs the head and draws every row - against the oracle on the stored logits."""
    rows, d, vocab = 1024, 4096, 151_936
    gen = torch.Generator(device=dev())
    gen.manual_seed(2024)
    w_f32 = torch.randn(vocab, d, device=dev(), generator=gen) * (2.0 / d ** 0.5)
    hid = torch.randn(rows, d, device=dev(), generator=gen)
    for r in range(24):   # peaks, so that the checked rows have candidates worth drawing
        ids = torch.randint(0, vocab, (40,), device=dev(), generator=gen)
        gain = (torch.rand(40, 1, device=dev(), generator=gen) * 0.7 + 0.3) * (6.0 / d)
        w_f32[ids] += gain * hid[r][None, :]
    hb, wb = hid.to(torch.bfloat16), w_f32.to(torch.bfloat16)
    del w_f32, hid
    tiles = (vocab + TILE - 1) // TILE
    logits = torch.zeros(rows, vocab, dtype=torch.bfloat16, device=dev())
    tmax = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    tsum = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    params_kw = [dict(temperature=0.8, top_k=64, top_p=0.9, seed=5000 + r) for r in range(rows)]
    params = [ls_params(**kw) for kw in params_kw]
    steps = [4] * rows
    out = torch.full((rows,), -1, dtype=torch.int32, device=dev())
    lp = torch.zeros(rows, dtype=torch.float32, device=dev())
    sampler.lm_head_sample_rows(hb, wb, logits, tmax, tsum, params, steps, out, out_logprobs=lp)
    sampler.synchronize()
    # ---- a seeded subset of tiles: the first, the last (ragged: 151 936 = 1 187 x 128) and 30 others
    rng = np.random.default_rng(99)
    pick = np.unique(np.concatenate([[0, tiles - 1], rng.integers(0, tiles, 30)]))
    c2 = np.float32(1.4426950408889634 / 0.8)
    for t in pick:
        lo, hi = int(t) * TILE, min((int(t) + 1) * TILE, vocab)
        ref = (hb.double() @ wb[lo:hi].double().T).cpu().numpy()
        got = W.bf16_bits_to_f32(_bits(logits[:, lo:hi].contiguous()))
        tol = np.abs(ref) * 2.0 ** -7 + 1e-4
        assert np.all(np.abs(got - ref) <= tol), (int(t), float(np.max(np.abs(got - ref) - tol)))
        assert np.array_equal(tmax[:, int(t)].cpu().numpy(), got.max(axis=1)), int(t)
        top = (got.max(axis=1).astype(np.float32) * c2).astype(np.float64)
        want = np.exp2(got.astype(np.float64) * np.float64(c2) - top[:, None]).sum(axis=1)
        assert np.allclose(tsum[:, int(t)].cpu().numpy(), want, rtol=4e-6, atol=0), int(t)
    # ---- the draws of 24 rows against the oracle on what was stored
    ids, lps = out.cpu().numpy().astype(np.int64), lp.cpu().numpy()
    assert ids.min() >= 0 and ids.max() < vocab
    stored = _bits(logits[:24].contiguous())
    for r in range(24):
        dd = O.sample(stored[r], None, o_params(**params_kw[r]), steps[r], want_logprob=True)
        assert ids[r] == dd.chosen, (r, ids[r], dd.chosen)
        assert abs(lps[r] - dd.logprob) <= LOGPROB_RTOL * max(1.0, abs(dd.logprob)), (r, lps[r], dd.logprob)


def test_sums_formed_at_another_temperature_are_not_used(sampler):
    """The producer ran with other temperatures than the rows are drawn at (or with none): the
    sums of the summaries would give a wrong log-probability beside the right token, so rows that
    ask for one are drawn from their logits - ids and log-probabilities are the oracle's, and the
    path statistics show the selects that read the row."""
    rows, d, vocab = 6, 128, 20_000
    rng = np.random.default_rng(515)
    hidden, weight = _peaked_head(rng, rows, d, vocab)
    params_kw = [dict(temperature=0.7, top_k=20, top_p=0.9, seed=60 + r) for r in range(rows)]
    params = [ls_params(**kw) for kw in params_kw]
    steps = [2] * rows
    for temps in ([1.3] * rows, None, [0.7, 0.7, 0.7, 1.3, 0.7, 0.7]):
        h, w, buf, logits, tmax, tsum = _produce(sampler, hidden, weight, temps, rows, vocab)
        stored = _bits(logits.contiguous())
        stats = torch.zeros(4, dtype=torch.int32, device=dev())
        sampler.set_path_stats(stats)
        ids, lps, cand, counts = _draw_all(
            sampler, lambda out, lp, di, dc: sampler.sample_rows_tiled(
                logits, tmax, tsum, params, steps, out, out_logprobs=lp, dbg_ids=di, dbg_counts=dc),
            logits, params_kw, steps)
        sampler.set_path_stats(None)
        _check_draws(stored, ids, lps, cand, counts, params_kw, steps)
        wrong = rows if temps is None else sum(1 for t in temps if t != 0.7)
        assert stats.cpu().numpy()[0] >= wrong, (temps, stats.cpu().tolist())


def _f32_bound(h, w):
    """What the f32 accumulation of d products may differ from the f64 product by (w: the
    magnitudes that are summed)."""
    return (h.double().abs() @ w.double().abs().T).cpu().numpy() * 2.0 ** -21 + 1e-6


def _check_f32_product(h, w, logits, tmax, tsum, temps, summed=None):
    rows, vocab = logits.shape
    got = logits.cpu().numpy()
    ref = (h.double() @ w.double().T).cpu().numpy()
    tol = _f32_bound(h, w if summed is None else summed)
    assert np.all(np.abs(got - ref) <= tol), float(np.max(np.abs(got - ref) - tol))
    tiles = tmax.shape[1]
    g = np.pad(got, ((0, 0), (0, tiles * TILE - vocab)), constant_values=-np.inf).reshape(rows, tiles, TILE)
    assert np.array_equal(tmax.cpu().numpy(), g.max(axis=2))
    for r in range(rows):
        t = temps[r] if temps is not None else 0.0
        if not t > 0.0:
            continue
        c2 = np.float32(1.4426950408889634 / t)
        top = (g[r].max(axis=1).astype(np.float32) * c2).astype(np.float64)
        want = np.exp2(g[r].astype(np.float64) * np.float64(c2) - top[:, None]).sum(axis=1)
        assert np.allclose(tsum[r].cpu().numpy(), want, rtol=4e-6, atol=0), r


@pytest.mark.parametrize("rows,d,vocab", [(4, 256, 20_000), (70, 128, 3000 + 4), (150, 192, 2000)])
def test_f32_logits_and_draws_from_their_summaries(sampler, rows, d, vocab):
    """The producer with f32 logits (what the reference's sampler reads, src/kernels/sample.rs:263):
    the stored values are the f32 sums, the summaries describe them, and the draws from the
    summaries are the oracle's on the stored f32 logits."""
    rng = np.random.default_rng(rows + d)
    hidden, weight = _peaked_head(rng, rows, d, vocab, peaks=min(40, vocab // 8))
    params_kw = _mixed_params(rows)
    params = [ls_params(**kw) for kw in params_kw]
    temps = [p.effective()[0] for p in params]
    steps = [2 + r for r in range(rows)]
    h, w = _bf16(hidden), _bf16(weight)
    stride = ((vocab + 3) // 4) * 4 + 4
    buf = torch.full((rows, stride), 7.0, dtype=torch.float32, device=dev())
    logits = buf[:, :vocab]
    tiles = (vocab + TILE - 1) // TILE
    tmax = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    tsum = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    sampler.lm_head(h, w, temps, logits, tmax, tsum)
    sampler.synchronize()
    _check_f32_product(h, w, logits, tmax, tsum, temps)
    assert torch.all(buf[:, vocab:] == 7.0)
    stored = logits.contiguous().cpu().numpy()
    ids, lps, cand, counts = _draw_all(
        sampler, lambda out, lp, di, dc: sampler.sample_rows_tiled(
            logits, tmax, tsum, params, steps, out, out_logprobs=lp, dbg_ids=di, dbg_counts=dc),
        logits, params_kw, steps)
    _check_draws(stored, ids, lps, cand, counts, params_kw, steps)
    # and the one call for both
    logits.zero_()
    ids2, lps2, cand2, counts2 = _draw_all(
        sampler, lambda out, lp, di, dc: sampler.lm_head_sample_rows(
            h, w, logits, tmax, tsum, params, steps, out, out_logprobs=lp, dbg_ids=di, dbg_counts=dc),
        logits, params_kw, steps)
    assert np.array_equal(logits.contiguous().cpu().numpy(), stored)
    assert np.array_equal(ids, ids2)


def _quantised(rng, vocab, d, bits, group):
    """Random affine weights in the reference's layout; what dequant_q4/q8_bf16 makes of them
    (src/kernels/metal/quant.metal:179-233: q * scale + bias in f32 (fused), rounded to bf16), the
    weights themselves (f64: what gemv_q4/q8_bf16_f32out multiply by, quant.metal:8-60 and
    130-176) and the magnitudes the few-row form sums in f32 (4-bit codes enter as 128 + q and the
    128 leaves with the bias)."""
    q = rng.integers(0, 1 << bits, (vocab, d)).astype(np.uint32)
    scales = W.to_bf16_bits(rng.uniform(0.5, 1.5, (vocab, d // group)).astype(np.float32) * (2.0 / (1 << bits)) / np.sqrt(d))
    biases = W.to_bf16_bits(-W.bf16_bits_to_f32(scales) * np.float32((1 << bits) / 2) +
                            rng.normal(0, 0.02 / np.sqrt(d), (vocab, d // group)).astype(np.float32))
    per = 32 // bits
    words = np.zeros((vocab, d // per), dtype=np.uint32)
    for j in range(per):
        words |= q[:, j::per] << np.uint32(bits * j)
    s = np.repeat(W.bf16_bits_to_f32(scales), group, axis=1)
    b = np.repeat(W.bf16_bits_to_f32(biases), group, axis=1)
    # (one fused operation: the exact q * s + b rounded once to f32 - exact in f64, whose 53 bits
    # hold an 8-bit code times an 8-bit scale plus a bias of like magnitude)
    exact = q.astype(np.float64) * s.astype(np.float64) + b.astype(np.float64)
    dense = W.to_bf16_bits(exact.astype(np.float32))
    off = 128.0 if bits == 4 else 0.0
    summed = (q + off) * s.astype(np.float64) + np.abs(b.astype(np.float64) - off * s)
    t = lambda a, dt: torch.from_numpy(a.view(np.int16) if dt is torch.bfloat16 else a.view(np.int32)).to(dev())
    qw = LS.QuantWeights(t(words, torch.int32), t(scales, torch.bfloat16).view(torch.bfloat16),
                         t(biases, torch.bfloat16).view(torch.bfloat16), group, bits)
    return (qw, torch.from_numpy(dense.view(np.int16)).to(dev()).view(torch.bfloat16),
            torch.from_numpy(exact).to(dev()), torch.from_numpy(summed).to(dev()))


@pytest.mark.parametrize("bits,group", [(4, 64), (8, 64), (4, 32), (8, 128)])
@pytest.mark.parametrize("rows", [1, 3, 16, 17, 40, 100, 300])
def test_heads_of_affine_codes(sampler, bits, group, rows):
    """The reference's quantised head formats (QuantWeights, src/weights.rs:27-36; lm_head is 4 bits
    in groups of 64, 8 under --q8 head).  Up to 16 rows of groups of 64 or more take the
    reference's form for few rows - the codes are not turned into weights - and are held against
    the f64 product with the affine weights themselves; the others against the f64 product with
    the weights as dequant_q4/q8_bf16 give them, for every tile shape the codes pass through.
    Greedy rows drawn by the same call pick the oracle's token on the stored logits.  (d = 1280:
    five or ten stages of the few-row form, which walks them three at a time.)"""
    d, vocab = 1280, 2000 + 8 * bits
    rng = np.random.default_rng(1000 * bits + group + rows)
    hidden = rng.normal(0, 1, (rows, d)).astype(np.float32)
    qw, dense, exact, summed = _quantised(rng, vocab, d, bits, group)
    few = rows <= 16 and group >= 64 and (d // group) % 2 == 0 and d % (1024 // bits) == 0
    h = _bf16(hidden)
    params_kw = [dict(temperature=0.8, top_k=20, top_p=0.9, seed=r) if r % 2 else dict() for r in range(rows)]
    params = [ls_params(**kw) for kw in params_kw]
    temps = [p.effective()[0] for p in params]
    logits = torch.zeros(rows, vocab, dtype=torch.float32, device=dev())
    tiles = (vocab + TILE - 1) // TILE
    tmax = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    tsum = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
    steps = [1] * rows
    ids, lps, cand, counts = _draw_all(
        sampler, lambda out, lp, di, dc: sampler.lm_head_sample_rows(
            h, qw, logits, tmax, tsum, params, steps, out, out_logprobs=lp, dbg_ids=di, dbg_counts=dc),
        logits, params_kw, steps)
    if few:
        _check_f32_product(h, exact, logits, tmax, tsum, temps, summed=summed)
    else:
        _check_f32_product(h, dense, logits, tmax, tsum, temps)
    _check_draws(logits.cpu().numpy(), ids, lps, cand, counts, params_kw, steps)


@pytest.mark.parametrize("form", ["own", "library"])
@pytest.mark.parametrize("rows,d,vocab,slack", [(130, 512, 4096 + 77, 8), (300, 128, 2000 + 3, 3),
                                                (1024, 256, 3000, 8), (5, 64, 700, 8)])
def test_batches_in_either_form(monkeypatch, form, rows, d, vocab, slack):
    """A batch through this library's own tiles and through the platform's GEMM library followed
    by the pass that forms the summaries (LILY_SAMPLER_HEAD, read when a sampler is created):
    bf16 logits, f32 logits and both widths of codes meet the producer's bar either way, nothing
    behind a row's last column is written, and the sampler counts the calls that took the
    library (none under `own`; every one under `library` where the rows of the logits start at
    multiples of 16 bytes, none where they do not: those stay with this library's own kernels)."""
    monkeypatch.setenv("LILY_SAMPLER_HEAD", form)
    s = LS.Sampler(0)
    try:
        rng = np.random.default_rng(rows + d)
        hidden, weight = _peaked_head(rng, rows, d, vocab, peaks=min(20, vocab // 8))
        temps = [0.0 if r % 5 == 4 else 0.5 + 0.1 * (r % 7) for r in range(rows)]
        stride = ((vocab + 7) // 8) * 8 + slack
        h, w, buf, logits, tmax, tsum = _produce(s, hidden, weight, temps, rows, vocab, stride)
        _check_product(h, w, logits, tmax, tsum, temps)
        assert torch.all(buf[:, vocab:] == 7.0)
        calls = s.lm_head_library_calls()
        assert calls == (1 if form == "library" and slack == 8 else 0)
        tiles = (vocab + TILE - 1) // TILE
        buf32 = torch.full((rows, stride), 7.0, dtype=torch.float32, device=dev())
        s.lm_head(h, w, temps, buf32[:, :vocab], tmax, tsum)
        s.synchronize()
        _check_f32_product(h, w, buf32[:, :vocab], tmax, tsum, temps)
        assert torch.all(buf32[:, vocab:] == 7.0)
        if form == "library" and slack == 8:
            assert s.lm_head_library_calls() == 2
        for bits, group in ((4, 64), (8, 32)):
            qw, dense, _, _ = _quantised(rng, vocab, d, bits, group)
            buf32.fill_(7.0)
            before = s.lm_head_library_calls()
            s.lm_head(h, qw, temps, buf32[:, :vocab], tmax, tsum)
            s.synchronize()
            if form == "library" and slack == 8:
                assert s.lm_head_library_calls() == before + 1
            if form == "own" and rows <= 16 and group >= 64 and (d // group) % 2 == 0 and d % (1024 // bits) == 0:
                continue   # (the form for few rows has a test of its own)
            _check_f32_product(h, dense, buf32[:, :vocab], tmax, tsum, temps)
            assert torch.all(buf32[:, vocab:] == 7.0)
        # a hidden row with a NaN: every logit of the row is a NaN, which counts as -inf in the
        # summaries (largest value -inf, sum 0); the other rows are what they were
        h2 = h.clone()
        h2[1, 3] = float("nan")
        s.lm_head(h2, w, temps, logits, tmax, tsum)
        s.synchronize()
        assert bool(torch.all(torch.isnan(logits[1].float())))
        assert bool(torch.all(tmax[1] == float("-inf"))) and bool(torch.all(tsum[1] == 0.0))
        keep = [r for r in range(rows) if r != 1]
        _check_product(h[keep], w, logits[keep], tmax[keep], tsum[keep], [temps[r] for r in keep])
    finally:
        s.close()


@pytest.mark.parametrize("block", range(4))
def test_random_rows_from_summaries(sampler, block):
    """Seeded random batches through lily_sample_rows_tiled: bf16 or f32 logits of heads with few
    or many peaks, 1 to 23 rows, vocabularies of 777 to 151 936, any k and temperature, lowering
    penalties over histories that may hold the rows' best ids, bias lists of 0 to 64 pairs with
    deltas from -inf to +60, and six kinds of allow-mask (a few of the best ids barred, a run
    around one of the best tiles, ids barred at random with any density, a sparse set, the best
    ids barred by the dozen, none).  Whatever way each row goes - the summaries, a decline on the
    device, the kernels that read the row - ids, candidates, kept counts, counts of the scratch
    and log-probabilities are the oracle's on the stored logits."""
    for trial in range(block * 10, block * 10 + 10):
        rng = np.random.default_rng(990_000 + trial)
        f32 = bool(rng.integers(0, 2))
        rows, d = int(rng.integers(1, 24)), int(rng.choice([64, 128, 256]))
        vocab = int(rng.choice([777, 5000, 20000 + int(rng.integers(0, 130)), 151936]))
        hidden, weight = _peaked_head(rng, rows, d, vocab, peaks=min(int(rng.choice([5, 40, 200])), vocab // 8),
                                      gain=float(rng.choice([3.0, 6.0, 9.0, 14.0])))
        kws = []
        for r in range(rows):
            kw = dict(temperature=float(rng.choice([0.3, 0.7, 1.0, 1.5])),
                      top_k=int(rng.choice([1, 2, 5, 20, 64, 64, 100])), top_p=float(rng.choice([1.0, 0.9, 0.5])),
                      min_p=float(rng.choice([0.0, 0.0, 0.05])), seed=int(rng.integers(0, 1 << 30)))
            if rng.random() < 0.5:
                kw.update(repetition_penalty=float(rng.choice([1.0, 1.1, 1.3])),
                          presence_penalty=float(rng.choice([0.0, 0.2])),
                          frequency_penalty=float(rng.choice([0.0, 0.1])))
            kws.append(dict() if rng.random() < 0.1 else kw)
        params = [ls_params(**kw) for kw in kws]
        temps = [p.effective()[0] for p in params]
        h, w = _bf16(hidden), _bf16(weight)
        tiles = (vocab + TILE - 1) // TILE
        stride = ((vocab + 7) // 8) * 8
        buf = torch.zeros(rows, stride, dtype=torch.float32 if f32 else torch.bfloat16, device=dev())
        logits = buf[:, :vocab]
        tmax = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
        tsum = torch.zeros(rows, tiles, dtype=torch.float32, device=dev())
        sampler.lm_head(h, w, temps, logits, tmax, tsum)
        sampler.synchronize()
        stored = logits.contiguous().cpu().numpy() if f32 else _bits(logits.contiguous())
        stored_f = stored if f32 else W.bf16_bits_to_f32(stored)
        words = (vocab + 31) // 32
        masks = np.zeros((rows, words), dtype=np.uint32)
        use_mask = rng.random() < 0.6
        bias, scratch, hist = [], [], []
        for r in range(rows):
            order = np.argsort(-stored_f[r])
            allowed = np.ones(vocab, dtype=bool)
            kind = int(rng.integers(0, 6))
            if kind == 0:
                allowed[order[rng.choice(min(30, vocab), 6, replace=False)]] = False
            elif kind == 1:
                t = int(order[int(rng.integers(0, 3))]) // TILE
                allowed[max(0, t * TILE - int(rng.integers(0, 200))):min(vocab, (t + 1) * TILE + int(rng.integers(0, 200)))] = False
            elif kind == 2:
                allowed[rng.random(vocab) < rng.choice([0.001, 0.03, 0.5])] = False
            elif kind == 3:
                allowed[:] = False
                allowed[order[rng.choice(min(200, vocab), int(rng.integers(1, 100)), replace=False)]] = True
            elif kind == 4:
                allowed[order[:int(rng.integers(1, 80))]] = False
            bits = np.zeros(words * 32, dtype=bool)
            bits[:vocab] = allowed
            masks[r] = np.packbits(bits.reshape(words, 32), axis=1, bitorder="little").view(np.uint32).reshape(words)
            nb = int(rng.choice([0, 0, 1, 5, 40, 64]))
            ids = np.concatenate([order[rng.integers(0, min(100, vocab), nb // 2)], rng.integers(0, vocab, nb - nb // 2)])
            deltas = rng.choice([-100.0, -5.0, -0.5, 0.25, 3.0, 20.0, 60.0, float("-inf")], nb)
            bias.append([(int(i), float(dl)) for i, dl in zip(ids, deltas)])
            best = order[:20].astype(np.int32)
            hh = np.concatenate([rng.integers(0, vocab, int(rng.integers(0, 2000))).astype(np.int32),
                                 np.repeat(best[:5], int(rng.integers(0, 4))), best[:int(rng.integers(0, 20))]])
            sc = LS.SamplerScratch(sampler, vocab)
            if len(hh):
                sc.add_history(torch.from_numpy(hh).to(dev()))
            scratch.append(sc)
            hist.append(np.bincount(hh, minlength=vocab).astype(np.uint32))
        steps = [int(rng.integers(0, 1000)) for _ in range(rows)]
        allow_t = torch.from_numpy(masks.view(np.int32)).to(dev()) if use_mask else None
        ids, lps, cand, counts = _draw_all(
            sampler, lambda out, lp, di, dc: sampler.sample_rows_tiled(
                logits, tmax, tsum, params, steps, out, scratch=scratch, bias=bias, allow=allow_t, out_logprobs=lp,
                dbg_ids=di, dbg_counts=dc),
            logits, kws, steps)
        for r, kw in enumerate(kws):
            p = o_params(**kw)
            dd = O.sample(stored[r], hist[r], p, steps[r], allow=masks[r] if use_mask else None, bias=bias[r],
                          want_logprob=True)
            assert ids[r] == dd.chosen, (trial, r)
            if p.temperature == 0.0 or kw.get("top_k") == 1:
                continue   # (a greedy row reports its token only)
            n_fin = int(np.sum(dd.cand_adj > -np.inf))
            assert counts[r, 0] == n_fin and counts[r, 1] == dd.n_kept, (trial, r)
            assert np.array_equal(cand[r, :n_fin], dd.cand_ids[:n_fin].astype(np.int64)), (trial, r)
            if np.isfinite(dd.logprob):
                assert abs(lps[r] - dd.logprob) <= LOGPROB_RTOL * max(1.0, abs(dd.logprob)), (trial, r, lps[r], dd.logprob)
        for r in range(rows):
            assert np.array_equal(scratch[r].read_counts().numpy().view(np.uint32), hist[r]), (trial, r)
            scratch[r].close()


def test_one_row_of_an_odd_vocabulary(sampler):
    """A batch of one row has no second row whose start the stride would decide: 777 columns,
    said as the stride too, are drawn from the summaries like any other row."""
    rows, d, vocab = 1, 64, 777
    rng = np.random.default_rng(3)
    hidden, weight = _peaked_head(rng, rows, d, vocab, peaks=20)
    params_kw = [dict(temperature=0.8, top_k=20, top_p=0.9, seed=4)]
    params = [ls_params(**kw) for kw in params_kw]
    h, w, buf, logits, tmax, tsum = _produce(sampler, hidden, weight, [0.8], rows, vocab, stride=vocab)
    ids, lps, cand, counts = _draw_all(
        sampler, lambda out, lp, di, dc: sampler.sample_rows_tiled(
            logits, tmax, tsum, params, [2], out, out_logprobs=lp, dbg_ids=di, dbg_counts=dc),
        logits, params_kw, [2])
    _check_draws(_bits(logits.contiguous()), ids, lps, cand, counts, params_kw, [2])


def test_codes_ask_for_f32_logits(sampler):
    rng = np.random.default_rng(5)
    qw, _, _, _ = _quantised(rng, 256, 64, 8, 64)
    h = torch.zeros(2, 64, dtype=torch.bfloat16, device=dev())
    tmax = torch.zeros(2, 2, dtype=torch.float32, device=dev())
    tsum = torch.zeros(2, 2, dtype=torch.float32, device=dev())
    with pytest.raises(LS.SamplerError):
        sampler.lm_head(h, qw, None, torch.zeros(2, 256, dtype=torch.bfloat16, device=dev()), tmax, tsum)
    bad = LS.QuantWeights(qw.codes, qw.scales, qw.biases, 48, 8)
    with pytest.raises(LS.SamplerError):
        sampler.lm_head(h, bad, None, torch.zeros(2, 256, dtype=torch.float32, device=dev()), tmax, tsum)
    sampler.synchronize()
