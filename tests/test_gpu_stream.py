"""The streaming select (k <= 64, no allow-mask) and the scratch's (id, count) list.

Rows of this kind are scanned once; penalised and biased ids come from the scratch's list
and the row's bias list, not from the stream.  These tests drive that path against the
oracle where it is most likely to go wrong: penalties that raise or lower values, bias on
penalised ids, counts beyond the packed range, rows whose best values are all penalised,
lists that outgrow the workgroup's or the scratch's capacity, the list after uncount /
reset / copy / a dense rewrite, and log-probabilities of peaked and of flat rows.
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


def make_sampler(slices):
    old = os.environ.get("LILY_SAMPLER_SLICES")
    os.environ["LILY_SAMPLER_SLICES"] = str(slices)
    try:
        return LS.Sampler(0)
    finally:
        if old is None:
            os.environ.pop("LILY_SAMPLER_SLICES", None)
        else:
            os.environ["LILY_SAMPLER_SLICES"] = old


@pytest.fixture(scope="module", params=[0, 1, 5], ids=lambda s: f"slices{s}")
def sampler(request):
    s = make_sampler(request.param)
    yield s
    s.close()


def _scratches(sampler, hist, vocab):
    out, counts = [], []
    for h in hist:
        sc = LS.SamplerScratch(sampler, vocab)
        sc.add_history(torch.from_numpy(np.ascontiguousarray(h, dtype=np.int32)).to(dev()))
        out.append(sc)
        counts.append(np.bincount(h, minlength=vocab).astype(np.uint32))
    return out, counts


def _check_logprob(r, i, d, tag):
    if np.isfinite(d.logprob):
        assert abs(r.logprobs[i] - d.logprob) <= 1e-5 * max(1.0, abs(d.logprob)), (tag, i)


def test_the_streaming_select_serves_the_throughput_shape(sampler):
    """Every slice of a config-5 shaped batch is produced by the streaming select."""
    c = W.config5(rows=16)
    vocab = c["logits"].shape[1]
    sc, counts = _scratches(sampler, c["history"], vocab)
    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    sampler.set_path_stats(stats)
    try:
        r = run_rows(sampler, c["logits"], c["params"], [2] * 16, scratch=sc, logprobs=True)
    finally:
        sampler.set_path_stats(None)
    st = stats.cpu().tolist()
    assert st[0] == 16 * sampler.slices_for(16, 64, vocab, bf16=True) and st[1] == 0 and st[2] == 0, st
    for i in range(16):
        d = O.sample(c["logits"][i], counts[i], o_params(**c["params"][i]), 2, want_logprob=True)
        check_row_against_oracle(r, i, d)
        _check_logprob(r, i, d, "config5")
    for x in sc:
        x.close()


@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
@pytest.mark.parametrize("vocab", [151_936, 30_011])
def test_penalties_and_bias_of_every_sign(sampler, vocab, bf16):
    """Penalties that lower and that raise, repetition below and above 1, bias on penalised and
    on plain ids with duplicates, one id counted beyond the packed 12 bits."""
    rng = np.random.default_rng(vocab + bf16)
    rows = 8
    x = rng.normal(0, 3, (rows, vocab)).astype(np.float32)
    x[:, : vocab // 3] -= 2.0
    xs = W.to_bf16_bits(x) if bf16 else x
    hist = [rng.integers(0, vocab, 2500) for _ in range(rows)]
    for r in range(rows):
        top = np.argsort(W.bf16_bits_to_f32(xs[r]) if bf16 else xs[r])[::-1]
        hist[r][:40] = top[:40]                      # the best ids are penalised
        hist[r][40:40 + 5000 // 8] = top[3]          # repeated
    hist[0] = np.concatenate([hist[0], np.full(5000, hist[0][0])])  # count 5001 > 4095
    sc, counts = _scratches(sampler, hist, vocab)
    signs = [dict(repetition_penalty=1.3, presence_penalty=0.4, frequency_penalty=0.05),
             dict(repetition_penalty=0.8, presence_penalty=-0.5, frequency_penalty=-0.02),
             dict(repetition_penalty=1.0, presence_penalty=2.0, frequency_penalty=0.0),
             dict(repetition_penalty=2.5, presence_penalty=0.0, frequency_penalty=0.3)]
    bias = []
    for r in range(rows):
        ids = list(rng.integers(0, vocab, 20)) + [int(hist[r][1]), int(hist[r][2])]
        b = [(int(i), float(d)) for i, d in zip(ids, rng.choice([-6.0, 4.0, 9.0], len(ids)))]
        bias.append(b + [b[0], b[-1]])               # duplicates accumulate in list order
    for trial, k in enumerate((1, 7, 20, 64)):
        kw = [dict(temperature=0.8, top_k=k, top_p=0.92, min_p=0.01, seed=300 + r, **signs[r % 4])
              for r in range(rows)]
        r = run_rows(sampler, xs, kw, [trial] * rows, scratch=sc, bias=bias, logprobs=True)
        for i in range(rows):
            d = O.sample(xs[i], counts[i], o_params(**kw[i]), trial, bias=bias[i], want_logprob=True)
            check_row_against_oracle(r, i, d)
            _check_logprob(r, i, d, ("signs", k))
        for i in range(rows):
            got = sc[i].read_counts().numpy().view(np.uint32)
            bad = np.flatnonzero(got != counts[i])
            assert bad.size == 0, (i, k, bad[:8], got[bad[:8]], counts[i][bad[:8]])
    for s_ in sc:
        s_.close()


def test_rows_that_defeat_the_bound(sampler):
    """All the best raw values penalised away, ascending order, constant rows, few finite
    values: the result stays the oracle's whichever select ends up producing it."""
    rng = np.random.default_rng(77)
    vocab, rows = 20_000, 6
    x = rng.normal(0, 1, (rows, vocab)).astype(np.float32)
    hist = [rng.integers(0, vocab, 64) for _ in range(rows)]
    top = np.argsort(x[0])[::-1][:300]
    hist[0] = np.repeat(top, 3)                      # the 300 best: each counted three times
    x[1] = np.sort(x[1])                             # ascending
    hist[1] = np.arange(vocab - 100, vocab)          # and the last ones penalised
    x[2] = 0.25                                      # constant
    x[3, :] = -np.inf
    x[3, rng.integers(0, vocab, 30)] = rng.normal(0, 1, 30)   # 30 finite values
    hist[3] = np.flatnonzero(np.isfinite(x[3]))[:10]
    x[4] = -50.0                                     # listed ids carry all the mass below the bound
    lid = rng.choice(vocab, 3000, replace=False)
    x[4, lid] = 5.0
    x[4, rng.choice(vocab, 200, replace=False)] = 6.0
    hist[4] = lid
    hist[5] = np.arange(0, vocab, 3)                 # a third of the vocabulary listed
    sc, counts = _scratches(sampler, hist, vocab)
    for trial, k in enumerate((64, 20, 1)):
        kw = [dict(temperature=0.9, top_k=k, top_p=0.95, seed=900 + r, repetition_penalty=1.5,
                   presence_penalty=4.0, frequency_penalty=1.0) for r in range(rows)]
        r = run_rows(sampler, x, kw, [trial] * rows, scratch=sc, logprobs=True)
        for i in range(rows):
            d = O.sample(x[i], counts[i], o_params(**kw[i]), trial, want_logprob=True)
            check_row_against_oracle(r, i, d)
            _check_logprob(r, i, d, ("defeat", k))
    for s_ in sc:
        s_.close()


def test_lists_beyond_the_workgroup_and_the_scratch(sampler):
    """4 000 listed ids (more than a workgroup buckets), 20 000 (spread over slices) and
    70 000 (more than a scratch lists): the draws agree whichever select serves them, and
    later draws keep agreeing."""
    rng = np.random.default_rng(5)
    vocab = 90_001
    x = W.to_bf16_bits(rng.normal(0, 2, (3, vocab)).astype(np.float32))
    hist = [rng.choice(vocab, n, replace=False) for n in (4000, 20_000, 70_000)]
    sc, counts = _scratches(sampler, hist, vocab)
    for step in range(3):
        kw = [dict(temperature=0.7, top_k=40, top_p=0.9, seed=r, repetition_penalty=1.1,
                   presence_penalty=0.2, frequency_penalty=0.1) for r in range(3)]
        r = run_rows(sampler, x, kw, [step] * 3, scratch=sc, logprobs=True)
        for i in range(3):
            d = O.sample(x[i], counts[i], o_params(**kw[i]), step, want_logprob=True)
            check_row_against_oracle(r, i, d)
            _check_logprob(r, i, d, ("long", step))
    for s_ in sc:
        s_.close()


def test_long_lists_are_read_in_place():
    """6 000 listed ids per row, far more than a workgroup could bucket in LDS: the sorted list
    is read from memory block by block, so the streaming select serves every slice at the
    slice count the batch size alone asks for."""
    s = LS.Sampler(0)
    rng = np.random.default_rng(15)
    vocab, rows = 151_936, 300
    x = W.to_bf16_bits(rng.normal(0, 2, (rows, vocab)).astype(np.float32))
    hist = [rng.choice(vocab, 6000, replace=False) for _ in range(rows)]
    sc, counts = _scratches(s, hist, vocab)
    kw = [dict(temperature=0.7, top_k=40, top_p=0.9, seed=r, repetition_penalty=1.1,
               presence_penalty=0.2, frequency_penalty=0.1) for r in range(rows)]
    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    s.set_path_stats(stats)
    r = run_rows(s, x, kw, [0] * rows, scratch=sc, logprobs=True)
    s.set_path_stats(None)
    st = stats.cpu().tolist()
    assert st[0] == rows * s.slices_for(rows, 40, vocab, bf16=True) and st[1] == 0 and st[2] == 0, st
    for i in range(0, rows, 7):
        d = O.sample(x[i], counts[i], o_params(**kw[i]), 0, want_logprob=True)
        check_row_against_oracle(r, i, d)
        _check_logprob(r, i, d, "long lists")
    for s_ in sc:
        s_.close()
    s.close()


def test_the_list_follows_every_scratch_operation(sampler):
    """Draws after uncount (to zero and back), reset, copy and a dense rewrite of the counts
    see exactly the counts the reference's histogram would hold (the oracle's draw adds the
    emitted id to the counts it is given, as the kernel does)."""
    rng = np.random.default_rng(31)
    vocab = 50_003
    x = rng.normal(0, 2.5, (1, vocab)).astype(np.float32)
    kw = [dict(temperature=0.6, top_k=12, top_p=0.9, seed=4, repetition_penalty=1.4,
               presence_penalty=1.0, frequency_penalty=0.5)]
    a = LS.SamplerScratch(sampler, vocab)
    b = LS.SamplerScratch(sampler, vocab)
    counts = np.zeros(vocab, np.uint32)

    def draw(sc, cnt, step):
        r = run_rows(sampler, x, kw, [step], scratch=[sc])
        d = O.sample(x[0], cnt, o_params(**kw[0]), step)
        check_row_against_oracle(r, 0, d)
        assert np.array_equal(sc.read_counts().numpy().view(np.uint32), cnt)
        return int(d.chosen)

    first = draw(a, counts, 0)
    a.uncount(first)                       # back to zero: the id stays listed with count 0
    counts[first] -= 1
    a.uncount(first)                       # saturates
    again = [draw(a, counts, s) for s in range(1, 6)]
    a.uncount(again[-1])
    counts[again[-1]] -= 1
    draw(a, counts, 6)
    b.copy_counts_from(a)                  # b continues from a's state
    cb = counts.copy()
    for s in range(7, 10):
        draw(b, cb, s)
        draw(a, counts, s)
    dense = np.zeros(vocab, np.uint32)
    dense[rng.integers(0, vocab, 500)] = rng.integers(1, 9, 500).astype(np.uint32)
    a.write_counts(torch.from_numpy(dense.view(np.int32)))
    counts = dense.copy()
    for s in range(10, 13):
        draw(a, counts, s)
    a.reset_counts()
    counts[:] = 0
    for s in range(13, 15):
        draw(a, counts, s)
    a.close()
    b.close()


def test_log_probabilities_of_peaked_and_flat_rows(sampler):
    """A row with one huge value (its bulk terms are skipped as negligible), the same with that
    value penalised, a flat row (nothing may be skipped) and a row of large negative values."""
    rng = np.random.default_rng(8)
    vocab, rows = 151_936, 6
    x = rng.normal(0, 2, (rows, vocab)).astype(np.float32)
    x[0, 1234] = 150.0
    x[1, 77] = 150.0
    x[2] = rng.normal(0, 0.05, vocab)
    x[3] -= 300.0
    x[4, 5:40] += 30.0
    x[5, vocab - 3] = 60.0
    xs = W.to_bf16_bits(x)
    hist = [rng.integers(0, vocab, 1500) for _ in range(rows)]
    hist[1][:4] = 77
    hist[4][:10] = np.arange(5, 15)
    sc, counts = _scratches(sampler, hist, vocab)
    for step, temp in enumerate((0.8, 0.3, 1.7)):
        kw = [dict(temperature=temp, top_k=64, top_p=0.9, seed=40 + r, repetition_penalty=1.2,
                   presence_penalty=0.3, frequency_penalty=0.1) for r in range(rows)]
        r = run_rows(sampler, xs, kw, [step] * rows, scratch=sc, logprobs=True)
        for i in range(rows):
            d = O.sample(xs[i], counts[i], o_params(**kw[i]), step, want_logprob=True)
            check_row_against_oracle(r, i, d)
            _check_logprob(r, i, d, ("lse", temp))
    for s_ in sc:
        s_.close()


def test_skipped_terms_are_measured_against_the_largest_true_value(sampler):
    """The largest raw value belongs to a heavily penalised id: terms may only be skipped
    relative to what that id is worth after the penalties, or the mass of the values in between
    would be lost."""
    rng = np.random.default_rng(21)
    vocab, rows = 151_936, 3
    x = rng.normal(0, 2, (rows, vocab)).astype(np.float32)
    hist = []
    for r in range(rows):
        x[r, 4000 + r] = 150.0                                   # worth 150 / 2.5 - 41 = 19 after penalties
        x[r, rng.choice(vocab, 3000, replace=False)] = 18.0      # real mass just below it
        hist.append(np.concatenate([np.full(40, 4000 + r), rng.integers(0, vocab, 1000)]))
    x[2, 9000] = 60.0                                            # row 2: a plain id above everything
    xs = W.to_bf16_bits(x)
    sc, counts = _scratches(sampler, hist, vocab)
    kw = [dict(temperature=0.8, top_k=64, top_p=0.9, seed=r, repetition_penalty=2.5,
               presence_penalty=1.0, frequency_penalty=1.0) for r in range(rows)]
    for step in range(2):
        r = run_rows(sampler, xs, kw, [step] * rows, scratch=sc, logprobs=True)
        for i in range(rows):
            d = O.sample(xs[i], counts[i], o_params(**kw[i]), step, want_logprob=True)
            check_row_against_oracle(r, i, d)
            _check_logprob(r, i, d, ("true max", step))
    for s_ in sc:
        s_.close()


def test_a_batch_replays(sampler):
    """The same batch from the same counts: identical ids, log-probabilities equal to 2e-6
    (the listed ids' terms are summed in the order their bucket slots were taken)."""
    c = W.config5(rows=24)
    vocab = c["logits"].shape[1]
    outs = []
    for _ in range(2):
        sc, _ = _scratches(sampler, c["history"], vocab)
        r = run_rows(sampler, c["logits"], c["params"], [1] * 24, scratch=sc, logprobs=True)
        outs.append(r)
        for x in sc:
            x.close()
    assert np.array_equal(outs[0].ids, outs[1].ids)
    assert np.allclose(outs[0].logprobs, outs[1].logprobs, rtol=0, atol=2e-6)
