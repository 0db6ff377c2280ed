"""Pins the CPU oracle: the reference's literal known answers, published vectors and
closed forms.  No GPU.  Each check is chosen so that a plausible mistake in the
restatement (wrong tie rule, dropped penalty term, transposed p/q, off-by-one in a
prefix) fails it; none re-types the oracle's own formula.
"""
import math

import numpy as np
import pytest

import oracle as O


def _row(spec):
    x = np.zeros(spec["v"], dtype=np.float32)
    for k, v in spec["set"].items():
        x[int(k)] = v
    return x


def _num(x):
    return float(x) if isinstance(x, str) else x


# ---------------------------------------------------------------- uniform_for

def test_uniform_is_splitmix64(kat):
    for seed, outs in kat["splitmix64"].items():
        for j, word in enumerate(outs, start=1):
            z = int(word, 0)
            assert O.uniform_for(int(seed), j) == (z >> 40) / 16777216.0


def test_uniform_step0_of_seed0_and_range():
    assert O.uniform_for(0, 0) == 0.0  # the finaliser of 0 is 0
    us = [O.uniform_for(0xDEADBEEF, s) for s in range(4096)]
    assert all(0.0 <= u < 1.0 for u in us)
    assert all((u * 16777216.0).is_integer() for u in us)
    # 64 equal bins of 4096 draws: chi-square, 63 dof, 99.9th percentile ~ 103.
    h = np.histogram(us, bins=64, range=(0, 1))[0]
    assert ((h - 64.0) ** 2 / 64.0).sum() < 103.0


def test_rng_domains_are_disjoint():
    assert O.lib().lo_draft_step(5) == 5 | 0x40000000
    a = O.uniform_for(9, 5)
    b = O.uniform_for(9, 5 | 0x40000000)
    c = O.uniform_for(9, 5 | 0x80000000)
    assert len({a, b, c}) == 3


# ---------------------------------------------------------------- expf

def test_expf_against_double_exp():
    rng = np.random.default_rng(1)
    xs = np.concatenate([
        rng.uniform(-104.5, 0.0, 200000), rng.uniform(0.0, 89.0, 20000),
        -np.logspace(-30, 2, 5000), np.array([0.0, -0.0, -1e-45, -87.33, -87.34, -103.9, -104.0]),
    ]).astype(np.float32)
    worst = 0.0
    for x in xs:
        got = O.expf(float(x))
        want = math.exp(float(x)) if x < 88.73 else math.inf
        want32 = np.float32(want) if want < 3.4028235e38 else np.float32(np.inf)
        if want32 == 0 or not np.isfinite(want32):
            assert abs(got - float(want32)) <= 2e-45 or got == float(want32)
            continue
        ulp = float(np.spacing(want32))
        worst = max(worst, abs(got - want) / ulp)
    assert worst <= 1.5, worst
    assert O.expf(0.0) == 1.0
    assert O.expf(-math.inf) == 0.0
    assert O.expf(-200.0) == 0.0


def test_expf_is_monotone_near_zero():
    xs = np.float32(-1.0) + np.arange(2000, dtype=np.float32) * np.float32(6e-8)
    ys = [O.expf(float(x)) for x in np.unique(xs)]
    assert all(b >= a for a, b in zip(ys, ys[1:]))


# ---------------------------------------------------------------- argmax / greedy

def test_greedy_lowest_id_on_ties(kat):
    k = kat["greedy_ties"]
    x = _row(k)
    assert O.argmax(x) == k["expect"]
    d = O.sample(x, np.zeros(x.size, np.uint32), O.greedy(), 0)
    assert d.chosen == k["expect"]


def test_argmax_first_max(kat):
    k = kat["argmax_ties"]
    rng = np.random.default_rng(8)
    x = rng.uniform(-8, 8, k["v"]).astype(np.float32)
    for i, v in k["set"].items():
        x[int(i)] = v
    assert O.argmax(x) == k["expect"]
    assert O.argmax(np.full(100, -np.inf, np.float32)) == 0
    assert O.argmax(np.full(100, 3.0, np.float32)) == 0
    for _ in range(20):
        y = rng.integers(-3, 4, 999).astype(np.float32)  # many ties
        assert O.argmax(y) == int(np.argmax(y))  # numpy's argmax is first-max too


# ---------------------------------------------------------------- penalties

def test_penalties_literal(kat):
    k = kat["penalties"]
    x = _row(k)
    counts = np.zeros(k["v"], np.uint32)
    for i, c in k["counts"].items():
        counts[int(i)] = c
    p = O.params(presence_penalty=k["presence"], frequency_penalty=k["frequency"],
                 repetition_penalty=k["repetition"])
    adj = O.adjust(x, counts, p)
    assert abs(adj[10] - k["adjusted_10"]) < k["adjusted_10_tol"]
    assert adj[20] == k["adjusted_20"]
    d = O.sample(x, counts, p, 0)
    assert d.chosen == k["expect_id"]
    for i, c in k["counts_after"].items():
        assert counts[int(i)] == c


def test_penalty_sign_cases_closed_form():
    x = np.array([2.0, -2.0, 0.0, 3.0], np.float32)
    counts = np.array([1, 2, 4, 0], np.uint32)
    p = O.params(temperature=0.5, top_k=0, presence_penalty=0.25, frequency_penalty=0.125,
                 repetition_penalty=2.0)
    adj = O.adjust(x, counts, p)
    # positive divides, non-positive multiplies; then presence + frequency*c; then /T
    assert adj[0] == (2.0 / 2.0 - (0.25 + 0.125 * 1)) / 0.5
    assert adj[1] == (-2.0 * 2.0 - (0.25 + 0.125 * 2)) / 0.5
    assert adj[2] == (0.0 * 2.0 - (0.25 + 0.125 * 4)) / 0.5
    assert adj[3] == 3.0 / 0.5  # count 0: untouched
    # penalties off: counts ignored
    assert np.array_equal(O.adjust(x, counts, O.params(temperature=0.5, top_k=0)), x / 0.5)


def test_counts_ops(kat):
    k = kat["counts_move"]
    v = k["v"]
    engine = np.zeros(v, np.uint32)
    for i, c in k["counts"].items():
        engine[int(i)] = c
    slot = engine.copy()
    engine[:] = 0
    assert slot[v - 1] == 5
    O.lib().lo_uncount(slot.ctypes.data, v, 7)
    assert slot[7] == 1
    O.lib().lo_uncount(slot.ctypes.data, v, 8)   # saturating
    assert slot[8] == 0
    O.lib().lo_uncount(slot.ctypes.data, v, v + 5)  # out of range: nothing
    assert slot.sum() == 6


# ---------------------------------------------------------------- params

def test_effective_table(kat):
    for row in kat["effective"]:
        p = O.params(temperature=row["temperature"], top_k=row["top_k"])
        assert bool(O.lib().lo_is_greedy(p)) == row["greedy"]
        assert O.effective(p) == (float(np.float32(row["T"])), row["k"])


def test_validate_table(kat):
    for over, rule in kat["validate"]:
        p = O.params(**{k: _num(v) for k, v in over.items()})
        assert O.lib().lo_validate(p) == rule, over


def test_samples_rule():
    assert not O.lib().lo_samples(O.greedy())
    assert O.lib().lo_samples(O.params(presence_penalty=0.1))          # greedy + penalties
    assert O.lib().lo_samples(O.params(temperature=0.7, top_k=20))
    d = O.draft_params(O.params(temperature=0.7, top_k=20, presence_penalty=1.0,
                                frequency_penalty=2.0, repetition_penalty=3.0, seed=5))
    assert (d.presence_penalty, d.frequency_penalty, d.repetition_penalty) == (0.0, 0.0, 1.0)
    assert (d.top_k, d.seed) == (20, 5)


# ---------------------------------------------------------------- top-k / top-p / min-p / draw

def _logits_of(probs, v=64, fill=-30.0):
    x = np.full(v, fill, np.float32)
    x[: len(probs)] = np.log(np.asarray(probs, np.float64)).astype(np.float32)
    return x


def test_top_p_prefix_closed_form():
    x = _logits_of([0.5, 0.3, 0.15, 0.05], v=4)
    z = np.zeros(4, np.uint32)
    for top_p, n in ((0.49, 1), (0.5, 1), (0.51, 2), (0.8, 2), (0.81, 3), (0.95, 3), (0.96, 4),
                     (1.0, 4)):
        d = O.sample(x, z, O.params(temperature=1.0, top_k=0, top_p=top_p), 0)
        assert d.n_kept == n, (top_p, d.n_kept)
        assert list(d.kept_ids) == list(range(n))


def test_min_p_is_relative_to_the_top():
    x = _logits_of([0.5, 0.3, 0.15, 0.05], v=4)
    z = np.zeros(4, np.uint32)
    for min_p, n in ((0.0, 4), (0.09, 4), (0.11, 3), (0.31, 2), (0.61, 1), (1.0, 1)):
        d = O.sample(x, z, O.params(temperature=1.0, top_k=0, min_p=min_p), 0)
        assert d.n_kept == n, (min_p, d.n_kept)


def test_top_k_set_is_the_brute_force_top_k_with_lowest_ids_on_ties():
    rng = np.random.default_rng(3)
    for v, k in ((1000, 20), (5000, 64), (3000, 1024), (700, 0), (50, 64)):
        x = rng.integers(-20, 21, v).astype(np.float32) / 4  # heavy ties
        d = O.sample(x, None, O.params(temperature=0.9, top_k=k), 0)
        n = min(k if k else 1024, v)
        brute = sorted(range(v), key=lambda i: (-x[i], i))[:n]
        assert list(d.cand_ids) == brute
        assert d.n_cand == n


def test_full_vs_partial_sort_agree():
    rng = np.random.default_rng(4)
    x = rng.normal(0, 3, 20000).astype(np.float32)
    p = O.params(temperature=0.7, top_k=20, top_p=0.95, seed=1)
    a = O.sample(x, None, p, 3)
    b = O.sample(x, None, p, 3, sort_mode=O.SORT_FULL)
    assert a.chosen == b.chosen and list(a.kept_ids) == list(b.kept_ids)


def test_draw_is_the_inverse_cdf():
    x = _logits_of([0.4, 0.3, 0.2, 0.1], v=4)
    p = O.params(temperature=1.0, top_k=0)
    for u, want in ((0.0, 0), (0.39, 0), (0.41, 1), (0.69, 1), (0.71, 2), (0.89, 2), (0.91, 3),
                    (0.9999999, 3)):
        assert O.sample(x, None, p, 0, uniform=u).chosen == want, u
    # temperature sharpens: T=0.5 squares the probabilities (0.16,0.09,0.04,0.01)/0.30
    p2 = O.params(temperature=0.5, top_k=0)
    assert O.sample(x, None, p2, 0, uniform=0.52).chosen == 0   # 0.16/0.30 = 0.533
    assert O.sample(x, None, p2, 0, uniform=0.54).chosen == 1
    # seeded replay uses uniform_for(seed, step)
    p3 = O.params(temperature=1.0, top_k=0, seed=99)
    d = O.sample(x, None, p3, 3)
    assert d.uniform == O.uniform_for(99, 3)
    assert d.chosen == O.sample(x, None, p3, 3).chosen


def test_gap_reports_boundary_distance():
    x = _logits_of([0.5, 0.5], v=2)
    d = O.sample(x, None, O.params(temperature=1.0, top_k=0), 0, uniform=0.5000001)
    assert d.gap < 1e-6 and d.chosen == 1


def test_draws_are_distributed_as_softmax():
    rng = np.random.default_rng(5)
    x = rng.uniform(-2, 2, 48).astype(np.float32)
    p = O.params(temperature=1.0, top_k=0, seed=31)
    probs = np.exp(x.astype(np.float64))
    probs /= probs.sum()
    n = 8192
    h = np.zeros(48)
    for s in range(n):
        h[O.sample(x, None, p, s).chosen] += 1
    chi2 = ((h - n * probs) ** 2 / (n * probs)).sum()
    assert chi2 < 82.0  # 47 dof, 99.9th percentile


# ---------------------------------------------------------------- draft export / spec

def test_kept_matches_sample_and_sums_to_one():
    rng = np.random.default_rng(21)
    head = rng.uniform(-8, 8, 5003).astype(np.float32)
    p = O.params(temperature=1.0, top_k=20, top_p=0.95, seed=5)
    ids, q = O.kept(head, O.draft_params(p))
    d = O.sample(head, None, O.draft_params(p), 0)
    assert list(ids) == list(d.kept_ids)
    assert np.array_equal(q, d.kept_q)
    assert abs(float(q.astype(np.float64).sum()) - 1.0) < 1e-6
    assert np.all(np.diff(q) <= 0)


def test_spec_closed_forms():
    ids = np.array([7, 3, 9], np.uint32)
    p = np.array([0.5, 0.3, 0.2], np.float32)
    # q == p: always accepted, for any uniform
    for u in (0.0, 0.5, 0.999999):
        tok, acc, _, _ = O.spec(ids, p, ids, p, 3, 0, 0, u1=u, u2=0.3)
        assert (tok, acc) == (3, True)
    # proposal outside p's support: always rejected, residual never returns it
    q_ids = np.array([7, 3, 11], np.uint32)
    q = np.array([0.2, 0.3, 0.5], np.float32)
    for u2 in np.linspace(0, 0.999, 50):
        tok, acc, _, _ = O.spec(ids, p, q_ids, q, 11, 0, 0, u1=0.0, u2=float(u2))
        assert not acc and tok in (7, 9)  # residual = (0.3, 0, 0.2): id 3 has no mass
    # accept iff u1*q(d) < p(d): p(7)=0.5, q(7)=0.8 -> ratio 0.625
    q2 = np.array([0.8, 0.1, 0.1], np.float32)
    assert O.spec(ids, p, ids, q2, 7, 0, 0, u1=0.62, u2=0.0)[1]
    assert not O.spec(ids, p, ids, q2, 7, 0, 0, u1=0.63, u2=0.0)[1]
    # rejected: residual (0, 0.2, 0.1)/0.3 -> u2 < 2/3 gives id 3, else id 9
    assert O.spec(ids, p, ids, q2, 7, 0, 0, u1=0.9, u2=0.6)[0] == 3
    assert O.spec(ids, p, ids, q2, 7, 0, 0, u1=0.9, u2=0.7)[0] == 9
    # seeded form draws u1 at step and u2 at step | 0x80000000
    tok = O.spec(ids, p, ids, q2, 7, 77, 4)[0]
    u1, u2 = O.uniform_for(77, 4), O.uniform_for(77, 4 | 0x80000000)
    assert tok == O.spec(ids, p, ids, q2, 7, 0, 0, u1=u1, u2=u2)[0]


def test_speculative_draw_is_distributed_as_the_trunk():
    """tests/unit/kernels/sample.rs:414-487 restated on the oracle."""
    rng = np.random.default_rng(25)
    v = 48
    head = rng.uniform(-2, 2, v).astype(np.float32)
    trunk = (head + rng.uniform(-1.5, 1.5, v)).astype(np.float32)
    p = O.params(temperature=1.0, top_k=0, top_p=1.0, seed=31)
    p_ids, p_pr = O.kept(trunk, p)
    q_ids, q_pr = O.kept(head, p)
    qd = dict(zip(q_ids.tolist(), q_pr.tolist()))
    overlap = sum(min(float(x), qd.get(int(i), 0.0)) for i, x in zip(p_ids, p_pr))
    n = 8192
    hist = np.zeros(v)
    accepted = 0
    for step in range(n):
        d = O.sample(head, None, p, O.lib().lo_draft_step(step)).chosen
        tok, acc, _, _ = O.spec(p_ids, p_pr, q_ids, q_pr, d, p.seed, step)
        assert acc == (tok == d) or tok == d
        hist[tok] += 1
        accepted += tok == d
    chi2 = 0.0
    for i, x in zip(p_ids, p_pr):
        e = float(x) * n
        chi2 += (hist[i] - e) ** 2 / e
        assert abs(hist[i] / n - float(x)) < 0.02
    assert chi2 < 82.0
    assert abs(accepted / n - overlap) < 0.03


def test_spec_accept_cases(kat):
    k = kat["spec_accept"]
    for case in k["cases"]:
        ctrl = O.spec_accept(case["draws"], case["ids"], k["pos0"], k["ratio"], k["chain"],
                             k["stride"])
        slot = lambda s: int(ctrl[s * k["stride"]])
        a = case["a"]
        assert slot(0) == a and slot(1) == a + 1
        for i in range(k["chain"]):
            pos = k["pos0"] + a + 1 + i
            assert slot(2 + 3 * i) == pos
            assert slot(3 + 3 * i) == pos // k["ratio"]
            assert slot(4 + 3 * i) == int((pos + 1) % k["ratio"] == 0)
        dr = np.array(case["draws"], np.uint32)
        ids = np.array(case["ids"], np.uint32)
        assert O.lib().lo_host_accept(dr.ctypes.data, ids.ctypes.data, dr.size) == a


# ---------------------------------------------------------------- extensions (unpinned by the reference)

def test_bf16_widening_is_exact():
    h = np.array([0x3F80, 0xC000, 0x0000, 0x8000, 0x7F80, 0x4049], np.uint16)
    want = np.array([1.0, -2.0, 0.0, -0.0, np.inf, 3.140625], np.float32)
    got = O.adjust(h, None, O.params(temperature=1.0, top_k=0))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_bias_mask_forced_logprob():
    x = np.array([1.0, 2.0, 3.0, 4.0, 0.5], np.float32)
    p = O.params(temperature=1.0, top_k=0, presence_penalty=1.0)
    counts = np.array([0, 0, 0, 2, 0], np.uint32)
    allow = np.array([0b01111], np.uint32)             # id 4 masked out
    bias = [(0, 5.0), (0, -1.0), (2, -3.0)]             # duplicates accumulate in order
    adj = O.adjust(x, counts, p, allow=allow, bias=bias)
    assert list(adj) == [(1.0 + 5.0) - 1.0, 2.0, 0.0, 4.0 - 1.0, -np.inf]
    d = O.sample(x, counts.copy(), p, 0, allow=allow, bias=bias, uniform=0.0, want_logprob=True)
    assert d.chosen == 0 and 4 not in d.kept_ids
    lse = math.log(sum(math.exp(v) for v in (5.0, 2.0, 0.0, 3.0)))
    assert abs(d.logprob - (5.0 - lse)) < 1e-12
    c2 = counts.copy()
    f = O.sample(x, c2, p, 0, allow=allow, bias=bias, forced=1, want_logprob=True)
    assert f.chosen == 1 and c2[1] == 1
    assert abs(f.logprob - (2.0 - lse)) < 1e-12


def test_libm_exp_mode_agrees_to_tolerance():
    rng = np.random.default_rng(6)
    x = rng.normal(0, 3, 6007).astype(np.float32)
    p = O.params(temperature=0.8, top_k=40, top_p=0.9, min_p=0.02, seed=0xDEADBEEF)
    agree = 0
    for s in range(64):
        a = O.sample(x, None, p, s)
        b = O.sample(x, None, p, s, exp_mode=O.EXP_LIBM)
        assert np.allclose(a.cand_prob, b.cand_prob, rtol=1e-5, atol=0)
        agree += a.chosen == b.chosen or min(a.gap, b.gap) < 1e-6
    assert agree == 64
