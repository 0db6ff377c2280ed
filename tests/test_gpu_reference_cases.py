"""The reference's own sampler tests (tests/unit/kernels/sample.rs, spec.rs,
elementwise.rs), restated against the HIP path through the C ABI, with the CPU oracle
as the checker.  Where the reference allows float-noise mismatches (>= 62/64, >= 93/96)
this build requires every draw to match the oracle bit for bit; the oracle run with
the C library's expf (the reference's libm stand-in) must agree except within 1e-6 of a
cumulative-mass boundary (counted).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import lily_sampler as LS
import oracle as O
from gpu_util import both_params, dev, ls_params, o_params, run_rows, check_row_against_oracle


@pytest.fixture(scope="module")
def sampler():
    s = LS.Sampler(0)
    yield s
    s.close()


def _i32(a):
    return torch.tensor(np.asarray(a, dtype=np.int64), dtype=torch.int32, device=dev())


def _draw(sampler, logits_np, counts_np, lp, step):
    """run_kernel of the reference test: one sample_f32 on a fresh scratch."""
    v = logits_np.size
    logits = torch.from_numpy(logits_np).to(dev())
    scratch = LS.SamplerScratch(sampler, v)
    if counts_np is not None:
        scratch.write_counts(torch.from_numpy(counts_np.view(np.int32)))
    out = torch.zeros(1, dtype=torch.int32, device=dev())
    sampler.sample_f32(logits, scratch, lp, step, out)
    sampler.synchronize()
    got = int(out.item())
    counts = scratch.read_counts().numpy().view(np.uint32)
    scratch.close()
    return got, counts


def test_greedy_matches_argmax_with_lowest_id_on_ties(sampler, kat):
    k = kat["greedy_ties"]
    x = np.zeros(k["v"], np.float32)
    for i, v in k["set"].items():
        x[int(i)] = v
    got, _ = _draw(sampler, x, np.zeros(k["v"], np.uint32), ls_params(), 0)
    assert got == k["expect"]


def test_argmax_f32_first_max(sampler, kat):
    k = kat["argmax_ties"]
    rng = np.random.default_rng(8)
    x = rng.uniform(-8, 8, k["v"]).astype(np.float32)
    for i, v in k["set"].items():
        x[int(i)] = v
    out = torch.zeros(1, dtype=torch.int32, device=dev())
    sampler.argmax_f32(torch.from_numpy(x).to(dev()), out)
    sampler.synchronize()
    assert int(out.item()) == k["expect"]
    for n in (1, 63, 4097, 151_936):
        for trial in range(3):
            y = rng.integers(-3, 4, n).astype(np.float32) if trial else np.full(n, -np.inf, np.float32)
            sampler.argmax_f32(torch.from_numpy(y).to(dev()), out)
            sampler.synchronize()
            assert int(out.item()) == O.argmax(y)


def test_draws_match_the_cpu_reference(sampler):
    rng = np.random.default_rng(7)
    v = 6007
    x = rng.uniform(-8, 8, v).astype(np.float32)
    kw = dict(temperature=0.8, top_k=40, top_p=0.9, min_p=0.02, seed=0xDEADBEEF)
    lp, op = both_params(**kw)
    near = 0
    for step in range(64):
        got, _ = _draw(sampler, x, np.zeros(v, np.uint32), lp, step)
        d = O.sample(x, None, op, step)
        assert got in d.kept_ids
        assert got == d.chosen, step
        m = O.sample(x, None, op, step, exp_mode=O.EXP_LIBM)
        if got != m.chosen:
            assert min(d.gap, m.gap) < 1e-6
            near += 1
    print("draws within 1e-6 of a boundary against the libm oracle:", near)


def test_full_vocabulary_top_p_and_seed_replay(sampler):
    rng = np.random.default_rng(11)
    v = 700
    x = rng.uniform(-3, 3, v).astype(np.float32)
    lp, op = both_params(temperature=1.0, top_k=0, top_p=0.5, seed=99)
    a, _ = _draw(sampler, x, None, lp, 3)
    b, _ = _draw(sampler, x, None, lp, 3)
    assert a == b
    d = O.sample(x, None, op, 3)
    assert a == d.chosen and d.n_kept < v


def test_penalties_suppress_repeated_ids_and_update_counts(sampler, kat):
    k = kat["penalties"]
    x = np.zeros(k["v"], np.float32)
    for i, v in k["set"].items():
        x[int(i)] = v
    counts = np.zeros(k["v"], np.uint32)
    for i, c in k["counts"].items():
        counts[int(i)] = c
    lp = ls_params(presence_penalty=k["presence"], frequency_penalty=k["frequency"],
                   repetition_penalty=k["repetition"])
    got, after = _draw(sampler, x, counts, lp, 0)
    assert got == k["expect_id"]
    for i, c in k["counts_after"].items():
        assert after[int(i)] == c
    assert after.sum() == counts.sum() + 1


def test_penalty_counts_move_between_samplers_whole(sampler, kat):
    k = kat["counts_move"]
    v = k["v"]
    engine = LS.SamplerScratch(sampler, v)
    slot = LS.SamplerScratch(sampler, v)
    counts = np.zeros(v, np.int32)
    for i, c in k["counts"].items():
        counts[int(i)] = c
    engine.write_counts(torch.from_numpy(counts))
    slot.write_counts(torch.full((v,), k["stale"], dtype=torch.int32))
    slot.copy_counts_from(engine)
    assert np.array_equal(slot.read_counts().numpy(), counts)
    engine.reset_counts()
    assert slot.read_counts()[v - 1] == 5
    assert engine.read_counts().sum() == 0
    slot.uncount(7)
    slot.uncount(8)        # saturating
    slot.uncount(v + 3)    # out of range: ignored
    engine.copy_counts_from(slot)
    e = engine.read_counts().numpy()
    assert e[7] == 1 and e[8] == 0 and e.sum() == 6
    other = LS.SamplerScratch(sampler, v + 1)
    with pytest.raises(LS.SamplerError) as err:
        other.copy_counts_from(engine)
    assert err.value.code == -3 and "different vocabularies" in str(err.value)
    for s in (engine, slot, other):
        s.close()


def _draft_and_spec(sampler, trunk, head, lp, step, dists=None):
    v = trunk.size
    t_trunk = torch.from_numpy(trunk).to(dev())
    t_head = torch.from_numpy(head).to(dev())
    scratch = LS.SamplerScratch(sampler, v)
    own = dists is None
    if own:
        dists = LS.DraftDists(sampler, 2)
    dist = dists.slot(1)
    drafted = torch.zeros(1, dtype=torch.int32, device=dev())
    out = torch.zeros(1, dtype=torch.int32, device=dev())
    dp = LS.draft_params(lp)
    sampler.sample_draft_f32(t_head, scratch, dp, LS.draft_step(step), drafted, dist)
    sampler.sample_spec_f32(t_trunk, scratch, lp, step, dist, drafted, out)
    sampler.synchronize()
    ids, probs = dists.read(1)
    scratch.close()
    if own:
        dists.close()
    return int(drafted.item()), int(out.item()), ids.numpy().astype(np.int64), probs.numpy()


def test_draft_draw_exports_the_kept_distribution(sampler):
    rng = np.random.default_rng(21)
    v = 5003
    head = rng.uniform(-8, 8, v).astype(np.float32)
    trunk = (head + rng.uniform(-1, 1, v)).astype(np.float32)
    kw = dict(temperature=1.0, top_k=20, top_p=0.95, seed=5)
    lp, op = both_params(**kw)
    d, _, ids, q = _draft_and_spec(sampler, trunk, head, lp, 4)
    want_ids, want_q = O.kept(head, O.draft_params(op))
    assert np.array_equal(ids, want_ids.astype(np.int64))
    assert np.array_equal(q.view(np.uint32), want_q.view(np.uint32))
    assert d in ids
    lib_ids, lib_q = O.kept(head, O.draft_params(op), exp_mode=O.EXP_LIBM)
    assert np.array_equal(ids, lib_ids.astype(np.int64)) and np.max(np.abs(q - lib_q)) < 1e-5


def test_speculative_draw_matches_the_cpu_reference(sampler):
    rng = np.random.default_rng(23)
    v = 4099
    head = rng.uniform(-6, 6, v).astype(np.float32)
    trunk = (head + rng.uniform(-2.5, 2.5, v)).astype(np.float32)
    cases = (
        ("server defaults", dict(temperature=1.0, top_k=20, top_p=0.95, seed=77)),
        ("wide", dict(temperature=1.3, top_k=0, top_p=1.0, min_p=0.001, seed=78)),
    )
    dists = LS.DraftDists(sampler, 2)
    for name, kw in cases:
        lp, op = both_params(**kw)
        p_ids, p_pr = O.kept(trunk, op)
        q_ids, q_pr = O.kept(head, O.draft_params(op))
        accepted = 0
        for step in range(96):
            d, got, _, _ = _draft_and_spec(sampler, trunk, head, lp, step, dists)
            assert d == O.sample(head, None, O.draft_params(op), O.lib().lo_draft_step(step)).chosen
            want, acc, zero, gap = O.spec(p_ids, p_pr, q_ids, q_pr, d, op.seed, step)
            assert got in p_ids
            assert zero or got == want, (name, step, got, want)
            accepted += got == d
        assert 0 < accepted < 96, (name, accepted)
    dists.close()


def test_speculative_draw_with_given_uniforms(sampler):
    """The two draws given instead of seeded (accept test on u1, residual draw on u2,
    sample.metal:626-651): every pair agrees with cpu_spec, including the corners u1 = 0
    (accepts whenever p(d) > 0) and u2 just below 1 (the last residual entry)."""
    rng = np.random.default_rng(29)
    v = 4099
    head = rng.normal(0, 2.5, v).astype(np.float32)
    trunk = (head + rng.normal(0, 0.6, v)).astype(np.float32)
    kw = dict(temperature=1.0, top_k=20, top_p=0.95, seed=3)
    lp, op = both_params(**kw)
    p_ids, p_pr = O.kept(trunk, op)
    q_ids, q_pr = O.kept(head, O.draft_params(op))
    t_trunk = torch.from_numpy(trunk).to(dev())
    t_head = torch.from_numpy(head).to(dev())
    scratch = LS.SamplerScratch(sampler, v)
    dists = LS.DraftDists(sampler, 1)
    dist = dists.slot(0)
    drafted = torch.zeros(1, dtype=torch.int32, device=dev())
    out = torch.zeros(1, dtype=torch.int32, device=dev())
    # a draft step whose proposal the trunk keeps with p(d) < q(d): both outcomes occur
    pd, qd = dict(zip(p_ids.tolist(), p_pr.tolist())), dict(zip(q_ids.tolist(), q_pr.tolist()))
    def proposal(t):
        return O.sample(head, None, O.draft_params(op), O.lib().lo_draft_step(t)).chosen

    dstep = next(t for t in range(200) if 0.0 < pd.get(proposal(t), 0.0) < 0.7 * qd[proposal(t)])
    sampler.sample_draft_f32(t_head, scratch, LS.draft_params(lp), LS.draft_step(dstep), drafted,
                             dist)
    sampler.synchronize()
    d = int(drafted.item())
    pairs = [(0.0, 0.0), (0.0, 0.99999994), (0.99999994, 0.0), (0.99999994, 0.99999994)]
    pairs += [(float(a), float(b)) for a, b in rng.random((60, 2)).astype(np.float32)]
    outcomes = set()
    for u1, u2 in pairs:
        sampler.sample_spec_f32(t_trunk, scratch, lp, 5, dist, drafted, out, uniforms=(u1, u2))
        sampler.synchronize()
        want, acc, zero, gap = O.spec(p_ids, p_pr, q_ids, q_pr, d, op.seed, 5, u1=u1, u2=u2)
        assert not zero
        assert int(out.item()) == want, (u1, u2, int(out.item()), want)
        outcomes.add(acc)
    assert outcomes == {True, False}
    for bad in ((1.0, 0.5), (0.5, -0.1), (float("nan"), 0.5)):
        with pytest.raises(LS.SamplerError):
            sampler.sample_spec_f32(t_trunk, scratch, lp, 5, dist, drafted, out, uniforms=bad)
    scratch.close()
    dists.close()


def test_massless_residual_draws_from_the_trunk_on_the_second_uniform(sampler):
    """A rejected proposal whose residual has no mass: the kernel draws from p on the second
    uniform (sample.metal:650-651) where the CPU test takes p's last entry
    (tests/unit/kernels/sample.rs:282).  Exact arithmetic never gets there (p <= q on p's
    support with sum 1 forces q == p, which always accepts), so the exported distribution is
    written by hand: q == p except q(d) = 2 p(d), and u1 = 0.75 rejects.  The oracle reports
    the case; the draw must be the plain inverse-CDF pick of u2 over the trunk's kept set."""
    rng = np.random.default_rng(31)
    v = 2048
    row = rng.uniform(-4, 4, v).astype(np.float32)
    kw = dict(temperature=1.0, top_k=12, top_p=1.0, seed=9)
    lp, op = both_params(**kw)
    t_row = torch.from_numpy(row).to(dev())
    scratch = LS.SamplerScratch(sampler, v)
    dists = LS.DraftDists(sampler, 1)
    dist = dists.slot(0)
    out = torch.zeros(1, dtype=torch.int32, device=dev())
    p_ids, p_pr = O.kept(row, op)
    for which in (0, 5, len(p_ids) - 1):
        d = int(p_ids[which])
        q_pr = p_pr.copy()
        q_pr[which] = np.float32(2.0) * p_pr[which]
        dists.write(0, p_ids, q_pr)
        drafted = torch.tensor([d], dtype=torch.int32, device=dev())
        for u2 in (0.0, 0.3, 0.77, 0.99999994):
            sampler.sample_spec_f32(t_row, scratch, lp, 0, dist, drafted, out, uniforms=(0.75, u2))
            sampler.synchronize()
            want, acc, zero, gap = O.spec(p_ids, p_pr, p_ids, q_pr, d, op.seed, 0, u1=0.75, u2=u2)
            assert zero and not acc
            plain = O.sample(row, None, op, 0, uniform=u2)
            assert int(out.item()) == plain.chosen, (which, u2, int(out.item()), plain.chosen)
        # the same hand-written q accepts below one half
        sampler.sample_spec_f32(t_row, scratch, lp, 0, dist, drafted, out, uniforms=(0.25, 0.5))
        sampler.synchronize()
        assert int(out.item()) == d
    scratch.close()
    dists.close()


def test_speculative_draw_is_distributed_as_the_trunk(sampler):
    rng = np.random.default_rng(25)
    v = 48
    head = rng.uniform(-2, 2, v).astype(np.float32)
    trunk = (head + rng.uniform(-1.5, 1.5, v)).astype(np.float32)
    lp, op = both_params(temperature=1.0, top_k=0, top_p=1.0, seed=31)
    p_ids, p_pr = O.kept(trunk, op)
    q_ids, q_pr = O.kept(head, op)
    qd = dict(zip(q_ids.tolist(), q_pr.tolist()))
    overlap = sum(min(float(x), qd.get(int(i), 0.0)) for i, x in zip(p_ids, p_pr))
    n = 8192
    t_trunk = torch.from_numpy(trunk).to(dev())
    t_head = torch.from_numpy(head).to(dev())
    scratch = LS.SamplerScratch(sampler, v)
    dists = LS.DraftDists(sampler, 1)
    dist = dists.slot(0)
    drafted = torch.zeros(n, dtype=torch.int32, device=dev())
    outs = torch.zeros(n, dtype=torch.int32, device=dev())
    for step in range(n):
        sampler.sample_draft_f32(t_head, scratch, lp, LS.draft_step(step), drafted[step:step + 1], dist)
        sampler.sample_spec_f32(t_trunk, scratch, lp, step, dist, drafted[step:step + 1],
                                outs[step:step + 1])
    sampler.synchronize()
    d = drafted.cpu().numpy()
    got = outs.cpu().numpy()
    hist = np.bincount(got, minlength=v)
    chi2 = 0.0
    for i, x in zip(p_ids, p_pr):
        e = float(x) * n
        chi2 += (hist[i] - e) ** 2 / e
        assert abs(hist[i] / n - float(x)) < 0.02
    assert chi2 < 82.0
    assert abs(float(np.mean(d == got)) - overlap) < 0.03
    # and every one of the 8192 draws equals the oracle's
    for step in range(0, n, 37):
        want = O.spec(p_ids, p_pr, q_ids, q_pr, int(d[step]), op.seed, step)
        assert want[2] or got[step] == want[0]
    scratch.close()
    dists.close()


def test_accept_counts_leading_matches_and_describes_the_chain(sampler, kat):
    k = kat["spec_accept"]
    for case in k["cases"]:
        ctrl = torch.zeros(LS.ctrl_words(k["chain"]), dtype=torch.int32, device=dev())
        sampler.spec_accept(_i32(case["draws"]), _i32(case["ids"]), ctrl, k["pos0"], k["ratio"],
                            k["chain"])
        sampler.synchronize()
        words = ctrl.cpu().numpy()
        want = O.spec_accept(case["draws"], case["ids"], k["pos0"], k["ratio"], k["chain"])
        assert np.array_equal(words.view(np.uint32), want)
        assert words[LS.SLOT_ACCEPTED * LS.CTRL_STRIDE] == case["a"]
        assert words[LS.SLOT_KEEP * LS.CTRL_STRIDE] == case["a"] + 1
        for i in range(k["chain"]):
            p = k["pos0"] + case["a"] + 1 + i
            assert words[LS.slot_pos(i) * LS.CTRL_STRIDE] == p
            assert words[LS.slot_block(i) * LS.CTRL_STRIDE] == p // k["ratio"]
            assert words[LS.slot_count(i) * LS.CTRL_STRIDE] == int((p + 1) % k["ratio"] == 0)
    with pytest.raises(LS.SamplerError):
        sampler.spec_accept(_i32([1]), _i32([1]), torch.zeros(4, dtype=torch.int32, device=dev()),
                            0, 4, 3)
    with pytest.raises(LS.SamplerError):
        sampler.spec_accept(_i32([1]), _i32([1]),
                            torch.zeros(8, dtype=torch.int32, device=dev()), 0, 0, 0)


def test_copy_row_reads_a_gpu_supplied_index(sampler):
    rows, words = 3, 300
    src = (np.arange(rows * words, dtype=np.int64) * 7 + 1).astype(np.int32).reshape(rows, words)
    src_t = torch.from_numpy(src).to(dev())
    m = 4
    for wanted in (0, 2, 3, 4):
        dst = torch.full((words,), 0x5EADBEEF, dtype=torch.int32, device=dev())
        draws = [100 + j if j < wanted else 0 for j in range(m)]
        ids = [1] + [100 + j for j in range(m - 1)]
        ctrl = torch.zeros(LS.ctrl_words(0), dtype=torch.int32, device=dev())
        sampler.spec_accept(_i32(draws), _i32(ids), ctrl, 0, 4, 0)
        sampler.copy_row(src_t, ctrl[0:1], dst)
        sampler.synchronize()
        a = int(ctrl[0].item())
        assert a == min(wanted, m - 1)
        got = dst.cpu().numpy()
        if a < rows:
            assert np.array_equal(got, src[a])
        else:
            assert np.all(got == 0x5EADBEEF)


def test_error_behaviour(sampler):
    v = 1000
    x = torch.zeros(v, device=dev())
    out = torch.zeros(1, dtype=torch.int32, device=dev())
    wrong = LS.SamplerScratch(sampler, v + 1)
    with pytest.raises(LS.SamplerError) as e:
        sampler.sample_f32(x, wrong, ls_params(temperature=0.7, top_k=5), 0, out)
    assert e.value.code == -3
    for bad in (dict(temperature=-1.0), dict(temperature=0.7, top_p=0.0),
                dict(temperature=0.7, min_p=2.0), dict(repetition_penalty=0.0),
                dict(presence_penalty=float("inf"))):
        with pytest.raises(LS.SamplerError) as e:
            sampler.sample_f32(x, None, ls_params(**bad), 0, out)
        assert e.value.code == -2
    with pytest.raises(LS.SamplerError):  # penalties need a scratch
        sampler.sample_f32(x, None, ls_params(presence_penalty=0.5), 0, out)
    wrong.close()


def test_rows_that_share_a_scratch(sampler):
    """A row touches its scratch only under penalties: a scratch may stand in several rows of one
    call as long as at most one of them uses penalties - in either order; two penalised rows on
    one scratch would count into one histogram at once and are refused."""
    rng = np.random.default_rng(61)
    v = 4096
    x = rng.normal(0, 2, (3, v)).astype(np.float32)
    hist = rng.integers(0, v, 100).astype(np.int32)
    hist[:5] = np.argsort(-x[1])[:5]
    plain = dict(temperature=0.8, top_k=10, top_p=0.9, seed=4)
    pen = dict(plain, repetition_penalty=1.3, presence_penalty=0.5, frequency_penalty=0.2)
    t = torch.from_numpy(x).to(dev())
    out = torch.zeros(3, dtype=torch.int32, device=dev())
    for kws in ([plain, pen, plain], [pen, plain, plain], [plain, plain, pen]):
        sc = LS.SamplerScratch(sampler, v)
        sc.add_history(torch.from_numpy(hist).to(dev()))
        counts = np.bincount(hist, minlength=v).astype(np.uint32)
        sampler.sample_rows(t, [ls_params(**kw) for kw in kws], [2, 2, 2], out, scratch=[sc, sc, sc])
        sampler.synchronize()
        got = out.cpu().numpy()
        for r, kw in enumerate(kws):
            d = O.sample(x[r], counts if kw is pen else None, o_params(**kw), 2)   # bumps counts under penalties
            assert got[r] == d.chosen, (r, got[r], d.chosen)
        assert np.array_equal(sc.read_counts().numpy().view(np.uint32), counts)
        sc.close()
    sc = LS.SamplerScratch(sampler, v)
    with pytest.raises(LS.SamplerError) as e:
        sampler.sample_rows(t, [ls_params(**pen), ls_params(**plain), ls_params(**pen)], [0, 0, 0], out,
                            scratch=[sc, sc, sc])
    assert e.value.code == -1 and "share a scratch" in str(e.value)
    sampler.synchronize()
    sc.close()
