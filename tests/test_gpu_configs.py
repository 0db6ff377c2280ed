"""The five BASELINE configurations on the HIP path against the CPU oracle.

Bar: token ids, top-k index sets (in order) and kept counts bit-exact against the
oracle with the shared expf; candidate probabilities bit-exact too.  Against the oracle
with the C library's expf (the reference's libm stand-in) ids may differ only where the
draw lies within 1e-6 of a cumulative-mass boundary; such rows are counted and printed.
Log-probabilities: |gpu - f64 oracle| <= 1e-5 * max(1, |logprob|).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import lily_sampler as LS
import lily_workloads as W
import oracle as O
from gpu_util import check_row_against_oracle, dev, ls_params, o_params, run_rows

LOGPROB_RTOL = 1e-5


@pytest.fixture(scope="module")
def sampler():
    s = LS.Sampler(0)
    yield s
    s.close()


def _scratches(sampler, history, vocab):
    out = []
    for h in history:
        sc = LS.SamplerScratch(sampler, vocab)
        sc.add_history(torch.from_numpy(np.ascontiguousarray(h)).to(dev()))
        out.append(sc)
    return out


def _counts_of(h, vocab):
    return np.bincount(h, minlength=vocab).astype(np.uint32)


def _libm_report(name, rows, near):
    print(f"{name}: {rows} rows, {near} within 1e-6 of a boundary against the libm oracle")


@pytest.mark.parametrize("vocab", [W.VOCAB, 6007])
def test_config1_single_row_greedy_and_sampled(sampler, vocab):
    c = W.config1(vocab=vocab)
    x = c["logits"]
    g = run_rows(sampler, x, [dict()], [0])
    assert g.ids[0] == O.argmax(x[0])
    r = run_rows(sampler, x, [c["params"]], [0], uniforms=[c["uniform"]])
    d = O.sample(x[0], None, o_params(**c["params"]), 0, uniform=c["uniform"])
    check_row_against_oracle(r, 0, d)
    m = O.sample(x[0], None, o_params(**c["params"]), 0, uniform=c["uniform"], exp_mode=O.EXP_LIBM)
    assert r.ids[0] == m.chosen or min(d.gap, m.gap) < 1e-6
    # seeded: 32 steps of the same row
    near = 0
    for step in range(32):
        kw = dict(c["params"], seed=123)
        r = run_rows(sampler, x, [kw], [step])
        d = O.sample(x[0], None, o_params(**kw), step)
        check_row_against_oracle(r, 0, d)
        m = O.sample(x[0], None, o_params(**kw), step, exp_mode=O.EXP_LIBM)
        if r.ids[0] != m.chosen:
            assert min(d.gap, m.gap) < 1e-6
            near += 1
    _libm_report("config1", 32, near)


@pytest.mark.parametrize("use_plan", [False, True])
def test_config2_batch_of_four_with_penalties(sampler, use_plan):
    c = W.config2()
    x, hist = c["logits"], c["history"]
    rows, vocab = x.shape
    sc = _scratches(sampler, hist, vocab)
    counts = [_counts_of(h, vocab) for h in hist]
    near = 0
    for step in range(3):  # three decode steps: the counts evolve with the draws
        r = run_rows(sampler, x, c["params"], [step] * rows, scratch=sc, use_plan=use_plan)
        for i in range(rows):
            before = counts[i].copy()
            d = O.sample(x[i], counts[i], o_params(**c["params"][i]), step)
            check_row_against_oracle(r, i, d)
            m = O.sample(x[i], before, o_params(**c["params"][i]), step, exp_mode=O.EXP_LIBM)
            if r.ids[i] != m.chosen:
                assert min(d.gap, m.gap) < 1e-6
                near += 1
        for i in range(rows):
            assert np.array_equal(sc[i].read_counts().numpy().view(np.uint32), counts[i])
    _libm_report("config2", 3 * rows, near)
    for s in sc:
        s.close()


@pytest.mark.parametrize("given", [False, True])
def test_config3_speculative_verify(sampler, given):
    """given: the configuration's fixed (u1, u2) per position replace the seeded draws
    (accept test and plain draw on u1, residual draw on u2: sample.metal:626-651)."""
    c = W.config3()
    us = c["u"] if given else None
    target, draft = c["target"], c["draft"]
    m, vocab = target.shape
    t_target = torch.from_numpy(target).to(dev())
    t_draft = torch.from_numpy(draft).to(dev())
    pending = 42
    for kw, step0 in ((dict(), 0), (c["params"], 10),
                      (dict(c["params"], presence_penalty=0.4, repetition_penalty=1.1), 20)):
        lp, op = ls_params(**kw), o_params(**kw)
        scratch = LS.SamplerScratch(sampler, vocab)
        dists = LS.DraftDists(sampler, m)
        proposals = torch.zeros(m, dtype=torch.int32, device=dev())
        dp = LS.draft_params(lp)
        # the draft head's draws: proposal j is checked by verify row j (draw index step0 + j)
        for j in range(m - 1):
            sampler.sample_draft_f32(t_draft[j], scratch, dp, LS.draft_step(step0 + j),
                                     proposals[j:j + 1], dists.slot(j))
        sampler.synchronize()
        props = proposals.cpu().numpy()
        ids = torch.tensor([pending] + [int(props[j]) for j in range(m - 1)], dtype=torch.int32,
                           device=dev())
        verify = torch.zeros(m, dtype=torch.int32, device=dev())
        ctrl = torch.zeros(LS.ctrl_words(2), dtype=torch.int32, device=dev())
        sampler.spec_verify(t_target, scratch, lp, step0, dists, ids, verify, ctrl, pos0=100,
                            ratio=4, chain=2, uniforms=us)
        sampler.synchronize()
        got = verify.cpu().numpy()
        # oracle: the same sequence with the counts flowing from row to row
        counts = np.zeros(vocab, np.uint32)
        want = []
        odp = O.draft_params(op)
        for j in range(m):
            if j + 1 < m and O.lib().lo_samples(op):
                dd = O.sample(draft[j], None, odp, O.lib().lo_draft_step(step0 + j))
                assert dd.chosen == props[j]
                trunk = O.sample(target[j], counts.copy(), op, step0 + j)
                tok, acc, zero, gap = O.spec(trunk.kept_ids, trunk.kept_q, dd.kept_ids, dd.kept_q,
                                             int(props[j]), op.seed, step0 + j,
                                             u1=float(us[j, 0]) if given else None,
                                             u2=float(us[j, 1]) if given else None)
                if zero:
                    tok = int(got[j])
                if O.lib().lo_uses_penalties(op):
                    counts[tok] += 1
            else:
                if j + 1 < m:
                    assert props[j] == O.argmax(draft[j])
                ukw = dict(uniform=float(us[j, 0])) if given and O.lib().lo_samples(op) else {}
                tok = O.sample(target[j], counts, op, step0 + j, **ukw).chosen
            want.append(tok)
        assert list(got) == want, (kw, got, want)
        if O.lib().lo_uses_penalties(op):
            assert np.array_equal(scratch.read_counts().numpy().view(np.uint32), counts)
        wctrl = O.spec_accept(got, ids.cpu().numpy(), 100, 4, 2)
        assert np.array_equal(ctrl.cpu().numpy().view(np.uint32), wctrl)
        scratch.close()
        dists.close()


def test_rollback_of_rejected_draws_on_the_device(sampler):
    """finish_speculation's rollback (src/qwen4exp/spec.rs:213-217) with the accepted row read
    from the control block on the device: the counts equal the oracle's uncount over
    sampled[accepted + 1:], the list the draws read stays consistent with them (a further
    penalised draw agrees with the oracle), and an earlier stop of the engine caps the row."""
    rng = np.random.default_rng(77)
    vocab = 151_936
    x = rng.normal(0, 3, (2, vocab)).astype(np.float32)
    kw = dict(temperature=0.7, top_k=20, top_p=0.95, seed=5, repetition_penalty=1.3,
              presence_penalty=0.5, frequency_penalty=0.25)
    hist = rng.integers(0, vocab, 600).astype(np.int32)
    top = np.argsort(-x[0])[:6].astype(np.int32)          # ids a penalised draw looks at
    hist[:12] = np.repeat(top[:4], 3)
    cases = [
        # draws, accepted word, cap
        ([int(top[0]), int(top[1]), int(top[1]), int(top[2])], 1, 0xFFFFFFFF),
        ([int(top[0]), int(top[1]), int(top[2]), int(top[3])], 3, 0xFFFFFFFF),   # all accepted
        ([int(top[0]), int(top[1]), int(top[2]), int(top[3])], 3, 0),            # engine stopped at row 0
        ([int(top[3]), vocab + 9, 12345, int(top[3])], 0, 0xFFFFFFFF),           # out of range, never counted
        ([int(top[0])], 0, 0xFFFFFFFF),                                          # one row: nothing after it
        ([int(top[5])] * 8, 2, 5),                                               # saturates at 0
    ]
    for draws, acc, cap in cases:
        sc = LS.SamplerScratch(sampler, vocab)
        sc.add_history(torch.from_numpy(hist).to(dev()))
        counts = np.bincount(hist, minlength=vocab).astype(np.uint32)
        m = len(draws)
        t_draws = torch.from_numpy(np.array(draws, dtype=np.uint32).view(np.int32)).to(dev())
        ctrl = torch.zeros(LS.ctrl_words(2), dtype=torch.int32, device=dev())
        ctrl[LS.SLOT_ACCEPTED * LS.CTRL_STRIDE] = acc
        sc.uncount_after(t_draws, ctrl[LS.SLOT_ACCEPTED * LS.CTRL_STRIDE:], cap)
        for t in draws[min(acc, cap) + 1:]:
            O.lib().lo_uncount(counts.ctypes.data, vocab, t)
        assert np.array_equal(sc.read_counts().numpy().view(np.uint32), counts), (draws, acc, cap)
        for step in (3, 4):
            r = run_rows(sampler, x[:1], [kw], [step], scratch=[sc])
            d = O.sample(x[0], counts, o_params(**kw), step)   # bumps counts[chosen] like the kernel
            check_row_against_oracle(r, 0, d)
        assert np.array_equal(sc.read_counts().numpy().view(np.uint32), counts)
        sc.close()
    with pytest.raises(LS.SamplerError):
        sc2 = LS.SamplerScratch(sampler, vocab)
        try:
            sc2.uncount_after(torch.zeros(9, dtype=torch.int32, device=dev()),
                              torch.zeros(1, dtype=torch.int32, device=dev()))
        finally:
            sc2.close()


def test_config4_constrained_bf16(sampler):
    c = W.config4(rows=64)
    x = c["logits"]
    rows, vocab = x.shape
    r = run_rows(sampler, x, c["params"], [7] * rows, allow=c["allow"], bias=c["bias"],
                 forced=c["forced"], logprobs=True)
    near = 0
    for i in range(rows):
        ext = dict(allow=c["allow"][i], bias=c["bias"][i], want_logprob=True)
        op = o_params(**c["params"][i])
        if c["forced"][i] is not None:
            d = O.sample(x[i], None, op, 7, forced=c["forced"][i], **ext)
            assert r.ids[i] == c["forced"][i]
        else:
            d = O.sample(x[i], None, op, 7, **ext)
            check_row_against_oracle(r, i, d)
            assert (c["allow"][i][r.ids[i] >> 5] >> (r.ids[i] & 31)) & 1
            m = O.sample(x[i], None, op, 7, exp_mode=O.EXP_LIBM, **ext)
            if r.ids[i] != m.chosen:
                assert min(d.gap, m.gap) < 1e-6
                near += 1
        if np.isfinite(d.logprob):
            assert abs(r.logprobs[i] - d.logprob) <= LOGPROB_RTOL * max(1.0, abs(d.logprob)), i
        else:
            assert r.logprobs[i] == -np.inf
    _libm_report("config4", rows, near)


def _check_config5_rows(sampler, c, pick, r, step):
    near = 0
    x, hist = c["logits"], c["history"]
    vocab = x.shape[1]
    for i in pick:
        counts = _counts_of(hist[i], vocab)
        op = o_params(**c["params"][i])
        d = O.sample(x[i], counts.copy(), op, step, want_logprob=True)
        check_row_against_oracle(r, i, d)
        assert abs(r.logprobs[i] - d.logprob) <= LOGPROB_RTOL * max(1.0, abs(d.logprob)), i
        m = O.sample(x[i], counts, op, step, exp_mode=O.EXP_LIBM)
        if r.ids[i] != m.chosen:
            assert min(d.gap, m.gap) < 1e-6
            near += 1
    return near


def test_config5_throughput_shape_against_the_oracle(sampler):
    rows = 96
    c = W.config5(rows=rows)
    x, hist = c["logits"], c["history"]
    vocab = x.shape[1]
    sc = _scratches(sampler, hist, vocab)
    r = run_rows(sampler, x, c["params"], [3] * rows, scratch=sc, logprobs=True)
    near = _check_config5_rows(sampler, c, range(rows), r, 3)
    _libm_report("config5", rows, near)
    for s in sc:
        s.close()


def test_config5_full_size_properties(sampler):
    """1024 x 151 936 bf16: replay determinism, membership, and 24 rows against the oracle."""
    rows = 1024
    c = W.config5(rows=rows)
    x, hist = c["logits"], c["history"]
    vocab = x.shape[1]
    logits = torch.from_numpy(x.view(np.int16)).to(dev()).view(torch.bfloat16)
    params = [ls_params(**kw) for kw in c["params"]]
    outs = []
    for rep in range(2):
        sc = _scratches(sampler, hist, vocab)
        out = torch.zeros(rows, dtype=torch.int32, device=dev())
        lp = torch.zeros(rows, dtype=torch.float32, device=dev())
        dbg_ids = torch.full((rows, 1024), -1, dtype=torch.int32, device=dev())
        dbg_probs = torch.zeros((rows, 1024), dtype=torch.float32, device=dev())
        dbg_counts = torch.zeros((rows, 2), dtype=torch.int32, device=dev())
        torch.cuda.synchronize()
        plan = sampler.plan(logits, params, [3] * rows, out, scratch=sc, out_logprobs=lp,
                            dbg_ids=dbg_ids, dbg_probs=dbg_probs, dbg_counts=dbg_counts)
        plan.run(0)
        sampler.synchronize()
        plan.close()
        outs.append((out.cpu().numpy(), lp.cpu().numpy(), dbg_ids.cpu().numpy(),
                     dbg_counts.cpu().numpy(), dbg_probs.cpu().numpy()))
        if rep == 0:
            # the emitted id was counted exactly once
            for i in (0, 511, 1023):
                after = sc[i].read_counts().numpy().view(np.uint32)
                want = _counts_of(hist[i], vocab)
                want[outs[0][0][i]] += 1
                assert np.array_equal(after, want)
        for s in sc:
            s.close()
    a, b = outs
    assert np.array_equal(a[0], b[0])           # token ids replay exactly
    # log-probabilities are sums whose order depends on wave arrival: equal to tolerance
    assert np.allclose(a[1], b[1], rtol=0, atol=2e-6)
    ids, lps, cand, cnt, probs = a
    assert np.all(cnt[:, 0] == 64) and np.all(cnt[:, 1] >= 1) and np.all(cnt[:, 1] <= 64)
    for i in range(rows):
        assert ids[i] in cand[i, : cnt[i, 1]]
        assert len(set(cand[i, :64].tolist())) == 64
    assert np.all(lps <= 0) and np.all(np.isfinite(lps))
    assert np.all(np.diff(probs[:, :64], axis=1) <= 0) and np.all(probs[:, 0] == 1.0)

    class R:
        pass

    r = R()
    r.ids, r.logprobs, r.cand_ids, r.cand_probs = ids.astype(np.int64), lps, cand, probs
    r.n_cand, r.n_kept = cnt[:, 0], cnt[:, 1]
    pick = np.random.default_rng(0).choice(rows, 24, replace=False)
    near = _check_config5_rows(sampler, c, pick, r, 3)
    _libm_report("config5 full size (24 rows checked)", rows, near)
