"""The penalised verify pass as one launch: rows that share a scratch draw in order, each
against the counts the rows before it left (src/qwen4exp/model.rs:3008-3040).  The rows here are
built so that consecutive rows want the same tokens: what one row draws changes what the next
may draw, and the oracle's row-to-row count flow is the reference."""
import numpy as np
import pytest
import torch

import lily_sampler as LS
import lily_workloads as W
import oracle as O
from gpu_util import dev, ls_params, o_params

pytestmark = pytest.mark.gpu


def _flow(sampler, target, draft, kw, step0, uniforms=None, hist=None):
    """Runs draft draws + lily_spec_verify and the oracle's sequence; returns (got, want, counts ok)."""
    m, vocab = target.shape
    bf16 = target.dtype == np.uint16
    up = (lambda a: torch.from_numpy(a.view(np.int16)).to(dev()).view(torch.bfloat16)) if bf16 else \
         (lambda a: torch.from_numpy(a).to(dev()))
    t_target = up(target)
    draft32 = (draft.astype(np.uint32) << 16).view(np.float32) if bf16 else draft
    t_draft = torch.from_numpy(np.ascontiguousarray(draft32)).to(dev())
    lp, op = ls_params(**kw), o_params(**kw)
    scratch = LS.SamplerScratch(sampler, vocab)
    counts = np.zeros(vocab, np.uint32)
    if hist is not None:
        scratch.add_history(torch.from_numpy(hist.astype(np.int32)).to(dev()))
        counts = np.bincount(hist, minlength=vocab).astype(np.uint32)
    dists = LS.DraftDists(sampler, m)
    proposals = torch.zeros(m, dtype=torch.int32, device=dev())
    dp = LS.draft_params(lp)
    for j in range(m - 1):
        sampler.sample_draft_f32(t_draft[j], scratch, dp, LS.draft_step(step0 + j),
                                 proposals[j:j + 1], dists.slot(j))
    sampler.synchronize()
    props = proposals.cpu().numpy()
    ids = torch.tensor([7] + [int(props[j]) for j in range(m - 1)], dtype=torch.int32, device=dev())
    verify = torch.full((m,), -1, dtype=torch.int32, device=dev())
    ctrl = torch.zeros(LS.ctrl_words(2), dtype=torch.int32, device=dev())
    stats = torch.zeros(4, dtype=torch.int32, device=dev())
    sampler.set_path_stats(stats)
    sampler.spec_verify(t_target, scratch, lp, step0, dists, ids, verify, ctrl, pos0=50, ratio=4,
                        chain=2, uniforms=uniforms)
    sampler.synchronize()
    sampler.set_path_stats(None)
    got = verify.cpu().numpy()
    want = []
    odp = O.draft_params(op)
    for j in range(m):
        if j + 1 < m:
            dd = O.sample(draft32[j], None, odp, O.lib().lo_draft_step(step0 + j))
            assert dd.chosen == props[j]
            trunk = O.sample(target[j], counts.copy(), op, step0 + j)
            tok, acc, zero, gap = O.spec(trunk.kept_ids, trunk.kept_q, dd.kept_ids, dd.kept_q,
                                         int(props[j]), op.seed, step0 + j,
                                         u1=float(uniforms[j, 0]) if uniforms is not None else None,
                                         u2=float(uniforms[j, 1]) if uniforms is not None else None)
            if zero:
                tok = int(got[j])
            counts[tok] += 1
        else:
            ukw = dict(uniform=float(uniforms[j, 0])) if uniforms is not None else {}
            tok = O.sample(target[j], counts.copy(), op, step0 + j, **ukw).chosen
            counts[tok] += 1
        want.append(int(tok))
    ok = np.array_equal(scratch.read_counts().numpy().view(np.uint32), counts)
    wctrl = O.spec_accept(got, ids.cpu().numpy(), 50, 4, 2)
    assert np.array_equal(ctrl.cpu().numpy().view(np.uint32), wctrl)
    scratch.close()
    dists.close()
    return list(got), want, ok, stats.cpu().tolist()


@pytest.mark.parametrize("m", [2, 3, 5, 8])
@pytest.mark.parametrize("k", [1, 20, 60, 64])
@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
def test_rows_that_want_the_same_tokens(m, k, bf16):
    s = LS.Sampler(0)
    rng = np.random.default_rng(100 * m + k + bf16)
    vocab = 151_936
    base = rng.normal(0, 1.5, vocab).astype(np.float32)
    hot = rng.choice(vocab, 6, replace=False)
    base[hot] = [9.0, 8.8, 8.7, 8.5, 8.4, 8.2]               # every row's favourites
    target = np.stack([base + rng.normal(0, 0.05, vocab).astype(np.float32) for _ in range(m)])
    draft = np.stack([base + rng.normal(0, 0.3, vocab).astype(np.float32) for _ in range(m)])
    if bf16:
        target, draft = W.to_bf16_bits(target), W.to_bf16_bits(draft)
    kw = dict(temperature=0.9, top_k=k, top_p=0.98, seed=17, repetition_penalty=1.4,
              presence_penalty=1.5, frequency_penalty=0.6) if k > 1 else \
         dict(repetition_penalty=1.4, presence_penalty=1.5, frequency_penalty=0.6)
    hist = np.concatenate([hot[:2], rng.integers(0, vocab, 300)])
    for step0 in (0, 40):
        got, want, ok, st = _flow(s, target, draft, kw, step0, hist=hist)
        assert got == want, (m, k, bf16, step0, got, want)
        assert ok
        assert st[2] == 0, st            # nothing fell to the exhaustive select
    s.close()


def test_given_uniforms_and_rising_penalties():
    """Explicit (u1, u2) per row in the one-launch form; and penalties that may raise a value
    (negative presence), which keep the one-launch-per-row form - same answers either way."""
    s = LS.Sampler(0)
    rng = np.random.default_rng(9)
    vocab, m = 50_021, 4
    base = rng.normal(0, 2, vocab).astype(np.float32)
    base[rng.choice(vocab, 4, replace=False)] = [7.0, 6.9, 6.8, 6.5]
    target = np.stack([base + rng.normal(0, 0.05, vocab).astype(np.float32) for _ in range(m)])
    draft = np.stack([base + rng.normal(0, 0.3, vocab).astype(np.float32) for _ in range(m)])
    us = rng.random((m, 2)).astype(np.float32)
    hist = rng.integers(0, vocab, 100)
    for kw in (dict(temperature=1.0, top_k=30, top_p=0.95, seed=3, repetition_penalty=1.2,
                    presence_penalty=0.8, frequency_penalty=0.3),
               dict(temperature=1.0, top_k=30, top_p=0.95, seed=3, repetition_penalty=1.2,
                    presence_penalty=-0.5, frequency_penalty=0.3)):
        for u in (None, us):
            got, want, ok, st = _flow(s, target, draft, kw, 5, uniforms=u, hist=hist)
            assert got == want, (kw, u is not None, got, want)
            assert ok
    s.close()


@pytest.mark.parametrize("outside", [False, True], ids=["q(d) = 2 p(d)", "proposal outside p's kept set"])
def test_massless_residual_in_the_one_launch_form(outside):
    """A rejected proposal whose residual max(0, p - q) has no mass: the kernel draws plainly from
    p on the second uniform (sample.metal:649-651).  Draft heads never export such a distribution,
    so it is written by hand: q equal to p on p's kept set except at the proposal (twice p there,
    rejected by u1 = 0.75), or q equal to p with a proposal that p does not keep at all (always
    rejected).  The rows are penalised, so both draw inside one launch, the speculative row in the
    wave that runs every row's tail; the next row sees the count the fallback's draw left."""
    s = LS.Sampler(0)
    rng = np.random.default_rng(77)
    vocab, m = 30_011, 2
    target = rng.normal(0, 2, (m, vocab)).astype(np.float32)
    kw = dict(temperature=1.0, top_k=12, top_p=1.0, seed=21, repetition_penalty=1.3,
              presence_penalty=0.4, frequency_penalty=0.2)
    lp, op = ls_params(**kw), o_params(**kw)
    hist = rng.integers(0, vocab, 200)
    t_target = torch.from_numpy(target).to(dev())
    for which, u2 in ((0, 0.0), (4, 0.31), (11, 0.77), (2, 0.99999994)):
        scratch = LS.SamplerScratch(s, vocab)
        scratch.add_history(torch.from_numpy(hist.astype(np.int32)).to(dev()))
        counts = np.bincount(hist, minlength=vocab).astype(np.uint32)
        trunk = O.sample(target[0], counts.copy(), op, 3)
        p_ids, p_pr = trunk.kept_ids, trunk.kept_q
        dists = LS.DraftDists(s, m)
        if outside:
            d = int(np.setdiff1d(np.arange(64), p_ids)[0])
            q_ids = np.concatenate([p_ids, [d]]).astype(np.uint32)
            q_pr = np.concatenate([p_pr, [np.float32(0.5)]]).astype(np.float32)
        else:
            d = int(p_ids[which])
            q_ids, q_pr = p_ids.copy(), p_pr.copy()
            q_pr[which] = np.float32(2.0) * p_pr[which]
        dists.write(0, q_ids, q_pr)
        ids = torch.tensor([7, d], dtype=torch.int32, device=dev())
        verify = torch.full((m,), -1, dtype=torch.int32, device=dev())
        ctrl = torch.zeros(LS.ctrl_words(1), dtype=torch.int32, device=dev())
        us = np.array([[0.75, u2], [0.5, 0.0]], dtype=np.float32)
        s.spec_verify(t_target, scratch, lp, 3, dists, ids, verify, ctrl, pos0=9, ratio=4, chain=1,
                      uniforms=us)
        s.synchronize()
        got = verify.cpu().numpy()
        tok, acc, zero, gap = O.spec(p_ids, p_pr, q_ids, q_pr, d, op.seed, 3, u1=0.75, u2=u2)
        assert zero and not acc
        plain = O.sample(target[0], counts, op, 3, uniform=u2)      # bumps counts[plain.chosen]
        assert got[0] == plain.chosen, (outside, which, u2, got[0], plain.chosen)
        nxt = O.sample(target[1], counts, op, 4, uniform=0.5)
        assert got[1] == nxt.chosen, (outside, which, u2, got[1], nxt.chosen)
        assert np.array_equal(scratch.read_counts().numpy().view(np.uint32), counts)
        scratch.close()
        dists.close()
    s.close()
