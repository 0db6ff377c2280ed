"""The hand-over from a verify pass to the draws that follow it without a host read between
(src/qwen4exp/spec.rs:356-528: the draft pass is encoded before the host knows how many rows
were accepted; its dispatches read the control block).  The reference checks that such a
GPU-selected pass does what the host-driven one does (tests/unit/qwen4exp/spec.rs:186-281);
the same check here for the sampler's share of it: verify -> spec_accept -> rollback of the
rejected rows' counts -> the next draws, (a) all enqueued back to back with rows and steps read
from the control block on the device, (b) driven by the host after reading the control block,
(c) the oracle's sequence."""
import numpy as np
import pytest
import torch

import lily_sampler as LS
import oracle as O
from gpu_util import dev, ls_params, o_params

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_selected_on_the_device_equals_driven_by_the_host(seed):
    s = LS.Sampler(0)
    rng = np.random.default_rng(seed)
    vocab, m, chain = 30_011, 4, 2
    base = rng.normal(0, 2, vocab).astype(np.float32)
    base[rng.choice(vocab, 3, replace=False)] = [8.0, 7.6, 7.2]
    target = np.stack([base + rng.normal(0, 0.3, vocab).astype(np.float32) for _ in range(m)])
    draft = np.stack([base + rng.normal(0, 0.6, vocab).astype(np.float32) for _ in range(m)])
    nxt = rng.normal(0, 2, (m, vocab)).astype(np.float32)     # what the head would see after row a
    kw = dict(temperature=0.9, top_k=30, top_p=0.95, seed=11, repetition_penalty=1.2,
              presence_penalty=0.7, frequency_penalty=0.2)
    lp, op = ls_params(**kw), o_params(**kw)
    step0, pos0, ratio = 6, 40, 4
    t_target, t_draft, t_next = (torch.from_numpy(a).to(dev()) for a in (target, draft, nxt))
    hist = rng.integers(0, vocab, 200)

    def one(device_selected):
        scratch = LS.SamplerScratch(s, vocab)
        scratch.add_history(torch.from_numpy(hist.astype(np.int32)).to(dev()))
        dists = LS.DraftDists(s, m)
        props = torch.zeros(m, dtype=torch.int32, device=dev())
        dp = LS.draft_params(lp)
        for j in range(m - 1):
            s.sample_draft_f32(t_draft[j], scratch, dp, LS.draft_step(step0 + j), props[j:j + 1], dists.slot(j))
        ids = torch.cat([torch.tensor([5], dtype=torch.int32, device=dev()), props[:m - 1]])
        verify = torch.full((m,), -1, dtype=torch.int32, device=dev())
        ctrl = torch.zeros(LS.ctrl_words(chain), dtype=torch.int32, device=dev())
        out = torch.full((2,), -1, dtype=torch.int32, device=dev())
        bonus = torch.full((1,), -1, dtype=torch.int32, device=dev())
        s.spec_verify(t_target, scratch, lp, step0, dists, ids, verify, ctrl, pos0=pos0, ratio=ratio, chain=chain)
        accepted_dev = ctrl[LS.SLOT_ACCEPTED * LS.CTRL_STRIDE:LS.SLOT_ACCEPTED * LS.CTRL_STRIDE + 1]
        if device_selected:
            # nothing below waits for the verify pass
            scratch.uncount_after(verify, accepted_dev)
            s.copy_row(verify.view(m, 1), accepted_dev, bonus)          # the token that stands
            s.sample_f32_at(t_next, accepted_dev, scratch, lp, step0 + 1, accepted_dev, out[0:1])
            s.sample_draft_f32_at(t_next, accepted_dev, scratch, dp, LS.draft_step(step0 + 1),
                                  accepted_dev, out[1:2], dists.slot(0))
            s.synchronize()
            a = int(ctrl.cpu()[LS.SLOT_ACCEPTED * LS.CTRL_STRIDE])
        else:
            s.synchronize()
            a = int(ctrl.cpu()[LS.SLOT_ACCEPTED * LS.CTRL_STRIDE])       # the host read
            drawn = verify.cpu().numpy()
            for tok in drawn[a + 1:]:
                scratch.uncount(int(tok))
            bonus[0] = int(drawn[a])
            s.sample_f32(t_next[a], scratch, lp, step0 + 1 + a, out[0:1])
            s.sample_draft_f32(t_next[a], scratch, dp, LS.draft_step(step0 + 1) + a, out[1:2], dists.slot(0))
            s.synchronize()
        res = (a, verify.cpu().tolist(), int(bonus.cpu()[0]), out.cpu().tolist(),
               scratch.read_counts().numpy().copy(), props.cpu().tolist())
        scratch.close()
        dists.close()
        return res

    a_dev, v_dev, b_dev, o_dev, c_dev, props = one(True)
    a_host, v_host, b_host, o_host, c_host, _ = one(False)
    assert (a_dev, v_dev, b_dev, o_dev) == (a_host, v_host, b_host, o_host)
    assert np.array_equal(c_dev, c_host)
    # and the oracle's sequence
    counts = np.bincount(hist, minlength=vocab).astype(np.uint32)
    odp = O.draft_params(op)
    want = []
    for j in range(m):
        if j + 1 < m:
            dd = O.sample(draft[j], None, odp, O.lib().lo_draft_step(step0 + j))
            trunk = O.sample(target[j], counts.copy(), op, step0 + j)
            tok, acc, zero, gap = O.spec(trunk.kept_ids, trunk.kept_q, dd.kept_ids, dd.kept_q,
                                         int(props[j]), op.seed, step0 + j)
            tok = v_dev[j] if zero else tok
        else:
            tok = O.sample(target[j], counts.copy(), op, step0 + j).chosen
        counts[tok] += 1
        want.append(int(tok))
    assert v_dev == want
    a = 0
    while a + 1 < m and want[a] == props[a]:
        a += 1
    assert a_dev == a and b_dev == want[a]
    for tok in want[a + 1:]:
        counts[tok] -= 1
    d1 = O.sample(nxt[a], counts.copy(), op, step0 + 1 + a)
    counts[d1.chosen] += 1
    d2 = O.sample(nxt[a], None, odp, O.lib().lo_draft_step(step0 + 1) + a)
    assert o_dev == [int(d1.chosen), int(d2.chosen)]
    assert np.array_equal(c_dev.view(np.uint32), counts)
    s.close()
