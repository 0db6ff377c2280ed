"""Shared plumbing of the GPU parity tests: upload, run through the C ABI, fetch."""
import numpy as np
import torch

import lily_sampler as LS
import oracle as O

K_CAP = LS.SAMPLE_K_CAP


def dev():
    return torch.device("cuda", 0)


def ls_params(**kw):
    return LS.SamplingParams.greedy(**kw)


def o_params(**kw):
    return O.params(**kw)


def both_params(**kw):
    return ls_params(**kw), o_params(**kw)


def upload_logits(x):
    """numpy float32 or uint16 (bf16 bits) [rows, V] -> device tensor."""
    x = np.ascontiguousarray(x)
    if x.dtype == np.uint16:
        return torch.from_numpy(x.view(np.int16)).to(dev()).view(torch.bfloat16)
    return torch.from_numpy(x).to(dev())


class RowsOut:
    pass


def run_rows(sampler, logits_np, param_kw, steps, scratch=None, allow=None, bias=None,
             forced=None, uniforms=None, logprobs=False, use_plan=False):
    """One lily_sample_rows call with every diagnostic output; returns host arrays."""
    logits_np = np.atleast_2d(logits_np)
    rows, vocab = logits_np.shape
    logits = upload_logits(logits_np)
    out = torch.full((rows,), -1, dtype=torch.int32, device=dev())
    lp = torch.zeros(rows, dtype=torch.float32, device=dev()) if logprobs else None
    dbg_ids = torch.full((rows, K_CAP), -1, dtype=torch.int32, device=dev())
    dbg_probs = torch.zeros((rows, K_CAP), dtype=torch.float32, device=dev())
    dbg_counts = torch.zeros((rows, 2), dtype=torch.int32, device=dev())
    allow_t = None
    if allow is not None:
        allow_t = torch.from_numpy(np.ascontiguousarray(allow).view(np.int32)).to(dev())
    params = [ls_params(**kw) for kw in param_kw]
    torch.cuda.synchronize()
    kw = dict(scratch=scratch, allow=allow_t, bias=bias, forced=forced, uniforms=uniforms,
              out_logprobs=lp, dbg_ids=dbg_ids, dbg_probs=dbg_probs, dbg_counts=dbg_counts)
    if use_plan:
        plan = sampler.plan(logits, params, steps, out, **kw)
        plan.run(0)
        sampler.synchronize()
        plan.close()
    else:
        keep = sampler.sample_rows(logits, params, steps, out, **kw)
        sampler.synchronize()
        del keep
    r = RowsOut()
    r.ids = out.cpu().numpy().astype(np.int64)
    r.logprobs = lp.cpu().numpy() if logprobs else None
    r.cand_ids = dbg_ids.cpu().numpy()
    r.cand_probs = dbg_probs.cpu().numpy()
    r.n_cand = dbg_counts[:, 0].cpu().numpy()
    r.n_kept = dbg_counts[:, 1].cpu().numpy()
    return r


def check_row_against_oracle(r, row, d, exact=True):
    """Row `row` of a RowsOut against an oracle Draw: candidates, probabilities, kept, id."""
    n_fin = int(np.sum(d.cand_adj > -np.inf))
    assert r.n_cand[row] == n_fin, (row, r.n_cand[row], n_fin)
    assert np.array_equal(r.cand_ids[row, :n_fin], d.cand_ids[:n_fin].astype(np.int64)), row
    if exact:
        assert np.array_equal(r.cand_probs[row, :n_fin].view(np.uint32),
                              d.cand_prob[:n_fin].view(np.uint32)), row
        assert r.n_kept[row] == d.n_kept, (row, r.n_kept[row], d.n_kept)
        assert r.ids[row] == d.chosen, (row, r.ids[row], d.chosen)
    else:
        assert np.allclose(r.cand_probs[row, :n_fin], d.cand_prob[:n_fin], rtol=1e-5, atol=0), row
