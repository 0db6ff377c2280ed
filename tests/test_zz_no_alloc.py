"""lily_sample_f32_static - the draw that allocates nothing - against lily_sample_f32.

Two calls in a row on the same GPU share the library's static device array: the second, over
a shorter row, must not see anything the first left behind.  Token ids and the scratch's
counts are compared bit for bit with the existing entry point's (whose own parity against the
oracle the other tests hold), and with the oracle directly.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import lily_sampler as LS
import oracle as O
from gpu_util import dev, ls_params, o_params


def _draw_both(sampler, stream, x, kw, step, hist=None):
    """(static id, ordinary id, static counts, ordinary counts) for one row."""
    v = x.size
    t = torch.from_numpy(x).to(dev())
    p = ls_params(**kw)
    outs, counts = [], []
    for static in (True, False):
        sc = None
        if hist is not None:
            sc = LS.SamplerScratch(sampler, v)
            sc.add_history(torch.from_numpy(hist).to(dev()))
        out = torch.full((1,), -1, dtype=torch.int32, device=dev())
        sampler.synchronize()
        torch.cuda.synchronize()
        if static:
            LS.sample_f32_static(stream, t, sc, p, step, out)
            stream.synchronize()
        else:
            sampler.sample_f32(t, sc, p, step, out)
            sampler.synchronize()
        outs.append(int(out.item()))
        counts.append(sc.read_counts().numpy().copy() if sc is not None else None)
        if sc is not None:
            sc.close()
    return outs[0], outs[1], counts[0], counts[1]


def test_static_entry_needs_no_sampler_object():
    """In a process state where no lily_sampler exists any more: the entry point stands alone."""
    stream = torch.cuda.current_stream(0)
    rng = np.random.default_rng(43)
    x = rng.normal(0, 3, 151_936).astype(np.float32)
    t = torch.from_numpy(x).to(dev())
    out = torch.full((1,), -1, dtype=torch.int32, device=dev())
    kw = dict(temperature=0.9, top_k=50, top_p=0.9, min_p=0.01, seed=2)
    torch.cuda.synchronize()
    for step in range(4):
        LS.sample_f32_static(stream, t, None, ls_params(**kw), step, out)
        stream.synchronize()
        assert int(out.item()) == O.sample(x, None, o_params(**kw), step).chosen


def test_static_entry_matches_the_ordinary_one_on_two_calls_in_a_row():
    sampler = LS.Sampler(0)
    stream = sampler.stream
    rng = np.random.default_rng(41)
    big = rng.normal(0, 3, 151_936).astype(np.float32)     # 38 workgroups share the static array
    small = rng.normal(0, 3, 40_000).astype(np.float32)    # 10 workgroups, right behind it
    tiny = rng.normal(0, 3, 900).astype(np.float32)        # one workgroup: the array is not used
    kw = dict(temperature=0.7, top_k=20, top_p=0.95, seed=17)
    pen = dict(kw, repetition_penalty=1.2, presence_penalty=0.4, frequency_penalty=0.1)
    for x in (big, small, tiny, big):
        for step in (0, 1):
            got, ref, _, _ = _draw_both(sampler, stream, x, kw, step)
            want = O.sample(x, None, o_params(**kw), step).chosen
            assert got == ref == want, (x.size, step, got, ref, want)
    # greedy (several workgroups' argmax partials meet in the same array) and penalised draws
    for x in (big, small):
        got, ref, _, _ = _draw_both(sampler, stream, x, dict(), 0)
        assert got == ref == O.argmax(x)
        hist = rng.integers(0, x.size, 700).astype(np.int32)
        hist[:8] = np.argsort(-x)[:8]
        got, ref, c_got, c_ref = _draw_both(sampler, stream, x, pen, 3, hist)
        counts = np.bincount(hist, minlength=x.size).astype(np.uint32)
        want = O.sample(x, counts, o_params(**pen), 3).chosen
        assert got == ref == want
        assert np.array_equal(c_got, c_ref) and np.array_equal(c_got.view(np.uint32), counts)
    # back-to-back on the stream with no host wait between them: big, then small
    tb, ts = torch.from_numpy(big).to(dev()), torch.from_numpy(small).to(dev())
    outs = torch.full((2,), -1, dtype=torch.int32, device=dev())
    p = ls_params(**kw)
    torch.cuda.synchronize()
    LS.sample_f32_static(stream, tb, None, p, 5, outs[0:1])
    LS.sample_f32_static(stream, ts, None, p, 5, outs[1:2])
    stream.synchronize()
    got = outs.cpu().numpy()
    assert got[0] == O.sample(big, None, o_params(**kw), 5).chosen
    assert got[1] == O.sample(small, None, o_params(**kw), 5).chosen
    sampler.close()


def test_static_entry_rejects_what_it_cannot_hold():
    stream = torch.cuda.current_stream(0)
    x = torch.zeros(16, device=dev())
    out = torch.zeros(1, dtype=torch.int32, device=dev())
    with pytest.raises(LS.SamplerError) as e:
        LS._check(LS._lib.lily_sample_f32_static(
            None, LS._ptr(x), (1 << 20) + 1, None,
            LS.C.byref(ls_params(temperature=0.7, top_k=5)), 0, LS._ptr(out)))
    assert e.value.code == -6 and "at most" in str(e.value)
    with pytest.raises(LS.SamplerError) as e:      # the reference's validation still applies
        LS.sample_f32_static(stream, x, None, ls_params(temperature=-1.0), 0, out)
    assert e.value.code == -2
    with pytest.raises(LS.SamplerError):           # penalties need a scratch
        LS.sample_f32_static(stream, x, None, ls_params(presence_penalty=0.5), 0, out)


def test_static_entry_captured_into_a_graph():
    """Two static draws recorded into one HIP graph and replayed.  The first call on a device
    looks the static array's address up (a module load that a capture does not admit), so one
    call outside the capture comes first - as the header asks.  Every replay, with eager work
    and synchronisations between them, gives the oracle's tokens."""
    rng = np.random.default_rng(47)
    big = rng.normal(0, 3, 151_936).astype(np.float32)
    small = rng.normal(0, 3, 40_000).astype(np.float32)
    kw = dict(temperature=0.7, top_k=20, top_p=0.95, seed=23)
    p = ls_params(**kw)
    tb, ts = torch.from_numpy(big).to(dev()), torch.from_numpy(small).to(dev())
    outs = torch.full((2,), -1, dtype=torch.int32, device=dev())
    warm = torch.full((1,), -1, dtype=torch.int32, device=dev())
    side = torch.cuda.Stream(device=dev())
    torch.cuda.synchronize()
    LS.sample_f32_static(side, ts, None, p, 0, warm)          # the warm call, not captured
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        cur = torch.cuda.current_stream(0)
        LS.sample_f32_static(cur, tb, None, p, 6, outs[0:1])
        LS.sample_f32_static(cur, ts, None, p, 6, outs[1:2])
    want = [O.sample(big, None, o_params(**kw), 6).chosen, O.sample(small, None, o_params(**kw), 6).chosen]
    for replay in range(4):
        outs.fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert outs.cpu().tolist() == want, (replay, outs.cpu().tolist(), want)
        # eager work on the same array between the replays
        LS.sample_f32_static(side, tb, None, p, 100 + replay, warm)
        side.synchronize()
        assert int(warm.item()) == O.sample(big, None, o_params(**kw), 100 + replay).chosen
