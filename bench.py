#!/usr/bin/env python3
"""Benchmark of the logits-to-token stage on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one pass of the sampler over one batch of synthetic logits already
resident in HBM: the throughput configuration of BASELINE.json (1 024 rows x 151 936
bf16 logits, top-k 64, top-p 0.9, T 0.8, penalties over a 2 048-id history per row,
output = token ids + chosen-token log-probabilities).  Every timed step reads other
logits than the step before it (LOGITS_SETS resident batches taken in turn: a decode
step never sees the same logits twice, and a sampler that is handed the same rows again
and again finds the token it drew most often to be the row's dominant one, which it is
not in general); the figure with one batch replayed is reported beside it.  The 4-row decode-step
configuration (f32, 8 192-id history, k 20) is timed in the same run and reported in
the same JSON line under "decode_b4".  The CPU oracle is timed on a bounded sample
of the same rows on the host's cores as a reported baseline.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "lily-qwen3.8-flash-next_amd", "python"))

HBM_PEAK_GBS = 8000.0
LOGITS_SETS = 8   # resident batches of logits the timed steps take in turn
# HBM bytes per 1024-row launch come from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# very command, summarised in this file (a line "traffic_bytes_per_launch: N"; 1024 rows only).
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "k_rows_table_bf16_config5_b1024.md")


def measured_traffic(rows):
    """Bytes per launch from the committed counter summary, or None (other sizes, no summary)."""
    if rows != 1024 or not os.path.exists(TRAFFIC_SUMMARY):
        return None
    for line in open(TRAFFIC_SUMMARY):
        if line.startswith("traffic_bytes_per_launch:"):
            return float(line.split(":", 1)[1])
    return None


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--rows", type=int, default=1024)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--no-others", action="store_true",
                    help="skip configurations 1, 3 and 4 (profiles of the two headline launches)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one 256 MiB device copy (a known-size kernel that counter runs "
                         "under rocprofv3 --pmc are scaled by)")
    return ap.parse_args()


def time_steps(stream, fn, steps, warmup):
    """Average milliseconds per call of fn, HIP events on the sampler's own stream."""
    import torch
    for i in range(warmup):
        fn(i)
    stream.synchronize()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record(stream)
    for i in range(steps):
        fn(warmup + i)
    stop.record(stream)
    stop.synchronize()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def median_ms(stream, fn, reps, warmup):
    """Median milliseconds of single calls of fn, each between its own pair of events."""
    import torch
    for i in range(warmup):
        fn(i)
    stream.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for i, (e0, e1) in enumerate(pairs):
        e0.record(stream)
        fn(warmup + i)
        e1.record(stream)
    pairs[-1][1].synchronize()
    times = sorted(e0.elapsed_time(e1) for e0, e1 in pairs)
    return times[len(times) // 2]


def queued_ms(stream, fn, reps, warmup, rounds=3):
    """Milliseconds per call of fn over `reps` calls queued back to back between one pair of
    events (the host's work for a call hides behind the device's work for the one before), the
    best of `rounds`."""
    import torch
    for i in range(warmup):
        fn(i)
    best = None
    for _ in range(rounds):
        stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(reps):
            fn(i)
        e1.record(stream)
        e1.synchronize()
        t = e0.elapsed_time(e1) / reps
        best = t if best is None else min(best, t)
    return best


def cpp_caller(rows, vocab, calls):
    """lily_sample_rows with host descriptors on every call, from the C++ program that the tests
    build against the public header (a child process): host time a call takes to return,
    device time per call, host time with an idle stream."""
    import subprocess
    exe = os.path.join(ROOT, "tests", "abi_harness", "harness.bin")
    if not os.path.exists(exe):
        return None
    try:
        res = subprocess.run([exe, "time", str(rows), str(vocab), str(calls)], capture_output=True,
                             text=True, timeout=240)
    except (OSError, subprocess.TimeoutExpired):
        return None
    for line in res.stdout.splitlines():
        w = line.split()
        if w[:1] == ["time"]:
            kv = dict(zip(w[1::2], w[2::2]))
            return {"rows": rows, "calls": calls,
                    "host_us_per_call": float(kv["host_us_per_call"]),
                    "device_us_per_call": float(kv["device_us_per_call"]),
                    "host_us_per_call_idle_stream": float(kv["host_us_per_call_idle_stream"]),
                    "logits": "a language-model-shaped row rotated per row (the program's own), replayed"}
    return None


def paths_of(sampler, fn):
    """Which selects served one more (untimed) run of fn: workgroups by the streaming select, by
    the sparse / bitmap selects, by the exhaustive select, and the reasons the first gave up."""
    import torch
    stats = torch.zeros(4, dtype=torch.int32, device="cuda")
    sampler.set_path_stats(stats)
    fn(0)
    sampler.synchronize()
    sampler.set_path_stats(None)
    st = stats.cpu().tolist()
    return {"streaming": st[0], "sparse_or_bitmap": st[1], "exhaustive": st[2], "gave_up_bits": st[3]}


def make_scratches(LS, sampler, history, vocab, device):
    import numpy as np
    import torch
    out = []
    for h in history:
        sc = LS.SamplerScratch(sampler, vocab)
        sc.add_history(torch.from_numpy(np.ascontiguousarray(h)).to(device))
        out.append(sc)
    return out


def cpu_baseline(c, rows_total, seconds):
    """The oracle (reference-faithful full-vocabulary sort) on this host's cores."""
    import numpy as np
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as O
    avail = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    cores = max(1, min(avail, 16))   # the GPU box's CPU share is 16 whatever it shows
    x, hist = c["logits"], c["history"]
    vocab = x.shape[1]
    ext, _ = O.make_ext(sort_mode=O.SORT_FULL, want_logprob=True)

    def run(n):
        n = min(n, rows_total)
        counts = np.stack([np.bincount(hist[i], minlength=vocab).astype(np.uint32) for i in range(n)])
        params = [O.params(**c["params"][i]) for i in range(n)]
        t0 = time.perf_counter()
        O.sample_rows(x[:n], counts, params, [3] * n, exts=[ext] * n, threads=cores)
        return n, time.perf_counter() - t0

    n, dt = run(cores)                       # probe: one row per core
    total_rows, total_dt = 0, 0.0
    chunk = int(max(cores, min(rows_total, cores * max(1.0, 2.0 / max(dt, 1e-3)))))
    while total_dt < seconds:                # bounded sample: about `seconds` of wall time
        n, dt = run(chunk)
        total_rows += n
        total_dt += dt
    n, dt = total_rows, total_dt
    return {"value": n / dt, "unit": "rows/s", "cores": cores, "nproc": os.cpu_count(),
            "cores_available_to_this_process": avail, "kind": "port",
            "sample": f"{n} row draws (rows 0..{min(chunk, rows_total) - 1} of the {rows_total}, repeated), full-vocabulary index sort per row "
                      f"(as tests/unit/kernels/sample.rs:31-34), id + f64 log-probability, "
                      f"{dt:.1f} s wall"}


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py measures one GPU: rows are independent, so more GPUs only split the "
              "batch; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch
    import lily_sampler as LS
    import lily_workloads as W

    if not torch.cuda.is_available():
        print("no GPU visible", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda", 0)
    stream = torch.cuda.Stream(device=device)
    sampler = LS.Sampler(0, stream=stream)

    # ---- throughput configuration: rows x 151 936 bf16
    rows = a.rows
    c5 = W.config5(rows=rows)
    vocab = c5["logits"].shape[1]
    history = c5["history"].shape[1]
    logits = torch.from_numpy(c5["logits"].view(np.int16)).to(device).view(torch.bfloat16)
    params = [LS.SamplingParams.greedy(**kw) for kw in c5["params"]]
    scratches = make_scratches(LS, sampler, c5["history"], vocab, device)
    out_ids = torch.zeros(rows, dtype=torch.int32, device=device)
    out_lp = torch.zeros(rows, dtype=torch.float32, device=device)
    # The other batches: the same rows handed to other requests and turned along the vocabulary
    # (row r of batch j is row r - 131 j of the first, its ids moved on by 32 792 j), so that a
    # request's scratch meets other logits at every step.
    sets = [logits] + [torch.roll(logits, shifts=(131 * j, 32_792 * j), dims=(0, 1)).contiguous()
                       for j in range(1, LOGITS_SETS)]
    torch.cuda.synchronize()
    plans = [sampler.plan(x, params, [0] * rows, out_ids, scratch=scratches, out_logprobs=out_lp)
             for x in sets]
    ms = time_steps(stream, lambda i: plans[i % LOGITS_SETS].run(i), a.steps, a.warmup)
    bytes_row = W.algorithmic_bytes_per_row(vocab, 2, history=history, logprob=True)
    achieved = rows * bytes_row / (ms * 1e-3) / 1e9
    ids_host = out_ids.cpu().numpy()
    assert ids_host.min() >= 0 and ids_host.max() < vocab
    paths5 = paths_of(sampler, lambda i: plans[1].run(a.warmup + a.steps))
    # for comparison: one batch replayed (what the figure of earlier builds was measured on)
    ms_replay = time_steps(stream, lambda i: plans[0].run(2 * (a.warmup + a.steps) + i), a.steps, a.warmup)
    for p_ in plans:
        p_.close()
    del sets[1:]
    # the reference's call shape at this size: host descriptors packed and uploaded every step
    ms_call = time_steps(stream, lambda i: sampler.sample_rows(logits, params, [i] * rows, out_ids,
                                                               scratch=scratches, out_logprobs=out_lp),
                         max(5, a.steps // 5), 2)
    # the ceiling of a row-per-workgroup launch of this size: the same rows only read
    probe_out = torch.zeros(rows, dtype=torch.int32, device=device)
    ms_read = time_steps(stream, lambda i: sampler.probe_read(logits, probe_out), a.steps, a.warmup)
    plain_read = rows * vocab * 2 / (ms_read * 1e-3) / 1e9

    if a.copy_probe:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=device).normal_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)                      # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    # ---- decode-step configuration: 4 x 151 936 f32, 8 192-id history
    c2 = W.config2()
    l2 = torch.from_numpy(c2["logits"]).to(device)
    p2 = [LS.SamplingParams.greedy(**kw) for kw in c2["params"]]
    s2 = make_scratches(LS, sampler, c2["history"], vocab, device)
    o2 = torch.zeros(4, dtype=torch.int32, device=device)
    torch.cuda.synchronize()
    plan2 = sampler.plan(l2, p2, [0] * 4, o2, scratch=s2)
    ms2 = time_steps(stream, lambda i: plan2.run(i), max(a.steps, 200), max(a.warmup, 20))
    # the reference's call shape: host descriptors every step (lily_sample_rows)
    paths2 = paths_of(sampler, lambda i: plan2.run(1000))
    ms2_call = time_steps(stream, lambda i: sampler.sample_rows(l2, p2, [i] * 4, o2, scratch=s2),
                          max(a.steps, 200), max(a.warmup, 20))
    bytes2 = 4 * W.algorithmic_bytes_per_row(vocab, 4, history=c2["history"].shape[1])
    plan2.close()

    # ---- the other BASELINE configurations, for the record (latency-bound launches)
    others = {}
    if not a.no_others:
        n_lat, w_lat = max(a.steps, 100), max(a.warmup, 10)
        c1 = W.config1()
        l1 = torch.from_numpy(c1["logits"]).to(device)
        o1 = torch.zeros(1, dtype=torch.int32, device=device)
        for name, kw in (("config1_greedy", dict()), ("config1_sampled", c1["params"])):
            torch.cuda.synchronize()
            p1 = sampler.plan(l1, [LS.SamplingParams.greedy(**kw)], [0], o1)
            others[name] = {"us_per_step": time_steps(stream, lambda i: p1.run(i), n_lat, w_lat) * 1e3}
            p1.close()
        # the decode step of config 2 without top_k: the reference then keeps 1024 candidates
        # (src/kernels/sample.rs:326-331), the case of a request that names no top_k
        lp2 = torch.zeros(4, dtype=torch.float32, device=device)
        for name, with_lp in (("decode_b4_default_top_k", False), ("decode_b4_default_top_k_logprob", True)):
            pk = [LS.SamplingParams.greedy(**dict(kw, top_k=0)) for kw in c2["params"]]
            torch.cuda.synchronize()
            p1 = sampler.plan(l2, pk, [0] * 4, o2, scratch=s2, out_logprobs=lp2 if with_lp else None)
            others[name] = {"us_per_step": time_steps(stream, lambda i: p1.run(i), n_lat, w_lat) * 1e3, "rows": 4,
                            "k": 1024, "paths": paths_of(sampler, lambda i: p1.run(0))}
            p1.close()
        c3 = W.config3()
        m3 = c3["target"].shape[0]
        t3 = torch.from_numpy(c3["target"]).to(device)
        d3 = torch.from_numpy(c3["draft"]).to(device)
        for name, kw in (("config3_verify_greedy", dict()), ("config3_verify_sampled", c3["params"]),
                         ("config3_verify_penalised", dict(c3["params"], presence_penalty=0.4,
                                                           repetition_penalty=1.1))):
            lp3 = LS.SamplingParams.greedy(**kw)
            sc3 = LS.SamplerScratch(sampler, vocab)
            dists = LS.DraftDists(sampler, m3)
            props = torch.zeros(m3, dtype=torch.int32, device=device)
            torch.cuda.synchronize()
            for j in range(m3 - 1):
                sampler.sample_draft_f32(d3[j], sc3, LS.draft_params(lp3), LS.draft_step(j),
                                         props[j:j + 1], dists.slot(j))
            sampler.synchronize()
            ids3 = torch.cat([torch.tensor([42], dtype=torch.int32, device=device), props[:m3 - 1]])
            ver = torch.zeros(m3, dtype=torch.int32, device=device)
            ctrl = torch.zeros(LS.ctrl_words(2), dtype=torch.int32, device=device)
            torch.cuda.synchronize()
            us = time_steps(stream, lambda i: sampler.spec_verify(t3, sc3, lp3, i, dists, ids3, ver, ctrl,
                                                                  pos0=100, ratio=4, chain=2),
                            n_lat, w_lat) * 1e3
            others[name] = {"us_per_step": us, "rows": m3}
            sampler.synchronize()
            sc3.close()
            dists.close()
        c4 = W.config4(rows=64)
        l4 = torch.from_numpy(c4["logits"].view(np.int16)).to(device).view(torch.bfloat16)
        o4 = torch.zeros(64, dtype=torch.int32, device=device)
        lp4 = torch.zeros(64, dtype=torch.float32, device=device)
        allow4 = torch.from_numpy(np.ascontiguousarray(c4["allow"]).view(np.int32)).to(device)
        torch.cuda.synchronize()
        p4 = sampler.plan(l4, [LS.SamplingParams.greedy(**kw) for kw in c4["params"]], [7] * 64, o4,
                          allow=allow4, bias=c4["bias"], forced=c4["forced"], out_logprobs=lp4)
        us4 = time_steps(stream, lambda i: p4.run(i), n_lat, w_lat) * 1e3
        bytes4 = 64 * W.algorithmic_bytes_per_row(vocab, 2, mask_words=c4["allow"].shape[1], bias_pairs=32,
                                                  logprob=True)
        others["config4_constrained"] = {"us_per_step": us4, "rows": 64,
                                         "achieved_GBs": bytes4 / (us4 * 1e-6) / 1e9,
                                         "paths": paths_of(sampler, lambda i: p4.run(0))}
        p4.close()
        torch.cuda.synchronize()
        p4 = sampler.plan(l4, [LS.SamplingParams.greedy(**kw) for kw in c4["params"]], [7] * 64, o4)
        us4 = time_steps(stream, lambda i: p4.run(i), n_lat, w_lat) * 1e3
        others["config4_rows_unconstrained"] = {"us_per_step": us4, "rows": 64, "k": 1024,
                                                "paths": paths_of(sampler, lambda i: p4.run(0))}
        p4.close()

    # ---- the logits' producer (bf16 head on the matrix cores, d = 4096) and the draws from its
    # summaries: config 5's draw settings without penalties (rows under penalties read the row)
    head = None
    if not a.no_others:
        head = {}
        d_model = 4096
        tiles = (vocab + LS.LOGIT_TILE_COLS - 1) // LS.LOGIT_TILE_COLS
        gen = torch.Generator(device=device)
        gen.manual_seed(11)
        w_f32 = torch.randn(vocab, d_model, device=device, generator=gen) * (2.0 / d_model ** 0.5)
        # one weight row in ten scaled by 2|t(3)|: the logits then are, like config 5's, a bulk
        # N(0, 2^2) with a heavy-tailed tenth
        t3 = torch.from_numpy(np.random.default_rng(13).standard_t(3.0, vocab).astype(np.float32)).to(device)
        heavy = torch.rand(vocab, device=device, generator=gen) < 0.1
        w_f32 *= torch.where(heavy, 2.0 * t3.abs(), torch.ones_like(t3))[:, None]
        del t3, heavy
        for b_rows in (4, rows):
            hid = torch.randn(b_rows, d_model, device=device, generator=gen)
            # and, per row, 40 ids whose weights point along the row's hidden state
            for r in range(min(b_rows, 128)):
                ids = torch.randint(0, vocab, (40,), device=device, generator=gen)
                gain = (torch.rand(40, 1, device=device, generator=gen) * 0.7 + 0.3) * (6.0 / d_model)
                w_f32[ids] += gain * hid[r][None, :]
            hb, wb = hid.to(torch.bfloat16), w_f32.to(torch.bfloat16)
            lg = torch.zeros(b_rows, vocab, dtype=torch.bfloat16, device=device)
            tmax = torch.zeros(b_rows, tiles, dtype=torch.float32, device=device)
            tsum = torch.zeros(b_rows, tiles, dtype=torch.float32, device=device)
            hp = [LS.SamplingParams.greedy(temperature=0.8, top_k=64, top_p=0.9, seed=5000 + r)
                  for r in range(b_rows)]
            ho = torch.zeros(b_rows, dtype=torch.int32, device=device)
            hl = torch.zeros(b_rows, dtype=torch.float32, device=device)
            torch.cuda.synchronize()
            n_h = 30
            ms_head = queued_ms(stream, lambda i: sampler.lm_head(hb, wb, [0.8] * b_rows, lg, tmax, tsum),
                                n_h, 3)
            ms_fused = median_ms(stream, lambda i: sampler.lm_head_sample_rows(
                hb, wb, lg, tmax, tsum, hp, [i] * b_rows, ho, out_logprobs=hl), n_h, 3)
            # what was timed is checked: the drawn ids lie in the vocabulary, and a seeded handful
            # of the stored logits equal the f64 product of the same bf16 operands to one bf16 step
            sampler.synchronize()
            ids_h = ho.cpu().numpy()
            assert ids_h.min() >= 0 and ids_h.max() < vocab, (ids_h.min(), ids_h.max())
            pick = np.random.default_rng(17 + b_rows)
            rr = torch.from_numpy(pick.integers(0, b_rows, 64)).to(device)
            cc = torch.from_numpy(pick.integers(0, vocab, 64)).to(device)
            want = (hb[rr].double() * wb[cc].double()).sum(dim=1)
            have = lg[rr, cc].double()
            assert bool(torch.all((have - want).abs() <= want.abs() * 2.0 ** -7 + 1e-3)), \
                float((have - want).abs().max())

            def behind_a_head(draw, n=4):
                """GPU time of a draw call: n of them queued while head launches still run (three
                for a batch: the mirror packs 1 024 penalised rows for longer than one lasts),
                so that the host's packing is off the clock."""
                for _ in range(3 if b_rows > 64 else 1):
                    sampler.lm_head(hb, wb, [0.8] * b_rows, lg, tmax, tsum)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for i in range(n):
                    draw(i)
                e1.record(stream)
                e1.synchronize()
                return e0.elapsed_time(e1) / n * 1e3

            us_tiled = behind_a_head(lambda i: sampler.sample_rows_tiled(lg, tmax, tsum, hp, [i] * b_rows, ho,
                                                                        out_logprobs=hl))
            us_rows = behind_a_head(lambda i: sampler.sample_rows(lg, hp, [i] * b_rows, ho, out_logprobs=hl))
            # config 5's draw settings in full: penalties over a 2 048-id history per row
            pp = [LS.SamplingParams.greedy(temperature=0.8, top_k=64, top_p=0.9, repetition_penalty=1.1,
                                           presence_penalty=0.2, frequency_penalty=0.1, seed=5000 + r)
                  for r in range(b_rows)]
            hist = np.random.default_rng(12).integers(0, vocab, (b_rows, 2048)).astype(np.int32)
            hs = make_scratches(LS, sampler, hist, vocab, device)
            torch.cuda.synchronize()
            us_tiled_pen = behind_a_head(lambda i: sampler.sample_rows_tiled(
                lg, tmax, tsum, pp, [i] * b_rows, ho, scratch=hs, out_logprobs=hl))
            paths_pen = paths_of(sampler, lambda i: sampler.sample_rows_tiled(
                lg, tmax, tsum, pp, [99] * b_rows, ho, scratch=hs, out_logprobs=hl))
            us_rows_pen = behind_a_head(lambda i: sampler.sample_rows(lg, pp, [i] * b_rows, ho, scratch=hs,
                                                                     out_logprobs=hl))
            # ... and config 5 in full as one call: the head and the penalised draws
            ms_fused_pen = median_ms(stream, lambda i: sampler.lm_head_sample_rows(
                hb, wb, lg, tmax, tsum, pp, [i] * b_rows, ho, scratch=hs, out_logprobs=hl), n_h, 3)
            sampler.synchronize()
            for sc_ in hs:
                sc_.close()
            # the same head held in the reference's affine formats (random codes, scales of the
            # weights' size; lm_head is 4 bits in groups of 64, 8 under --q8 head), f32 logits
            quant = {}
            lg32 = torch.zeros(b_rows, vocab, dtype=torch.float32, device=device)
            for bits in (8, 4):
                per = 32 // bits
                q = torch.randint(0, 1 << bits, (vocab, d_model // per, per), device=device, generator=gen,
                                  dtype=torch.int64)
                words = (q << (bits * torch.arange(per, device=device, dtype=torch.int64))).sum(dim=2)
                words = torch.where(words >= 2 ** 31, words - 2 ** 32, words).to(torch.int32).contiguous()
                del q
                sc = (torch.rand(vocab, d_model // 64, device=device, generator=gen) + 0.5) * (4.0 / (1 << bits) / d_model ** 0.5)
                bi = -sc * (1 << bits) / 2
                qw = LS.QuantWeights(words, sc.to(torch.bfloat16), bi.to(torch.bfloat16), 64, bits)
                ms_q = queued_ms(stream, lambda i: sampler.lm_head(hb, qw, [0.8] * b_rows, lg32, tmax, tsum), n_h, 3)
                code_bytes = vocab * d_model * bits / 8 + 2 * vocab * (d_model // 64) * 2
                quant[f"q{bits}_g64"] = {"head_us": ms_q * 1e3, "weight_GBs": code_bytes / (ms_q * 1e-3) / 1e9,
                                         "TFLOPs": 2.0 * b_rows * d_model * vocab / (ms_q * 1e-3) / 1e12}
                del words, qw
            ms_f32 = queued_ms(stream, lambda i: sampler.lm_head(hb, wb, [0.8] * b_rows, lg32, tmax, tsum), n_h, 3)
            del lg32
            # which way the producer took (a batch goes through hipBLASLt and a pass that forms
            # the summaries where that library can be opened), and this library's own kernel for
            # the same batch beside it
            before = sampler.lm_head_library_calls()
            sampler.lm_head(hb, wb, [0.8] * b_rows, lg, tmax, tsum)
            through_library = sampler.lm_head_library_calls() > before
            ms_own = None
            if through_library:
                asked = os.environ.get("LILY_SAMPLER_HEAD")
                os.environ["LILY_SAMPLER_HEAD"] = "own"
                own = LS.Sampler(0, stream=stream)
                if asked is None:
                    del os.environ["LILY_SAMPLER_HEAD"]
                else:
                    os.environ["LILY_SAMPLER_HEAD"] = asked
                ms_own = queued_ms(stream, lambda i: own.lm_head(hb, wb, [0.8] * b_rows, lg, tmax, tsum), n_h, 3)
                own.synchronize()
                own.close()
            # for reference only: the library's GEMM (torch.matmul, hipBLASLt) on the same
            # operands, bf16 in and out, without the summaries the head's epilogue leaves
            ref_out = torch.empty(b_rows, vocab, dtype=torch.bfloat16, device=device)
            with torch.cuda.stream(stream):
                ms_lib = queued_ms(stream, lambda i: torch.matmul(hb, wb.t(), out=ref_out), n_h, 3)
            del ref_out
            flops = 2.0 * b_rows * d_model * vocab
            head[f"b{b_rows}"] = {
                "rows": b_rows, "d": d_model,
                "head_us": ms_head * 1e3,
                "head_TFLOPs": flops / (ms_head * 1e-3) / 1e12,
                "head_frac_of_mfma_peak": flops / (ms_head * 1e-3) / 1e12 / 2500.0,
                "head_weight_GBs": vocab * d_model * 2 / (ms_head * 1e-3) / 1e9,
                "head_form": "hipBLASLt GEMM + k_head_summaries" if through_library else "own kernel",
                "head_own_kernel_us": ms_own * 1e3 if ms_own is not None else ms_head * 1e3,
                "library_gemm_us": ms_lib * 1e3,
                "timing": f"the producers alone: per launch over {n_h} queued back to back, best of 3; "
                          f"head_plus_draws_us: median of {n_h} single calls",
                "head_f32_logits_us": ms_f32 * 1e3,
                "quantised_heads_f32_logits": quant,
                "head_plus_draws_us": ms_fused * 1e3,
                "head_plus_penalised_draws_us": ms_fused_pen * 1e3,
                "draws_from_summaries_us": us_tiled,
                "draws_from_rows_us": us_rows,
                "penalised_draws_from_summaries_us": us_tiled_pen,
                "penalised_draws_from_rows_us": us_rows_pen,
                "penalised_paths": paths_pen,
            }
            del hb, wb, lg
        del w_f32

    # lily_sample_rows as a C++ caller sees it (the Python mirror packs 1 024 descriptors in
    # Python on every call, which is what "us_per_step_host_descriptors" times)
    sampler.synchronize()
    torch.cuda.synchronize()
    cpp = cpp_caller(rows, vocab, 100)

    line = {
        "metric": "rows/s and us/step at B=4 and B=1024 x151,936 vocab; achieved HBM GB/s",
        "value": rows / (ms * 1e-3),
        "unit": "rows/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{rows} rows x {vocab} bf16 logits (90% N(0,2^2) + 10% Student-t(3)x4), "
                        f"top-k 64, top-p 0.9, T 0.8, penalties over a {history}-id history per "
                        "row, output ids + chosen-token logprobs (BASELINE config 5)",
            "rows": rows, "vocab": vocab, "logits": "bf16",
        },
        "us_per_step": ms * 1e3,
        "logits_per_step": f"{LOGITS_SETS} resident batches taken in turn (row and vocabulary rotations of one "
                           "generated batch): no step reads the logits of the step before it",
        "us_per_step_replayed_logits": ms_replay * 1e3,
        "us_per_step_host_descriptors": ms_call * 1e3,
        "host_descriptors_from_cpp": cpp,
        "paths": paths5,
        "decode_b4": {
            "workload": "4 rows x 151936 f32 logits, 8192-id Zipf history, rep 1.05 / pres 0.3 / "
                        "freq 0.2, k 20, p 0.95, min_p 0.05, T 0.6 (BASELINE config 2)",
            "us_per_step": ms2 * 1e3,
            "us_per_step_host_descriptors": ms2_call * 1e3,
            "paths": paths2,
            "rows_per_s": 4 / (ms2 * 1e-3),
            "achieved_GBs": bytes2 / (ms2 * 1e-3) / 1e9,
            "target_us": 20.0,
        },
        "other_configs": others,
        "lm_head": head,
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": measured_traffic(rows),
            "plain_read_GBs": plain_read,
            "frac_of_plain_read": (rows * vocab * 2 / (ms * 1e-3) / 1e9) / plain_read,
            "kernel": "k_rows_table<bf16, streaming select, log-sum-exp>",
            "bytes_per_row": bytes_row,
        },
    }
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(c5, rows, a.cpu_seconds)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
