"""Seeded synthetic inputs of the five BASELINE configurations (numpy, host side).

The same arrays feed the GPU path, the CPU oracle in the tests and the CPU baseline
leg of the benchmark.  bf16 rows are returned as uint16 bit patterns.
"""
import numpy as np

VOCAB = 151_936


def to_bf16_bits(x):
    """float32 -> bf16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + 0x7FFF
    return ((u + r) >> 16).astype(np.uint16)


def bf16_bits_to_f32(h):
    return (h.astype(np.uint32) << 16).view(np.float32)


def zipf_history(rng, n, vocab, a=1.1):
    """n ids with P(rank r) ~ r^-a over the vocabulary, ranks mapped to shuffled ids."""
    ranks = np.arange(1, vocab + 1, dtype=np.float64)
    p = ranks ** (-a)
    p /= p.sum()
    r = rng.choice(vocab, size=n, p=p)
    perm = rng.permutation(vocab)
    return perm[r].astype(np.int32)


def allow_mask(rng, vocab, frac=0.02, max_run=64):
    """Packed u32 allow mask: about `frac` of the ids, in runs of 1..max_run."""
    bits = np.zeros(vocab, dtype=bool)
    target = int(vocab * frac)
    have = 0
    while have < target:
        run = int(rng.integers(1, max_run + 1))
        at = int(rng.integers(0, vocab - run))
        have += run - int(bits[at:at + run].sum())
        bits[at:at + run] = True
    words = (vocab + 31) // 32
    padded = np.zeros(words * 32, dtype=bool)
    padded[:vocab] = bits
    return np.packbits(padded.reshape(words, 32), axis=1, bitorder="little").view(np.uint32).ravel()


def config1(seed=1, vocab=VOCAB):
    """1 x V f32, N(0, 3^2), 8 ids +12; greedy and T=.7/k=20/p=.95 with a fixed uniform."""
    rng = np.random.default_rng(seed)
    x = rng.normal(0.0, 3.0, vocab).astype(np.float32)
    x[rng.choice(vocab, 8, replace=False)] += np.float32(12.0)
    return {"logits": x[None, :], "uniform": float(rng.random()),
            "params": dict(temperature=0.7, top_k=20, top_p=0.95)}


def config2(seed=2, rows=4, vocab=VOCAB, history=8192):
    """rows x V f32 N(0,3^2) + Zipf(1.1) history; rep 1.05, pres .3, freq .2, k 20, p .95, min_p .05, T .6."""
    rng = np.random.default_rng(seed)
    x = rng.normal(0.0, 3.0, (rows, vocab)).astype(np.float32)
    hist = np.stack([zipf_history(rng, history, vocab) for _ in range(rows)])
    params = [dict(temperature=0.6, top_k=20, top_p=0.95, min_p=0.05, repetition_penalty=1.05,
                   presence_penalty=0.3, frequency_penalty=0.2, seed=1000 + r) for r in range(rows)]
    return {"logits": x, "history": hist, "params": params}


def config3(seed=3, positions=3, vocab=VOCAB):
    """Speculative verify: target rows and draft-head rows (target + N(0,.5^2))."""
    rng = np.random.default_rng(seed)
    target = rng.normal(0.0, 3.0, (positions, vocab)).astype(np.float32)
    draft = (target + rng.normal(0.0, 0.5, (positions, vocab))).astype(np.float32)
    return {"target": target, "draft": draft, "u": rng.random((positions, 2)).astype(np.float32),
            "params": dict(temperature=0.7, top_k=20, top_p=0.95, seed=77)}


def config4(seed=4, rows=64, vocab=VOCAB, n_bias=32):
    """rows x V bf16 N(0,2^2); 2% allow mask, 32 (id, +-5) bias pairs, forced id on 25% rows; T 1, p .9."""
    rng = np.random.default_rng(seed)
    x = to_bf16_bits(rng.normal(0.0, 2.0, (rows, vocab)).astype(np.float32))
    masks = np.stack([allow_mask(rng, vocab) for _ in range(rows)])
    bias = [[(int(i), float(s)) for i, s in zip(rng.choice(vocab, n_bias, replace=False),
                                                 rng.choice([-5.0, 5.0], n_bias))]
            for _ in range(rows)]
    forced = [int(rng.integers(0, vocab)) if rng.random() < 0.25 else None for _ in range(rows)]
    params = [dict(temperature=1.0, top_k=0, top_p=0.9, seed=4000 + r) for r in range(rows)]
    return {"logits": x, "allow": masks, "bias": bias, "forced": forced, "params": params}


def config5(seed=5, rows=1024, vocab=VOCAB, history=2048):
    """rows x V bf16, 90% N(0,2^2) + 10% Student-t(3)*4; k 64, p .9, T .8, 2048-id history; id + logprob."""
    rng = np.random.default_rng(seed)
    x = np.empty((rows, vocab), dtype=np.uint16)
    step = 64
    for r0 in range(0, rows, step):
        n = min(step, rows - r0)
        g = rng.normal(0.0, 2.0, (n, vocab)).astype(np.float32)
        heavy = rng.random((n, vocab)) < 0.1
        t = (rng.standard_t(3.0, (n, vocab)) * 4.0).astype(np.float32)
        x[r0:r0 + n] = to_bf16_bits(np.where(heavy, t, g))
    hist = rng.integers(0, vocab, (rows, history)).astype(np.int32)
    params = [dict(temperature=0.8, top_k=64, top_p=0.9, repetition_penalty=1.1,
                   presence_penalty=0.2, frequency_penalty=0.1, seed=5000 + r)
              for r in range(rows)]
    return {"logits": x, "history": hist, "params": params}


def algorithmic_bytes_per_row(vocab, dtype_bytes, history=0, mask_words=0, bias_pairs=0,
                              logprob=False):
    """logits + history ids + mask words + bias pairs + outputs."""
    return vocab * dtype_bytes + 4 * history + 4 * mask_words + 8 * bias_pairs + 4 + (4 if logprob else 0)
