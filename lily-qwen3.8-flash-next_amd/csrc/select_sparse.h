// select_sparse.h - rows whose allow-mask admits few ids: nothing of the row is streamed.
#pragma once

#include "device_common.h"

namespace lily {

// ------------------------------------------------------------------ sparse select
//
// Rows whose allow-mask admits few ids: the slice's allowed ids are listed from the mask
// (two passes over its words: count, then place by an exclusive scan of the threads'
// counts, so the order is the same in every run), each is evaluated exactly (bias,
// penalties), adds its term to the row sum and becomes a candidate.  Nothing of the row is
// streamed: the mask's words and one logit per allowed id are all that is read.  Returns
// false, with nothing changed, when the slice admits more ids than `cap` candidates.
template <int DT, bool LSE>
__device__ __forceinline__ bool select_sparse(const RowArgs& a, const Geo<DT>& g, uint32_t k, uint64_t* cand,
                                              uint32_t cap, Shared& sh, bool& sorted) {
    static_assert(STREAM_BIAS_CAP <= NT, "one thread stages one bias entry");
    const uint32_t tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    const bool want_lse = LSE && a.out_logprob != nullptr;
    const bool pen = (a.flags & F_PEN) != 0;
    const uint32_t w_lo = g.id_lo >> 5, w_hi = (g.id_hi + 31u) >> 5;
    auto word = [&](uint32_t i) -> uint32_t {
        return gload(a.allow + i) & range32_at(g.id_lo, g.id_hi, (int64_t)i * 32);
    };
    // A short bias list is kept in the last slots of the buffer (id, delta) and walked from
    // there for every candidate; a longer one is read from memory.
    const uint32_t n_bias = a.n_bias;
    const bool bias_lds = n_bias != 0 && n_bias <= STREAM_BIAS_CAP && cap > 2u * STREAM_BIAS_CAP;
    if (bias_lds) {
        cap -= STREAM_BIAS_CAP;
        if (tid < n_bias) {
            cand[cap + tid] = ((uint64_t)lilym_f32_bits(gload(&a.bias[tid].delta)) << 32) |
                              gload(&a.bias[tid].id);
        }
    }
    uint32_t mine = 0;
    for (uint32_t i = w_lo + tid; i < w_hi; i += NT) {
        mine += (uint32_t)__popc(word(i));
    }
    // Exclusive scan of the threads' counts: inside the wave, then over the waves.
    uint32_t incl = mine;
    for (int o = 1; o < 64; o <<= 1) {
        const uint32_t t = __shfl_up(incl, o);
        if ((int)lane >= o) {
            incl += t;
        }
    }
    if (lane == 63u) {
        sh.red_i[w] = incl;
    }
    __syncthreads();
    uint32_t base = incl - mine, total = 0;
    for (int i = 0; i < NWAVE; ++i) {
        const uint32_t c = sh.red_i[i];
        base += (uint32_t)i < w ? c : 0u;
        total += c;
    }
    __syncthreads();
    if (total > cap) {
        return false;
    }
    for (uint32_t i = w_lo + tid; i < w_hi; i += NT) {
        uint32_t bits = word(i);
        while (bits != 0u) {
            cand[base++] = (uint64_t)(i * 32u + (uint32_t)__builtin_ctz(bits));
            bits &= bits - 1u;
        }
    }
    __syncthreads();
    LseAcc lse;
    lse.init();
    for (uint32_t i = tid; i < total; i += NT) {
        const uint32_t id = (uint32_t)cand[i];
        float l = load_logit<DT>(a.logits, id);
        const uint32_t c = pen ? gload(a.counts + id) : 0u;
        float u;
        if (bias_lds) {
            for (uint32_t j = 0; j < n_bias; ++j) {
                const uint64_t e = cand[cap + j];
                if ((uint32_t)e == id) {
                    l += lilym_bits_f32((uint32_t)(e >> 32));
                }
            }
            if (c > 0u) {
                l = l > 0.0f ? l / a.repetition : l * a.repetition;
                l -= a.presence + a.frequency * (float)c;
            }
            u = l;
        } else {
            u = finish_pre_temperature(a, id, l, c, true);
        }
        if (want_lse) {
            lse.add_one(u, a.c2);
        }
        cand[i] = composite_of(u / a.temperature, id);  // 0 for -inf: dropped by the select
    }
    if (want_lse) {
        lse_reduce(sh, lse);
    } else {
        __syncthreads();
    }
    sorted = false;
    const uint32_t n = select_topk(cand, total, k, sh, sorted);
    if (tid == 0) {
        sh.n_cand = n;
    }
    __syncthreads();
    return true;
}


}  // namespace lily
