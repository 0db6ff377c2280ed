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
//
// Diagnostic stamps with -DLILY_SPARSE_TRACE (LaunchCfg::phase_trace): 1 ids counted, 2 ids
// listed, 3 ids evaluated, 13 row sum reduced (the caller stamps 4 behind the select).
#ifdef LILY_SPARSE_TRACE
#define SPARSE_MARK(i) phase(cfg, i)
#else
#define SPARSE_MARK(i)
#endif
template <int DT, bool LSE>
__device__ __forceinline__ bool select_sparse(const RowArgs& a, const Geo<DT>& g, uint32_t k, uint64_t* cand,
                                              uint32_t cap, Shared& sh, bool& sorted, const LaunchCfg& cfg) {
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
    // The mask's words are asked for eight at a time (every load issued, a word past the
    // slice replaced by the slice's last and not counted): a load per turn of the loop is a
    // trip to the L2 per turn.
    constexpr int WB = 8;
    const uint32_t n_words = w_hi - w_lo;
    auto words_of = [&](uint32_t i0, uint32_t (&wv)[WB]) {
#pragma unroll
        for (int u = 0; u < WB; ++u) {
            const uint32_t i = i0 + (uint32_t)u * NT + tid;
            const uint32_t got = word(w_lo + min(i, n_words - 1u));
            wv[u] = i < n_words ? got : 0u;
        }
    };
    uint32_t mine = 0;
    for (uint32_t i0 = 0; i0 < n_words; i0 += WB * NT) {
        uint32_t wv[WB];
        words_of(i0, wv);
#pragma unroll
        for (int u = 0; u < WB; ++u) {
            mine += (uint32_t)__popc(wv[u]);
        }
    }
    // Exclusive scan of the threads' counts: inside the wave, then over the waves.
    const uint32_t incl = wave_scan_u32(mine);
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
    SPARSE_MARK(1);
    for (uint32_t i0 = 0; i0 < n_words; i0 += WB * NT) {
        uint32_t wv[WB];
        words_of(i0, wv);
#pragma unroll
        for (int u = 0; u < WB; ++u) {
            const uint32_t i = w_lo + i0 + (uint32_t)u * NT + tid;
            uint32_t bits = wv[u];
            // A mask's bits come in clusters (a grammar's token classes): a lane that listed a
            // full word bit by bit would keep its wave 32 turns.  Words of more than 8 bits are
            // listed by the wave together, a bit a lane, the word, its place in the list and
            // its number read from the lane that holds them; the others bit by bit.
            const uint32_t n_bits = (uint32_t)__popc(bits), place = base;
            base += n_bits;
            const bool dense = n_bits > 8u;
            uint64_t votes = __ballot(dense);
            while (votes != 0ull) {
                const int from = __builtin_ctzll(votes);
                votes &= votes - 1ull;
                const uint32_t w_bits = (uint32_t)__builtin_amdgcn_readlane((int)bits, from);
                const uint32_t w_place = (uint32_t)__builtin_amdgcn_readlane((int)place, from);
                const uint32_t w_index = (uint32_t)__builtin_amdgcn_readlane((int)i, from);
                if (lane < 32u && ((w_bits >> lane) & 1u) != 0u) {
                    cand[w_place + (uint32_t)__popc(w_bits & ((1u << lane) - 1u))] =
                        (uint64_t)(w_index * 32u + lane);
                }
            }
            if (!dense) {
                uint32_t at = place;
                while (bits != 0u) {
                    cand[at++] = (uint64_t)(i * 32u + (uint32_t)__builtin_ctz(bits));
                    bits &= bits - 1u;
                }
            }
        }
    }
    __syncthreads();
    SPARSE_MARK(2);
    LseAcc lse;
    lse.init();
    // Four ids a thread at a time, their logits and counts asked for together (an id past the
    // list is replaced by id 0 and dropped).
    constexpr int EB = 4;
    for (uint32_t i0 = 0; i0 < total; i0 += EB * NT) {
        uint32_t ids[EB], cs[EB];
        float ls[EB];
#pragma unroll
        for (int q = 0; q < EB; ++q) {
            const uint32_t i = i0 + (uint32_t)q * NT + tid;
            ids[q] = i < total ? (uint32_t)cand[i] : 0u;
        }
#pragma unroll
        for (int q = 0; q < EB; ++q) {
            ls[q] = load_logit<DT>(a.logits, ids[q]);
            cs[q] = pen ? gload(a.counts + ids[q]) : 0u;
        }
#pragma unroll
        for (int q = 0; q < EB; ++q) {
            const uint32_t i = i0 + (uint32_t)q * NT + tid;
            if (i >= total) {
                continue;
            }
            const uint32_t id = ids[q], c = cs[q];
            float l = ls[q];
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
    }
    SPARSE_MARK(3);
    if (want_lse) {
        lse_reduce(sh, lse);
    } else {
        __syncthreads();
    }
    SPARSE_MARK(13);
    sorted = false;
    const uint32_t n = select_topk(cand, total, k, sh, sorted);
    if (tid == 0) {
        sh.n_cand = n;
    }
    __syncthreads();
    return true;
}


}  // namespace lily
