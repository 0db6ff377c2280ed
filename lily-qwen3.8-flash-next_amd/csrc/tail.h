// tail.h - from a row's candidates to its token: sort, softmax over the candidates, the
// sequential top-p / min-p prefix, the draw, the draft export and the speculative accept /
// residual draw, and the bookkeeping of the emitted id.
#pragma once

#include "device_common.h"

namespace lily {

// ------------------------------------------------------------------ sort

// The value lane ^ M holds, every lane of the wave at work - by moves inside the vector unit for
// every M, never through the LDS crossbar, whose latency a sort of dependent exchanges would wait
// out stage by stage.  1 and 2: a permutation inside each group of four lanes.  4: the lanes of
// the even groups of four read four lanes up, those of the odd groups four lanes down (two moves,
// each written to its groups only).  8: a rotation by eight within each row of 16.  16 and 32:
// the swaps of whole rows and of the wave's halves (v_permlane16_swap / v_permlane32_swap with
// the value as both operands leave one copy with rows 0 0 2 2 / the lower half twice and the
// other with rows 1 1 3 3 / the upper half twice).
template <uint32_t M>
__device__ __forceinline__ uint32_t from_lane_xor32(uint32_t x) {
    static_assert(M == 1u || M == 2u || M == 4u || M == 8u || M == 16u || M == 32u, "a power of two inside the wave");
    const int v = (int)x;
    if (M == 1u) {
        return (uint32_t)__builtin_amdgcn_update_dpp(0, v, 0xb1, 0xf, 0xf, true);   // quad_perm [1, 0, 3, 2]
    }
    if (M == 2u) {
        return (uint32_t)__builtin_amdgcn_update_dpp(0, v, 0x4e, 0xf, 0xf, true);   // quad_perm [2, 3, 0, 1]
    }
    if (M == 4u) {
        const int up = __builtin_amdgcn_update_dpp(0, v, 0x104, 0xf, 0x5, false);    // row_shl:4 into groups 0 and 2
        return (uint32_t)__builtin_amdgcn_update_dpp(up, v, 0x114, 0xf, 0xa, false); // row_shr:4 into groups 1 and 3
    }
    if (M == 8u) {
        return (uint32_t)__builtin_amdgcn_update_dpp(0, v, 0x128, 0xf, 0xf, false);  // row_ror:8
    }
    const uint32_t lane = threadIdx.x & 63u;
    if (M == 16u) {
        const auto two = __builtin_amdgcn_permlane16_swap(x, x, false, false);
        return (lane & 16u) != 0u ? two[0] : two[1];
    }
    const auto two = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return (lane & 32u) != 0u ? two[0] : two[1];
}

template <uint32_t M>
__device__ __forceinline__ uint64_t from_lane_xor(uint64_t v) {
    return ((uint64_t)from_lane_xor32<M>((uint32_t)(v >> 32)) << 32) | from_lane_xor32<M>((uint32_t)v);
}

// Descending bitonic sort of cand[0..n), n <= 4 * NT, four entries per thread (entry
// 4 * tid + r in register r; absent entries are 0, the smallest).  Exchanges at distance
// 1 and 2 stay inside a thread, 4 .. 128 are moves between the lanes of a wave, and only the
// three at distance 256 and 512 go through LDS with a barrier.
__device__ __forceinline__ void sort_desc_regs(uint64_t* cand, uint32_t n) {
    static_assert(NT == 256, "four entries per thread cover 1024");
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    uint64_t v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t i = tid * 4u + (uint32_t)r;
        v[r] = i < n ? cand[i] : 0ull;
    }
    __syncthreads();
    auto exchange = [](uint64_t& lo, uint64_t& hi, bool desc) {  // lo sits at the lower index
        const bool swap = (lo < hi) == desc;  // equal entries may swap: nothing changes
        const uint64_t t = lo;
        lo = swap ? hi : lo;
        hi = swap ? t : hi;
    };
#pragma unroll
    for (int lsize = 1; lsize <= 10; ++lsize) {
#pragma unroll
        for (int lstride = lsize - 1; lstride >= 0; --lstride) {
            const uint32_t size = 1u << lsize, stride = 1u << lstride;
            if (stride >= 4u * 64u) {
                const uint32_t other = tid ^ (stride >> 2);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    cand[tid * 4u + (uint32_t)r] = v[r];
                }
                __syncthreads();
                const bool desc = ((tid * 4u) & size) == 0;
                const bool take_max = ((tid & (stride >> 2)) == 0) == desc;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint64_t o = cand[other * 4u + (uint32_t)r];
                    v[r] = ((o > v[r]) == take_max) ? o : v[r];
                }
                __syncthreads();
            } else if (stride >= 4u) {
                const uint32_t m = stride >> 2;   // (a constant once the loops are unrolled)
                const bool desc = ((tid * 4u) & size) == 0;
                const bool take_max = ((lane & m) == 0) == desc;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint64_t o = m == 1u ? from_lane_xor<1>(v[r]) : m == 2u ? from_lane_xor<2>(v[r])
                                     : m == 4u ? from_lane_xor<4>(v[r]) : m == 8u ? from_lane_xor<8>(v[r])
                                     : m == 16u ? from_lane_xor<16>(v[r]) : from_lane_xor<32>(v[r]);
                    v[r] = ((o > v[r]) == take_max) ? o : v[r];
                }
            } else if (stride == 2u) {
                const bool desc = ((tid * 4u) & size) == 0;  // size >= 4 here
                exchange(v[0], v[2], desc);
                exchange(v[1], v[3], desc);
            } else {
                if (size == 2u) {
                    exchange(v[0], v[1], true);   // index bit 1 clear: descending
                    exchange(v[2], v[3], false);  // set: ascending
                } else {
                    const bool desc = ((tid * 4u) & size) == 0;
                    exchange(v[0], v[1], desc);
                    exchange(v[2], v[3], desc);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        cand[tid * 4u + (uint32_t)r] = v[r];
    }
    __syncthreads();
}

// Descending sort of cand[0..n).  Up to 64 entries: one wave, in registers.  Up to 4 * NT:
// four per thread in registers.  More: bitonic in LDS over the next power of two (the
// buffer holds it).
// BIG = false leaves the register sort out (kernels whose rows never sort more than 64).
template <bool BIG>
__device__ __forceinline__ void sort_desc(uint64_t* cand, uint32_t n) {
    if (n <= 64) {
        if (threadIdx.x < 64) {
            const uint32_t lane = threadIdx.x;
            uint64_t c = lane < n ? cand[lane] : 0ull;
#pragma unroll
            for (uint32_t size = 2; size <= 64; size <<= 1) {
#pragma unroll
                for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
                    const uint64_t o = stride == 1u ? from_lane_xor<1>(c) : stride == 2u ? from_lane_xor<2>(c)
                                     : stride == 4u ? from_lane_xor<4>(c) : stride == 8u ? from_lane_xor<8>(c)
                                     : stride == 16u ? from_lane_xor<16>(c) : from_lane_xor<32>(c);
                    const bool desc = (lane & size) == 0;
                    const bool lower = (lane & stride) == 0;
                    const bool take_max = lower == desc;
                    c = take_max ? (o > c ? o : c) : (o < c ? o : c);
                }
            }
            cand[lane] = c;
        }
        __syncthreads();
        return;
    }
    if (BIG && n <= 4u * NT) {
        sort_desc_regs(cand, n);
        return;
    }
    uint32_t p = 128;
    while (p < n) {
        p <<= 1;
    }
    for (uint32_t i = n + threadIdx.x; i < p; i += NT) {
        cand[i] = 0;
    }
    __syncthreads();
    for (uint32_t size = 2; size <= p; size <<= 1) {
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            for (uint32_t i = threadIdx.x; i < (p >> 1); i += NT) {
                const uint32_t pos = ((i / stride) * (stride << 1)) + (i % stride);
                const uint32_t partner = pos + stride;
                const bool desc = (pos & size) == 0;
                const uint64_t x = cand[pos], y = cand[partner];
                if (desc ? x < y : x > y) {
                    cand[pos] = y;
                    cand[partner] = x;
                }
            }
            __syncthreads();
        }
    }
}

// ------------------------------------------------------------------ tail

// Counts one emission of `id` in a scratch: the dense count, the id's bit in the bitmap of the
// ids that were ever counted, the largest count any id has reached (the first spare word behind
// the bitmap: never lowered, so an upper bound after un-counting) and an id that reached it (the
// second spare word).  That id is a hint only - writers race, un-counting leaves it alone - and
// readers take its count from the histogram.  Returns the count before.
__device__ __forceinline__ uint32_t count_token(const RowArgs& a, uint32_t id, uint32_t vocab) {
    // The largest count so far is read beside the increment (one round trip for both): a launch
    // has one writer per scratch, so what the maximum becomes follows from the two, and nothing
    // waits for the maximum's own update.
    const uint32_t words = (vocab + 31u) / 32u;
    const uint32_t top = gload(&a.touched[words]);
    const uint32_t before = atomicAdd(&a.counts[id], 1u);
    atomicOr(&a.touched[id >> 5], 1u << (id & 31u));
    if (top <= before + 1u) {
        atomicMax(&a.touched[words], before + 1u);
        a.touched[words + 1u] = id;
    }
    return before;
}

// `sh`: where a launch whose rows draw in order learns what this row drew and the count the id
// has now (null otherwise: nobody then waits for the increment to come back).
// The increments alone, nothing waited for: for rows that draw in order within one launch, whose
// workgroup knows the counts itself and brings the largest count up to date once at the end.
__device__ __forceinline__ void count_token_blind(const RowArgs& a, uint32_t id) {
    atomicAdd(&a.counts[id], 1u);
    atomicOr(&a.touched[id >> 5], 1u << (id & 31u));
}

// `sh`: where a launch whose rows draw in order learns what this row drew (null otherwise).
__device__ __forceinline__ void emit(const RowArgs& a, uint32_t id, uint32_t vocab, Shared* sh = nullptr) {
    *a.out_id = id;
    if ((a.flags & F_PEN) && id < vocab) {
        if (sh != nullptr) {
            count_token_blind(a, id);
        } else {
            count_token(a, id, vocab);
        }
    }
    if (sh != nullptr) {
        sh->emitted_id = id;
    }
}

// First slot of prefix[0..n) whose value exceeds target, else the last slot.
__device__ __forceinline__ uint32_t pick_sequential(const float* prefix, uint32_t n, float target) {
    for (uint32_t i = 0; i < n; ++i) {
        if (target < prefix[i]) {
            return i;
        }
    }
    return n - 1;
}

// log p(id) = (u*c2 - mc - log2 s) * ln 2, with the id's exponent u*c2 formed exactly as
// the row sum formed its terms, so the two cancel when the id carries all the mass.
// Emits `id` and, when asked, its log-probability, with the memory operations of both in one
// round trip: the count's atomic increment returns the count the penalties used, and the logit
// loads beside it.
template <int DT>
__device__ __forceinline__ void finish_token(const RowArgs& a, Shared& sh, uint32_t id, uint32_t vocab,
                                             bool in_order = false) {
    *a.out_id = id;
    const bool pen = (a.flags & F_PEN) != 0;
    const bool want = a.out_logprob != nullptr;
    if (id >= vocab) {
        if (want) {
            *a.out_logprob = NEG_INF;
        }
        if (in_order) {
            sh.emitted_id = id;
        }
        return;
    }
    // The id's logit is asked for before the increments (it comes back with the count), and
    // the logarithm of the row's sum is formed while they are on their way.
    const float l = want ? load_logit<DT>(a.logits, id) : 0.0f;
    const bool allowed = !want || a.allow == nullptr || bit_of(a.allow, id);
    uint32_t before = 0, top = 0;
    const uint32_t words = (vocab + 31u) / 32u;
    if (in_order) {
        // Rows that draw in order: the next row learns the id; nobody waits for the increments.
        sh.emitted_id = id;
        if (pen) {
            count_token_blind(a, id);
        }
    } else if (pen) {
        // (count_token(), taken apart so that nothing between here and the logarithm below
        // waits for memory)
        top = gload(&a.touched[words]);
        before = atomicAdd(&a.counts[id], 1u);
        atomicOr(&a.touched[id >> 5], 1u << (id & 31u));
    }
    const double base = want ? sh.lse_mc + log2(sh.lse_s) : 0.0;
    if (pen && !in_order && top <= before + 1u) {
        atomicMax(&a.touched[words], before + 1u);
        a.touched[words + 1u] = id;
    }
    if (want) {
        const float u = finish_pre_temperature(a, id, l, before, allowed);
        float lp = NEG_INF;
        if (u > NEG_INF) {
            const double e = (double)u * (double)a.c2 - base;
            lp = fminf((float)(e * 0.6931471805599453), 0.0f);  // the sum is approximate: clamp
        }
        *a.out_logprob = lp;
    }
}

// cand[0..n) holds the row's candidates (at least its top-k); finishes the row.
// SPEC_WAVE: compile the speculative draw of at most 64 candidates as one wave too (the kernel
// of rows that draw in order, where every row's tail is a step of a chain; elsewhere its scalar
// registers would be taken from the scan).
template <int DT, bool BIG, bool SPEC_WAVE = false>
__device__ __forceinline__ void tail(const RowArgs& a, uint32_t vocab, uint32_t step, uint32_t n, bool sorted,
                     uint64_t* cand, Shared& sh, const LaunchCfg& cfg) {
#ifdef LILY_TAIL_TRACE
#define TAIL_MARK(i) phase(cfg, i)
#else
#define TAIL_MARK(i)
#endif
    const uint32_t tid = threadIdx.x;
    if (n == 0) {
        // No finite value anywhere: the oracle's order then starts at id 0.
        if (tid == 0) {
            if (a.out_logprob) {
                *a.out_logprob = NEG_INF;
            }
            emit(a, 0, vocab, cfg.chain_rows != 0u ? &sh : nullptr);
            if (a.dbg_counts) {
                a.dbg_counts[0] = 0;
                a.dbg_counts[1] = 1;  // the reference keeps rank 0 whatever its value
            }
            if (a.mode == MODE_DRAFT) {
                *a.q_n = 0;
            }
        }
        return;
    }
    // The speculative draw's proposal and the length of the draft's distribution are asked
    // for now, so that they have arrived when the candidates are ranked and summed.
    uint32_t spec_d = 0, spec_qn = 0;
    if (a.mode == MODE_SPEC) {
        spec_d = *a.draft;
        spec_qn = *a.q_n;
    }
    if (!sorted) {
        sort_desc<BIG>(cand, n);
    }
    TAIL_MARK(8);
    const uint32_t k = min(a.k, n);
    const float top = composite_value(cand[0]);
    if (k <= 64u && (a.mode != MODE_SPEC || (SPEC_WAVE && spec_qn <= 64u))) {
        // One wave, a candidate per lane.  The sums keep the reference's left-to-right f32
        // order: every lane runs the same chain of 64 additions on values read lane by lane
        // (lanes past k hold 0, which changes nothing), so nothing waits on LDS.
        if (tid >= 64u) {
            return;
        }
        const uint32_t lane = tid;
        const uint64_t c = lane < k ? cand[lane] : 0ull;
        const float p = lane < k ? lilym_expf(composite_value(c) - top) : 0.0f;
        if (lane < k) {
            if (a.dbg_ids) {
                a.dbg_ids[lane] = composite_id(c);
            }
            if (a.dbg_probs) {
                a.dbg_probs[lane] = p;
            }
        }
        const int pbits = (int)lilym_f32_bits(p);
        float cum = 0.0f, before = 0.0f, mine = 0.0f;
#pragma unroll
        for (int i = 0; i < 64; ++i) {
            before = lane == (uint32_t)i ? cum : before;
            cum += lilym_bits_f32((uint32_t)__builtin_amdgcn_readlane(pbits, i));
            mine = lane == (uint32_t)i ? cum : mine;
        }
        // (the chain's last value is the row total: the same additions in the same order)
        const float limit = a.top_p * cum;
        const bool stop = lane >= 1u && lane < k && !(before < limit && p >= a.min_p);
        const uint64_t stops = __ballot(stop);
        const uint32_t kept = stops != 0ull ? (uint32_t)__builtin_ctzll(stops) : k;
        const float mass = __shfl(mine, (int)kept - 1);
        if (lane == 0 && a.dbg_counts) {
            a.dbg_counts[0] = k;
            a.dbg_counts[1] = kept;
        }
        if (a.mode == MODE_DRAFT) {
            if (lane < kept) {
                a.q_ids[lane] = composite_id(c);
                a.q_probs[lane] = p / mass;
            }
            if (lane == 0) {
                *a.q_n = kept;
            }
        }
        const float u1 = (a.flags & F_UNIFORM) ? a.uniform : lilym_uniform_for(a.seed, step);
        if (SPEC_WAVE && a.mode == MODE_SPEC) {
            // Speculative draw (sample.metal:596-658, cpu_spec at tests/unit/kernels/sample.rs:264-283)
            // in the same wave: the draft's distribution (at most 64 entries here) sits an entry
            // per lane, lookups are ballots and lane reads, and the residual's sums run the same
            // left-to-right chains as above.
            const uint32_t d = spec_d, qn = spec_qn;
            const uint32_t my_id = composite_id(c);
            const uint32_t q_id = lane < qn ? a.q_ids[lane] : 0xffffffffu;
            const float q_p = lane < qn ? a.q_probs[lane] : 0.0f;
            const float p_norm = p / mass;
            const uint64_t at_p = __ballot(lane < kept && my_id == d);
            const uint64_t at_q = __ballot(lane < qn && q_id == d);
            const float p_d = at_p != 0ull ? __shfl(p_norm, (int)__builtin_ctzll(at_p)) : 0.0f;
            const float q_d = at_q != 0ull ? __shfl(q_p, (int)__builtin_ctzll(at_q)) : 0.0f;
            if (u1 * q_d < p_d) {
                if (lane == 0) {
                    finish_token<DT>(a, sh, d, vocab, cfg.chain_rows != 0u);
                }
                return;
            }
            // The draft's probability of each candidate, then the residual max(0, p - q).
            int match = -1;   // the lane that holds this candidate's id in the draft's list
            const int qid_bits = (int)q_id;
#pragma unroll
            for (int j = 0; j < 64; ++j) {
                const uint32_t idj = (uint32_t)__builtin_amdgcn_readlane(qid_bits, j);
                match = ((uint32_t)j < qn && idj == my_id) ? j : match;
            }
            const float q_there = __shfl(q_p, match < 0 ? 0 : match);
            const float q_mine = match < 0 ? 0.0f : q_there;
            const float res = lane < kept ? fmaxf(p_norm - q_mine, 0.0f) : 0.0f;
            const int rbits = (int)lilym_f32_bits(res);
            const float u2 = (a.flags & F_UNIFORM) ? a.uniform2
                                                   : lilym_uniform_for(a.seed, lilym_residual_step(step));
            float r_cum = 0.0f, r_mine = 0.0f;
#pragma unroll
            for (int i = 0; i < 64; ++i) {
                r_cum += lilym_bits_f32((uint32_t)__builtin_amdgcn_readlane(rbits, i));
                r_mine = lane == (uint32_t)i ? r_cum : r_mine;
            }
            const float r_total = r_cum;   // lanes past `kept` added 0
            uint64_t picks;
            if (r_total > 0.0f) {
                picks = __ballot(lane < kept && u2 * r_total < r_mine);
            } else {
                // Only rounding gives a rejected proposal a massless residual: draw from p.
                picks = __ballot(lane < kept && u2 * mass < mine);
            }
            const uint32_t slot = picks != 0ull ? (uint32_t)__builtin_ctzll(picks) : kept - 1u;
            const uint32_t id = ~(uint32_t)__shfl((int)(uint32_t)c, (int)slot);
            if (lane == 0) {
                finish_token<DT>(a, sh, id, vocab, cfg.chain_rows != 0u);
            }
            return;
        }
        const uint64_t hits = __ballot(lane < kept && u1 * mass < mine);
        const uint32_t slot = hits != 0ull ? (uint32_t)__builtin_ctzll(hits) : kept - 1u;
        const uint32_t id = ~(uint32_t)__shfl((int)(uint32_t)c, (int)slot);
        if (lane == 0) {
            finish_token<DT>(a, sh, id, vocab, cfg.chain_rows != 0u);
        }
        return;
    }
    for (uint32_t i = tid; i < k; i += NT) {
        const float p = lilym_expf(composite_value(cand[i]) - top);
        sh.prob[i] = p;
        if (a.dbg_ids) {
            a.dbg_ids[i] = composite_id(cand[i]);
        }
        if (a.dbg_probs) {
            a.dbg_probs[i] = p;
        }
    }
    __syncthreads();
    TAIL_MARK(9);
    // The reference's left-to-right f32 sums, by one wave, 64 candidates at a time with a
    // candidate per lane; every prefix is kept.  The row total is the last prefix, and the sum
    // the reference holds before rank r is the prefix of rank r - 1: the cut by top-p and min-p
    // and the inverse-CDF pick then are searches every thread takes part in.
    //
    // While the running sum S stays inside one binade it is an integer m in units of its last
    // place u, and adding p <= S rounds to m + floor(p / u) + (frac(p / u) > 1/2): integer
    // additions, which a wave sums in six data-parallel moves, exactly.  (p / u, its integer
    // part and its fraction are exact in f32: u is a power of two and p has no more bits than
    // S.)  A block of 64 in which some fraction is exactly 1/2 (the rounding then depends on
    // m's parity) or the sum leaves its binade - and the first block, whose sum starts at 0 -
    // is added the slow way: a chain of 63 additions, each step adding the lane's value to the
    // running sum of the lane below (a shift by one lane across the whole wave; lane 0 has no
    // lane below and keeps what it has), after which every lane holds its final prefix.  The
    // candidates' weights are at most 1 and the first is 1, so the sum crosses at most ten
    // binades and a peaked row none.  (Restarting inside a block at the lane that leaves the
    // binade, instead of giving the block to the chain, was slower: a round of the exact form
    // costs a third of a chain, and a flat row then takes 25 rounds.)
    if (tid < 64u) {
        float carry = 0.0f;
        for (uint32_t r0 = 0; r0 < k; r0 += 64u) {
            const uint32_t i = r0 + tid;
            const float p = i < k ? sh.prob[i] : 0.0f;
            float run;
            bool done = false;
            const uint32_t sbits = lilym_f32_bits(carry), sexp = (sbits >> 23) & 0xffu;
            // (a normal, positive sum whose last place and its inverse are normal numbers too)
            if ((int32_t)sbits > 0 && sexp >= 24u && sexp <= 253u) {
                const float inv_u = lilym_bits_f32((277u - sexp) << 23);   // 2^(23 - e)
                const float u = lilym_bits_f32((sexp - 23u) << 23);        // 2^(e - 23)
                const uint32_t m0 = (sbits & 0x7fffffu) | 0x800000u;
                const float q = p * inv_u;
                const uint32_t n = (uint32_t)q;
                const float frac = q - (float)n;
                const bool fits = p >= 0.0f && p <= carry;
                const uint32_t m = m0 + wave_scan_u32(n + (frac > 0.5f ? 1u : 0u));
                const uint32_t last = (uint32_t)__builtin_amdgcn_readlane((int)m, 63);
                if (__ballot(frac == 0.5f || !fits) == 0ull && last < 0x1000000u) {
                    run = (float)m * u;
                    done = true;
                }
            }
            if (!done) {
                run = carry + p;  // final in lane 0
#pragma unroll
                for (int j = 1; j < 64; ++j) {
                    // Two idle cycles between a lane's write and the neighbour's read of it.
                    asm volatile("s_nop 1\n\tv_add_f32_dpp %0, %0, %1 wave_shr:1 row_mask:0xf bank_mask:0xf"
                                 : "+v"(run)
                                 : "v"(p));
                }
            }
            if (i < k) {
                sh.cum[i] = run;
            }
            carry = lilym_bits_f32((uint32_t)__builtin_amdgcn_readlane((int)lilym_f32_bits(run), 63));
        }
    }
    __syncthreads();
    TAIL_MARK(10);
    auto first_of = [&](uint32_t mine_first) -> uint32_t {  // the lowest index any thread found
        mine_first = wave_min_u32(mine_first);
        if ((tid & 63u) == 0) {
            sh.red_i[tid >> 6] = mine_first;
        }
        __syncthreads();
        uint32_t r = sh.red_i[0];
        for (int i = 1; i < NWAVE; ++i) {
            r = min(r, sh.red_i[i]);
        }
        __syncthreads();
        return r;
    };
    const float limit = a.top_p * sh.cum[k - 1];
    uint32_t stop = k;
    for (uint32_t r = 1 + tid; r < k; r += NT) {
        if (!(sh.cum[r - 1] < limit && sh.prob[r] >= a.min_p)) {
            stop = min(stop, r);
        }
    }
    if (tid == 0) {
        sh.p_d = 0.0f;
        sh.q_d = 0.0f;
    }
    const uint32_t n_keep = first_of(stop);
    const float mass = sh.cum[n_keep - 1];
    TAIL_MARK(11);
    const float u1 = (a.flags & F_UNIFORM) ? a.uniform : lilym_uniform_for(a.seed, step);
    if (tid == 0) {
        if (a.dbg_counts) {
            a.dbg_counts[0] = k;
            a.dbg_counts[1] = n_keep;
        }
    }
    // First slot of cum[0..n) whose value exceeds target, else the last slot.
    auto pick = [&](const float* prefix, uint32_t n, float target) -> uint32_t {
        uint32_t hit = n - 1u;
        for (uint32_t i = tid; i < n; i += NT) {
            if (target < prefix[i]) {
                hit = min(hit, i);
            }
        }
        return first_of(hit);
    };

    if (a.mode == MODE_DRAFT) {
        for (uint32_t i = tid; i < n_keep; i += NT) {
            a.q_ids[i] = composite_id(cand[i]);
            a.q_probs[i] = sh.prob[i] / mass;
        }
        if (tid == 0) {
            *a.q_n = n_keep;
        }
    }

    if (a.mode != MODE_SPEC) {
        const uint32_t slot = pick(sh.cum, n_keep, u1 * mass);
        TAIL_MARK(12);
        if (tid == 0) {
            const uint32_t id = composite_id(cand[slot]);
            finish_token<DT>(a, sh, id, vocab, cfg.chain_rows != 0u);
        }
        return;
    }

    // Speculative draw (sample.metal:596-658, cpu_spec at tests/unit/kernels/sample.rs:264-283).
    const uint32_t d = spec_d;
    const uint32_t qn = min(spec_qn, K_CAP);
    for (uint32_t i = tid; i < n_keep; i += NT) {
        if (composite_id(cand[i]) == d) {
            sh.p_d = sh.prob[i] / mass;
        }
    }
    for (uint32_t j = tid; j < qn; j += NT) {
        if (a.q_ids[j] == d) {
            sh.q_d = a.q_probs[j];
        }
    }
    __syncthreads();
    if (u1 * sh.q_d < sh.p_d) {
        if (tid == 0) {
            finish_token<DT>(a, sh, d, vocab, cfg.chain_rows != 0u);
        }
        return;
    }
    for (uint32_t i = tid; i < n_keep; i += NT) {
        const uint32_t id = composite_id(cand[i]);
        // The draft's probability of this id: its entries eight at a time, loaded whatever they
        // hold (a loop that stops at the match is a memory round trip per entry; ids are
        // listed once, so going on changes nothing).
        float q_i = 0.0f;
        for (uint32_t j0 = 0; j0 < qn; j0 += 8u) {
            uint32_t qi[8];
            float qp[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const uint32_t j = min(j0 + (uint32_t)q, qn - 1u);
                qi[q] = a.q_ids[j];
                qp[q] = a.q_probs[j];
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                if (j0 + (uint32_t)q < qn && qi[q] == id) {
                    q_i = qp[q];
                }
            }
        }
        sh.res[i] = fmaxf(sh.prob[i] / mass - q_i, 0.0f);
    }
    __syncthreads();
    if (tid == 0) {
        const float u2 = (a.flags & F_UNIFORM) ? a.uniform2
                                               : lilym_uniform_for(a.seed, lilym_residual_step(step));
        float total = 0.0f;
        for (uint32_t i = 0; i < n_keep; ++i) {
            total += sh.res[i];
        }
        uint32_t slot;
        if (total > 0.0f) {
            const float target = u2 * total;
            float cum = 0.0f;
            slot = n_keep - 1;
            for (uint32_t i = 0; i < n_keep; ++i) {
                cum += sh.res[i];
                if (target < cum) {
                    slot = i;
                    break;
                }
            }
        } else {
            // Only rounding gives a rejected proposal a massless residual: draw from p.
            slot = pick_sequential(sh.cum, n_keep, u2 * mass);
        }
        const uint32_t id = composite_id(cand[slot]);
        finish_token<DT>(a, sh, id, vocab, cfg.chain_rows != 0u);
    }
}


}  // namespace lily
