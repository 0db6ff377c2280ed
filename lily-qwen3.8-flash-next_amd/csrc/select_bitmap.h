// select_bitmap.h - the select of rows that cannot be streamed: allow-masks that are neither
// sparse nor nearly full, and every row with k > 64.
//
// How a slice is scanned:
//   * 16-byte loads, 8 bf16 or 4 f32 per lane, four loads in flight per lane.
//   * Ids that need more than "widen and compare" - masked out, penalised (count > 0) or
//     biased - are marked in an LDS bitmap built once per slice; the stream treats them as
//     -inf and the few that are allowed are evaluated exactly afterwards ("specials").
//   * The filter works on the value BEFORE the division by the temperature (the division is
//     monotone), so the hot loop has no division.  Candidates that pass go to an LDS buffer;
//     the exact arithmetic runs on those only.
//   * k <= 64: single pass.  Every lane keeps its running maximum; the minimum over G >= k
//     lane groups of the group maximum is a lower bound of the k-th largest value (G distinct
//     elements reach it), refreshed every block of loads; elements at or above it (less a
//     4-ulp slack for values the division merges) are appended.
//   * k > 64: two passes.  The k-th largest of the per-lane-per-slot running maxima is the
//     bound; the second pass (L2 / MALL hits) collects.
//   * Too many candidates (huge tie classes, adversarial order) or a failed slack check: the
//     caller redoes the slice with select_exhaustive.
#pragma once

#include "device_common.h"

namespace lily {

// The exact top-k of the slice in cand[0..n) as adjusted-value composites (n through
// sh.n_cand, `sorted` tells whether they are in order); false when the slice must be
// redone exhaustively.  Also leaves the slice's log-sum-exp in sh when LSE.
//
// Rows with an allow-mask keep every masked, penalised or biased id out of the stream
// through the LDS bitmap (`mask_stream`).  Rows with penalties or a bias list only are
// streamed raw ("patch"): candidates that turn out to be penalised or biased are
// dropped, all such ids are evaluated exactly afterwards and re-enter with their true
// value, the row sum is corrected by their raw and true terms, and the a-posteriori
// check below covers the case where a raw value had lifted the threshold too far.
template <int DT, bool EXCL, bool LSE>
__device__ __forceinline__ bool select_fast(const RowArgs& a, const Geo<DT>& g, uint32_t k, bool two_pass,
                            uint64_t* cand, uint32_t cap, uint32_t* excl, Shared& sh,
                            const LaunchCfg& cfg, bool& sorted) {
    constexpr int E = Geo<DT>::E;
    constexpr int U = UNROLL;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    const uint32_t nchunks = g.ce - g.cb;
    const uint32_t nwords = (nchunks * E + 31u) / 32u;
    const uint32_t row_words = (g.vocab + 31u) / 32u;
    const uint32_t nblocks = (nchunks + NT * U - 1) / (NT * U);
    const int64_t slice_id0 = (int64_t)g.cb * E - g.pad;
    const float c2 = a.c2;
    const bool pen = (a.flags & F_PEN) != 0;
    const bool special_row = EXCL && (a.allow != nullptr || pen || a.n_bias != 0);
    const bool mask_stream = EXCL && a.allow != nullptr;
    const bool patch = special_row && !mask_stream;
    const bool want_lse = LSE && a.out_logprob != nullptr;
    uint32_t* list = excl + cfg.excl_words;
    const uint32_t list_cap = cfg.list_cap;

    auto fetch = [&](u32x4 (&dst)[U], uint32_t b) {
        for (int u = 0; u < U; ++u) {
            dst[u] = g.load_raw(g.cb + (b * U + u) * NT + tid);
        }
    };
    u32x4 cur[U];
    if (nblocks > 0) {
        fetch(cur, 0);  // in flight while the bitmap is built
    }

    if (tid == 0) {
        sh.n_cand = 0;
        sh.need = 0;
    }
    if (tid < NWAVE) {
        sh.wthr[tid] = NEG_INF;
        sh.wthr_f[tid] = F32_LOWEST;
    }
    if (mask_stream) {
        // Bit b of the slice bitmap <-> id cb*E - pad + b.  Set = not streamed.
        for (uint32_t i0 = tid; i0 < nwords; i0 += 4 * NT) {
            uint32_t x[4];
            for (int q = 0; q < 4; ++q) {  // four words' loads in flight before any store
                const uint32_t i = i0 + (uint32_t)q * NT;
                const int64_t id0 = slice_id0 + (int64_t)i * 32;
                x[q] = ~range32_at(g.id_lo, g.id_hi, id0);
                if (i < nwords) {
                    x[q] |= ~bits32_at(a.allow, row_words, id0);
                    if (pen) {
                        x[q] |= bits32_at(a.touched, row_words, id0);
                    }
                }
            }
            for (int q = 0; q < 4; ++q) {
                const uint32_t i = i0 + (uint32_t)q * NT;
                if (i < nwords) {
                    excl[i] = x[q];
                }
            }
        }
        __syncthreads();
        for (uint32_t i = tid; i < a.n_bias; i += NT) {
            const uint32_t id = gload(&a.bias[i].id);
            if (id >= g.id_lo && id < g.id_hi) {
                const uint32_t b = id + g.pad - g.cb * E;
                atomicOr(&excl[b >> 5], 1u << (b & 31u));
            }
        }
    }
    __syncthreads();
    phase(cfg, 1);

    // Lanes per group: the largest power of two with NT / L >= k groups (at most a wave).
    uint32_t group = 64;
    while (group > 1 && NT / group < k) {
        group >>= 1;
    }

    float lane_max = NEG_INF;
    float ms[8];
    for (int j = 0; j < 8; ++j) {
        ms[j] = NEG_INF;
    }
    WaveLse wl;
    wl.init();
    float thr_f = F32_LOWEST;
    const uint8_t* excl_bytes = reinterpret_cast<const uint8_t*>(excl);
    // While scanning, wave w appends to cand[w * seg, (w + 1) * seg); wcount is its fill.
    const uint32_t seg = cap / NWAVE;
    uint64_t* region = cand + w * seg;
    uint32_t wcount = 0;

    // Lower bound of the k-th largest value from the lanes' running maxima: the minimum
    // over groups of the group maximum (other waves' entries may be older: still bounds).
    auto update_threshold = [&](bool first) {
        float t = lane_max;
        for (uint32_t o = 1; o < group; o <<= 1) {
            t = fmaxf(t, __shfl_xor(t, (int)o));
        }
        for (uint32_t o = group; o < 64; o <<= 1) {
            t = fminf(t, __shfl_xor(t, (int)o));
        }
        if (lane == 0) {
            __hip_atomic_store(&sh.wthr[w], t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        if (first) {
            __syncthreads();  // every wave has published its first statistic
        }
        for (int i = 0; i < NWAVE; ++i) {
            t = fminf(t, __hip_atomic_load(&sh.wthr[i], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_WORKGROUP));
        }
        thr_f = fmaxf(thr_f, lower_by_slack(t));
    };

    // Stages of the scan.  Single pass (k <= 64): MAIN.  Two passes: BOUND then COLLECT.
    // A failed a-posteriori check re-enters at COLLECT with a fixed threshold.
    enum { MAIN = 0, BOUND = 1, COLLECT = 2 };
    int stage = two_pass ? BOUND : MAIN;
    bool have_first = nblocks > 0;

    LseAcc lse_true, lse_raw;  // specials: true terms, and (patch) the raw terms streamed
    lse_true.init();
    lse_raw.init();
    bool lse_done = !want_lse;
    bool rescued = false;

    for (int round = 0; round < 4; ++round) {
        const bool stats = stage == MAIN;
        const bool submax = stage == BOUND;
        const bool lse_on = want_lse && stage != COLLECT;
        const bool filter = stage != BOUND;
        // One pass over the slice, double-buffered: block b+1 is in flight while b is
        // processed.
        if (nblocks > 0 && !have_first) {
            fetch(cur, 0);
        }
        have_first = false;
        if (stats && nblocks > 0) {
            // Block 0's own maxima first, so that its elements already meet a real threshold.
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t c = g.cb + (uint32_t)u * NT + tid;
                float v[E];
                unpack<DT>(cur[u], v);
                if (mask_stream && c >= g.main_lo && c < g.main_hi) {
                    const uint32_t rel = c - g.cb;
                    const uint32_t m = E == 8 ? excl_bytes[rel]
                                              : ((excl_bytes[rel >> 1] >> ((rel & 1u) * 4u)) & 15u);
#pragma unroll
                    for (int j = 0; j < E; ++j) {
                        v[j] = ((m >> j) & 1u) ? NEG_INF : v[j];
                    }
                }
#pragma unroll
                for (int j = 0; j < E; ++j) {
                    lane_max = fmaxf(lane_max, v[j]);
                }
            }
            update_threshold(true);
        }
        for (uint32_t b = 0; b < nblocks; ++b) {
            if (b > 0) {
                fetch(cur, b);
            }
            {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint32_t c = g.cb + (b * U + u) * NT + tid;
                    float v[E];
                    unpack<DT>(cur[u], v);
                    if (mask_stream && c >= g.main_lo && c < g.main_hi) {
                        const uint32_t rel = c - g.cb;
                        uint32_t m;
                        if (E == 8) {
                            m = excl_bytes[rel];
                        } else {
                            m = (excl_bytes[rel >> 1] >> ((rel & 1u) * 4u)) & 15u;
                        }
#pragma unroll
                        for (int j = 0; j < E; ++j) {
                            // all-ones when bit j is set: the element reads as -inf
                            const uint32_t on = (uint32_t)((int32_t)(m << (31 - j)) >> 31);
                            v[j] = lilym_bits_f32((lilym_f32_bits(v[j]) & ~on) | (0xff800000u & on));
                        }
                    }
                    float m8 = v[0];
#pragma unroll
                    for (int j = 1; j < E; ++j) {
                        m8 = fmaxf(m8, v[j]);
                    }
                    if (stats) {
                        lane_max = fmaxf(lane_max, m8);
                    }
                    if (submax) {
#pragma unroll
                        for (int j = 0; j < E; ++j) {
                            const int slot = (E == 8) ? j : ((u & 1) * 4 + j);
                            ms[slot] = fmaxf(ms[slot], v[j]);
                        }
                    }
                    if (LSE && lse_on) {
                        wl.template add<E>(v, m8, c2);
                    }
                    if (filter && __ballot(m8 >= thr_f) != 0ull) {
#pragma unroll
                        for (int j = 0; j < E; ++j) {
                            append(v[j] >= thr_f, v[j], g.id_of(c, j), region, seg, wcount);
                        }
                    }
                }
            }
            if (stats) {
                update_threshold(false);
            }
        }
        if (stage == MAIN && nblocks == 0) {
            update_threshold(true);  // keeps the barrier count the same in every workgroup
        }
        if (stage == BOUND) {
            // The k-th largest of the NT x 8 sub-stream maxima bounds the k-th largest
            // element; a margin covers maxima that belong to ids evaluated separately.
            const uint32_t kb = patch ? min(k + k / 8u + 16u, (uint32_t)(NT * 8)) : k;
            thr_f = lower_by_slack(wg_kth_largest(ms, kb, sh));
            stage = COLLECT;
            continue;
        }
        if (round == 0 || (two_pass && round == 1)) {
            phase(cfg, 2);
        }

        if (lane == 0) {
            sh.wthr_f[w] = thr_f;
        }
        __syncthreads();
        float filt = sh.wthr_f[0];
        for (int i = 1; i < NWAVE; ++i) {
            filt = fmaxf(filt, sh.wthr_f[i]);
        }
        // Close the gaps between the waves' regions (entries travel through registers).
        if (lane == 0) {
            sh.red_i[w] = wcount;
        }
        __syncthreads();
        uint32_t n = 0, my_base = 0;
        bool overflow = false;
        for (int i = 0; i < NWAVE; ++i) {
            const uint32_t ci = sh.red_i[i];
            overflow = overflow || ci > seg;
            if ((uint32_t)i == w) {
                my_base = n;
            }
            n += min(ci, seg);
        }
        if (overflow) {
            return false;
        }
        {
            constexpr int PERW = CAND_CAP / NT;  // a wave moves its own region, PERW per lane
            uint64_t keep[PERW];
            const uint32_t mine = min(wcount, seg);
#pragma unroll
            for (int q = 0; q < PERW; ++q) {
                const uint32_t i = lane + (uint32_t)q * 64u;
                keep[q] = i < mine ? region[i] : 0ull;
            }
            __syncthreads();
#pragma unroll
            for (int q = 0; q < PERW; ++q) {
                const uint32_t i = lane + (uint32_t)q * 64u;
                if (i < mine) {
                    cand[my_base + i] = keep[q];
                }
            }
        }
        if (tid == 0) {
            sh.n_cand = n;
        }
        wcount = 0;
        __syncthreads();
        // Buffered composites hold the pre-temperature value: divide now, exactly.  In
        // patch mode a candidate that is penalised or biased carried its raw value: drop
        // it, the specials below bring it back with the true one.
        for (uint32_t i = tid; i < n; i += NT) {
            const uint64_t c = cand[i];
            const uint32_t id = composite_id(c);
            const bool drop = patch && ((pen && bit_of(a.touched, id)) || in_bias_list(a, id));
            cand[i] = drop ? 0ull : composite_of(composite_value(c) / a.temperature, id);
        }
        phase(cfg, 8);
        if (special_row) {
            // Specials: the ids that need exact evaluation, compacted into an LDS list and
            // walked four per thread at a time so a batch's gathers are independent loads.
            if (tid == 0) {
                sh.need = 0;
            }
            __syncthreads();
            auto one = [&](uint32_t id, float l, uint32_t cnt) {
                const float u = finish_pre_temperature(a, id, l, cnt, true);
                if (!lse_done) {
                    lse_true.add_one(u, c2);
                    // The raw term is taken off only where the stream added it: ids of the
                    // partial chunks at the row's ends were never streamed.
                    const uint32_t ch = (id + g.pad) / E;
                    if (patch && ch >= g.main_lo && ch < g.main_hi) {
                        lse_raw.add_one(l, c2);
                    }
                }
                if (u >= filt) {
                    const uint32_t at = atomicAdd(&sh.n_cand, 1u);
                    if (at < cap) {
                        cand[at] = composite_of(u / a.temperature, id);
                    }
                }
            };
            auto slow_one = [&](uint32_t id) {
                one(id, load_logit<DT>(a.logits, id), pen ? gload(a.counts + id) : 0u);
            };
            for (uint32_t i0 = 0; i0 < nwords; i0 += NT) {
                const uint32_t i = i0 + tid;
                const int64_t id0 = slice_id0 + (int64_t)i * 32;
                uint32_t bits = 0;
                if (i < nwords) {
                    if (mask_stream) {
                        bits = excl[i] & range32_at(g.id_lo, g.id_hi, id0) &
                               bits32_at(a.allow, row_words, id0);
                    } else if (pen) {
                        bits = bits32_at(a.touched, row_words, id0) &
                               range32_at(g.id_lo, g.id_hi, id0);
                    }
                }
                while (__ballot(bits != 0u) != 0ull) {
                    const bool has = bits != 0u;
                    const uint32_t id = has ? (uint32_t)(id0 + __builtin_ctz(bits)) : 0u;
                    bits &= bits - 1u;
                    if (!list_push(has, id, list, list_cap, sh)) {
                        slow_one(id);  // more specials than the list holds
                    }
                }
            }
            if (patch) {
                // Biased ids that are not penalised (those are listed already), once each.
                for (uint32_t i0 = 0; i0 < a.n_bias; i0 += NT) {
                    const uint32_t i = i0 + tid;
                    bool has = false;
                    uint32_t id = 0;
                    if (i < a.n_bias) {
                        id = gload(&a.bias[i].id);
                        has = id >= g.id_lo && id < g.id_hi && !(pen && bit_of(a.touched, id));
                        for (uint32_t j = 0; has && j < i; ++j) {
                            has = gload(&a.bias[j].id) != id;
                        }
                    }
                    if (!list_push(has, id, list, list_cap, sh)) {
                        slow_one(id);
                    }
                }
            }
            __syncthreads();
            phase(cfg, 9);
            const uint32_t m = min(sh.need, list_cap);
            for (uint32_t i0 = tid; i0 < m; i0 += 4 * NT) {
                uint32_t ids[4];
                float l[4];
                uint32_t cnt[4];
                for (int q = 0; q < 4; ++q) {
                    const uint32_t i = i0 + (uint32_t)q * NT;
                    ids[q] = i < m ? list[i] : 0xffffffffu;
                }
                for (int q = 0; q < 4; ++q) {
                    const bool ok = ids[q] != 0xffffffffu;
                    l[q] = ok ? load_logit<DT>(a.logits, ids[q]) : 0.0f;
                    cnt[q] = (ok && pen) ? gload(a.counts + ids[q]) : 0u;
                }
                for (int q = 0; q < 4; ++q) {
                    if (ids[q] != 0xffffffffu) {
                        one(ids[q], l[q], cnt[q]);
                    }
                }
            }
        }
        phase(cfg, 10);
        // Edge ids (partial 16-byte chunks at the row's ends) were not streamed: the ones
        // that are not specials (those were just handled) enter here with their raw value.
        for (int side = 0; side < 2; ++side) {
            const uint32_t lo = side == 0 ? g.id_lo : g.edge_hi_begin;
            const uint32_t hi = side == 0 ? g.edge_lo_end : g.id_hi;
            for (uint32_t id = lo + tid; id < hi; id += NT) {
                const bool allowed = a.allow == nullptr || bit_of(a.allow, id);
                const bool is_special =
                    special_row && ((pen && bit_of(a.touched, id)) || in_bias_list(a, id));
                if (allowed && !is_special) {
                    const float u = load_logit<DT>(a.logits, id);
                    if (!lse_done) {
                        lse_true.add_one(u, c2);
                    }
                    if (u >= filt && u > NEG_INF) {
                        const uint32_t at = atomicAdd(&sh.n_cand, 1u);
                        if (at < cap) {
                            cand[at] = composite_of(u / a.temperature, id);
                        }
                    }
                }
            }
        }
        phase(cfg, 11);
        if (!lse_done) {
            // Row sum = streamed sum - raw terms of the specials (patch) + their true terms.
            double m_s, s_s, m_t, s_t, m_r = 0.0, s_r = 0.0;
            bool bad = wg_merge_lse(sh, wl.ref, wl.s, m_s, s_s);   // a NaN logit among the streamed ones
            wg_merge_lse(sh, lse_true.mc, lse_true.s, m_t, s_t);
            if (patch) {
                wg_merge_lse(sh, lse_raw.mc, lse_raw.s, m_r, s_r);
            }
            double rest = s_s;
            if (patch && s_r > 0.0) {
                rest = s_s - s_r * exp2(m_r - m_s);
                bad = bad || !(rest > 0.05 * s_s);  // cancellation: the streamed sum is too coarse
            }
            if (bad) {
                phase(cfg, 12);
                // Rare: penalised ids held nearly all the raw mass, or a logit is a NaN.  Redo
                // the sum exactly.
                LseAcc exact;
                exact.init();
                exact_terms<DT>(a, g.id_lo, g.id_hi, c2, exact);
                double m_e, s_e;
                wg_merge_lse(sh, exact.mc, exact.s, m_e, s_e);
                if (tid == 0) {
                    sh.lse_mc = m_e;
                    sh.lse_s = s_e;
                }
            } else if (tid == 0) {
                const bool has_s = rest > 0.0, has_t = s_t > 0.0;
                const double m = has_s && has_t ? fmax(m_s, m_t) : (has_s ? m_s : m_t);
                double total = 0.0;
                if (has_s) {
                    total += rest * exp2(m_s - m);
                }
                if (has_t) {
                    total += s_t * exp2(m_t - m);
                }
                sh.lse_mc = m;
                sh.lse_s = total;
            }
            lse_done = true;
        }
        __syncthreads();
        n = sh.n_cand;
        phase(cfg, 3);
        if (n > cap) {
            return false;
        }
        sorted = false;
        n = select_topk(cand, n, k, sh, sorted);  // also drops the zeros
        // Every element that was not collected lies strictly below `filt`.  The result is
        // exact if k candidates were found and the k-th lies strictly above anything the
        // division could map an uncollected value to.
        bool good = true;
        float lowest_value = 0.0f;
        if (filt > F32_LOWEST) {
            uint32_t lowest = 0xffffffffu;
            for (uint32_t i = tid; i < n; i += NT) {
                lowest = min(lowest, (uint32_t)(cand[i] >> 32));
            }
            lowest = wave_min_u32(lowest);
            if (lane == 0) {
                sh.red_i[w] = lowest;
            }
            __syncthreads();
            lowest = sh.red_i[0];
            for (int i = 1; i < NWAVE; ++i) {
                lowest = min(lowest, sh.red_i[i]);
            }
            __syncthreads();
            const float below = lilym_key_value(lilym_order_key(filt) - 1u) / a.temperature;
            good = n >= k && lilym_order_key(below) < lowest;
            lowest_value = n > 0 ? lilym_key_value(lowest) : 0.0f;
        }
        if (good) {
            if (tid == 0) {
                sh.n_cand = n;
            }
            __syncthreads();
            return true;
        }
        if (rescued || n < k) {
            return false;
        }
        // k true candidates exist, so everything at or above the k-th of them (taken back
        // before the division, with slack) is enough: collect exactly that.
        rescued = true;
        stage = COLLECT;
        thr_f = lower_by_slack(lower_by_slack(lowest_value * a.temperature));
        if (tid == 0) {
            sh.n_cand = 0;
        }
        __syncthreads();
    }
    return false;
}


}  // namespace lily
