// select_stream.h - the one-pass streaming select (k <= 64).
#pragma once

#include "device_common.h"

namespace lily {

// ------------------------------------------------------------------ streaming select
//
// The select of rows with k <= STREAM_K_MAX and no allow-mask.  One pass, one barrier per
// block of NT x STREAM_UNROLL chunks, every 16-byte chunk read from memory once:
//
//   * Bound.  Each lane keeps the maximum of what it has seen; each wave takes the kw-th
//     largest of its 64 lane maxima (kw = ceil(k' / NWAVE), a 16-step ballot search on the
//     top half of the order key).  At least k' distinct elements are at or above the
//     minimum of the waves' values, so that minimum is a lower bound of the k'-th largest
//     value; it is refreshed after every block and is the same in every wave while a
//     block is processed, which makes the run reproducible.
//   * Owner side.  A lane whose chunk holds a value at or above the bound appends the whole
//     chunk (16 raw bytes + its index) to its wave's queue and leaves it out of the running
//     sum of exponentials; all other chunks only feed the lane maximum and the sum.
//   * Listed ids (penalised: the scratch's (id, count) list; biased: the row's bias list)
//     are sorted into per-block buckets in LDS before the scan.  While block b streams,
//     thread t also loads the chunk of "its" listed id of block b (the same cache lines
//     the owners are loading), evaluates the id exactly, offers it as a candidate, adds its
//     true term to the sum and - when the chunk was not queued, which it can tell from the
//     chunk's maximum and the block's bound - books the raw term the owner added, to be
//     taken off at the end.  Listed ids inside queued chunks go to a short drop list.
//   * After the scan the queued chunks are expanded: elements that are not on the drop list
//     add their term and, at or above the final bound, become candidates.
//
// Values are compared before the division by the temperature; candidates are divided
// exactly and the caller's check (k-th candidate strictly above anything a value below
// the bound can map to) decides whether the result stands.  Any overflow returns false.

struct StreamLds {
    u32x4* qraw;
    uint32_t* qidx;
    uint32_t* spec;
    uint64_t* fc;
    uint32_t* drop;
    uint32_t* dmask;   // per queue slot, a byte: bit j set = element j is a listed id
    uint32_t* bkt;
    uint32_t* bfill;
    uint2* hseg;
    uint32_t* bias_id;
    float* bias_delta;
    __device__ __forceinline__ void init() {
        char* b = reinterpret_cast<char*>(dyn_lds);
        qraw = reinterpret_cast<u32x4*>(b + OFF_QRAW);
        qidx = reinterpret_cast<uint32_t*>(b + OFF_QIDX);
        spec = reinterpret_cast<uint32_t*>(b + OFF_SPEC);
        fc = reinterpret_cast<uint64_t*>(b + OFF_FC);
        drop = reinterpret_cast<uint32_t*>(b + OFF_DROP);
        dmask = reinterpret_cast<uint32_t*>(b + OFF_DMASK);
        bkt = reinterpret_cast<uint32_t*>(b + OFF_BKT);
        bfill = reinterpret_cast<uint32_t*>(b + OFF_BFILL);
        bias_id = reinterpret_cast<uint32_t*>(b + OFF_BIAS);
        bias_delta = reinterpret_cast<float*>(b + OFF_BIAS + STREAM_BIAS_CAP * 4);
        hseg = reinterpret_cast<uint2*>(b + OFF_HSEG);
    }
};

// 2^(v*c - ref) as a double for any argument (0 below 2^-1000).
// 2^d for d in (-1000, 1000]: the fraction through the hardware exponential, the integer
// part as a power of two.
__device__ __forceinline__ double pow2_d(double d) {
    const double di = __builtin_floor(d);
    return __builtin_ldexp((double)__builtin_amdgcn_exp2f((float)(d - di)), (int)di);
}

// The largest 16-bit prefix P with at least `need` lanes holding key16 >= P; 0 when fewer
// than `need` lanes hold a non-zero key.
__device__ __forceinline__ uint32_t wave_kth_key16(uint32_t key16, uint32_t need) {
    uint32_t P = 0;
#pragma unroll
    for (int bit = 15; bit >= 0; --bit) {
        const uint32_t c = P | (1u << bit);
        const uint32_t cnt = (uint32_t)__popcll(__ballot(key16 >= c));
        P = cnt >= need ? c : P;
    }
    return P;
}

__device__ __forceinline__ double wg_sum_d(Shared& sh, double v) {
    v = wave_sum_d(v);
    if ((threadIdx.x & 63u) == 0) {
        sh.red_d[threadIdx.x >> 6] = v;
    }
    __syncthreads();
    double t = 0.0;
    for (int i = 0; i < NWAVE; ++i) {
        t += sh.red_d[i];
    }
    __syncthreads();
    return t;
}

// Records why the streaming select gave up (bit `why` of path_stats[3]) and returns false.
__device__ __forceinline__ bool stream_fail(const LaunchCfg& cfg, uint32_t why) {
    if (cfg.path_stats != nullptr && threadIdx.x == 0) {
        atomicOr(&cfg.path_stats[3], 1u << why);
    }
    return false;
}

template <int DT, bool LSE, bool MASKS>
__device__ __forceinline__ bool select_stream(const RowArgs& a, const Geo<DT>& g, uint32_t k, Shared& sh,
                                              const LaunchCfg& cfg, bool& sorted, uint64_t*& out) {
    constexpr int E = Geo<DT>::E;
    constexpr int U = STREAM_UNROLL;
    constexpr uint32_t BLOCK = NT * U;
    constexpr uint32_t QSEG = Q_CAP / NWAVE;
    constexpr uint32_t NONE = 0xffffffffu;
    constexpr uint32_t ID_MASK = (1u << SPEC_ID_BITS) - 1u;
    constexpr int PREG = 2;   // tail entries a thread keeps in registers between the two bucket passes
    const uint32_t tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    const uint32_t nchunks = g.ce - g.cb;
    const uint32_t nblocks = (nchunks + BLOCK - 1) / BLOCK;
    const bool pen = (a.flags & F_PEN) != 0;
    const uint32_t n_bias = a.n_bias;
    const bool want_lse = LSE && a.out_logprob != nullptr;
    const float c2 = a.c2;
    if (nblocks > MAX_BUCKETS || n_bias > STREAM_BIAS_CAP || g.vocab > (1u << SPEC_ID_BITS)) {
        return stream_fail(cfg, 1u);
    }
    StreamLds L;
    L.init();

    // Every load of a block is issued whatever its chunk: a conditional load makes the wait
    // for its result drain every load in flight, the blocks requested ahead included.  Chunks
    // past the slice's end read its last chunk instead (every chunk of the slice holds an
    // element of the row, so the 16 bytes are readable); chunks that are not streamed are
    // replaced by -inf when the block is worked on (`full_block`).
    const uint32_t c_last = g.ce - 1u;  // nblocks > 0 wherever a block is fetched
    auto fetch = [&](u32x4 (&dst)[U], uint32_t b) {
        const uint32_t c0 = g.cb + b * BLOCK + tid;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t c = min(c0 + (uint32_t)u * NT, c_last);
            dst[u] = gload(reinterpret_cast<const u32x4*>(g.base + (c << 4)));  // rows are below 4 GiB
        }
    };
    auto full_block = [&](uint32_t b) -> bool {
        const uint32_t c0 = g.cb + b * BLOCK;
        return c0 >= g.main_lo && c0 + BLOCK <= g.main_hi;
    };
    // ---- the slice's listed ids
    // The scratch's list comes in two parts.  Its sorted part (ascending ids, indexed by
    // buckets of 1 << SORT_SHIFT ids) is read straight from memory while the row streams:
    // block b's entries lie between two bucket starts, requested here by thread b.  Its tail
    // (the ids first counted since the list was last sorted: a few, the host has the list
    // sorted again before there are many) is bucketed by block in LDS below, together with
    // the bias list's ids and a dense mask's barred ids.  The tail's first PREG x NT entries
    // are requested together with the two lengths (the tail grows downwards from the end of
    // the list's memory, so their addresses depend on nothing), ahead of the first block of
    // the row, which is then in flight while they are bucketed.
    uint32_t n_sorted = 0, n_tail = 0, loaded = 0;
    uint32_t seg_s = 0, seg_e = 0;   // thread b: block b's entries of the sorted part
    uint32_t early[PREG];
    const ListEntry* list = a.pairs;
    if (pen) {
        // The lengths come through the scalar path (nothing writes them while the slices of
        // their row still read them): a vector load of a value that is the same in every lane
        // is moved to a scalar register at once, and that move would hold the loads below
        // back until the lengths had arrived.
        const LILY_CONST uint32_t* hdr = (const LILY_CONST uint32_t*)a.list_hdr;
        n_sorted = hdr[HDR_SORTED];
        n_tail = hdr[HDR_TAIL];
        if (tid < nblocks) {
            const uint32_t c0 = max(g.cb + tid * BLOCK, g.main_lo);
            const uint32_t c1 = min(g.cb + (tid + 1u) * BLOCK, g.main_hi);
            if (c1 > c0) {
                const uint32_t id_first = c0 * E - g.pad, id_last = c1 * E - g.pad - 1u;
                const uint32_t* start = a.list_hdr + LIST_HDR_WORDS;
                seg_s = gload(start + (id_first >> SORT_SHIFT));
                seg_e = gload(start + (id_last >> SORT_SHIFT) + 1u);
            }
        }
        // The host's bound of the tail's length says how much to request; a longer tail is
        // still read completely (by the loop further down), a shorter one costs idle loads.
        const uint64_t hint = (cfg.hint_replace != 0u ? 0u : a.tail_hint) + (uint64_t)cfg.hint_growth;
        const uint64_t want = (hint + NT - 1) / NT * NT;
        loaded = (uint32_t)min(want, (uint64_t)min(a.pairs_cap, (uint32_t)(PREG * NT)));
#pragma unroll
        for (int q = 0; q < PREG; ++q) {
            const uint32_t p = (uint32_t)q * NT + tid;
            early[q] = p < loaded ? gload(list + (a.pairs_cap - 1u - p)) : NONE;
        }
    }
    u32x4 buf_a[U], buf_b[U], buf_c[U];
    if (nblocks > 0) {
        fetch(buf_a, 0);
    }
    if (tid <= MAX_BUCKETS) {
        L.bkt[tid] = 0;
    }
    if (tid < MAX_BUCKETS) {
        L.bfill[tid] = 0;
    }
    if (tid < Q_CAP / 4) {
        L.dmask[tid] = 0;
    }
    if (tid < MAX_BUCKETS) {
        // A list that does not fit its memory is not used (checked below); its bucket starts
        // then mean nothing, and a start is never taken beyond the sorted part.
        seg_e = min(seg_e, n_sorted);
        seg_s = min(seg_s, seg_e);
        L.hseg[tid] = uint2{seg_s, seg_e};
        // A block with more listed ids than the workgroup has threads (see row_max below).
        const uint64_t big = __ballot(seg_e - seg_s > (uint32_t)NT);
        if (tid == 0) {
            sh.dense_listed = big != 0ull ? 1u : 0u;
        }
    }
    if (tid == 0) {
        sh.n_fc = 0;
        sh.n_drop = 0;
        sh.fail = 0;
    }
    for (uint32_t i = tid; i < n_bias; i += NT) {
        L.bias_id[i] = gload(&a.bias[i].id);
        L.bias_delta[i] = gload(&a.bias[i].delta);
    }
    __syncthreads();
    phase(cfg, 13);
    if ((uint64_t)n_sorted + n_tail > a.pairs_cap) {
        return stream_fail(cfg, 2u);  // the list overflowed: the bitmap and the counts hold the truth
    }
    // A row with an allow-mask is streamed when the mask is dense: its disallowed ids join the
    // listed ids (true value -inf).  Otherwise the row is left to the selects made for masks.
    // (MASKS is false in kernels whose launches hold no masked row.)
    const bool masked = MASKS && a.allow != nullptr;
    const uint32_t w_lo = g.id_lo >> 5, w_hi = (g.id_hi + 31u) >> 5;
    auto barred = [&](uint32_t i) -> uint32_t {  // disallowed ids of mask word i inside the slice
        return ~gload(a.allow + i) & range32_at(g.id_lo, g.id_hi, (int64_t)i * 32);
    };
    uint32_t n_barred = 0;
    if (masked) {
        uint32_t mine = 0;
        for (uint32_t i = w_lo + tid; i < w_hi; i += NT) {
            mine += (uint32_t)__popc(barred(i));
        }
        for (int o = 32; o > 0; o >>= 1) {
            mine += __shfl_xor(mine, o);
        }
        if (lane == 0) {
            sh.red_i[w] = mine;
        }
        __syncthreads();
        for (int i = 0; i < NWAVE; ++i) {
            n_barred += sh.red_i[i];
        }
        __syncthreads();
        if ((uint64_t)n_barred + n_tail + n_bias > SPEC_CAP - SPEC_CAP / 10u) {
            return false;  // not a failure: the mask is not dense enough for this select
        }
    }
    // `bucketed`: some listed ids reach the scan through the LDS buckets; `listed_row`: the row
    // has listed ids at all (the sorted part included).
    const bool bucketed = n_tail != 0 || n_bias != 0 || n_barred != 0;
    const bool listed_row = bucketed || n_sorted != 0;
    // Block of a streamed id of this slice, NONE for ids outside it or in a partial chunk.
    auto block_of = [&](uint32_t id) -> uint32_t {
        if (id >= g.vocab) {
            return NONE;
        }
        const uint32_t c = (id + g.pad) / E;
        if (c < g.main_lo || c >= g.main_hi) {
            return NONE;
        }
        return (c - g.cb) / BLOCK;
    };
    // The bias entry i opens a bucket slot when it is the first of its id and the id is
    // not on the scratch's list (that entry covers it).
    auto bias_block = [&](uint32_t i) -> uint32_t {
        const uint32_t id = L.bias_id[i];
        for (uint32_t j = 0; j < i; ++j) {
            if (L.bias_id[j] == id) {
                return NONE;
            }
        }
        const uint32_t b = block_of(id);
        if (b != NONE && pen && bit_of(a.touched, id)) {
            return NONE;
        }
        return b;
    };
    // The disallowed ids that open a bucket slot of their own: streamed ones that neither
    // the scratch's list nor the bias list covers already.
    auto each_barred = [&](auto&& fn) {
        if (n_barred == 0u) {
            return;
        }
        for (uint32_t i = w_lo + tid; i < w_hi; i += NT) {
            uint32_t bits = barred(i);
            while (bits != 0u) {
                const uint32_t id = i * 32u + (uint32_t)__builtin_ctz(bits);
                bits &= bits - 1u;
                const uint32_t b = block_of(id);
                bool open = b != NONE && !(pen && bit_of(a.touched, id));
                for (uint32_t j = 0; open && j < n_bias; ++j) {
                    open = L.bias_id[j] != id;
                }
                if (open) {
                    fn(id, b);
                }
            }
        }
    };
    if (bucketed && nblocks == 1u) {
        // One block: its bucket starts at slot 0, so a single atomic places each entry and
        // there is nothing to count first.
        auto put = [&](uint32_t entry) {
            const uint32_t at = atomicAdd(&L.bfill[0], 1u);
            if (at < SPEC_CAP) {
                L.spec[at] = entry;
            }
        };
#pragma unroll
        for (int q = 0; q < PREG; ++q) {
            const uint32_t p = (uint32_t)q * NT + tid;
            if (p < n_tail && p < loaded && block_of(early[q] & ID_MASK) != NONE) {
                put(early[q]);
            }
        }
        for (uint32_t p = loaded + tid; p < n_tail; p += NT) {
            const uint32_t e = gload(list + (a.pairs_cap - 1u - p));
            if (block_of(e & ID_MASK) != NONE) {
                put(e);
            }
        }
        for (uint32_t i = tid; i < n_bias; i += NT) {
            if (bias_block(i) != NONE) {
                put(L.bias_id[i]);
            }
        }
        each_barred([&](uint32_t id, uint32_t) { put(id); });
        __syncthreads();
        const uint32_t total = L.bfill[0];
        if (total > SPEC_CAP) {
            return stream_fail(cfg, 3u);
        }
        // Every wave writes the bucket's end for its own later reads (the same value).
        if (lane == 0) {
            L.bkt[1] = total;
            L.bkt[MAX_BUCKETS] = total;
            if (total + (L.hseg[0].y - L.hseg[0].x) > (uint32_t)NT) {
                sh.dense_listed = 1u;
            }
        }
    } else if (bucketed) {
        uint32_t packed[PREG];  // id | min(count, 4095) << 20, NONE when not of this slice
#pragma unroll
        for (int q = 0; q < PREG; ++q) {
            const uint32_t p = (uint32_t)q * NT + tid;
            packed[q] = NONE;
            if (p < n_tail && p < loaded && block_of(early[q] & ID_MASK) != NONE) {
                packed[q] = early[q];
            }
        }
        // Entries held in registers take their place inside the bucket with the first pass's
        // atomic (counted in bfill); everything else is counted in bkt and placed behind them
        // by a second atomic in the second pass.
        uint32_t place[PREG];
        for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
            for (int q = 0; q < PREG; ++q) {
                if (packed[q] != NONE) {
                    const uint32_t b = block_of(packed[q] & ID_MASK);
                    if (pass == 0) {
                        place[q] = atomicAdd(&L.bfill[b], 1u);
                    } else {
                        L.spec[L.bkt[b] + place[q]] = packed[q];
                    }
                }
            }
            for (uint32_t p = loaded + tid; p < n_tail; p += NT) {  // what the registers do not hold
                const uint32_t e = gload(list + (a.pairs_cap - 1u - p));
                const uint32_t b = block_of(e & ID_MASK);
                if (b != NONE) {
                    if (pass == 0) {
                        atomicAdd(&L.bkt[b], 1u);
                    } else {
                        L.spec[L.bkt[b] + atomicAdd(&L.bfill[b], 1u)] = e;
                    }
                }
            }
            for (uint32_t i = tid; i < n_bias; i += NT) {
                const uint32_t b = bias_block(i);
                if (b != NONE) {
                    if (pass == 0) {
                        atomicAdd(&L.bkt[b], 1u);
                    } else {
                        L.spec[L.bkt[b] + atomicAdd(&L.bfill[b], 1u)] = L.bias_id[i];
                    }
                }
            }
            each_barred([&](uint32_t id, uint32_t b) {
                if (pass == 0) {
                    atomicAdd(&L.bkt[b], 1u);
                } else {
                    L.spec[L.bkt[b] + atomicAdd(&L.bfill[b], 1u)] = id;
                }
            });
            __syncthreads();
            if (pass == 0) {
                phase(cfg, 14);
                if (tid < 64) {  // counts -> exclusive offsets, total in bkt[MAX_BUCKETS]
                    const uint32_t cnt = L.bkt[tid] + L.bfill[tid];
                    const uint64_t big =
                        __ballot(cnt + (L.hseg[tid].y - L.hseg[tid].x) > (uint32_t)NT);
                    if (tid == 0 && big != 0ull) {
                        sh.dense_listed = 1u;
                    }
                    uint32_t incl = cnt;
                    for (int o = 1; o < 64; o <<= 1) {
                        const uint32_t t = __shfl_up(incl, o);
                        if ((int)tid >= o) {
                            incl += t;
                        }
                    }
                    L.bkt[tid] = incl - cnt;
                    if (tid == 63) {
                        L.bkt[MAX_BUCKETS] = incl;
                    }
                }
                __syncthreads();
                phase(cfg, 15);
                if (L.bkt[MAX_BUCKETS] > SPEC_CAP) {
                    return stream_fail(cfg, 3u);
                }
            }
        }
    }
    phase(cfg, 1);

    // ---- scan
    const uint32_t keff = min(k + k / 8u + 2u, 64u * NWAVE);
    const uint32_t kw = (keff + NWAVE - 1) / NWAVE;
    float lane_max = NEG_INF;
    float T = F32_LOWEST;       // the block's bound, the same in every thread
    float ref_s = 0.0f;         // reference of the double sums
    float row_max = NEG_INF;    // lower bound of the row's largest true value, as of the last refresh
    float listed_raw_max = NEG_INF, listed_true_max = NEG_INF;  // this thread's listed ids so far
    float skip_b = NEG_INF;     // the block's cut: chunks whose maximum is not above it are not summed
    uint32_t wq = 0;            // this wave's queue fill
    WaveLse wl;
    wl.init();
    double acc_t = 0.0, acc_r = 0.0, acc_q = 0.0;
    constexpr int UP_UNSET = INT_MIN;
    int up = UP_UNSET;          // this thread's double sums are relative to ref_s + up
    uint32_t parity = 0;
    // One term 2^(v*c2 - ref_s - up) of a double sum.  The exponent is formed in double: a
    // row's largest value may lie hundreds of units above the reference (fixed after the
    // first block), where an f32 difference is good to 1e-5 only.  The thread's own
    // reference ref_s + up starts at its first term and moves up (its three sums scaled down
    // by the same power of two) when a term lies beyond 2^900 of it, so what a thread drops
    // as too small is small against something it holds - the row's raw maximum, which ref_s
    // comes from, may belong to an id that a mask or a bias takes out.  The threads'
    // references are brought together at the end.
    double base = -1.0e300;     // ref_s + up; far below anything while up is unset
    const double c2d = (double)c2;
    auto term_d = [&](float v) -> double {
        double d = __builtin_fma((double)v, c2d, -base);
        if (d > 900.0) {
            // The thread's first term, or one beyond 2^900 of its reference: the reference
            // moves to the term (the three sums, if any, scaled down by the same power of two).
            double e = (double)v * c2d - (double)ref_s;
            e = e < 1.0e9 ? (e > -1.0e9 ? e : -1.0e9) : 1.0e9;
            const int now = (int)__builtin_floor(e);
            if (up != UP_UNSET) {
                const int step = now - up;
                acc_t = __builtin_ldexp(acc_t, -step);
                acc_r = __builtin_ldexp(acc_r, -step);
                acc_q = __builtin_ldexp(acc_q, -step);
            }
            up = now;
            base = (double)ref_s + (double)up;
            d = e - (double)up;
        }
        if (!(d > -1000.0)) {
            return 0.0;  // -inf, NaN, or nothing against what the thread already holds
        }
        return pow2_d(d);
    };

    // Brings T up to date with everything the lanes have seen, the current block included.
    auto refresh_bound = [&](bool first, bool maxima) {
        const uint32_t key16 = lane_max > NEG_INF ? (lilym_order_key(lane_max) >> 16) : 0u;
        const uint32_t P = wave_kth_key16(key16, kw);
        const float mine = P != 0u ? lilym_key_value(P << 16) : F32_LOWEST;
        float wm[3] = {0.0f, 0.0f, 0.0f};
        if (maxima) {
            wm[0] = wave_max_dpp(lane_max);
            if (want_lse && listed_row) {
                wm[1] = wave_max_dpp(listed_raw_max);
                wm[2] = wave_max_dpp(listed_true_max);
            }
        }
        if (lane == 0) {
            sh.bound[parity][w] = mine;
            if (maxima) {
                for (int q = 0; q < 3; ++q) {
                    sh.wmax[parity][q][w] = wm[q];
                }
            }
        }
        __syncthreads();
        float t = sh.bound[parity][0];
        for (int i = 1; i < NWAVE; ++i) {
            t = fminf(t, sh.bound[parity][i]);
        }
        T = fmaxf(T, lower_by_slack(t));
        if (maxima) {
            float m[3];
            for (int q = 0; q < 3; ++q) {
                m[q] = sh.wmax[parity][q][0];
                for (int i = 1; i < NWAVE; ++i) {
                    m[q] = fmaxf(m[q], sh.wmax[parity][q][i]);
                }
            }
            // A lower bound of the row's largest TRUE value: the largest raw value when it
            // exceeds every listed id's raw value (then it belongs to an id that keeps its
            // value), and the largest true value of the listed ids in any case.  All three
            // maxima cover the same blocks.  A block with more listed ids than threads breaks
            // that (its later rounds lag), so such rows skip nothing.
            if (!listed_row) {
                row_max = m[0];
            } else if (sh.dense_listed != 0u) {
                row_max = NEG_INF;
            } else {
                row_max = m[0] > m[1] ? fmaxf(m[0], m[2]) : m[2];
            }
            if (first) {
                // Finite and far from overflow: every term is formed as 2^(v*c2 - ref_s).
                ref_s = m[0] > NEG_INF ? fminf(fmaxf(m[0] * c2, -1.0e30f), 1.0e30f) : 0.0f;
            }
        }
        parity ^= 1u;
    };

    struct Listed {
        uint32_t ent;
        u32x4 chunk;
    };
    // A thread's place among block b's listed ids in round `round` (rotated from block to
    // block so that the same threads do not serve every block's first entries).
    auto slot_of = [&](uint32_t b, uint32_t round) -> uint32_t {
        return round * NT + ((tid + NT - ((b * 64u) % NT)) % NT);
    };
    // Block b's entries are those of the sorted part between its two bucket starts (ids of
    // the neighbouring blocks at either end are dropped when the entry is used), then those
    // of its LDS bucket.  The load is unconditional as well: a thread without an entry reads
    // some entry of the list (rows without a list read the row's first bytes).
    const ListEntry* ent_base = pen ? list : reinterpret_cast<const ListEntry*>(g.base);
    const uint32_t ent_last = pen ? a.pairs_cap - 1u : 0u;
    auto entry_load = [&](uint32_t b, uint32_t round) -> uint32_t {
        return gload(ent_base + min(L.hseg[b].x + slot_of(b, round), ent_last));
    };
    // `pre`: what entry_load(b, round) returned.  Issues the gather of the entry's chunk; a
    // thread without an entry reads the slice's last chunk.
    auto listed_fetch = [&](Listed& r, uint32_t pre, uint32_t b, uint32_t round) {
        const uint2 seg = L.hseg[b];
        const uint32_t nh = seg.y - seg.x;
        const uint32_t lo = L.bkt[b], nl = L.bkt[b + 1] - lo;
        const uint32_t j = slot_of(b, round);
        uint32_t ent = NONE;
        if (j < nh) {
            if (block_of(pre & ID_MASK) == b) {
                ent = pre;
            }
        } else if (j - nh < nl) {
            ent = L.spec[min(lo + (j - nh), SPEC_CAP - 1u)];
        }
        r.ent = ent;
        const uint32_t c = min(((ent & ID_MASK) + g.pad) / E, c_last);
        r.chunk = gload(reinterpret_cast<const u32x4*>(g.base + (c << 4)));
    };
    // The id's own logit out of its chunk (one gather per listed id, not two).
    // Element j of a chunk: one compare picks the 8-byte half, one 64-bit shift the element.
    auto elem_of = [&](const u32x4& q, uint32_t j) -> float {
        const bool upper = (j & (uint32_t)(E / 2)) != 0u;
        const uint64_t half = upper ? (((uint64_t)q.w << 32) | q.z) : (((uint64_t)q.y << 32) | q.x);
        if (E == 8) {
            return lilym_bits_f32((uint32_t)(half >> ((j & 3u) * 16u)) << 16);
        }
        return lilym_bits_f32((uint32_t)(half >> ((j & 1u) * 32u)));
    };
    auto raw_of = [&](const u32x4& q, uint32_t id) -> float {
        return elem_of(q, (id + g.pad) % E);
    };
    // Penalties with a repetition factor of at least 1 and non-negative presence and frequency
    // terms can only lower a value, and a barred id's value is -inf: without a bias list a
    // listed id's true value never exceeds its raw one.
    const bool lowering = n_bias == 0u && a.repetition >= 1.0f && a.presence >= 0.0f &&
                          a.frequency >= 0.0f;
    // A listed id's raw value, into the thread's maximum of listed raw values (which must
    // cover every listed id: see row_max).
    auto listed_raw = [&](const Listed& r) {
        if (r.ent != NONE) {
            listed_raw_max = fmaxf(listed_raw_max, raw_of(r.chunk, r.ent & ID_MASK));
        }
    };
    // A listed id's true value before the temperature (bias in list order, then penalties);
    // also feeds the thread's maximum of listed true values (a lower bound of the row's largest
    // true value whichever ids it covers).
    auto listed_true = [&](const Listed& r, float raw) -> float {
        const uint32_t id = r.ent & ID_MASK;
        uint32_t cnt = r.ent >> SPEC_ID_BITS;
        if (cnt == 4095u) {
            cnt = gload(a.counts + id);
            // The value is waited for here, inside the branch: waiting after it would make
            // every thread drain the loads it has in flight.
            asm volatile("" : "+v"(cnt));
        }
        float t = raw;
        for (uint32_t j = 0; j < n_bias; ++j) {
            if (L.bias_id[j] == id) {
                t += L.bias_delta[j];
            }
        }
        if (cnt > 0u) {
            t = t > 0.0f ? t / a.repetition : t * a.repetition;
            t -= a.presence + a.frequency * (float)cnt;
        }
        if (masked && !bit_of(a.allow, id)) {
            t = NEG_INF;
        }
        listed_true_max = fmaxf(listed_true_max, t);
        return t;
    };
    // After the block's bound is known: was the id's chunk queued or summed by its owner (the
    // owner's tests on the same bits), the id's terms, and the id as a candidate.  When values
    // can only be lowered, an id whose chunk was neither queued nor summed is below the bound
    // and below the sum's cut with its true value too: nothing of it is evaluated (most blocks
    // of most rows hold no other kind, and their waves skip all of this).
    auto listed_finish = [&](const Listed& r, bool nonneg) {
        const bool has = r.ent != NONE;
        const float cm = nonneg ? chunk_max_nonneg<DT>(r.chunk) : chunk_max<DT>(r.chunk);
        const bool queued = cm >= T;
        const bool summed = !queued && cm > skip_b;  // the cut is -inf without a row sum
        if (!has || (lowering && !queued && !(want_lse && summed))) {
            return;
        }
        const uint32_t id = r.ent & ID_MASK;
        const float raw = raw_of(r.chunk, id);
        const float t = listed_true(r, raw);
        if (want_lse) {
            if (t > skip_b) {  // the same cut as for streamed terms
                acc_t += term_d(t);
            }
            if (summed) {
                acc_r += term_d(raw);
            }
        }
        if (queued) {
            const uint32_t at = atomicAdd(&sh.n_drop, 1u);
            if (at < DROP_CAP) {
                L.drop[at] = id;
            }
        }
        if (t >= T && t > NEG_INF) {
            const uint32_t at = atomicAdd(&sh.n_fc, 1u);
            if (at < FC_CAP) {
                L.fc[at] = composite_of(t / a.temperature, id);
            }
        }
    };

    // Blocks b + 1 and b + 2 are on their way while block b is worked on (three register
    // buffers that swap roles): one block in flight per wave leaves the memory idle whenever
    // a wave's arithmetic outlasts its load.
    const float lse_cut = (log2f((float)g.vocab) + 21.0f) * (a.temperature * 0.6931471805599453f);
    // Memory operations of a wave complete in the order they were issued: a block's listed
    // gathers are requested BEFORE the next stream block, so using them never waits for it.
    Listed lst_a, lst_b, lst_c;
    lst_a.ent = NONE;
    lst_b.ent = NONE;
    lst_c.ent = NONE;
    // The waves of a compute unit's oldest workgroup win the issue slots and its youngest
    // finishes last, alone.  Rows that carry both listed ids and a row sum (the most
    // instructions per block) lower their waves' priority as they advance, so a workgroup
    // that fell behind catches up; lighter rows lose by it and leave the priority alone.
    const bool paced = listed_row && want_lse;
    auto work = [&](u32x4 (&cur)[U], Listed& lcur, uint32_t b) {
        if (paced) {
            const uint32_t q = b * 4u / nblocks;
            if (q == 0u) {
                __builtin_amdgcn_s_setprio(3);
            } else if (q == 1u) {
                __builtin_amdgcn_s_setprio(2);
            } else if (q == 2u) {
                __builtin_amdgcn_s_setprio(1);
            } else {
                __builtin_amdgcn_s_setprio(0);
            }
        }
        if (!full_block(b)) {
            const uint32_t ninf = DT == LILY_BF16 ? 0xff80ff80u : 0xff800000u;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t c = g.cb + (b * U + u) * NT + tid;
                if (c < g.main_lo || c >= g.main_hi) {
                    cur[u] = u32x4{ninf, ninf, ninf, ninf};
                }
            }
        }
        if (listed_row) {
            listed_raw(lcur);
        }
        // The block's own maxima enter the bound before the block is filtered.  Chunks below
        // the previous bound cannot be queued: their terms are summed right away.
        const float T_prev = T;
        // Once the bound is positive only chunks with a positive element can matter to it:
        // their maximum comes from the cheaper form, which reports +0 for all others (the sum
        // then takes such a chunk unless the cut is positive too, and the lanes' maxima are
        // only overstated up to 0, below the bound they could move).
        const bool nonneg = DT == LILY_BF16 && __builtin_amdgcn_readfirstlane((int)(T_prev > 0.0f)) != 0;
        float m8[U];
        float block_max = NEG_INF;
        if (nonneg) {
            // No value here is below +0: their bit patterns order like integers, and such a
            // pattern exceeds that of any negative value the lane's maximum may still hold.
            int bm = 0;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                m8[u] = chunk_max_nonneg<DT>(cur[u]);
                bm = max(bm, (int)lilym_f32_bits(m8[u]));
            }
            block_max = lilym_bits_f32((uint32_t)bm);
            lane_max = lilym_bits_f32((uint32_t)max((int)lilym_f32_bits(lane_max), bm));
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                m8[u] = chunk_max<DT>(cur[u]);
                block_max = max2_raw(block_max, m8[u]);
            }
            lane_max = max2_raw(lane_max, block_max);
        }
        if (LSE && want_lse) {
            // A term 2^(v*c2) below 2^-21 / vocab of the largest one seen cannot move the row
            // sum by more than 2^-21 of it, even with every element of the row at that level:
            // such chunks are left out, by a rule every thread of the block can evaluate.
            skip_b = row_max - lse_cut;
            wl.skip_below = skip_b;
            // Rows with a dominant value skip nearly every block as a whole.
            if (__ballot(block_max > skip_b) != 0ull) {
                wl.prepare(block_max < T_prev ? block_max : T_prev, c2);  // nothing above T_prev is added
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    wl.template add_prepared<DT>(cur[u], m8[u], c2, !(m8[u] >= T_prev));
                }
            }
        }
        // The bound moves most in the first blocks: refresh it for each of them, then for
        // every fourth block (each refresh is a ballot search and a barrier).  The row's
        // maxima behind the sum's cut follow with every other of those.
        if (b < 4u || (b & 3u) == 0u) {
            refresh_bound(b == 0, b == 0 || (LSE && want_lse && (b < 4u || (b & 7u) == 0u)));
        }
        const bool any_late = LSE && want_lse && T != T_prev &&
                              __ballot(block_max >= T_prev && block_max > skip_b) != 0ull;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t c = g.cb + (b * U + u) * NT + tid;
            const bool pass = m8[u] >= T;
            const uint64_t mask = __ballot(pass);
            if (mask != 0ull) {
                const uint32_t rank = __builtin_amdgcn_mbcnt_hi(
                    (uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
                const uint32_t at = wq + rank;
                if (pass && at < QSEG) {
                    L.qraw[w * QSEG + at] = cur[u];
                    L.qidx[w * QSEG + at] = c;
                }
                wq += (uint32_t)__popcll(mask);
            }
            if (any_late) {
                // At or above the previous bound but below the new one: not queued after all.
                const bool late = m8[u] >= T_prev && !pass;
                if (__ballot(late) != 0ull) {
                    wl.prepare(late ? m8[u] : NEG_INF, c2);
                    wl.template add_prepared<DT>(cur[u], m8[u], c2, late);
                }
            }
        }
        if (listed_row) {
            listed_finish(lcur, nonneg);
            const uint32_t n_b = (L.hseg[b].y - L.hseg[b].x) + (L.bkt[b + 1] - L.bkt[b]);
            for (uint32_t round = 1; round * NT < n_b; ++round) {
                // Rare (a block with more listed ids than threads).  Both loads are waited for
                // right here, inside the loop: left to the first use, their waits would be
                // placed where every path meets and drain the blocks requested ahead.
                Listed extra;
                uint32_t e = entry_load(b, round);
                asm volatile("" : "+v"(e));
                listed_fetch(extra, e, b, round);
                asm volatile("" : "+v"(extra.chunk.x), "+v"(extra.chunk.y), "+v"(extra.chunk.z),
                             "+v"(extra.chunk.w));
                listed_raw(extra);
                listed_finish(extra, nonneg);
            }
        }
    };
    // A request past the last block asks for the last block again (its lines are in the
    // cache and nothing uses the result): with the same loads in flight on every path the
    // wait for a block's data leaves the blocks requested after it in flight, where a request
    // that may be skipped makes that wait count as if it had been.
    // A block's entry of the sorted part is requested two requests ahead of its gather, which
    // therefore never waits for anything younger than the block the next `work` needs anyway:
    // `pre` is this block's entry, `ahead` receives the one of the block after next.
    auto request = [&](u32x4 (&dst)[U], Listed& ldst, uint32_t pre, uint32_t& ahead, uint32_t b) {
        const uint32_t bb = min(b, nblocks - 1u);
        if (listed_row) {
            listed_fetch(ldst, pre, bb, 0);
            ahead = entry_load(min(b + 2u, nblocks - 1u), 0);
        }
        fetch(dst, bb);
    };
    if (nblocks == 0) {
        refresh_bound(true, true);  // the same barriers in every workgroup
    } else {
        uint32_t pre_a = 0, pre_b = 0, pre_c = 0;
        if (listed_row) {
            pre_a = entry_load(0, 0);
            pre_b = entry_load(min(1u, nblocks - 1u), 0);
            pre_c = entry_load(min(2u, nblocks - 1u), 0);
            listed_fetch(lst_a, pre_a, 0, 0);
        }
        request(buf_b, lst_b, pre_b, pre_a, 1);
        for (uint32_t b = 0; b < nblocks; b += 3) {
            request(buf_c, lst_c, pre_c, pre_b, b + 2);
            work(buf_a, lst_a, b);
            if (b + 1 < nblocks) {
                request(buf_a, lst_a, pre_a, pre_c, b + 3);
                work(buf_b, lst_b, b + 1);
                if (b + 2 < nblocks) {
                    request(buf_b, lst_b, pre_b, pre_a, b + 4);
                    work(buf_c, lst_c, b + 2);
                }
            }
        }
    }
    if (paced) {
        __builtin_amdgcn_s_setprio(0);  // a row of fewer than four blocks never reached it
    }
    phase(cfg, 2);

    // ---- after the scan
    if (lane == 0) {
        sh.qfill[w] = wq;
    }
    __syncthreads();
    const float filt = T;
    {
        bool overflow = sh.n_drop > DROP_CAP;
        for (int i = 0; i < NWAVE; ++i) {
            overflow = overflow || sh.qfill[i] > QSEG;
        }
        if (overflow) {
            return stream_fail(cfg, 4u);
        }
    }
    // Listed ids inside queued chunks: mark their element in the chunk's queue slot.  A
    // wave's segment is in ascending chunk order, so the slot is found by bisection.
    for (uint32_t d = tid; d < sh.n_drop; d += NT) {
        const uint32_t id = L.drop[d];
        const uint32_t c = (id + g.pad) / E, j = (id + g.pad) % E;
        const uint32_t ow = ((c - g.cb) % NT) / 64u;
        uint32_t lo = ow * QSEG, hi = lo + sh.qfill[ow];
        while (lo < hi) {
            const uint32_t mid = (lo + hi) >> 1;
            if (L.qidx[mid] < c) {
                lo = mid + 1;
            } else {
                hi = mid;
            }
        }
        atomicOr(&L.dmask[lo >> 2], (1u << j) << ((lo & 3u) * 8u));
    }
    __syncthreads();
    auto offer = [&](float u, uint32_t id) {
        if (u >= filt && u > NEG_INF) {
            const uint32_t at = atomicAdd(&sh.n_fc, 1u);
            if (at < FC_CAP) {
                L.fc[at] = composite_of(u / a.temperature, id);
            }
        }
    };
    {
        // One thread per queued chunk (the waves' segments counted through in order): its
        // elements that are not listed ids add their term and are offered.
        uint32_t seg_end[NWAVE], total = 0;
#pragma unroll
        for (int i = 0; i < NWAVE; ++i) {
            total += sh.qfill[i];
            seg_end[i] = total;
        }
        for (uint32_t ch = tid; ch < total; ch += NT) {
            uint32_t ww = 0, before = 0;
#pragma unroll
            for (int i = 0; i + 1 < NWAVE; ++i) {
                if (ch >= seg_end[i]) {
                    ww = (uint32_t)i + 1u;
                    before = seg_end[i];
                }
            }
            const uint32_t slot = ww * QSEG + (ch - before);
            const u32x4 q = L.qraw[slot];
            const uint32_t c = L.qidx[slot];
            const uint32_t dm = (L.dmask[slot >> 2] >> ((slot & 3u) * 8u)) & 0xffu;
            float v[E];
            unpack<DT>(q, v);
            // Few elements of a queued chunk matter (usually the one that got it queued):
            // they are marked first and then taken one at a time, in ascending order, instead
            // of eight branches that some lane of the wave enters every time.
            uint32_t todo = 0;
#pragma unroll
            for (int j = 0; j < E; ++j) {
                const bool term = want_lse && v[j] > skip_b;  // the cut of the streamed terms
                const bool cand = v[j] >= filt && v[j] > NEG_INF;
                todo |= (term || cand) ? 1u << j : 0u;
            }
            todo &= ~dm;
            while (todo != 0u) {
                const uint32_t j = (uint32_t)__builtin_ctz(todo);
                todo &= todo - 1u;
                const float x = elem_of(q, j);
                if (want_lse && x > skip_b) {
                    acc_q += term_d(x);
                }
                offer(x, g.id_of(c, (int)j));
            }
        }
    }
    phase(cfg, 8);
    // Ids of partial 16-byte chunks at the row's ends were not streamed: exact, one by one.
    for (int side = 0; side < 2; ++side) {
        const uint32_t lo = side == 0 ? g.id_lo : g.edge_hi_begin;
        const uint32_t hi = side == 0 ? g.edge_lo_end : g.id_hi;
        for (uint32_t id = lo + tid; id < hi; id += NT) {
            const float u = pre_temperature_of<DT>(a, id);
            if (want_lse) {
                acc_q += term_d(u);
            }
            offer(u, id);
        }
    }
    phase(cfg, 9);
    if (want_lse) {
        // Each wave brings its sums to one reference of its own: the highest of its threads'
        // references and of the streamed sums' (wave-uniform) reference.  The waves' partial
        // sums and references meet in LDS and are brought together after one barrier.
        int ref_w = up;
        for (int o = 32; o > 0; o >>= 1) {
            ref_w = max(ref_w, __shfl_xor(ref_w, o));
        }
        const double stream_at = (double)wl.ref - (double)ref_s;  // exact
        if (__ballot(wl.s > 0.0f) != 0ull) {
            const double e = stream_at < 1.0e9 ? (stream_at > -1.0e9 ? stream_at : -1.0e9) : 1.0e9;
            ref_w = max(ref_w, (int)__builtin_floor(e));
        }
        const int down = up == UP_UNSET ? 0 : up - ref_w;  // <= 0
        double part[3];
        {
            double d = stream_at - (double)ref_w;  // <= 1 where there is a sum
            d = d < -1000.0 ? -1000.0 : d;
            part[0] = wl.s > 0.0f ? (double)wl.s * pow2_d(d) : 0.0;
        }
        part[1] = __builtin_ldexp(acc_r, down);
        part[2] = __builtin_ldexp(acc_t + acc_q, down);
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            part[i] = wave_sum_d(part[i]);
            if (lane == 0) {
                sh.red3[i][w] = part[i];
            }
        }
        if (lane == 0) {
            sh.red_i[w] = (uint32_t)ref_w;
        }
        __syncthreads();
        int ref_all = (int)sh.red_i[0];
        for (int i = 1; i < NWAVE; ++i) {
            ref_all = max(ref_all, (int)sh.red_i[i]);
        }
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            part[i] = 0.0;
            for (int ww = 0; ww < NWAVE; ++ww) {
                const int at = (int)sh.red_i[ww];
                part[i] += at == UP_UNSET ? 0.0 : __builtin_ldexp(sh.red3[i][ww], at - ref_all);
            }
        }
        if (ref_all == UP_UNSET) {
            ref_all = 0;  // no term anywhere: the sums are zero
        }
        const double streamed = part[0], booked = part[1], exact = part[2];
        const double rest = streamed - booked;
        // Listed ids held nearly all of what was streamed: the difference is too coarse.
        const bool coarse = booked > 0.0 && !(rest > 0.05 * streamed);
        phase(cfg, 10);
        if (coarse) {
            phase(cfg, 11);
            LseAcc all;
            all.init();
            exact_terms<DT>(a, g.id_lo, g.id_hi, c2, all);
            double m_e, s_e;
            wg_merge_lse(sh, all.mc, all.s, m_e, s_e);
            if (tid == 0) {
                sh.lse_mc = m_e;
                sh.lse_s = s_e;
            }
        } else if (tid == 0) {
            sh.lse_mc = (double)ref_s + (double)ref_all;
            sh.lse_s = (rest > 0.0 ? rest : 0.0) + exact;
        }
    }
    __syncthreads();
    uint32_t n = sh.n_fc;
    phase(cfg, 3);
    if (n > FC_CAP) {
        return stream_fail(cfg, 5u);
    }
    sorted = false;
    n = select_topk(L.fc, n, k, sh, sorted);
    phase(cfg, 12);
    // Everything that is not a candidate lies strictly below `filt`: the result is exact if
    // k candidates were found and the k-th lies strictly above anything the division can
    // map such a value to.
    if (filt > F32_LOWEST) {
        uint32_t lowest = 0xffffffffu;
        if (sorted) {
            // Ranked candidates are in descending order: the last one is the lowest.
            lowest = n > 0u ? (uint32_t)(L.fc[n - 1u] >> 32) : lowest;
        } else {
            for (uint32_t i = tid; i < n; i += NT) {
                lowest = min(lowest, (uint32_t)(L.fc[i] >> 32));
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
        }
        const float below = lilym_key_value(lilym_order_key(filt) - 1u) / a.temperature;
        if (!(n >= k && lilym_order_key(below) < lowest)) {
            return stream_fail(cfg, 6u);
        }
    }
    // The candidates stay where they are (the tail's arrays and the merge's buffer lie below
    // them in dynamic LDS).
    out = L.fc;
    if (tid == 0) {
        sh.n_cand = n;
    }
    __syncthreads();
    return true;
}


}  // namespace lily
