// rows_wide.hip - rows that draw among many candidates (k > 64, up to the reference's cap of 1024,
// which is what a request without top_k gets: src/kernels/sample.rs:17, :326-331), spread over
// as many workgroups as rows of few candidates are.
//
// Two launches.  In the first every workgroup reads its slice of the row once and leaves its
// lanes' largest values (penalised ids at their penalised worth).  In the second every
// workgroup first takes the k-th largest of all the row's lane maxima: k lanes reach it, so k
// values do - a lower bound of the row's k-th largest value that about k * (1 + a few per cent)
// values reach -, then reads its slice again (from the L2 now) and appends the values that
// reach the bound to the row's list; the one that finishes last reads the list - a thousand and
// some, whatever the number of slices -, selects, and runs the common tail.  (The select of the
// other kernels keeps k candidates per slice and can therefore spread a row with k = 1024 over
// 4 workgroups only.)
#include <algorithm>

#ifdef LILY_WIDE_TRACE
#define LILY_TAIL_TRACE
#endif

#include "row_kernel.h"

namespace lily {

// Diagnostic stamps (LaunchCfg::phase_trace), compiled in with -DLILY_WIDE_TRACE (which also
// turns on the tail's: slots 8 to 12).  First launch: 0 start, 1 slice read, 2 maxima stored;
// second: 5 start, 6 slice read, 7 last slice in, 13 list read, 14 selected.
#ifdef LILY_WIDE_TRACE
#define WIDE_MARK(i) phase(cfg, i)
#else
#define WIDE_MARK(i)
#endif

// What the two launches share beyond LaunchCfg.
struct WideArgs {
    Handed<float> lane_max;   // [rows][slices][lanes]
    Handed<float> slice_bound;   // [rows][slices] a value that k / slices of the slice's lanes reach
    uint32_t lanes;       // values a slice leaves: NT, or NT / 2 (the larger of each pair of lanes)
    uint32_t* count;      // [rows] candidates the row's slices have left so far (0 between launches)
};

template <bool INLINE>
__device__ __forceinline__ const LILY_CONST RowArgs* wide_table(const LaunchCfg& cfg) {
    if (INLINE) {
        // the rows are the kernel's first argument: index the kernel-argument segment itself
        return (const LILY_CONST RowArgs*)__builtin_amdgcn_kernarg_segment_ptr();
    }
    return (const LILY_CONST RowArgs*)cfg.table;
}

// One pass over the slice's chunks, four loads in flight per thread, every load unconditional
// (a chunk number past the slice is replaced by the slice's last; `use` says whether it counts).
template <int DT, class F>
__device__ __forceinline__ void wide_scan(const Geo<DT>& g, F&& per_chunk) {
    const uint32_t tid = threadIdx.x;
    if (g.main_hi <= g.main_lo) {
        return;
    }
    for (uint32_t c0 = g.main_lo; c0 < g.main_hi; c0 += 4u * NT) {
        u32x4 q[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t c = min(c0 + (uint32_t)u * NT + tid, g.main_hi - 1u);
            q[u] = gload(reinterpret_cast<const u32x4*>(g.base + (size_t)c * 16));
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t c = c0 + (uint32_t)u * NT + tid;
            if (c < g.main_hi) {
                per_chunk(q[u], c);
            }
        }
    }
}

// What a raw value is worth under the row's penalties (the arithmetic of finish_pre_temperature).
__device__ __forceinline__ float wide_worth(const RowArgs& a, float x, uint32_t id) {
    if (bit_of(a.touched, id)) {
        uint32_t cnt = gload(a.counts + id);
        asm volatile("" : "+v"(cnt));   // waited for here, inside the branch
        if (cnt > 0u) {
            x = x > 0.0f ? x / a.repetition : x * a.repetition;
            x -= a.presence + a.frequency * (float)cnt;
        }
    }
    return x;
}

// Bits id0 .. id0 + E - 1 of the bitmap of penalised ids (all below the vocabulary; the word
// behind the bitmap's last is the row's largest count, so the second load stays in bounds).
template <int E>
__device__ __forceinline__ uint32_t wide_bits(const uint32_t* words, uint32_t id0) {
    const uint32_t w = id0 >> 5, sh = id0 & 31u;
    uint32_t b = gload(words + w) >> sh;
    if (sh + (uint32_t)E > 32u) {
        b |= gload(words + w + 1u) << (32u - sh);
    }
    return b & ((1u << E) - 1u);
}

// The ids of the partial 16-byte chunks at the slice's ends, one by one.
template <int DT, class F>
__device__ __forceinline__ void wide_edges(const RowArgs& a, const Geo<DT>& g, F&& per_id) {
    for (int side = 0; side < 2; ++side) {
        const uint32_t lo = side == 0 ? g.id_lo : g.edge_hi_begin;
        const uint32_t hi = side == 0 ? g.edge_lo_end : g.id_hi;
        for (uint32_t id = lo + threadIdx.x; id < hi; id += NT) {
            per_id(load_logit<DT>(a.logits, id), id);
        }
    }
}

// The row's ticket: true in every thread of the workgroup that arrives last (last_to_arrive()).
__device__ __forceinline__ bool wide_last(const LaunchCfg& cfg, uint32_t row, uint32_t S, Shared& sh) {
    return last_to_arrive(&cfg.ws_ticket[row], S, sh.last, cfg.relaxed_handover != 0u);
}

// ---- first launch: lane maxima, the slice's sum of exponentials

template <int DT, bool LSE, bool INLINE>
__global__ __launch_bounds__(NT, 4) void k_wide_bound(InlineRows rows_arg, LaunchCfg cfg, WideArgs w) {
    __shared__ Shared sh;
    constexpr int E = Geo<DT>::E;
    const uint32_t tid = threadIdx.x, s = blockIdx.x, row = blockIdx.y, S = cfg.slices;
    if (cfg.served != nullptr && *(const LILY_CONST uint32_t*)(cfg.served + row) != 0u) {
        return;   // drawn by an earlier launch of the same call
    }
    WIDE_MARK(0);
    RowArgs a;
    load_row_args(a, wide_table<INLINE>(cfg) + row);
    apply_selection(a);
    const bool want_lse = LSE && a.out_logprob != nullptr;
    Geo<DT> g;
    g.init(a.logits, cfg.vocab, s, S);
    const bool pen = (a.flags & F_PEN) != 0;
    float lane_max = NEG_INF;
    LseAcc lse;
    lse.init();
    wide_scan<DT>(g, [&](const u32x4& q, uint32_t c) {
        float v[E];
        unpack<DT>(q, v);
        float m;
        if (pen) {
            const uint32_t id0 = g.id_of(c, 0);
            const uint32_t bits = wide_bits<E>(a.touched, id0);
            if (bits != 0u) {
#pragma unroll
                for (int j = 0; j < E; ++j) {
                    if ((bits >> j) & 1u) {
                        v[j] = wide_worth(a, v[j], id0 + (uint32_t)j);
                    }
                }
            }
            m = NEG_INF;
#pragma unroll
            for (int j = 0; j < E; ++j) {
                m = fmaxf(m, v[j]);   // (a NaN operand loses)
            }
        } else {
            m = chunk_max<DT>(q);   // (NaN operands lose)
        }
        lane_max = fmaxf(lane_max, m);
        if (want_lse && m > NEG_INF) {
            const float safe = lse.rebase(m, a.c2);
#pragma unroll
            for (int j = 0; j < E; ++j) {
                if (v[j] > NEG_INF) {   // (false for a NaN: worth -inf)
                    lse.term(v[j], a.c2, safe);
                }
            }
        }
    });
    wide_edges<DT>(a, g, [&](float x, uint32_t id) {
        if (pen) {
            x = wide_worth(a, x, id);
        }
        if (x > NEG_INF) {
            lane_max = fmaxf(lane_max, x);
            if (want_lse) {
                lse.add_one(x, a.c2);
            }
        }
    });
    WIDE_MARK(1);
    const size_t slot = (size_t)row * S + s;
    const float pair_max = lane_max;
    if (w.lanes == NT) {
        handed_store(w.lane_max, slot * NT + tid, lane_max);
    } else {
        // (with slices enough that half the lanes still are four times k, half the keys make
        // the select of the bound half as long)
        const int other = __builtin_amdgcn_update_dpp(0, (int)lilym_f32_bits(lane_max), 0xb1, 0xf, 0xf, true);   // quad_perm [1, 0, 3, 2]
        lane_max = fmaxf(lane_max, lilym_bits_f32((uint32_t)other));
        if ((tid & 1u) == 0u) {
            handed_store(w.lane_max, slot * (NT / 2) + tid / 2u, lane_max);
        }
    }
    // ... and one value per slice that at least ceil(k / slices) of its lanes reach: in each wave
    // the ceil(k / (4 * slices))-th largest of the 64 lane maxima (a 16-step ballot search on the
    // leading 16 bits of the order key, as the streaming select takes its bound), the least of the
    // four.  The least of a row's slices' values is then reached by k lanes of the row, so by k
    // values: the second launch takes that as the row's bound without looking at the lanes'
    // maxima.  F32_LOWEST from a wave with fewer finite lane maxima than that: the second launch
    // then takes the bound from all the lanes' maxima.
    {
        const float whole = pair_max;   // (every lane's own maximum, whatever was stored above)
        const uint32_t per_wave = (a.k + 4u * S - 1u) / (4u * S);
        const uint32_t key16 = whole > NEG_INF ? (lilym_order_key(whole) >> 16) : 0u;
        const uint32_t P = per_wave <= 64u ? wave_kth_key16(key16, per_wave) : 0u;
        if ((tid & 63u) == 0u) {
            sh.bound[0][tid >> 6] = P != 0u ? lilym_key_value(P << 16) : F32_LOWEST;
        }
        __syncthreads();
        if (tid == 0) {
            float least = sh.bound[0][0];
            for (int i = 1; i < NWAVE; ++i) {
                least = fminf(least, sh.bound[0][i]);
            }
            handed_store(w.slice_bound, slot, least);
        }
    }
    if (want_lse) {
        lse_reduce(sh, lse);
        if (tid == 0) {
            handed_store(cfg.ws_lse, 2 * slot, sh.lse_mc);
            handed_store(cfg.ws_lse, 2 * slot + 1, sh.lse_s);
        }
    }
    WIDE_MARK(2);
}

// The row's bound: the k-th largest of its S x lanes lane maxima, by a radix select on the
// leading 16 bits of their order keys, 8 bits a pass: that key with the other 16 bits clear, at
// most 2^-7 of its magnitude below the k-th largest lane maximum, which lets a few per cent more
// values through.  Every workgroup of the second launch works it out for itself, from what the
// first launch left (a row's slices all arrive at the same value; a workgroup that did it for
// all of them would have to be waited for).  A thread keeps its keys in registers (the loops
// are unrolled over MAX_SLICES in groups of eight, a group past the last is skipped by the whole
// workgroup): a pass that fetched each key from LDS, or the values from the L2 a few at a time,
// would wait out that latency over and over.  F32_LOWEST when fewer than k lanes saw a finite
// value: every value is a candidate then.
__device__ __forceinline__ float wide_bound_of(const WideArgs& w, uint32_t row, uint32_t S, uint32_t k, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    static_assert(MAX_SLICES == 64, "the unrolled loops below cover 64 keys a thread");
    const uint32_t n = S * w.lanes, mine_n = (n + NT - 1u) / NT;   // keys in all, keys a thread
    float got[MAX_SLICES];
#pragma unroll
    for (int j0 = 0; j0 < (int)MAX_SLICES; j0 += 8) {
        if ((uint32_t)j0 < mine_n) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const uint32_t i = min((uint32_t)(j0 + u) * NT + tid, n - 1u);
                got[j0 + u] = handed_load(w.lane_max, (size_t)row * n + i);
            }
        }
    }
    uint32_t keys[MAX_SLICES];
#pragma unroll
    for (int j = 0; j < (int)MAX_SLICES; ++j) {
        const bool in = (uint32_t)j * NT + tid < n;   // (a group past the last was not loaded: what it holds is not read)
        keys[j] = in && got[j] > NEG_INF ? lilym_order_key(got[j]) : 0u;
    }
    uint32_t prefix = 0, pmask = 0, need = k;
    bool enough = true;
    for (int pass = 0; pass < 2 && enough; ++pass) {
        const int shift = 24 - 8 * pass;
        sh.hist[tid] = 0;
        __syncthreads();
        HistRun run;
        run.init();
#pragma unroll
        for (int j0 = 0; j0 < (int)MAX_SLICES; j0 += 8) {
            if ((uint32_t)j0 < mine_n) {
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const uint32_t key = keys[j0 + u];
                    run.add(sh.hist, (key >> shift) & 255u, key != 0u && (key & pmask) == prefix);
                }
            }
        }
        run.flush(sh.hist);
        __syncthreads();
        find_bin(sh, need);
        if (sh.all_taken != 0u) {
            enough = false;   // fewer than k lanes saw a finite value: every value is a candidate
        } else {
            prefix |= sh.sel_bin << shift;
            pmask |= 255u << shift;
            need = sh.need;
        }
        __syncthreads();
    }
    return enough ? lilym_key_value(prefix) : F32_LOWEST;
}

// ---- second launch: the values that reach the bound, then merge, select and tail

template <int DT, bool LSE, bool INLINE>
__global__ __launch_bounds__(NT, 4) void k_wide_draw(InlineRows rows_arg, LaunchCfg cfg, WideArgs w) {
    __shared__ Shared sh;
    __shared__ uint32_t n_mine;
    constexpr int E = Geo<DT>::E;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, s = blockIdx.x, row = blockIdx.y, S = cfg.slices;
    if (cfg.served != nullptr && *(const LILY_CONST uint32_t*)(cfg.served + row) != 0u) {
        return;
    }
    WIDE_MARK(5);
    if (tid == 0) {
        tail_arrays(sh);
        n_mine = 0;
    }
    RowArgs a;
    load_row_args(a, wide_table<INLINE>(cfg) + row);
    apply_selection(a);
    const uint32_t vocab = cfg.vocab;
    const uint32_t step = a.step + cfg.step_delta;
    const bool want_lse = LSE && a.out_logprob != nullptr;
    const bool pen = (a.flags & F_PEN) != 0;   // (of the kind that only lowers: the host sees to it)
    // The bound (of the values' worth under the penalties): the least of the slices' values, which
    // k lanes of the row reach; where a wave of some slice had too few finite lane maxima to name
    // one, the k-th largest of all the lanes' maxima.  Every wave reads the slices' values itself.
    float bound;
    {
        const float mine = lane < S ? handed_load(w.slice_bound, (size_t)row * S + lane) : __builtin_huge_valf();
        bound = -wave_max_dpp(-mine);
    }
    if (!(bound > F32_LOWEST)) {   // (the same in every wave)
        bound = wide_bound_of(w, row, S, a.k, sh);
    }
    Geo<DT> g;
    g.init(a.logits, vocab, s, S);
    uint64_t* cand = dyn_lds;
    const uint32_t cap = MERGE_CAP;   // what the slice's own list holds
    __syncthreads();
    auto offer = [&](float x, uint32_t id) {
        if (!(x >= bound)) {
            return;
        }
        if (pen) {
            x = wide_worth(a, x, id);   // (never more than the raw value: the host sees to it)
            if (!(x >= bound)) {
                return;
            }
        }
        const uint32_t at = atomicAdd(&n_mine, 1u);
        if (at < cap) {
            cand[at] = composite_of(x / a.temperature, id);
        }
    };
    wide_scan<DT>(g, [&](const u32x4& q, uint32_t c) {
        if (chunk_max<DT>(q) >= bound) {
            float v[E];
            unpack<DT>(q, v);
#pragma unroll
            for (int j = 0; j < E; ++j) {
                offer(v[j], g.id_of(c, j));
            }
        }
    });
    wide_edges<DT>(a, g, [&](float x, uint32_t id) { offer(x, id); });
    __syncthreads();
    WIDE_MARK(6);
    // The slice's candidates go behind those the row's other slices have left (any order: the
    // select does not care).  A row whose list would pass MERGE_CAP is counted on and not
    // written: the last workgroup sees the count and takes the exhaustive select.
    const uint32_t mine = n_mine;
    if (tid == 0) {
        n_mine = __hip_atomic_fetch_add(&w.count[row], mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    const uint32_t base = n_mine;
    if (base + mine <= MERGE_CAP) {
        for (uint32_t i = tid; i < mine; i += NT) {
            handed_store(cfg.ws_cand, (size_t)row * MERGE_CAP + base + i, cand[i]);
        }
    }
    if (!wide_last(cfg, row, S, sh)) {
        return;
    }
    WIDE_MARK(7);
    if (tid == 0) {
        sh.need = load_through(&w.count[row]);
        store_through(&w.count[row], 0u);
    }
    __syncthreads();
    const uint32_t total = sh.need;
    uint32_t n;
    bool sorted = false;
    if (total > MERGE_CAP) {
        // more than the buffers hold (values that tie by the thousand, a row in ascending
        // order): the select that is right for any input, over the whole row
        __syncthreads();
        select_exhaustive<DT>(a, 0, vocab, a.k, want_lse, cand, min(cfg.dyn_slots, MERGE_CAP), sh);
        n = min(sh.n_cand, min(cfg.dyn_slots, MERGE_CAP));
        if (cfg.path_stats != nullptr && tid == 0) {
            atomicAdd(&cfg.path_stats[2], 1u);
        }
    } else {
        constexpr int PER = MERGE_CAP / NT;
        for (int j0 = 0; j0 < PER; j0 += 8) {   // eight loads in flight
            if ((uint32_t)j0 * NT >= total) {
                break;
            }
            uint64_t got[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const uint32_t i = min((uint32_t)(j0 + u) * NT + tid, total - 1u);
                got[u] = handed_load(cfg.ws_cand, (size_t)row * MERGE_CAP + i);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const uint32_t i = (uint32_t)(j0 + u) * NT + tid;
                if (i < total) {
                    cand[i] = got[u];
                }
            }
        }
        if (want_lse && tid < 64u) {
            double mt = -__builtin_huge_val(), st = 0.0;
            if (lane < S) {
                mt = handed_load(cfg.ws_lse, 2 * ((size_t)row * S + lane));
                st = handed_load(cfg.ws_lse, 2 * ((size_t)row * S + lane) + 1);
                if (!(st > 0.0)) {
                    mt = -__builtin_huge_val();
                }
            }
            double m = mt;
            for (int o = 32; o > 0; o >>= 1) {
                m = fmax(m, __shfl_xor(m, o));
            }
            const double sum = wave_sum_d(st > 0.0 ? st * exp2(mt - m) : 0.0);
            if (tid == 0) {
                sh.lse_mc = m;
                sh.lse_s = sum;
            }
        }
        __syncthreads();
        WIDE_MARK(13);
        n = select_topk(cand, total, a.k, sh, sorted);
        WIDE_MARK(14);
        if (cfg.path_stats != nullptr && tid == 0) {
            atomicAdd(&cfg.path_stats[1], 1u);
        }
    }
    tail<DT, true>(a, vocab, step, n, sorted, cand, sh, cfg);
}

template <int DT, bool LSE, bool INLINE>
static hipError_t launch_wide_variant(hipStream_t stream, uint32_t rows, const LaunchCfg& cfg,
                                      const InlineRows* inline_rows, const WideArgs& w) {
    const dim3 grid(cfg.slices, rows), block(NT);
    static const InlineRows none = {};
    const InlineRows& r = inline_rows != nullptr ? *inline_rows : none;
    const size_t dyn2 = (size_t)cfg.dyn_slots * 8;
    hipLaunchKernelGGL((k_wide_bound<DT, LSE, INLINE>), grid, block, 0, stream, r, cfg, w);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        return e;
    }
    hipLaunchKernelGGL((k_wide_draw<DT, LSE, INLINE>), grid, block, dyn2, stream, r, cfg, w);
    return hipGetLastError();
}

hipError_t launch_rows_wide(hipStream_t stream, int dtype, bool lse, uint32_t rows, const LaunchCfg& cfg_in,
                            const InlineRows* inline_rows, float* lane_max, uint32_t* count) {
    LaunchCfg cfg = cfg_in;
    // the merging workgroup's candidates, then the tail's arrays behind the first K_CAP of them
    cfg.dyn_slots = MERGE_CAP;
    cfg.cand_cap = MERGE_CAP;
    WideArgs w;
    w.lane_max = Handed<float>{lane_max};
    w.slice_bound = Handed<float>{lane_max + (size_t)rows * cfg.slices * NT};   // (behind the lanes' maxima)
    w.lanes = (uint64_t)cfg.slices * (NT / 2) >= 4ull * cfg.ws_k ? NT / 2 : NT;
    w.count = count;
    const bool inl = inline_rows != nullptr;
#define LILY_WIDE(DT)                                                                               \
    (lse ? (inl ? launch_wide_variant<DT, true, true>(stream, rows, cfg, inline_rows, w)            \
                : launch_wide_variant<DT, true, false>(stream, rows, cfg, inline_rows, w))          \
         : (inl ? launch_wide_variant<DT, false, true>(stream, rows, cfg, inline_rows, w)           \
                : launch_wide_variant<DT, false, false>(stream, rows, cfg, inline_rows, w)))
    return dtype == LILY_BF16 ? LILY_WIDE(LILY_BF16) : LILY_WIDE(LILY_F32);
#undef LILY_WIDE
}

}  // namespace lily
