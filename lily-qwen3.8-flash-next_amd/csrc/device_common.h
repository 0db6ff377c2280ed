// device_common.h - what every select and the tail share: memory helpers, wave reductions,
// the workgroup's static LDS block, the radix-select plumbing over 64-bit composites, the
// slice geometry of a row read in 16-byte chunks, the running sums of exponentials and the
// per-chunk maxima.
//
// A candidate is a 64-bit composite: order key of the adjusted value << 32 | ~id.  A greater
// composite is a better candidate and the lowest id wins a tie.  Arithmetic that decides a
// token id follows tests/unit/kernels/sample.rs:8-54 of the reference operation for operation
// (IEEE division by the temperature, left-to-right f32 sums, lilym_expf); see
// include/lily_sampler_math.h.
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/lily_sampler_math.h"
#include "row_args.h"

namespace lily {

constexpr int NT = 256;
constexpr int NWAVE = NT / 64;
constexpr int UNROLL = 4;
constexpr uint32_t K_CAP = LILY_SAMPLE_K_CAP;
constexpr float F32_LOWEST = -3.4028234663852886e38f;

#define NEG_INF (-__builtin_huge_valf())

extern __shared__ uint64_t dyn_lds[];  // candidates, then the exclusion bitmap

// ------------------------------------------------------------------ small helpers

// Loads through a pointer known to be device memory: global_load instead of flat_load
// (the row's pointers arrive through LDS, so the compiler cannot tell by itself).
#define LILY_GLOBAL __attribute__((address_space(1)))
#define LILY_CONST __attribute__((address_space(4)))
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <class T>
__device__ __forceinline__ T gload(const T* p) {
    return *(const LILY_GLOBAL T*)p;
}
// Device-scope accesses that go through to memory, for data another workgroup (on any
// XCD, behind another L2) will read after taking the row's ticket.
template <class T>
__device__ __forceinline__ void store_through(T* p, T v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <class T>
__device__ __forceinline__ T load_through(const T* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <class T>
__device__ __forceinline__ void handed_store(const Handed<T>& h, size_t i, T v) {
    store_through(h.p + i, v);
}
template <class T>
__device__ __forceinline__ T handed_load(const Handed<T>& h, size_t i) {
    return load_through(h.p + i);
}

// The hand-over between the workgroups of a row (or the rows of a chained launch): every
// workgroup calls this after its handed_store()s; true, in every thread, in the workgroup that
// arrives last, which then reads with handed_load().  The counter is left at 0 for the next launch.
//
// Strict form (`relaxed` false): the ticket is a device-scope release, and an acquire fence of the
// same scope stands behind it - the hand-over the HIP memory model defines.
//
// Relaxed form: the ticket is a relaxed device atomic behind a wait for the thread's stores and a
// workgroup barrier, and nothing is invalidated behind it.  That leans on the hardware, not on the
// memory model: handed_store() writes through to memory (sc1) and has completed when
// s_waitcnt vmcnt(0) returns, handed_load() reads past the L2 of its XCD, so neither a write-back
// nor an invalidation of that L2 - what the release and the acquire cost, once per workgroup -
// adds anything.  A plain store to handed memory would break it silently, which is why Handed<T>
// admits none.  The host asks for this form only for launches of hundreds of workgroups
// (LaunchCfg::relaxed_handover; LILY_SAMPLER_HANDOVER=strict|relaxed overrides the choice), and
// -DLILY_STRICT_HANDOVER leaves it out of the build.
__device__ __forceinline__ bool last_to_arrive(uint32_t* ticket, uint32_t expected, uint32_t& last_lds,
                                               bool relaxed) {
#ifdef LILY_STRICT_HANDOVER
    relaxed = false;
#endif
    if (relaxed) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);   // every counter at 0: this thread's stores have completed
        __syncthreads();
        if (threadIdx.x == 0) {
            const uint32_t t = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_lds = t == expected - 1u ? 1u : 0u;
        }
        __syncthreads();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    } else {
        __syncthreads();   // (the other threads' stores happen before thread 0's release)
        if (threadIdx.x == 0) {
            const uint32_t t = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            last_lds = t == expected - 1u ? 1u : 0u;
        }
        __syncthreads();
        if (last_lds != 0u) {
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        }
    }
    const bool last = last_lds != 0u;
    if (last && threadIdx.x == 0) {
        store_through(ticket, 0u);
    }
    return last;
}

template <int DT>
__device__ __forceinline__ float load_logit(const void* p, uint32_t i) {
    if (DT == LILY_BF16) {
        return lilym_bits_f32((uint32_t)gload(static_cast<const uint16_t*>(p) + i) << 16);
    }
    return gload(static_cast<const float*>(p) + i);
}

__device__ __forceinline__ bool bit_of(const uint32_t* words, uint32_t id) {
    return (gload(words + (id >> 5)) >> (id & 31u)) & 1u;
}

__device__ __forceinline__ uint64_t composite_of(float adj, uint32_t id) {
    if (!(adj > NEG_INF)) {
        return 0;  // -inf (masked) and NaN are never candidates
    }
    return ((uint64_t)lilym_order_key(adj) << 32) | (uint32_t)(~id);
}
__device__ __forceinline__ uint32_t composite_id(uint64_t c) { return ~(uint32_t)c; }
__device__ __forceinline__ float composite_value(uint64_t c) {
    return lilym_key_value((uint32_t)(c >> 32));
}

// The oracle's map on a loaded logit l with emission count c: bias (list order), mask,
// penalties; the division by the temperature is the caller's.
__device__ __forceinline__ float finish_pre_temperature(const RowArgs& a, uint32_t id, float l,
                                                        uint32_t c, bool allowed) {
    // Eight pairs at a time, loaded whatever they hold (a delta that is loaded only on a match
    // makes every pair a memory round trip of its own); the additions keep the list's order.
    for (uint32_t j0 = 0; j0 < a.n_bias; j0 += 8u) {
        uint32_t bid[8];
        float delta[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const uint32_t j = min(j0 + (uint32_t)q, a.n_bias - 1u);
            bid[q] = gload(&a.bias[j].id);
            delta[q] = gload(&a.bias[j].delta);
        }
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            if (j0 + (uint32_t)q < a.n_bias && bid[q] == id) {
                l += delta[q];
            }
        }
    }
    if (!allowed) {
        return NEG_INF;
    }
    if (c > 0u) {
        l = l > 0.0f ? l / a.repetition : l * a.repetition;
        l -= a.presence + a.frequency * (float)c;
    }
    return l;
}

// The value before the temperature of one id, loads included.
template <int DT>
__device__ __forceinline__ float pre_temperature_of(const RowArgs& a, uint32_t id) {
    float l = load_logit<DT>(a.logits, id);
    const uint32_t c = (a.flags & F_PEN) ? gload(a.counts + id) : 0u;
    const bool allowed = a.allow == nullptr || bit_of(a.allow, id);
    return finish_pre_temperature(a, id, l, c, allowed);
}

template <int DT>
__device__ __forceinline__ float adjusted_of(const RowArgs& a, uint32_t id) {
    return pre_temperature_of<DT>(a, id) / a.temperature;
}

// The exact terms of ids [lo, hi), a thread's share sixteen at a time so that their loads
// are in flight together (the loop is a chain of memory round trips otherwise).  The slow way
// to a row sum, for the rare slices whose fast sum cancels.
template <int DT, typename Acc>
__device__ __forceinline__ void exact_terms(const RowArgs& a, uint32_t lo, uint32_t hi, float c2, Acc& acc) {
    constexpr int DEPTH = 16;
    const bool pen = (a.flags & F_PEN) != 0;
    for (uint32_t id0 = lo + threadIdx.x; id0 < hi; id0 += (uint32_t)DEPTH * NT) {
        float l[DEPTH];
        uint32_t c[DEPTH];
#pragma unroll
        for (int q = 0; q < DEPTH; ++q) {
            const uint32_t id = id0 + (uint32_t)q * NT;
            l[q] = id < hi ? load_logit<DT>(a.logits, id) : 0.0f;
            c[q] = (id < hi && pen) ? gload(a.counts + id) : 0u;
        }
#pragma unroll
        for (int q = 0; q < DEPTH; ++q) {
            const uint32_t id = id0 + (uint32_t)q * NT;
            if (id < hi) {
                const bool allowed = a.allow == nullptr || bit_of(a.allow, id);
                acc.add_one(finish_pre_temperature(a, id, l[q], c[q], allowed), c2);
            }
        }
    }
}

__device__ __forceinline__ float wave_max_f(float v) {
    for (int o = 32; o > 0; o >>= 1) {
        v = fmaxf(v, __shfl_xor(v, o));
    }
    return v;
}
// The wave's maximum in every lane, without LDS traffic: an inclusive running maximum inside
// each row of 16 lanes by DPP row shifts (a lane whose source lies outside the row keeps its
// own value), then the four row results read from lanes 15, 31, 47 and 63.
__device__ __forceinline__ float wave_max_dpp(float v) {
#define LILY_ROW_SHR_MAX(n)                                                                \
    v = fmaxf(v, lilym_bits_f32((uint32_t)__builtin_amdgcn_update_dpp(                       \
                     (int)lilym_f32_bits(v), (int)lilym_f32_bits(v), 0x110 + (n), 0xf, 0xf, false)))
    LILY_ROW_SHR_MAX(1);
    LILY_ROW_SHR_MAX(2);
    LILY_ROW_SHR_MAX(4);
    LILY_ROW_SHR_MAX(8);
#undef LILY_ROW_SHR_MAX
    const int b = (int)lilym_f32_bits(v);
    const float r0 = lilym_bits_f32((uint32_t)__builtin_amdgcn_readlane(b, 15));
    const float r1 = lilym_bits_f32((uint32_t)__builtin_amdgcn_readlane(b, 31));
    const float r2 = lilym_bits_f32((uint32_t)__builtin_amdgcn_readlane(b, 47));
    const float r3 = lilym_bits_f32((uint32_t)__builtin_amdgcn_readlane(b, 63));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}
__device__ __forceinline__ double wave_sum_d(double v) {
    for (int o = 32; o > 0; o >>= 1) {
        v += __shfl_xor(v, o);
    }
    return v;
}
// The wave's sum in every lane without LDS traffic: inclusive sums inside each row of 16 lanes
// by DPP row shifts (a lane without such a neighbour adds 0), then the four rows' totals read
// from lanes 15, 31, 47 and 63.
__device__ __forceinline__ double wave_sum_d_dpp(double v) {
#define LILY_ROW_SHR_ADD(n)                                                                      \
    {                                                                                            \
        const uint64_t b = __builtin_bit_cast(uint64_t, v);                                      \
        const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)b, 0x110 + (n), 0xf, 0xf, false);        \
        const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(b >> 32), 0x110 + (n), 0xf, 0xf, false); \
        v += __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);                              \
    }
    LILY_ROW_SHR_ADD(1)
    LILY_ROW_SHR_ADD(2)
    LILY_ROW_SHR_ADD(4)
    LILY_ROW_SHR_ADD(8)
#undef LILY_ROW_SHR_ADD
    const uint64_t b = __builtin_bit_cast(uint64_t, v);
    double t = 0.0;
#pragma unroll
    for (int l = 15; l < 64; l += 16) {
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, l);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), l);
        t += __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
    }
    return t;
}
__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int o) {
    const uint32_t lo = __shfl_xor((uint32_t)v, o);
    const uint32_t hi = __shfl_xor((uint32_t)(v >> 32), o);
    return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
    for (int o = 32; o > 0; o >>= 1) {
        const uint64_t w = shfl_xor_u64(v, o);
        v = w > v ? w : v;
    }
    return v;
}
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
    for (int o = 32; o > 0; o >>= 1) {
        const uint32_t w = __shfl_xor(v, o);
        v = w < v ? w : v;
    }
    return v;
}

// The value 4 order-key steps below t, not below the lowest finite float.
__device__ __forceinline__ float lower_by_slack(float t) {
    if (!(t > F32_LOWEST)) {
        return F32_LOWEST;
    }
    const uint32_t key = lilym_order_key(t) - 4u;
    return fmaxf(lilym_key_value(key), F32_LOWEST);
}

// ------------------------------------------------------------------ shared memory

struct Shared {
    // The tail's arrays live in dynamic LDS behind the (by then at most K_CAP) sorted
    // candidates; see tail_arrays().
    float* prob;         // [K_CAP] exp(adjusted - top) per sorted candidate
    float* cum;          // [K_CAP] inclusive prefix of the kept ones
    float* res;          // [K_CAP] residual of the speculative draw
    uint32_t hist[256];
    double red_d[NWAVE];
    float red_f[NWAVE];
    uint64_t red_u[NWAVE];
    uint32_t red_i[NWAVE];
    float wthr[NWAVE];      // each wave's threshold statistic (single-pass select)
    float wthr_f[NWAVE];    // each wave's last filter threshold
    uint32_t n_cand;
    uint32_t need;
    uint32_t sel_bin;
    uint32_t bin_count;
    uint32_t all_taken;
    uint32_t n_keep;
    uint32_t last;
    float mass;
    float p_d;
    float q_d;
    double lse_mc;   // log2-domain reference of the row's sum of exponentials
    double lse_s;    // sum of 2^(x * log2e / T - lse_mc) over the row
    // streaming select
    float bound[2][NWAVE];   // each wave's lower bound of its share of the k-th largest (two parities)
    float wmax[2][NWAVE];     // each wave's largest raw value
    uint32_t wfill[2][NWAVE]; // each wave's queue fill at the last refresh
    uint32_t wnote[2][NWAVE]; // each wave's count for the scan's choice of mode
    uint32_t qfill[NWAVE];   // chunks each wave queued
    uint32_t nfill[NWAVE];   // chunks each wave noted
    uint32_t n_fc;           // final candidates
    uint32_t n_pairs;  // (id, raw value) pairs listed from the queued chunks
    // rows that draw in order (one launch): what the rows before drew, the count each of those
    // ids had right after, the proposals the draws are compared with, and the last draw
    uint32_t drawn[LILY_MAX_VERIFY_ROWS];
    uint32_t drawn_count[LILY_MAX_VERIFY_ROWS];
    uint32_t proposal[LILY_MAX_VERIFY_ROWS];
    uint32_t chain_n[LILY_MAX_VERIFY_ROWS];   // candidates each row published
    uint32_t proposal_of[LILY_MAX_VERIFY_ROWS];   // each speculative row's proposal ...
    uint32_t q_n_of[LILY_MAX_VERIFY_ROWS];        // ... and the length of its draft distribution
    uint32_t emitted_id;
    uint32_t fail;
    double red3[4][NWAVE];
};

// Running sum of 2^(v*c - mc) of one thread with its own reference mc.
struct LseAcc {
    float mc;
    float s;
    __device__ __forceinline__ void init() {
        mc = NEG_INF;
        s = 0.0f;
    }
    // Raises the reference to cover block maximum cm; returns the reference to subtract.
    __device__ __forceinline__ float rebase(float cm, float c) {
        const float mcn = fmaxf(mc, cm * c);
        const float safe = fmaxf(mcn, F32_LOWEST);
        s *= __builtin_amdgcn_exp2f(mc - safe);
        mc = mcn;
        return safe;
    }
    __device__ __forceinline__ void term(float v, float c, float safe) {
        s += __builtin_amdgcn_exp2f(__builtin_fmaf(v, c, -safe));
    }
    __device__ __forceinline__ void add_one(float v, float c) {
        if (v > NEG_INF) {
            const float safe = rebase(v, c);
            term(v, c, safe);
        }
    }
};

// Workgroup-wide merge of the threads' accumulators into sh.lse_mc / sh.lse_s.
__device__ __forceinline__ void lse_reduce(Shared& sh, const LseAcc& l) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    float m = wave_max_f(l.mc);
    if (lane == 0) {
        sh.red_f[w] = m;
    }
    __syncthreads();
    m = sh.red_f[0];
    for (int i = 1; i < NWAVE; ++i) {
        m = fmaxf(m, sh.red_f[i]);
    }
    double s = 0.0;
    if (l.mc > NEG_INF) {
        s = (double)l.s * exp2((double)l.mc - (double)m);
    }
    s = wave_sum_d(s);
    if (lane == 0) {
        sh.red_d[w] = s;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int i = 0; i < NWAVE; ++i) {
            t += sh.red_d[i];
        }
        sh.lse_mc = (double)m;
        sh.lse_s = t;
    }
    __syncthreads();
}

// ------------------------------------------------------------------ radix-select plumbing

// Inclusive sums over the lanes of a wave (all 64 at work), lane 0 first, by six data-parallel
// moves between neighbours: by 1, 2, 4 and 8 lanes within each row of 16 (a lane without such
// a neighbour adds 0), then the last lane of row 0 into row 1 and of row 2 into row 3, then
// lane 31 into rows 2 and 3.
__device__ __forceinline__ uint32_t wave_scan_u32(uint32_t x) {
    int v = (int)x;
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);   // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);   // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);   // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);   // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);   // row_bcast:15 into rows 1, 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);   // row_bcast:31 into rows 2, 3
    return (uint32_t)v;
}

// With sh.hist complete: finds the bin in which the count from bin 255 downwards
// reaches `need`.  Leaves sh.sel_bin, sh.need (what is still needed inside that
// bin), sh.bin_count, and sh.all_taken = 1 when fewer than `need` were counted.
__device__ __forceinline__ void find_bin(Shared& sh, uint32_t need) {
    if (threadIdx.x < 64) {
        const uint32_t lane = threadIdx.x;
        uint32_t h[4], sum = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            h[j] = sh.hist[255u - (4u * lane + j)];
            sum += h[j];
        }
        const uint32_t incl = wave_scan_u32(sum);
        const uint32_t excl = incl - sum;
        const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        if (excl < need && need <= incl) {
            uint32_t seen = excl;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (seen < need && seen + h[j] >= need) {
                    sh.sel_bin = 255u - (4u * lane + j);
                    sh.need = need - seen;
                    sh.bin_count = h[j];
                }
                seen += h[j];
            }
        }
        if (lane == 0) {
            sh.all_taken = total < need ? 1u : 0u;
        }
    }
    __syncthreads();
}

// One thread's counts of one pass of a radix select.  The digit the thread meets first is
// counted in a register and added once at the end: the keys of a row of logits share their
// leading digits, adds by the lanes of a wave to one LDS word are served one after the other,
// and the workgroup's waves share the one LDS - counted key by key, the leading passes are
// that queue and little else.
struct HistRun {
    uint32_t d0, c0;
    __device__ __forceinline__ void init() {
        d0 = 0;
        c0 = 0;
    }
    __device__ __forceinline__ void add(uint32_t* hist, uint32_t digit, bool on) {
        // (no branch but around the add: selects, not jumps, for the common case)
        const bool same = on & ((c0 == 0u) | (digit == d0));
        d0 = same ? digit : d0;
        c0 += same ? 1u : 0u;
        if (on & !same) {
            atomicAdd(&hist[digit], 1u);
        }
    }
    __device__ __forceinline__ void flush(uint32_t* hist) {
        if (c0 != 0u) {
            atomicAdd(&hist[d0], c0);
        }
    }
};

// The top-k of cand[0..n) (zeros are invalid) compacted, unsorted, to the front;
// returns how many there are.
__device__ __forceinline__ uint32_t wg_select_topk(uint64_t* cand, uint32_t n, uint32_t k, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    constexpr int PER = MERGE_CAP / NT;  // n <= MERGE_CAP
    // Every pass works on the thread's own entries, read from LDS once.
    uint64_t mine[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const uint32_t i = tid + (uint32_t)j * NT;
        mine[j] = i < n ? cand[i] : 0ull;
    }
    uint64_t prefix = 0, pmask = 0;
    uint32_t need = k;
    bool all = false;
    for (int pass = 0; pass < 8; ++pass) {
        const int shift = 56 - 8 * pass;
        if (tid < 256) {
            sh.hist[tid] = 0;
        }
        __syncthreads();
        HistRun run;
        run.init();
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            run.add(sh.hist, (uint32_t)(mine[j] >> shift) & 255u, mine[j] != 0 && (mine[j] & pmask) == prefix);
        }
        run.flush(sh.hist);
        __syncthreads();
        find_bin(sh, need);
        if (sh.all_taken != 0u) {
            all = true;
            break;
        }
        prefix |= (uint64_t)sh.sel_bin << shift;
        pmask |= (uint64_t)255u << shift;
        const bool whole_bin = sh.bin_count == sh.need;
        const uint32_t in_bin = sh.bin_count;
        need = sh.need;
        if (whole_bin) {
            break;
        }
        if (in_bin <= 128u) {
            // Few entries left (rows of bf16 logits tie by the dozen at the k-th value and
            // would take every remaining pass to split by id): rank them against each
            // other; the one with `need - 1` above it is the k-th entry itself.
            uint64_t* left = reinterpret_cast<uint64_t*>(sh.hist);  // free after find_bin
            if (tid == 0) {
                sh.n_cand = 0;
            }
            __syncthreads();
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                if (mine[j] != 0 && (mine[j] & pmask) == prefix) {
                    left[atomicAdd(&sh.n_cand, 1u)] = mine[j];
                }
            }
            __syncthreads();
            if (tid < in_bin) {
                const uint64_t me = left[tid];
                uint32_t above = 0;
                for (uint32_t j = 0; j < in_bin; ++j) {
                    above += left[j] > me ? 1u : 0u;
                }
                if (above == need - 1u) {
                    sh.red_u[0] = me;
                }
            }
            __syncthreads();
            prefix = sh.red_u[0];
            __syncthreads();
            break;
        }
    }
    const uint64_t floor_c = all ? 1ull : prefix;
    if (tid == 0) {
        sh.n_cand = 0;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        if (mine[j] != 0 && mine[j] >= floor_c) {
            cand[atomicAdd(&sh.n_cand, 1u)] = mine[j];
        }
    }
    __syncthreads();
    return sh.n_cand;
}

// Small sets (n <= NT): every thread ranks one candidate against all the others (each a
// broadcast LDS read); the rank is the candidate's place in descending order, so the
// top-k come out sorted.  Returns how many there are (zeros are dropped).
__device__ __forceinline__ uint32_t wg_rank_select(uint64_t* cand, uint32_t n, uint32_t k, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    const uint64_t mine = tid < n ? cand[tid] : 0ull;
    uint32_t rank = 0;
    uint32_t j = 0;
    for (; j + 8 <= n; j += 8) {  // eight independent broadcast reads at a time
        uint64_t c[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            c[q] = cand[j + q];
        }
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            rank += c[q] > mine ? 1u : 0u;
        }
    }
    for (; j < n; ++j) {
        rank += cand[j] > mine ? 1u : 0u;
    }
    if (tid == 0) {
        sh.n_cand = 0;
    }
    __syncthreads();
    if (mine != 0ull && rank < k) {
        cand[rank] = mine;  // composites are distinct: ranks are too
        atomicAdd(&sh.n_cand, 1u);
    }
    __syncthreads();
    return sh.n_cand;
}

// Top-k of cand[0..n) to the front; `sorted` tells whether they are in descending order.
__device__ __forceinline__ uint32_t select_topk(uint64_t* cand, uint32_t n, uint32_t k, Shared& sh, bool& sorted) {
    if (n <= 256u) {
        sorted = true;
        return wg_rank_select(cand, n, k, sh);
    }
    sorted = false;
    return wg_select_topk(cand, n, k, sh);
}

// The k-th largest of the workgroup's NT x 8 per-lane values (-inf = absent) by a
// radix select on their order keys; F32_LOWEST when fewer than k are present.
__device__ __forceinline__ float wg_kth_largest(const float (&ms)[8], uint32_t k, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    uint32_t keys[8];
    for (int j = 0; j < 8; ++j) {
        keys[j] = ms[j] > NEG_INF ? lilym_order_key(ms[j]) : 0u;
    }
    uint32_t prefix = 0, pmask = 0, need = k;
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 24 - 8 * pass;
        if (tid < 256) {
            sh.hist[tid] = 0;
        }
        __syncthreads();
        HistRun run;
        run.init();
        for (int j = 0; j < 8; ++j) {
            run.add(sh.hist, (keys[j] >> shift) & 255u, keys[j] != 0u && (keys[j] & pmask) == prefix);
        }
        run.flush(sh.hist);
        __syncthreads();
        find_bin(sh, need);
        if (sh.all_taken != 0u) {
            return F32_LOWEST;
        }
        prefix |= sh.sel_bin << shift;
        pmask |= 255u << shift;
        need = sh.need;
    }
    return lilym_key_value(prefix);
}

// ------------------------------------------------------------------ slice geometry

// A row is read in 16-byte chunks from the 16-byte boundary at or below its first
// element; `pad` elements of chunk 0 lie before the row.  Chunk c holds ids
// c*E - pad .. c*E - pad + E - 1.
template <int DT>
struct Geo {
    static constexpr int E = DT == LILY_BF16 ? 8 : 4;
    const char* base;   // 16-byte aligned
    uint32_t pad;
    uint32_t cb, ce;    // this slice's chunks
    uint32_t full_lo, full_hi;  // chunks lying wholly inside the row
    uint32_t vocab;
    uint32_t id_lo, id_hi;      // this slice's ids
    uint32_t main_lo, main_hi;  // this slice's chunks that are streamed
    uint32_t edge_lo_end;       // ids [id_lo, edge_lo_end) and [edge_hi_begin, id_hi) are edges
    uint32_t edge_hi_begin;

    __device__ void init(const void* logits, uint32_t v, uint32_t s, uint32_t slices) {
        const uintptr_t addr = reinterpret_cast<uintptr_t>(logits);
        pad = (uint32_t)(addr & 15u) / (16u / E);
        base = reinterpret_cast<const char*>(addr & ~(uintptr_t)15u);
        vocab = v;
        const uint32_t nch = (pad + v + E - 1) / E;
        const uint32_t per = (nch + slices - 1) / slices;
        cb = min(s * per, nch);
        ce = min(cb + per, nch);
        full_lo = pad ? 1u : 0u;
        full_hi = (pad + v) / E;
        const int64_t lo = (int64_t)cb * E - pad, hi = (int64_t)ce * E - pad;
        id_lo = (uint32_t)max(lo, (int64_t)0);
        id_hi = (uint32_t)min(hi, (int64_t)v);
        if (id_hi < id_lo) {
            id_hi = id_lo;
        }
        main_lo = max(cb, full_lo);
        main_hi = max(min(ce, full_hi), main_lo);
        if (main_hi > main_lo) {
            edge_lo_end = main_lo * E - pad;
            edge_hi_begin = main_hi * E - pad;
        } else {
            edge_lo_end = id_hi;  // nothing is streamed: every id is an edge
            edge_hi_begin = id_hi;
        }
    }

    // Chunk c as its 16 raw bytes when it lies wholly inside the row and the slice
    // (main_lo <= c < main_hi), else sixteen bytes of -inf.  The few ids of partial chunks
    // at the ends of a row (edge_*) are not streamed; callers evaluate them one by one.
    __device__ __forceinline__ u32x4 load_raw(uint32_t c) const {
        u32x4 q;
        const uint32_t ninf = DT == LILY_BF16 ? 0xff80ff80u : 0xff800000u;
        q.x = q.y = q.z = q.w = ninf;
        if (c >= main_lo && c < main_hi) {
            q = gload(reinterpret_cast<const u32x4*>(base + (size_t)c * 16));
        }
        return q;
    }

    __device__ __forceinline__ uint32_t id_of(uint32_t c, int j) const {
        return c * E - pad + (uint32_t)j;
    }
};

// 32 bits of bitmap `words` (bit index = id) starting at id0 (may be negative or
// run past the end: those bits read 0).
__device__ __forceinline__ uint32_t bits32_at(const uint32_t* words, uint32_t nwords, int64_t id0) {
    const int64_t wi = id0 >> 5;
    const uint32_t sh = (uint32_t)(id0 & 31);
    const uint32_t w0 = (wi >= 0 && wi < (int64_t)nwords) ? gload(words + wi) : 0u;
    if (sh == 0) {
        return w0;
    }
    const uint32_t w1 = (wi + 1 >= 0 && wi + 1 < (int64_t)nwords) ? gload(words + wi + 1) : 0u;
    return (w0 >> sh) | (w1 << (32u - sh));
}

// Bits of [id0, id0 + 32) that are ids in [lo, hi).
__device__ __forceinline__ uint32_t range32_at(uint32_t lo, uint32_t hi, int64_t id0) {
    const int64_t a = (int64_t)lo - id0 > 0 ? (int64_t)lo - id0 : 0;
    const int64_t b = (int64_t)hi - id0 < 32 ? (int64_t)hi - id0 : 32;
    if (b <= a) {
        return 0u;
    }
    const uint32_t upto_b = b >= 32 ? 0xffffffffu : ((1u << b) - 1u);
    const uint32_t upto_a = a >= 32 ? 0xffffffffu : ((1u << a) - 1u);
    return upto_b & ~upto_a;
}

// ------------------------------------------------------------------ diagnostics, appends, row sums

// Diagnostic: thread 0 stamps the 100 MHz wall clock at phase i (see LaunchCfg::phase_trace).
__device__ __forceinline__ void phase(const LaunchCfg& cfg, uint32_t i) {
    if (cfg.phase_trace != nullptr && threadIdx.x == 0) {
        cfg.phase_trace[((size_t)blockIdx.y * cfg.slices + blockIdx.x) * PHASE_SLOTS + i] =
            wall_clock64();
        // The store is waited for here, where it is rare: a store still in flight next to
        // loads makes every later wait for a load drain all loads in flight (stores and
        // loads share one counter and complete in no fixed order).
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    }
}

// Appends the lanes with `pass` set to this wave's own region of the candidate buffer
// (`region`, `seg` slots); `count` is the wave's fill, the same in every lane.  No atomics:
// the slot is the fill plus the lane's rank among the passing lanes.
__device__ __forceinline__ void append(bool pass, float v, uint32_t id, uint64_t* region,
                                       uint32_t seg, uint32_t& count) {
    const uint64_t mask = __ballot(pass);
    if (mask == 0) {
        return;
    }
    const uint32_t rank =
        __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
    const uint32_t at = count + rank;
    if (pass && at < seg) {
        region[at] = ((uint64_t)lilym_order_key(v) << 32) | (uint32_t)(~id);
    }
    count += (uint32_t)__popcll(mask);
}

// Appends ids to the specials list (wave-aggregated); returns false for a lane whose id
// did not fit.
__device__ __forceinline__ bool list_push(bool has, uint32_t id, uint32_t* list, uint32_t list_cap,
                                          Shared& sh) {
    const uint64_t mask = __ballot(has);
    if (mask == 0) {
        return true;
    }
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t rank =
        __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
    const int leader = __builtin_ctzll(mask);
    uint32_t base = 0;
    if ((int)lane == leader) {
        base = atomicAdd(&sh.need, (uint32_t)__popcll(mask));
    }
    base = __shfl(base, leader);
    if (has) {
        if (base + rank < list_cap) {
            list[base + rank] = id;
            return true;
        }
        return false;
    }
    return true;
}

// A term's exponent v*c - ref is formed in f32: its rounding error grows with its size, and
// the terms that carry the sum are the ones above the reference.  The reference is raised
// before any exponent exceeds this (values below 32 are at most 0.95e-6 off: a relative
// error of 0.7e-6 in the term, well inside the log-probability's 1e-5).
constexpr float LSE_RAISE = 24.0f;

// One wave's sum of 2^(v*c - ref) with a reference that is the same in every lane.
struct WaveLse {
    float ref;
    float s;
    float booked;   // what the caller took off `s` again, kept relative to the same reference
    __device__ __forceinline__ void init() {
        ref = F32_LOWEST;
        s = 0.0f;
        booked = 0.0f;
    }
    // Adds the E terms of one load whose lane maximum is m; skipped by the whole wave when
    // every term is below 2^-40 of the reference.
    template <int E>
    __device__ __forceinline__ void add(const float (&v)[E], float m, float c) {
        if (__ballot(__builtin_fmaf(m, c, -ref) > LSE_RAISE) != 0ull) {
            // A term would dwarf the reference: raise it to the wave's maximum (rare).
            const float nref = fmaxf(ref, wave_max_f(m * c));
            const float down = __builtin_amdgcn_exp2f(ref - nref);
            s *= down;
            booked *= down;
            ref = nref;
        }
        if (__ballot(__builtin_fmaf(m, c, -ref) > -40.0f) == 0ull) {
            return;
        }
        for (int j = 0; j < E; ++j) {
            s += __builtin_amdgcn_exp2f(__builtin_fmaf(v[j], c, -ref));
        }
    }
    // As add(); an inactive lane contributes nothing.
    template <int E>
    __device__ __forceinline__ void add_if(const float (&v)[E], float m, float c, bool active) {
        const float d = __builtin_fmaf(active ? m : NEG_INF, c, -ref);
        if (__ballot(d > LSE_RAISE) != 0ull) {
            const float nref = fmaxf(ref, wave_max_f(active ? m * c : NEG_INF));
            const float down = __builtin_amdgcn_exp2f(ref - nref);
            s *= down;
            booked *= down;
            ref = nref;
        } else if (__ballot(d > -40.0f) == 0ull) {
            return;
        }
        if (active) {
#pragma unroll
            for (int j = 0; j < E; ++j) {
                s += __builtin_amdgcn_exp2f(__builtin_fmaf(v[j], c, -ref));
            }
        }
    }
    // As add_if() on the raw 16 bytes of one load (unpacked only when the wave does not skip
    // it).
    template <int DT>
    __device__ __forceinline__ void add_chunk(const u32x4& q, float m, float c, bool active);
    // Block-wise use: prepare() once with the largest value the lane will add in the block
    // (raises the reference when some lane's would dwarf it), then add_prepared() per load.
    float skip_below;  // loads whose maximum is not above this are left out (set by the caller)
    __device__ __forceinline__ void prepare(float block_max, float c) {
        if (__ballot(__builtin_fmaf(block_max, c, -ref) > LSE_RAISE) != 0ull) {
            const float nref = fmaxf(ref, wave_max_dpp(block_max * c));
            const float down = __builtin_amdgcn_exp2f(ref - nref);
            s *= down;
            booked *= down;
            ref = nref;
        }
    }
    template <int DT>
    __device__ __forceinline__ void add_prepared(const u32x4& q, float m, float c, bool active);
};

// Workgroup-wide merge of per-thread (reference, sum) pairs: returns through `m`, `sum`
// (double, valid in every thread).
// Returns whether some thread's sum is a NaN (a NaN logit went into it: such a logit is worth
// -inf, and the caller forms the row's sum again by the path that looks at every value).
__device__ __forceinline__ bool wg_merge_lse(Shared& sh, float mc, float s_in, double& m_out, double& sum_out) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    float m = wave_max_f(s_in > 0.0f ? mc : NEG_INF);
    if (lane == 0) {
        sh.red_f[w] = m;
    }
    const bool poisoned = __syncthreads_or(s_in != s_in ? 1 : 0) != 0;
    m = sh.red_f[0];
    for (int i = 1; i < NWAVE; ++i) {
        m = fmaxf(m, sh.red_f[i]);
    }
    double s = 0.0;
    if (s_in > 0.0f) {
        s = (double)s_in * exp2((double)mc - (double)m);
    }
    s = wave_sum_d(s);
    if (lane == 0) {
        sh.red_d[w] = s;
    }
    __syncthreads();
    double t = 0.0;
    for (int i = 0; i < NWAVE; ++i) {
        t += sh.red_d[i];
    }
    __syncthreads();
    m_out = (double)m;
    sum_out = t;
    return poisoned;
}

template <int DT>
__device__ __forceinline__ void unpack(const u32x4 q, float (&v)[Geo<DT>::E]) {
    if (DT == LILY_BF16) {
        v[0] = lilym_bits_f32(q.x << 16);
        v[1] = lilym_bits_f32(q.x & 0xffff0000u);
        v[2] = lilym_bits_f32(q.y << 16);
        v[3] = lilym_bits_f32(q.y & 0xffff0000u);
        v[4 % Geo<DT>::E] = lilym_bits_f32(q.z << 16);
        v[5 % Geo<DT>::E] = lilym_bits_f32(q.z & 0xffff0000u);
        v[6 % Geo<DT>::E] = lilym_bits_f32(q.w << 16);
        v[7 % Geo<DT>::E] = lilym_bits_f32(q.w & 0xffff0000u);
    } else {
        v[0] = lilym_bits_f32(q.x);
        v[1] = lilym_bits_f32(q.y);
        v[2] = lilym_bits_f32(q.z);
        v[3] = lilym_bits_f32(q.w);
    }
}

// max(a, b, c) / max(a, b) as single instructions (NaN operands lose, as with fmaxf); the
// compiler's fmaxf adds a canonicalising instruction per operand in front of each.
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float max2_raw(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

// The largest element of one 16-byte chunk.
template <int DT>
__device__ __forceinline__ float chunk_max(const u32x4& q) {
    float v[Geo<DT>::E];
    unpack<DT>(q, v);
    if (DT == LILY_BF16) {
        return max2_raw(max3_raw(v[0], v[1], v[2]),
                        max3_raw(v[3], v[4 % Geo<DT>::E], max3_raw(v[5 % Geo<DT>::E], v[6 % Geo<DT>::E], v[7 % Geo<DT>::E])));
    }
    return max2_raw(max3_raw(v[0], v[1], v[2]), v[3]);
}

// Signed 16-bit maximum of both halves of a and b.  bf16 patterns of values that are not
// negative order like the values; every negative one is below all of them.
typedef short s16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_max_i16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(s16x2, a),
                                                                   __builtin_bit_cast(s16x2, b)));
}

// The largest element of one 16-byte chunk when that element is not negative, +0 otherwise:
// exact wherever the result is compared with a positive bound, an upper bound elsewhere.
// Half the instructions of chunk_max() for bf16 (no unpacking); the same for f32.
template <int DT>
__device__ __forceinline__ float chunk_max_nonneg(const u32x4& q) {
    if (DT == LILY_BF16) {
        const uint32_t r = pk_max_i16(pk_max_i16(q.x, q.y), pk_max_i16(q.z, q.w));
        const int m = max(max((int)(r << 16), (int)(r & 0xffff0000u)), 0);
        return lilym_bits_f32((uint32_t)m);
    }
    return chunk_max<DT>(q);
}

template <int DT>
__device__ __forceinline__ void WaveLse::add_prepared(const u32x4& q, float m, float c, bool active) {
    constexpr int E = DT == LILY_BF16 ? 8 : 4;
    active = active && m > skip_below;
    if (active) {
        // The raw bits pass through an empty asm so that this unpack is not merged with the
        // one that fed the chunk maximum: merged, 8 values per chunk stay live across the
        // whole block for a path that rows with a dominant value never take.
        u32x4 r = q;
        asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w));
        float v[E];
        unpack<DT>(r, v);
#pragma unroll
        for (int j = 0; j < E; ++j) {
            s += __builtin_amdgcn_exp2f(__builtin_fmaf(v[j], c, -ref));
        }
    }
}

template <int DT>
__device__ __forceinline__ void WaveLse::add_chunk(const u32x4& q, float m, float c, bool active) {
    constexpr int E = DT == LILY_BF16 ? 8 : 4;
    float v[E];
    unpack<DT>(q, v);
    add_if<E>(v, m, c, active);
}

__device__ __forceinline__ bool in_bias_list(const RowArgs& a, uint32_t id) {
    for (uint32_t j = 0; j < a.n_bias; ++j) {
        if (gload(&a.bias[j].id) == id) {
            return true;
        }
    }
    return false;
}

}  // namespace lily
