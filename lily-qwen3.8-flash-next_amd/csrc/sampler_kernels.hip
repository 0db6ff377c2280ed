// sampler_kernels.hip - gfx950 kernels of the logits-to-token stage.
//
// One launch serves a batch of logits rows.  Row r is scanned by `slices`
// workgroups of 512 threads (grid = slices x rows).  Each workgroup finds the
// exact top-k of its slice as 64-bit composites (order key of the adjusted value
// << 32 | ~id: a greater composite is a better candidate, the lowest id wins a
// tie).  With several slices the last workgroup to arrive (an atomic ticket,
// nobody waits) merges them.  That workgroup then runs the tail: sort, softmax
// over the candidates, the sequential top-p / min-p prefix, the draw, and for
// the speculative modes the export or the accept / residual draw.
//
// How a slice is scanned (select_fast):
//   * 16-byte loads, 8 bf16 or 4 f32 per lane, four loads in flight per lane.
//   * Ids that need more than "widen and compare" - masked out, penalised
//     (count > 0) or biased - are marked in an LDS bitmap built once per slice;
//     the stream treats them as -inf and the few that are allowed are evaluated
//     exactly afterwards ("specials").
//   * The filter works on the value BEFORE the division by the temperature (the
//     division is monotone), so the hot loop has no division.  Candidates that
//     pass go to an LDS buffer; the exact arithmetic runs on those only.
//   * k <= 64: single pass.  Every lane keeps its running maximum; the minimum
//     over G >= k lane groups of the group maximum is a lower bound of the k-th
//     largest value (G distinct elements reach it), refreshed every block of
//     loads; elements at or above it (less a 4-ulp slack for values the division
//     merges) are appended.
//   * k > 64: two passes.  The k-th largest of the 4 096 per-lane-per-slot
//     running maxima is the bound; the second pass (L2 / MALL hits) collects.
//   * Too many candidates (huge tie classes, adversarial order) or a failed
//     slack check: the slice is redone by select_exhaustive, a radix select over
//     the composites that re-evaluates every element and is correct for any input.
//
// Arithmetic that decides a token id follows tests/unit/kernels/sample.rs:8-54 of
// the reference operation for operation (IEEE division by the temperature,
// left-to-right f32 sums, lilym_expf); see include/lily_sampler_math.h.
#include <hip/hip_runtime.h>

#include "../../include/lily_sampler_math.h"
#include "row_args.h"

namespace lily {

constexpr int NT = 256;
constexpr int NWAVE = NT / 64;
constexpr int UNROLL = 4;
constexpr bool PREFETCH = false;  // keep block b+1 in flight while block b is processed
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
    for (uint32_t j = 0; j < a.n_bias; ++j) {
        const uint32_t bid = gload(&a.bias[j].id);
        if (bid == id) {
            l += gload(&a.bias[j].delta);
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
    float wmax[2][3][NWAVE];  // each wave's largest raw value, largest raw and largest true value
                              // of listed ids so far
    uint32_t dense_listed;    // some block holds more listed ids than the workgroup has threads
    uint32_t qfill[NWAVE];   // chunks each wave queued
    uint32_t n_fc;           // final candidates
    uint32_t n_drop;         // listed ids found inside queued chunks
    uint32_t fail;
    double red3[3][NWAVE];
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

// With sh.hist complete: finds the bin in which the count from bin 255 downwards
// reaches `need`.  Leaves sh.sel_bin, sh.need (what is still needed inside that
// bin), sh.bin_count, and sh.all_taken = 1 when fewer than `need` were counted.
__device__ __forceinline__ void find_bin(Shared& sh, uint32_t need) {
    if (threadIdx.x < 64) {
        const uint32_t lane = threadIdx.x;
        uint32_t h[4], sum = 0;
        for (int j = 0; j < 4; ++j) {
            h[j] = sh.hist[255u - (4u * lane + j)];
            sum += h[j];
        }
        uint32_t incl = sum;
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t t = __shfl_up(incl, o);
            if ((int)lane >= o) {
                incl += t;
            }
        }
        const uint32_t excl = incl - sum;
        const uint32_t total = __shfl(incl, 63);
        if (excl < need && need <= incl) {
            uint32_t seen = excl;
            for (int j = 0; j < 4; ++j) {
                if (seen + h[j] >= need) {
                    sh.sel_bin = 255u - (4u * lane + j);
                    sh.need = need - seen;
                    sh.bin_count = h[j];
                    break;
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
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            if (mine[j] != 0 && (mine[j] & pmask) == prefix) {
                atomicAdd(&sh.hist[(uint32_t)(mine[j] >> shift) & 255u], 1u);
            }
        }
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
        for (int j = 0; j < 8; ++j) {
            if (keys[j] != 0u && (keys[j] & pmask) == prefix) {
                atomicAdd(&sh.hist[(keys[j] >> shift) & 255u], 1u);
            }
        }
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

// ------------------------------------------------------------------ fast select

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
    __device__ __forceinline__ void init() {
        ref = F32_LOWEST;
        s = 0.0f;
    }
    // Adds the E terms of one load whose lane maximum is m; skipped by the whole wave when
    // every term is below 2^-40 of the reference.
    template <int E>
    __device__ __forceinline__ void add(const float (&v)[E], float m, float c) {
        if (__ballot(__builtin_fmaf(m, c, -ref) > LSE_RAISE) != 0ull) {
            // A term would dwarf the reference: raise it to the wave's maximum (rare).
            const float nref = fmaxf(ref, wave_max_f(m * c));
            s *= __builtin_amdgcn_exp2f(ref - nref);
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
            s *= __builtin_amdgcn_exp2f(ref - nref);
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
            s *= __builtin_amdgcn_exp2f(ref - nref);
            ref = nref;
        }
    }
    template <int DT>
    __device__ __forceinline__ void add_prepared(const u32x4& q, float m, float c, bool active);
};

// Workgroup-wide merge of per-thread (reference, sum) pairs: returns through `m`, `sum`
// (double, valid in every thread).
__device__ __forceinline__ void wg_merge_lse(Shared& sh, float mc, float s_in, double& m_out, double& sum_out) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    float m = wave_max_f(s_in > 0.0f ? mc : NEG_INF);
    if (lane == 0) {
        sh.red_f[w] = m;
    }
    __syncthreads();
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
    u32x4 cur[U], nxt[U];
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
            if (PREFETCH) {
                if (b + 1 < nblocks) {
                    fetch(nxt, b + 1);
                }
            } else if (b > 0) {
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
            if (PREFETCH) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    cur[u] = nxt[u];
                }
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
            wg_merge_lse(sh, wl.ref, wl.s, m_s, s_s);
            wg_merge_lse(sh, lse_true.mc, lse_true.s, m_t, s_t);
            if (patch) {
                wg_merge_lse(sh, lse_raw.mc, lse_raw.s, m_r, s_r);
            }
            double rest = s_s;
            bool bad = false;
            if (patch && s_r > 0.0) {
                rest = s_s - s_r * exp2(m_r - m_s);
                bad = !(rest > 0.05 * s_s);  // cancellation: the streamed sum is too coarse
            }
            if (bad) {
                phase(cfg, 12);
                // Rare: penalised ids held nearly all the raw mass.  Redo the sum exactly.
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
    constexpr int PREG = 12;  // listed ids a thread keeps in registers between the two bucket passes
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
    // ---- the slice's listed ids, bucketed by block
    // The first PREG x NT list entries are requested together with the list's length (the
    // list's memory is valid up to pairs_cap whatever the length turns out to be), ahead of
    // the first block of the row, which is then in flight while the ids are bucketed.
    uint32_t n_pairs = 0, loaded = 0;
    uint64_t early[PREG];
    if (pen) {
        // The list's length comes through the scalar path (nothing writes it while the
        // slices of its row still read it): a vector load of a value that is the same in
        // every lane is moved to a scalar register at once, and that move would hold the
        // list's loads below back until the length had arrived.
        n_pairs = *(const LILY_CONST uint32_t*)a.n_pairs;
        // The host's bound of the length says how much to request; a longer list is still
        // read completely (by the loop further down), a shorter one costs idle loads.
        const uint64_t want = ((uint64_t)a.pairs_hint + cfg.hint_growth + NT - 1) / NT * NT;
        loaded = (uint32_t)min(want, (uint64_t)min(a.pairs_cap, (uint32_t)(PREG * NT)));
#pragma unroll
        for (int q = 0; q < PREG; ++q) {
            const uint32_t p = (uint32_t)q * NT + tid;
            early[q] = p < loaded ? gload(reinterpret_cast<const uint64_t*>(a.pairs) + p) : ~0ull;
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
    if (tid == 0) {
        sh.n_fc = 0;
        sh.n_drop = 0;
        sh.fail = 0;
        sh.dense_listed = 0;
    }
    for (uint32_t i = tid; i < n_bias; i += NT) {
        L.bias_id[i] = gload(&a.bias[i].id);
        L.bias_delta[i] = gload(&a.bias[i].delta);
    }
    __syncthreads();
    phase(cfg, 13);
    if (n_pairs > a.pairs_cap) {
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
        if ((uint64_t)n_barred + n_pairs + n_bias > SPEC_CAP - SPEC_CAP / 10u) {
            return false;  // not a failure: the mask is not dense enough for this select
        }
    }
    const bool listed_row = n_pairs != 0 || n_bias != 0 || n_barred != 0;
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
    if (listed_row && nblocks == 1u) {
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
            if (p < n_pairs && p < loaded && block_of((uint32_t)early[q]) != NONE) {
                put((uint32_t)early[q] | (min((uint32_t)(early[q] >> 32), 4095u) << SPEC_ID_BITS));
            }
        }
        for (uint32_t p = loaded + tid; p < n_pairs; p += NT) {
            const uint64_t e = gload(reinterpret_cast<const uint64_t*>(a.pairs) + p);
            if (block_of((uint32_t)e) != NONE) {
                put((uint32_t)e | (min((uint32_t)(e >> 32), 4095u) << SPEC_ID_BITS));
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
            if (total > (uint32_t)NT) {
                sh.dense_listed = 1u;
            }
        }
    } else if (listed_row) {
        uint32_t packed[PREG];  // id | min(count, 4095) << 20, NONE when not of this slice
#pragma unroll
        for (int q = 0; q < PREG; ++q) {
            const uint32_t p = (uint32_t)q * NT + tid;
            packed[q] = NONE;
            if (p < n_pairs && p < loaded && block_of((uint32_t)early[q]) != NONE) {
                packed[q] = (uint32_t)early[q] |
                            (min((uint32_t)(early[q] >> 32), 4095u) << SPEC_ID_BITS);
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
            for (uint32_t p = loaded + tid; p < n_pairs; p += NT) {  // what the registers do not hold
                const uint64_t e = gload(reinterpret_cast<const uint64_t*>(a.pairs) + p);
                const uint32_t id = (uint32_t)e;
                const uint32_t b = block_of(id);
                if (b != NONE) {
                    if (pass == 0) {
                        atomicAdd(&L.bkt[b], 1u);
                    } else {
                        L.spec[L.bkt[b] + atomicAdd(&L.bfill[b], 1u)] =
                            id | (min((uint32_t)(e >> 32), 4095u) << SPEC_ID_BITS);
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
                    const uint64_t big = __ballot(cnt > (uint32_t)NT);
                    if (tid == 0) {
                        sh.dense_listed = big != 0ull ? 1u : 0u;
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
        float raw;
        u32x4 chunk;
    };
    // Unconditional as well: a thread without an entry reads the slice's last chunk.
    auto listed_fetch = [&](Listed& r, uint32_t b, uint32_t round) {
        r.raw = 0.0f;
        const uint32_t lo = L.bkt[b], hi = L.bkt[b + 1];
        const uint32_t e = lo + round * NT + ((tid + NT - ((b * 64u) % NT)) % NT);
        r.ent = e < hi ? L.spec[min(e, SPEC_CAP - 1u)] : NONE;
        const uint32_t c = min(((r.ent & ID_MASK) + g.pad) / E, c_last);
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
    // A listed id's true value before the temperature (bias in list order, then penalties);
    // also feeds the thread's maxima of listed raw and true values.
    auto listed_value = [&](Listed& r) -> float {
        if (r.ent == NONE) {
            return NEG_INF;
        }
        const uint32_t id = r.ent & ID_MASK;
        r.raw = raw_of(r.chunk, id);
        uint32_t cnt = r.ent >> SPEC_ID_BITS;
        if (cnt == 4095u) {
            cnt = gload(a.counts + id);
            // The value is waited for here, inside the branch: waiting after it would make
            // every thread drain the loads it has in flight.
            asm volatile("" : "+v"(cnt));
        }
        float t = r.raw;
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
        listed_raw_max = fmaxf(listed_raw_max, r.raw);
        listed_true_max = fmaxf(listed_true_max, t);
        return t;
    };
    // After the block's bound is known: was the id's chunk queued or summed by its owner (the
    // owner's tests on the same bits), the id's terms, and the id as a candidate.
    auto listed_finish = [&](const Listed& r, float t, bool nonneg) {
        if (r.ent == NONE) {
            return;
        }
        const uint32_t id = r.ent & ID_MASK;
        const float cm = nonneg ? chunk_max_nonneg<DT>(r.chunk) : chunk_max<DT>(r.chunk);
        const bool queued = cm >= T;
        const bool summed = !queued && cm > skip_b;
        if (want_lse) {
            if (t > skip_b) {  // the same cut as for streamed terms
                acc_t += term_d(t);
            }
            if (summed) {
                acc_r += term_d(r.raw);
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
        const float lcur_t = listed_row ? listed_value(lcur) : NEG_INF;
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
            listed_finish(lcur, lcur_t, nonneg);
            const uint32_t n_b = L.bkt[b + 1] - L.bkt[b];
            for (uint32_t round = 1; round * NT < n_b; ++round) {
                Listed extra;
                listed_fetch(extra, b, round);
                listed_finish(extra, listed_value(extra), nonneg);
            }
        }
    };
    // A request past the last block asks for the last block again (its lines are in the
    // cache and nothing uses the result): with the same loads in flight on every path the
    // wait for a block's data leaves the blocks requested after it in flight, where a request
    // that may be skipped makes that wait count as if it had been.
    auto request = [&](u32x4 (&dst)[U], Listed& ldst, uint32_t b) {
        const uint32_t bb = min(b, nblocks - 1u);
        if (listed_row) {
            listed_fetch(ldst, bb, 0);
        }
        fetch(dst, bb);
    };
    if (nblocks == 0) {
        refresh_bound(true, true);  // the same barriers in every workgroup
    } else {
        if (listed_row) {
            listed_fetch(lst_a, 0, 0);
        }
        request(buf_b, lst_b, 1);
        for (uint32_t b = 0; b < nblocks; b += 3) {
            request(buf_c, lst_c, b + 2);
            work(buf_a, lst_a, b);
            if (b + 1 < nblocks) {
                request(buf_a, lst_a, b + 3);
                work(buf_b, lst_b, b + 1);
                if (b + 2 < nblocks) {
                    request(buf_b, lst_b, b + 4);
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

// ------------------------------------------------------------------ exhaustive select
//
// The exact top-k of ids [id_lo, id_hi) by a radix select on the composite: up to
// eight passes of 8 bits, each re-evaluating every element.  Slow and correct for
// any input (ties, masks, few finite values).  Leaves the winners (unsorted) in
// cand[0 .. sh.n_cand).
template <int DT>
__device__ __forceinline__ void select_exhaustive(const RowArgs& a, uint32_t e0, uint32_t e1, uint32_t k,
                                  bool want_lse, uint64_t* cand, uint32_t cap, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    uint64_t prefix = 0, pmask = 0;
    uint32_t need = k;
    LseAcc lse;
    lse.init();
    bool take_all = false;
    for (int pass = 0; pass < 8 && !take_all; ++pass) {
        const int shift = 56 - 8 * pass;
        if (tid < 256) {
            sh.hist[tid] = 0;
        }
        __syncthreads();
        for (uint32_t id = e0 + tid; id < e1; id += NT) {
            const float u = pre_temperature_of<DT>(a, id);
            if (pass == 0 && want_lse) {
                lse.add_one(u, a.c2);
            }
            const uint64_t c = composite_of(u / a.temperature, id);
            if (c != 0 && (c & pmask) == prefix) {
                atomicAdd(&sh.hist[(uint32_t)(c >> shift) & 255u], 1u);
            }
        }
        __syncthreads();
        find_bin(sh, need);
        take_all = sh.all_taken != 0u;
        if (!take_all) {
            prefix |= (uint64_t)sh.sel_bin << shift;
            pmask |= (uint64_t)255u << shift;
            need = sh.need;
        }
    }
    if (want_lse) {
        lse_reduce(sh, lse);
    }
    if (tid == 0) {
        sh.n_cand = 0;
    }
    __syncthreads();
    const uint64_t floor_c = take_all ? 1ull : prefix;
    for (uint32_t id = e0 + tid; id < e1; id += NT) {
        const uint64_t c = composite_of(adjusted_of<DT>(a, id), id);
        if (c >= floor_c && c != 0) {
            const uint32_t at = atomicAdd(&sh.n_cand, 1u);
            if (at < cap) {
                cand[at] = c;
            }
        }
    }
    __syncthreads();
}

// ------------------------------------------------------------------ sort

// Descending bitonic sort of cand[0..n), n <= 4 * NT, four entries per thread (entry
// 4 * tid + r in register r; absent entries are 0, the smallest).  Exchanges at distance
// 1 and 2 stay inside a thread, 4 .. 128 are lane shuffles inside a wave, and only the
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
                const uint32_t m = stride >> 2;
                const bool desc = ((tid * 4u) & size) == 0;
                const bool take_max = ((lane & m) == 0) == desc;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint64_t o = shfl_xor_u64(v[r], (int)m);
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
            for (uint32_t size = 2; size <= 64; size <<= 1) {
                for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
                    const uint64_t o = shfl_xor_u64(c, (int)stride);
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

// Counts one emission of `id` in a scratch: the dense count, and the id's entry in the list
// (appended with the first count; `touched` marks the listed ids).
__device__ __forceinline__ void count_token(uint32_t* counts, uint32_t* touched, CountPair* pairs,
                                            uint32_t* n_pairs, uint32_t* pos, uint32_t pairs_cap,
                                            uint32_t id) {
    const uint32_t before = atomicAdd(&counts[id], 1u);
    const uint32_t bit = 1u << (id & 31u);
    const uint32_t bits = atomicOr(&touched[id >> 5], bit);
    if ((bits & bit) == 0u) {
        const uint32_t p = atomicAdd(n_pairs, 1u);
        if (p < pairs_cap) {
            pairs[p].id = id;
            pairs[p].count = before + 1u;
        }
        pos[id] = p < pairs_cap ? p : 0xffffffffu;  // listed ids always have a meaningful pos
    } else {
        const uint32_t p = pos[id];
        if (p < pairs_cap) {
            pairs[p].count = before + 1u;
        }
    }
}

__device__ __forceinline__ void emit(const RowArgs& a, uint32_t id) {
    *a.out_id = id;
    if (a.flags & F_PEN) {
        count_token(a.counts, a.touched, a.pairs, a.n_pairs, a.pos, a.pairs_cap, id);
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
// round trip: the count's atomic increment returns the count the penalties used, the bitmap's
// atomic OR tells whether the id is listed already, and the logit and the list position load
// beside them.
template <int DT>
__device__ __forceinline__ void finish_token(const RowArgs& a, const Shared& sh, uint32_t id, uint32_t vocab) {
    *a.out_id = id;
    const bool pen = (a.flags & F_PEN) != 0;
    const bool want = a.out_logprob != nullptr;
    if (id >= vocab) {
        if (want) {
            *a.out_logprob = NEG_INF;
        }
        return;
    }
    uint32_t before = 0, bits = 0, p = 0xffffffffu;
    const uint32_t bit = 1u << (id & 31u);
    if (pen) {
        before = atomicAdd(&a.counts[id], 1u);
        bits = atomicOr(&a.touched[id >> 5], bit);
        p = gload(a.pos + id);
    }
    if (want) {
        const float l = load_logit<DT>(a.logits, id);
        const bool allowed = a.allow == nullptr || bit_of(a.allow, id);
        const float u = finish_pre_temperature(a, id, l, before, allowed);
        float lp = NEG_INF;
        if (u > NEG_INF) {
            const double e = (double)u * (double)a.c2 - sh.lse_mc - log2(sh.lse_s);
            lp = fminf((float)(e * 0.6931471805599453), 0.0f);  // the sum is approximate: clamp
        }
        *a.out_logprob = lp;
    }
    if (pen) {
        if ((bits & bit) == 0u) {
            const uint32_t at = atomicAdd(a.n_pairs, 1u);
            if (at < a.pairs_cap) {
                a.pairs[at].id = id;
                a.pairs[at].count = before + 1u;
            }
            a.pos[id] = at < a.pairs_cap ? at : 0xffffffffu;
        } else if (p < a.pairs_cap) {
            a.pairs[p].count = before + 1u;
        }
    }
}

// cand[0..n) holds the row's candidates (at least its top-k); finishes the row.
template <int DT, bool BIG>
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
            emit(a, 0);
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
    if (!sorted) {
        sort_desc<BIG>(cand, n);
    }
    TAIL_MARK(8);
    const uint32_t k = min(a.k, n);
    const float top = composite_value(cand[0]);
    if (k <= 64u && a.mode != MODE_SPEC) {
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
        float total = 0.0f;
#pragma unroll
        for (int i = 0; i < 64; ++i) {
            total += lilym_bits_f32((uint32_t)__builtin_amdgcn_readlane(pbits, i));
        }
        const float limit = a.top_p * total;
        float cum = 0.0f, before = 0.0f, mine = 0.0f;
#pragma unroll
        for (int i = 0; i < 64; ++i) {
            before = lane == (uint32_t)i ? cum : before;
            cum += lilym_bits_f32((uint32_t)__builtin_amdgcn_readlane(pbits, i));
            mine = lane == (uint32_t)i ? cum : mine;
        }
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
        const uint64_t hits = __ballot(lane < kept && u1 * mass < mine);
        const uint32_t slot = hits != 0ull ? (uint32_t)__builtin_ctzll(hits) : kept - 1u;
        const uint32_t id = ~(uint32_t)__shfl((int)(uint32_t)c, (int)slot);
        if (lane == 0) {
            finish_token<DT>(a, sh, id, vocab);
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
    // The reference's left-to-right f32 sums: one wave runs the chain of additions, 64
    // candidates at a time with a candidate per lane, and keeps every prefix.  Each step adds
    // the lane's value to the running sum of the lane below (a shift by one lane across the
    // whole wave; lane 0 has no lane below and keeps what it has): after step j the lanes up
    // to j hold their final prefix, which further steps only reproduce.  The row total is
    // the last prefix, and the sum the reference holds before rank r is the prefix of rank
    // r - 1: the cut by top-p and min-p and the inverse-CDF pick then are searches every
    // thread takes part in.
    if (tid < 64u) {
        float carry = 0.0f;
        for (uint32_t r0 = 0; r0 < k; r0 += 64u) {
            const uint32_t i = r0 + tid;
            const float p = i < k ? sh.prob[i] : 0.0f;
            float run = carry + p;  // final in lane 0
#pragma unroll
            for (int j = 1; j < 64; ++j) {
                // Two idle cycles between a lane's write and the neighbour's read of it.
                asm volatile("s_nop 1\n\tv_add_f32_dpp %0, %0, %1 wave_shr:1 row_mask:0xf bank_mask:0xf"
                             : "+v"(run)
                             : "v"(p));
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
            finish_token<DT>(a, sh, id, vocab);
        }
        return;
    }

    // Speculative draw (sample.metal:596-658, cpu_spec at tests/unit/kernels/sample.rs:264-283).
    const uint32_t d = *a.draft;
    const uint32_t qn = min(*a.q_n, K_CAP);
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
            finish_token<DT>(a, sh, d, vocab);
        }
        return;
    }
    for (uint32_t i = tid; i < n_keep; i += NT) {
        const uint32_t id = composite_id(cand[i]);
        float q_i = 0.0f;
        for (uint32_t j = 0; j < qn; ++j) {
            if (a.q_ids[j] == id) {
                q_i = a.q_probs[j];
                break;
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
        finish_token<DT>(a, sh, id, vocab);
    }
}

// ------------------------------------------------------------------ argmax

// First maximum under float comparison (NaN never wins, -0 == +0), lowest id on
// ties: elementwise.metal:145-150.  Result: the best (value, id) of the slice as a
// composite; id bits all zero when no element qualified.
template <int DT>
__device__ __forceinline__ uint64_t slice_argmax(const RowArgs& a, const Geo<DT>& g, Shared& sh) {
    constexpr int E = Geo<DT>::E;
    const uint32_t tid = threadIdx.x;
    float bv = NEG_INF;
    uint32_t bi = 0xffffffffu;
    for (uint32_t c0 = g.cb; c0 < g.ce; c0 += NT * UNROLL) {
        // Unconditional loads (chunks past the slice's end read its last chunk; `inside`
        // below discards them): a load that may be skipped is waited for as the last one issued.
        u32x4 raw[UNROLL];
        for (int u = 0; u < UNROLL; ++u) {
            const uint32_t c = min(c0 + u * NT + tid, g.ce - 1u);
            raw[u] = gload(reinterpret_cast<const u32x4*>(g.base + (size_t)c * 16));
        }
        for (int u = 0; u < UNROLL; ++u) {
            const uint32_t c = c0 + u * NT + tid;
            float v[E];
            unpack<DT>(raw[u], v);
            for (int j = 0; j < E; ++j) {
                const uint32_t id = g.id_of(c, j);
                const bool inside = c >= g.main_lo && c < g.main_hi;
                const float x = v[j];
                if (inside && (x > bv || (x == bv && id < bi))) {
                    bv = x;
                    bi = id;
                }
            }
        }
    }
    for (int side = 0; side < 2; ++side) {
        const uint32_t lo = side == 0 ? g.id_lo : g.edge_hi_begin;
        const uint32_t hi = side == 0 ? g.edge_lo_end : g.id_hi;
        for (uint32_t id = lo + tid; id < hi; id += NT) {
            const float x = load_logit<DT>(a.logits, id);
            if (x > bv || (x == bv && id < bi)) {
                bv = x;
                bi = id;
            }
        }
    }
    uint64_t best = ((uint64_t)lilym_order_key(bv + 0.0f) << 32) | (uint32_t)(~bi);
    best = wave_max_u64(best);
    if ((tid & 63u) == 0) {
        sh.red_u[tid >> 6] = best;
    }
    __syncthreads();
    best = sh.red_u[0];
    for (int i = 1; i < NWAVE; ++i) {
        best = sh.red_u[i] > best ? sh.red_u[i] : best;
    }
    __syncthreads();
    return best;
}

// ------------------------------------------------------------------ the row kernel

template <int DT, int KIND, bool LSE>
__device__ __forceinline__ void row_body(const RowArgs& a, const LaunchCfg& cfg, Shared& sh) {
    // KIND: 0 = rows without masks, penalties or bias lists, 1 = rows with any of them (the
    // bitmap select is compiled for them), 2 = streaming rows only (no bitmap select at all).
    constexpr bool EXCL = KIND == 1;
    const uint32_t tid = threadIdx.x;
    const uint32_t s = blockIdx.x, row = blockIdx.y, S = cfg.slices;
    const uint32_t vocab = cfg.vocab;
    const uint32_t step = a.step + cfg.step_delta;
    const bool want_lse = LSE && a.out_logprob != nullptr;
    uint64_t* cand = dyn_lds;
    uint64_t* found = cand;  // where the select left the slice's candidates
    uint32_t* excl = reinterpret_cast<uint32_t*>(dyn_lds + cfg.cand_cap);

    if ((a.flags & F_FORCED) && !want_lse) {
        if (s == 0 && tid == 0) {
            emit(a, a.forced);
        }
        return;
    }

    Geo<DT> g;
    g.init(a.logits, vocab, s, S);
    phase(cfg, 0);

    const bool argmax = a.mode == MODE_ARGMAX;
    uint64_t best = 0;
    bool sorted = false;
    if (argmax) {
        best = slice_argmax<DT>(a, g, sh);
    } else {
        // A forced row with a log-probability needs the row sum only: it takes the same
        // selects (their sums are the fast ones) and its candidates are dropped below.
        bool done = false;
        uint32_t took = 2;
        if (cfg.path == 0u && (a.flags & F_STREAM)) {
            done = select_stream<DT, LSE, KIND != 2>(a, g, a.k, sh, cfg, sorted, found);
            took = done ? 0u : took;
            if (!done) {
                __syncthreads();
            }
        }
        if (KIND == 1 && !done && cfg.path == 0u && a.allow != nullptr) {
            done = select_sparse<DT, LSE>(a, g, a.k, cand, min(cfg.dyn_slots, MERGE_CAP), sh, sorted);
            took = done ? 1u : took;
        }
        if (KIND != 2 && !done && cfg.path != 1u && cfg.old_layout != 0u) {
            const bool special = a.allow != nullptr || (a.flags & F_PEN) || a.n_bias != 0;
            if (EXCL || !special) {
                // A single pass whose running bound let too many candidates in is repeated
                // as two passes (bound first, then collect) before the exhaustive select.
#pragma nounroll
                for (int attempt = 0; attempt < 2 && !done; ++attempt) {
                    const bool two_pass = a.k > 64u || cfg.path == 2u || attempt == 1;
                    if (attempt == 1) {
                        __syncthreads();
                    }
                    done = select_fast<DT, EXCL, LSE>(a, g, a.k, two_pass, cand, cfg.cand_cap, excl, sh,
                                                      cfg, sorted);
                    if (a.k > 64u || cfg.path == 2u) {
                        break;  // it was two passes already
                    }
                }
                took = done ? 1u : took;
            }
        }
        if (cfg.path_stats != nullptr && tid == 0) {
            atomicAdd(&cfg.path_stats[took], 1u);
        }
        if (!done) {
            __syncthreads();
            sorted = false;
            select_exhaustive<DT>(a, g.id_lo, g.id_hi, a.k, want_lse, cand, cfg.cand_cap, sh);
        }
    }

    const bool forced = (a.flags & F_FORCED) != 0;
    uint32_t n = (argmax || forced) ? 0u : min(sh.n_cand, cfg.cand_cap);
    phase(cfg, 4);
    if (S > 1) {
        const size_t slot = (size_t)row * S + s;
        // Partials go through to memory (no dirty L2 lines to write back), the wave waits
        // for its stores, the workgroup meets, and one thread takes the row's ticket.
        if (argmax) {
            if (tid == 0) {
                store_through(&cfg.ws_cand[slot * cfg.ws_k], best);
            }
        } else {
            // Every slot is written (0 = no candidate), so the merge needs no counts.
            for (uint32_t i = tid; !forced && i < cfg.ws_k; i += NT) {
                store_through(&cfg.ws_cand[slot * cfg.ws_k + i], i < n ? found[i] : (uint64_t)0);
            }
            if (tid == 0) {
                store_through(&cfg.ws_lse[2 * slot], want_lse ? sh.lse_mc : 0.0);
                store_through(&cfg.ws_lse[2 * slot + 1], want_lse ? sh.lse_s : 0.0);
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            const uint32_t t = __hip_atomic_fetch_add(&cfg.ws_ticket[row], 1u, __ATOMIC_RELAXED,
                                                      __HIP_MEMORY_SCOPE_AGENT);
            sh.last = (t == S - 1) ? 1u : 0u;
        }
        __syncthreads();
        phase(cfg, 5);
        if (sh.last == 0u) {
            return;
        }
        if (tid == 0) {
            store_through(&cfg.ws_ticket[row], 0u);
        }
        const size_t base = (size_t)row * S;
        if (argmax) {
            best = 0;
            for (uint32_t t = tid; t < S; t += NT) {
                const uint64_t c = load_through(&cfg.ws_cand[(base + t) * cfg.ws_k]);
                best = c > best ? c : best;
            }
            best = wave_max_u64(best);
            if ((tid & 63u) == 0) {
                sh.red_u[tid >> 6] = best;
            }
            __syncthreads();
            best = sh.red_u[0];
            for (int i = 1; i < NWAVE; ++i) {
                best = sh.red_u[i] > best ? sh.red_u[i] : best;
            }
        } else {
            // Gather every slice's candidates (0 = no candidate) and the log-sum-exp partials
            // in one round trip.
            constexpr int PER = MERGE_CAP / NT;
            const uint32_t slots = S * cfg.ws_k;
            uint64_t mine[PER];
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                const uint32_t j = tid + (uint32_t)q * NT;
                mine[q] = (!forced && j < slots) ? load_through(&cfg.ws_cand[base * cfg.ws_k + j]) : 0ull;
            }
            if (want_lse && tid < 64) {
                double mt = -__builtin_huge_val(), st = 0.0;
                if (tid < S) {
                    mt = load_through(&cfg.ws_lse[2 * (base + tid)]);
                    st = load_through(&cfg.ws_lse[2 * (base + tid) + 1]);
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
            // A bound of the k-th largest from the lanes' best entries (as in the streaming
            // select: each wave's ceil(k / NWAVE)-th largest lane maximum, the minimum over the
            // waves), then only entries at or above it are ranked.
            uint64_t best_mine = 0;
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                best_mine = mine[q] > best_mine ? mine[q] : best_mine;
            }
            const uint32_t kw = (a.k + NWAVE - 1) / NWAVE;
            const uint32_t P = kw <= 64u ? wave_kth_key16((uint32_t)(best_mine >> 48), kw) : 0u;
            if ((tid & 63u) == 0) {
                sh.red_i[tid >> 6] = P;
            }
            if (tid == 0) {
                sh.n_cand = 0;
            }
            __syncthreads();
            uint32_t bound = sh.red_i[0];
            for (int i = 1; i < NWAVE; ++i) {
                bound = min(bound, sh.red_i[i]);
            }
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                if (mine[q] != 0ull && (uint32_t)(mine[q] >> 48) >= bound) {
                    cand[atomicAdd(&sh.n_cand, 1u)] = mine[q];
                }
            }
            __syncthreads();
            n = sh.n_cand;
            sorted = false;
            n = select_topk(cand, n, a.k, sh, sorted);
            found = cand;
        }
    }

    phase(cfg, 6);
    if (argmax) {
        if (tid == 0) {
            const uint32_t id = composite_id(best);
            *a.out_id = id == 0xffffffffu ? 0u : id;
        }
        return;
    }
    if (a.flags & F_FORCED) {
        if (tid == 0) {
            finish_token<DT>(a, sh, a.forced, vocab);
        }
        return;
    }
    tail<DT, KIND != 2>(a, vocab, step, n, sorted, found, sh, cfg);
    phase(cfg, 7);
}

// Dynamic LDS: [0, cand_cap) candidates while scanning, then the bitmap.  In the tail the
// first K_CAP slots hold the sorted candidates and the three float arrays follow them
// (the launcher sizes the region for at least K_CAP * 8 + 3 * K_CAP * 4 bytes).
__device__ __forceinline__ void tail_arrays(Shared& sh) {
    float* f = reinterpret_cast<float*>(dyn_lds + K_CAP);
    sh.prob = f;
    sh.cum = f + K_CAP;
    sh.res = f + 2 * K_CAP;
}

// The row's arguments are the same for every thread: read through the constant address
// space they arrive by scalar loads and stay in scalar registers.
__device__ __forceinline__ void load_row_args(RowArgs& a, const LILY_CONST RowArgs* src) {
    static_assert(sizeof(RowArgs) % 16 == 0, "RowArgs is copied in 16-byte pieces");
    const LILY_CONST u32x4* from = (const LILY_CONST u32x4*)src;
    u32x4* to = reinterpret_cast<u32x4*>(&a);
    for (unsigned i = 0; i < sizeof(RowArgs) / 16; ++i) {
        to[i] = from[i];
    }
}

template <int DT, int KIND, bool LSE>
__global__ __launch_bounds__(NT, KIND == 1 ? 3 : 4) void k_rows_inline(InlineRows rows, LaunchCfg cfg) {
    __shared__ Shared sh;
    // `rows` is the first kernel argument: index it in the kernel-argument segment itself
    // (indexing the by-value copy would move all of it to scratch memory).
    const LILY_CONST RowArgs* table =
        (const LILY_CONST RowArgs*)__builtin_amdgcn_kernarg_segment_ptr();
    RowArgs a;
    load_row_args(a, table + blockIdx.y);
    if (threadIdx.x == 0) {
        tail_arrays(sh);
    }
    __syncthreads();
    row_body<DT, KIND, LSE>(a, cfg, sh);
}

template <int DT, int KIND, bool LSE>
__global__ __launch_bounds__(NT, KIND == 1 ? 3 : 4) void k_rows_table(LaunchCfg cfg) {
    __shared__ Shared sh;
    const LILY_CONST RowArgs* table = (const LILY_CONST RowArgs*)cfg.table;
    RowArgs a;
    load_row_args(a, table + blockIdx.y);
    if (threadIdx.x == 0) {
        tail_arrays(sh);
    }
    __syncthreads();
    row_body<DT, KIND, LSE>(a, cfg, sh);
}

// ------------------------------------------------------------------ small kernels

__global__ void k_fill_u32(uint32_t* p, uint32_t n, uint32_t v) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

// counts[id] += 1 per occurrence; ids counted for the first time join the list (their
// count is filled in by k_refresh_pairs once every occurrence has been added).
__global__ void k_add_history(ScratchView sc, const uint32_t* ids, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const uint32_t id = ids[i];
        if (id < sc.vocab) {
            atomicAdd(&sc.counts[id], 1u);
            const uint32_t bit = 1u << (id & 31u);
            const uint32_t bits = atomicOr(&sc.touched[id >> 5], bit);
            if ((bits & bit) == 0u) {
                const uint32_t p = atomicAdd(sc.n_pairs, 1u);
                if (p < sc.pairs_cap) {
                    sc.pairs[p].id = id;
                }
                sc.pos[id] = p < sc.pairs_cap ? p : 0xffffffffu;
            }
        }
    }
}

// pairs[p].count = counts[pairs[p].id] for every listed id.
__global__ void k_refresh_pairs(ScratchView sc) {
    const uint32_t p = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t n = min(*sc.n_pairs, sc.pairs_cap);
    if (p < n) {
        sc.pairs[p].count = sc.counts[sc.pairs[p].id];
    }
}

// Saturating decrement; the id stays listed (with a count that may now be 0).
__device__ __forceinline__ void uncount_one(const ScratchView& sc, uint32_t token) {
    if (token >= sc.vocab) {
        return;
    }
    const uint32_t c = sc.counts[token];
    if (c > 0u) {
        sc.counts[token] = c - 1u;
        const uint32_t p = sc.pos[token];
        if (((sc.touched[token >> 5] >> (token & 31u)) & 1u) && p < sc.pairs_cap) {
            sc.pairs[p].count = c - 1u;
        }
    }
}

__global__ void k_uncount(ScratchView sc, uint32_t token) {
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        uncount_one(sc, token);
    }
}

// The rollback of the rejected rows' draws (src/qwen4exp/spec.rs:213-217) with the accepted
// row read on the device: draws[a + 1 .. m) are un-counted in order, a = min(accepted[0], cap).
__global__ void k_uncount_after(ScratchView sc, const uint32_t* draws, uint32_t m,
                                const uint32_t* accepted, uint32_t cap) {
    if (blockIdx.x != 0 || threadIdx.x != 0) {
        return;
    }
    const uint32_t a = min(accepted[0], cap);
    if (a >= m) {
        return;
    }
    for (uint32_t j = a + 1u; j < m; ++j) {
        uncount_one(sc, draws[j]);
    }
}

// After counts were written whole: touched[w] = bits of the non-zero counts in word w, and
// the list is rebuilt from them (n_pairs was cleared before the launch).
__global__ void k_rebuild_listed(ScratchView sc) {
    const uint32_t w = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t words = (sc.vocab + 31u) / 32u;
    if (w < words) {
        uint32_t bits = 0;
        for (uint32_t b = 0; b < 32u; ++b) {
            const uint32_t id = w * 32u + b;
            if (id < sc.vocab && sc.counts[id] != 0u) {
                bits |= 1u << b;
                const uint32_t p = atomicAdd(sc.n_pairs, 1u);
                if (p < sc.pairs_cap) {
                    sc.pairs[p].id = id;
                    sc.pairs[p].count = sc.counts[id];
                }
                sc.pos[id] = p < sc.pairs_cap ? p : 0xffffffffu;
            }
        }
        sc.touched[w] = bits;
    }
}

// spec.metal:14-38
__global__ void k_spec_accept(const uint32_t* draws, const uint32_t* ids, uint32_t* ctrl,
                              uint32_t m, uint32_t pos0, uint32_t ratio, uint32_t chain,
                              uint32_t stride) {
    if (blockIdx.x != 0 || threadIdx.x != 0) {
        return;
    }
    uint32_t a = 0;
    while (a + 1 < m && draws[a] == ids[a + 1]) {
        ++a;
    }
    ctrl[0] = a;
    ctrl[stride] = a + 1;
    for (uint32_t i = 0; i < chain; ++i) {
        const uint32_t p = pos0 + a + 1 + i;
        ctrl[(2 + 3 * i) * stride] = p;
        ctrl[(3 + 3 * i) * stride] = p / ratio;
        ctrl[(4 + 3 * i) * stride] = ((p + 1) % ratio == 0) ? 1u : 0u;
    }
}

// spec.metal:42-52
__global__ void k_copy_row_u32(const uint32_t* src, uint32_t* dst, uint32_t words, uint32_t rows,
                               const uint32_t* row_dev) {
    const uint32_t row = *row_dev;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows || i >= words) {
        return;
    }
    dst[i] = src[(size_t)row * words + i];
}

// ------------------------------------------------------------------ launchers (host)

template <int DT, int KIND, bool LSE>
static hipError_t launch_variant(hipStream_t stream, uint32_t rows, const LaunchCfg& cfg,
                                 const InlineRows* inline_rows, size_t dyn_bytes) {
    const dim3 grid(cfg.slices, rows), block(NT);
    if (inline_rows != nullptr) {
        hipLaunchKernelGGL((k_rows_inline<DT, KIND, LSE>), grid, block, dyn_bytes, stream,
                           *inline_rows, cfg);
    } else {
        hipLaunchKernelGGL((k_rows_table<DT, KIND, LSE>), grid, block, dyn_bytes, stream, cfg);
    }
    return hipGetLastError();
}

hipError_t launch_rows(hipStream_t stream, int dtype, int kind, bool lse, uint32_t rows,
                       const LaunchCfg& cfg_in, const InlineRows* inline_rows, size_t dyn_bytes) {
    LaunchCfg cfg = cfg_in;
    cfg.dyn_slots = (uint32_t)(dyn_bytes / 8);
#ifdef LILY_ONE_VARIANT
    // For looking at one kernel's generated code (seconds instead of minutes): only the
    // bf16 streaming kernels with a row sum are instantiated.  Never defined in a build that runs.
    (void)dtype;
    (void)kind;
    (void)lse;
    return launch_variant<LILY_BF16, 2, true>(stream, rows, cfg, inline_rows, dyn_bytes);
#else
#define LILY_DISPATCH(DT)                                                                     \
    switch (kind) {                                                                           \
        case 0:                                                                               \
            return lse ? launch_variant<DT, 0, true>(stream, rows, cfg, inline_rows, dyn_bytes)  \
                       : launch_variant<DT, 0, false>(stream, rows, cfg, inline_rows, dyn_bytes); \
        case 1:                                                                               \
            return lse ? launch_variant<DT, 1, true>(stream, rows, cfg, inline_rows, dyn_bytes)  \
                       : launch_variant<DT, 1, false>(stream, rows, cfg, inline_rows, dyn_bytes); \
        default:                                                                              \
            return lse ? launch_variant<DT, 2, true>(stream, rows, cfg, inline_rows, dyn_bytes)  \
                       : launch_variant<DT, 2, false>(stream, rows, cfg, inline_rows, dyn_bytes); \
    }
    if (dtype == LILY_BF16) {
        LILY_DISPATCH(LILY_BF16)
    }
    LILY_DISPATCH(LILY_F32)
#undef LILY_DISPATCH
#endif
}

hipError_t launch_fill_u32(hipStream_t stream, uint32_t* p, uint32_t n, uint32_t v) {
    if (n == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(k_fill_u32, dim3((n + 255) / 256), dim3(256), 0, stream, p, n, v);
    return hipGetLastError();
}

hipError_t launch_add_history(hipStream_t stream, const ScratchView& sc, const uint32_t* ids,
                              uint32_t n) {
    if (n == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(k_add_history, dim3((n + 255) / 256), dim3(256), 0, stream, sc, ids, n);
    hipLaunchKernelGGL(k_refresh_pairs, dim3((sc.pairs_cap + 255) / 256), dim3(256), 0, stream, sc);
    return hipGetLastError();
}

hipError_t launch_uncount(hipStream_t stream, const ScratchView& sc, uint32_t token) {
    hipLaunchKernelGGL(k_uncount, dim3(1), dim3(64), 0, stream, sc, token);
    return hipGetLastError();
}

hipError_t launch_uncount_after(hipStream_t stream, const ScratchView& sc, const uint32_t* draws,
                                uint32_t m, const uint32_t* accepted, uint32_t cap) {
    hipLaunchKernelGGL(k_uncount_after, dim3(1), dim3(64), 0, stream, sc, draws, m, accepted, cap);
    return hipGetLastError();
}

hipError_t launch_rebuild_listed(hipStream_t stream, const ScratchView& sc) {
    const uint32_t words = (sc.vocab + 31u) / 32u;
    hipLaunchKernelGGL(k_fill_u32, dim3(1), dim3(256), 0, stream, sc.n_pairs, 1u, 0u);
    hipLaunchKernelGGL(k_rebuild_listed, dim3((words + 255) / 256), dim3(256), 0, stream, sc);
    return hipGetLastError();
}

hipError_t launch_spec_accept(hipStream_t stream, const uint32_t* draws, const uint32_t* ids,
                              uint32_t* ctrl, uint32_t m, uint32_t pos0, uint32_t ratio,
                              uint32_t chain) {
    hipLaunchKernelGGL(k_spec_accept, dim3(1), dim3(64), 0, stream, draws, ids, ctrl, m, pos0, ratio,
                       chain, LILY_CTRL_STRIDE);
    return hipGetLastError();
}

hipError_t launch_copy_row(hipStream_t stream, const uint32_t* src, uint32_t* dst, uint32_t words,
                           uint32_t rows, const uint32_t* row_dev) {
    hipLaunchKernelGGL(k_copy_row_u32, dim3((words + 255) / 256), dim3(256), 0, stream, src, dst,
                       words, rows, row_dev);
    return hipGetLastError();
}

}  // namespace lily
