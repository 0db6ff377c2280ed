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

constexpr int NT = 512;
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
__device__ float pre_temperature_of(const RowArgs& a, uint32_t id) {
    float l = load_logit<DT>(a.logits, id);
    const uint32_t c = (a.flags & F_PEN) ? gload(a.counts + id) : 0u;
    const bool allowed = a.allow == nullptr || bit_of(a.allow, id);
    return finish_pre_temperature(a, id, l, c, allowed);
}

template <int DT>
__device__ __forceinline__ float adjusted_of(const RowArgs& a, uint32_t id) {
    return pre_temperature_of<DT>(a, id) / a.temperature;
}

__device__ __forceinline__ float wave_max_f(float v) {
    for (int o = 32; o > 0; o >>= 1) {
        v = fmaxf(v, __shfl_xor(v, o));
    }
    return v;
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
__device__ void lse_reduce(Shared& sh, const LseAcc& l) {
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
__device__ void find_bin(Shared& sh, uint32_t need) {
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
__device__ uint32_t wg_select_topk(uint64_t* cand, uint32_t n, uint32_t k, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    uint64_t prefix = 0, pmask = 0;
    uint32_t need = k;
    bool all = false;
    for (int pass = 0; pass < 8; ++pass) {
        const int shift = 56 - 8 * pass;
        if (tid < 256) {
            sh.hist[tid] = 0;
        }
        __syncthreads();
        for (uint32_t i = tid; i < n; i += NT) {
            const uint64_t c = cand[i];
            if (c != 0 && (c & pmask) == prefix) {
                atomicAdd(&sh.hist[(uint32_t)(c >> shift) & 255u], 1u);
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
        need = sh.need;
        if (whole_bin) {
            break;
        }
    }
    const uint64_t floor_c = all ? 1ull : prefix;
    uint64_t mine[8];
    for (int j = 0; j < 8; ++j) {
        const uint32_t i = tid + (uint32_t)j * NT;
        mine[j] = i < n ? cand[i] : 0ull;
    }
    if (tid == 0) {
        sh.n_cand = 0;
    }
    __syncthreads();
    for (int j = 0; j < 8; ++j) {
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
__device__ uint32_t wg_rank_select(uint64_t* cand, uint32_t n, uint32_t k, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    const uint64_t mine = tid < n ? cand[tid] : 0ull;
    uint32_t rank = 0;
    for (uint32_t j = 0; j < n; ++j) {
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
__device__ uint32_t select_topk(uint64_t* cand, uint32_t n, uint32_t k, Shared& sh, bool& sorted) {
    if (n <= 256u) {
        sorted = true;
        return wg_rank_select(cand, n, k, sh);
    }
    sorted = false;
    return wg_select_topk(cand, n, k, sh);
}

// The k-th largest of the workgroup's NT x 8 per-lane values (-inf = absent) by a
// radix select on their order keys; F32_LOWEST when fewer than k are present.
__device__ float wg_kth_largest(const float (&ms)[8], uint32_t k, Shared& sh) {
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
    }

    // Chunk c as floats; positions outside the row or the slice read as -inf.
    __device__ __forceinline__ void load(const void* logits, uint32_t c, float (&v)[E]) const {
        if (c >= full_lo && c < full_hi && c < ce) {
            const u32x4 q = gload(reinterpret_cast<const u32x4*>(base + (size_t)c * 16));
            if (DT == LILY_BF16) {
                v[0] = lilym_bits_f32(q.x << 16);
                v[1] = lilym_bits_f32(q.x & 0xffff0000u);
                v[2] = lilym_bits_f32(q.y << 16);
                v[3] = lilym_bits_f32(q.y & 0xffff0000u);
                v[4 % E] = lilym_bits_f32(q.z << 16);
                v[5 % E] = lilym_bits_f32(q.z & 0xffff0000u);
                v[6 % E] = lilym_bits_f32(q.w << 16);
                v[7 % E] = lilym_bits_f32(q.w & 0xffff0000u);
            } else {
                v[0] = lilym_bits_f32(q.x);
                v[1] = lilym_bits_f32(q.y);
                v[2] = lilym_bits_f32(q.z);
                v[3] = lilym_bits_f32(q.w);
            }
        } else {
            for (int j = 0; j < E; ++j) {
                const int64_t id = (int64_t)c * E - pad + j;
                v[j] = (c < ce && id >= 0 && id < (int64_t)vocab)
                           ? load_logit<DT>(logits, (uint32_t)id)
                           : NEG_INF;
            }
        }
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
    }
}


// Appends the lanes with `pass` set to the candidate buffer (wave-aggregated).
__device__ __forceinline__ void append(bool pass, float v, uint32_t id, uint64_t* cand,
                                       uint32_t cap, Shared& sh) {
    const uint64_t mask = __ballot(pass);
    if (mask == 0) {
        return;
    }
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t rank =
        __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
    const int leader = __builtin_ctzll(mask);
    uint32_t base = 0;
    if ((int)lane == leader) {
        base = atomicAdd(&sh.n_cand, (uint32_t)__popcll(mask));
    }
    base = __shfl(base, leader);
    if (pass) {
        const uint32_t at = base + rank;
        if (at < cap) {
            cand[at] = ((uint64_t)lilym_order_key(v) << 32) | (uint32_t)(~id);
        }
    }
}

// The exact top-k of the slice in cand[0..n) as adjusted-value composites,
// unsorted, n returned through sh.n_cand; false when the slice must be redone
// exhaustively.  Also leaves the slice's log-sum-exp in sh when LSE.
template <int DT, bool EXCL, bool LSE>
__device__ bool select_fast(const RowArgs& a, const Geo<DT>& g, uint32_t k, bool two_pass,
                            uint64_t* cand, uint32_t cap, uint32_t* excl, Shared& sh,
                            const LaunchCfg& cfg, bool& sorted) {
    constexpr int E = Geo<DT>::E;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    const uint32_t nchunks = g.ce - g.cb;
    const uint32_t nwords = (nchunks * E + 31u) / 32u;
    const uint32_t row_words = (g.vocab + 31u) / 32u;
    const float c2 = a.c2;

    if (tid == 0) {
        sh.n_cand = 0;
    }
    if (tid < NWAVE) {
        sh.wthr[tid] = NEG_INF;
        sh.wthr_f[tid] = F32_LOWEST;
    }
    if (EXCL) {
        // Bit b of the slice bitmap <-> id cb*E - pad + b.  Set = not streamed.
        for (uint32_t i0 = tid; i0 < nwords; i0 += 4 * NT) {
            uint32_t x[4];
            for (int q = 0; q < 4; ++q) {  // four words' loads in flight before any store
                const uint32_t i = i0 + (uint32_t)q * NT;
                const int64_t id0 = (int64_t)g.cb * E - g.pad + (int64_t)i * 32;
                x[q] = ~range32_at(g.id_lo, g.id_hi, id0);
                if (i < nwords) {
                    if (a.allow != nullptr) {
                        x[q] |= ~bits32_at(a.allow, row_words, id0);
                    }
                    if (a.flags & F_PEN) {
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
    LseAcc lse;
    lse.init();
    float thr_f = F32_LOWEST;
    const uint8_t* excl_bytes = reinterpret_cast<const uint8_t*>(excl);

    for (int pass = 0; pass < (two_pass ? 2 : 1); ++pass) {
        const bool filter = !two_pass || pass == 1;
        for (uint32_t c0 = g.cb; c0 < g.ce; c0 += NT * UNROLL) {
            float v[UNROLL][E];
            for (int u = 0; u < UNROLL; ++u) {
                g.load(a.logits, c0 + u * NT + tid, v[u]);
            }
            if (EXCL) {
                for (int u = 0; u < UNROLL; ++u) {
                    const uint32_t c = c0 + u * NT + tid;
                    if (c < g.ce) {
                        const uint32_t rel = c - g.cb;
                        uint32_t m;
                        if (E == 8) {
                            m = excl_bytes[rel];
                        } else {
                            m = (excl_bytes[rel >> 1] >> ((rel & 1u) * 4u)) & 15u;
                        }
                        for (int j = 0; j < E; ++j) {
                            // all-ones when bit j is set: the element reads as -inf
                            const uint32_t on = (uint32_t)((int32_t)(m << (31 - j)) >> 31);
                            v[u][j] = lilym_bits_f32((lilym_f32_bits(v[u][j]) & ~on) | (0xff800000u & on));
                        }
                    }
                }
            }
            if (pass == 0) {
                float cm = NEG_INF;
                for (int u = 0; u < UNROLL; ++u) {
                    for (int j = 0; j < E; ++j) {
                        cm = fmaxf(cm, v[u][j]);
                        if (two_pass) {
                            const int slot = (E == 8) ? j : ((u & 1) * 4 + j);
                            ms[slot] = fmaxf(ms[slot], v[u][j]);
                        }
                    }
                }
                lane_max = fmaxf(lane_max, cm);
                if (LSE) {
                    const float safe = lse.rebase(cm, c2);
                    for (int u = 0; u < UNROLL; ++u) {
                        for (int j = 0; j < E; ++j) {
                            lse.term(v[u][j], c2, safe);
                        }
                    }
                }
                if (!two_pass) {
                    // Lower bound of the k-th largest: min over groups of the group maximum.
                    float t = lane_max;
                    for (uint32_t o = 1; o < group; o <<= 1) {
                        t = fmaxf(t, __shfl_xor(t, (int)o));
                    }
                    for (uint32_t o = group; o < 64; o <<= 1) {
                        t = fminf(t, __shfl_xor(t, (int)o));
                    }
                    if (lane == 0) {
                        __hip_atomic_store(&sh.wthr[w], t, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
                    if (c0 == g.cb) {
                        __syncthreads();  // every wave has published its first statistic
                    }
                    for (int i = 0; i < NWAVE; ++i) {
                        // Other waves' values may be older: still lower bounds.
                        t = fminf(t, __hip_atomic_load(&sh.wthr[i], __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_WORKGROUP));
                    }
                    thr_f = fmaxf(thr_f, lower_by_slack(t));
                }
            }
            if (filter) {
                for (int u = 0; u < UNROLL; ++u) {
                    const uint32_t c = c0 + u * NT + tid;
                    for (int j = 0; j < E; ++j) {
                        append(v[u][j] >= thr_f, v[u][j], g.id_of(c, j), cand, cap, sh);
                    }
                }
            }
        }
        if (two_pass && pass == 0) {
            thr_f = lower_by_slack(wg_kth_largest(ms, k, sh));
        }
    }
    if (lane == 0) {
        sh.wthr_f[w] = thr_f;
    }
    __syncthreads();
    phase(cfg, 2);
    float filt = sh.wthr_f[0];
    for (int i = 1; i < NWAVE; ++i) {
        filt = fmaxf(filt, sh.wthr_f[i]);
    }
    uint32_t n = sh.n_cand;
    if (n > cap) {
        return false;
    }
    // Buffered composites hold the pre-temperature value: divide now, exactly.
    for (uint32_t i = tid; i < n; i += NT) {
        const uint64_t c = cand[i];
        cand[i] = composite_of(composite_value(c) / a.temperature, composite_id(c));
    }
    if (EXCL) {
        // Specials: ids kept out of the stream that are allowed (penalised or biased).
        // Their ids are compacted into an LDS list, then the workgroup walks the list four
        // ids per thread at a time, so the gathers of a batch (logit, count) are
        // independent loads and the work is balanced.
        const bool pen = (a.flags & F_PEN) != 0;
        const int64_t slice_id0 = (int64_t)g.cb * E - g.pad;
        auto special_bits = [&](uint32_t i) -> uint32_t {
            const int64_t id0 = slice_id0 + (int64_t)i * 32;
            uint32_t b = excl[i] & range32_at(g.id_lo, g.id_hi, id0);
            if (a.allow != nullptr) {
                b &= bits32_at(a.allow, row_words, id0);
            }
            return b;
        };
        auto process = [&](uint32_t id, float l, uint32_t cnt) {
            const float u = finish_pre_temperature(a, id, l, cnt, true);
            if (LSE) {
                lse.add_one(u, c2);
            }
            if (u >= filt) {
                const uint32_t at = atomicAdd(&sh.n_cand, 1u);
                if (at < cap) {
                    cand[at] = composite_of(u / a.temperature, id);
                }
            }
        };
        if (tid == 0) {
            sh.need = 0;
        }
        __syncthreads();
        uint32_t* list = excl + cfg.excl_words;  // SPECIAL_LIST_CAP ids behind the bitmap
        const uint32_t list_cap = SPECIAL_LIST_CAP;
        for (uint32_t i0 = 0; i0 < nwords; i0 += NT) {
            const uint32_t i = i0 + tid;
            uint32_t bits = i < nwords ? special_bits(i) : 0u;
            while (__ballot(bits != 0u) != 0ull) {
                const bool has = bits != 0u;
                const uint32_t id = has ? (uint32_t)(slice_id0 + (int64_t)i * 32 + __builtin_ctz(bits)) : 0u;
                bits &= bits - 1u;
                const uint64_t mask = __ballot(has);
                const uint32_t rank = __builtin_amdgcn_mbcnt_hi(
                    (uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
                const int leader = __builtin_ctzll(mask);
                uint32_t base = 0;
                if ((int)lane == leader) {
                    base = atomicAdd(&sh.need, (uint32_t)__popcll(mask));
                }
                base = __shfl(base, leader);
                if (has) {
                    if (base + rank < list_cap) {
                        list[base + rank] = id;
                    } else {  // more specials than the list holds: one at a time
                        process(id, load_logit<DT>(a.logits, id), pen ? gload(a.counts + id) : 0u);
                    }
                }
            }
        }
        __syncthreads();
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
                    process(ids[q], l[q], cnt[q]);
                }
            }
        }
    }
    if (LSE) {
        lse_reduce(sh, lse);
    } else {
        __syncthreads();
    }
    n = sh.n_cand;
    phase(cfg, 3);
    if (n > cap) {
        return false;
    }
    sorted = false;
    if (n > k) {
        n = select_topk(cand, n, k, sh, sorted);
    }
    // Every element that was not collected lies strictly below `filt`; it must also
    // lie strictly below the k-th adjusted value, or the division has merged it
    // into the boundary's tie class.
    if (filt > F32_LOWEST && n > 0) {
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
        if (!(lilym_order_key(below) < lowest)) {
            return false;
        }
    }
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
__device__ void select_exhaustive(const RowArgs& a, uint32_t e0, uint32_t e1, uint32_t k,
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

// Descending sort of cand[0..n).  Up to 64 entries: one wave, in registers.
// More: bitonic in LDS over the next power of two (the buffer holds it).
__device__ void sort_desc(uint64_t* cand, uint32_t n) {
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

__device__ __forceinline__ void emit(const RowArgs& a, uint32_t id) {
    *a.out_id = id;
    if (a.flags & F_PEN) {
        atomicAdd(&a.counts[id], 1u);
        atomicOr(&a.touched[id >> 5], 1u << (id & 31u));
    }
}

// First slot of prefix[0..n) whose value exceeds target, else the last slot.
__device__ uint32_t pick_sequential(const float* prefix, uint32_t n, float target) {
    for (uint32_t i = 0; i < n; ++i) {
        if (target < prefix[i]) {
            return i;
        }
    }
    return n - 1;
}

// log p(id) = (u*c2 - mc - log2 s) * ln 2, with the id's exponent u*c2 formed exactly as
// the row sum formed its terms, so the two cancel when the id carries all the mass.
template <int DT>
__device__ void write_logprob(const RowArgs& a, const Shared& sh, uint32_t id, uint32_t vocab) {
    if (a.out_logprob == nullptr) {
        return;
    }
    float lp = NEG_INF;
    if (id < vocab) {
        const float u = pre_temperature_of<DT>(a, id);
        if (u > NEG_INF) {
            const double e = (double)u * (double)a.c2 - sh.lse_mc - log2(sh.lse_s);
            lp = fminf((float)(e * 0.6931471805599453), 0.0f);  // the sum is approximate: clamp
        }
    }
    *a.out_logprob = lp;
}

// cand[0..n) holds the row's candidates (at least its top-k); finishes the row.
template <int DT>
__device__ void tail(const RowArgs& a, uint32_t vocab, uint32_t step, uint32_t n, bool sorted,
                     uint64_t* cand, Shared& sh) {
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
                a.dbg_counts[1] = 0;
            }
            if (a.mode == MODE_DRAFT) {
                *a.q_n = 0;
            }
        }
        return;
    }
    if (!sorted) {
        sort_desc(cand, n);
    }
    const uint32_t k = min(a.k, n);
    const float top = composite_value(cand[0]);
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
    if (tid == 0) {
        float total = 0.0f;
        for (uint32_t i = 0; i < k; ++i) {
            total += sh.prob[i];
        }
        const float limit = a.top_p * total;
        float cum = 0.0f;
        uint32_t kept = 0;
        for (uint32_t rank = 0; rank < k; ++rank) {
            const float p = sh.prob[rank];
            if (rank > 0 && !(cum < limit && p >= a.min_p)) {
                break;
            }
            cum += p;
            sh.cum[rank] = cum;
            ++kept;
        }
        sh.n_keep = kept;
        sh.mass = cum;
        sh.p_d = 0.0f;
        sh.q_d = 0.0f;
        if (a.dbg_counts) {
            a.dbg_counts[0] = k;
            a.dbg_counts[1] = kept;
        }
    }
    __syncthreads();
    const uint32_t n_keep = sh.n_keep;
    const float mass = sh.mass;
    const float u1 = (a.flags & F_UNIFORM) ? a.uniform : lilym_uniform_for(a.seed, step);

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
        if (tid == 0) {
            const uint32_t slot = pick_sequential(sh.cum, n_keep, u1 * mass);
            const uint32_t id = composite_id(cand[slot]);
            write_logprob<DT>(a, sh, id, vocab);  // before the id is counted
            emit(a, id);
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
            write_logprob<DT>(a, sh, d, vocab);
            emit(a, d);
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
        write_logprob<DT>(a, sh, id, vocab);
        emit(a, id);
    }
}

// ------------------------------------------------------------------ argmax

// First maximum under float comparison (NaN never wins, -0 == +0), lowest id on
// ties: elementwise.metal:145-150.  Result: the best (value, id) of the slice as a
// composite; id bits all zero when no element qualified.
template <int DT>
__device__ uint64_t slice_argmax(const RowArgs& a, const Geo<DT>& g, Shared& sh) {
    constexpr int E = Geo<DT>::E;
    const uint32_t tid = threadIdx.x;
    float bv = NEG_INF;
    uint32_t bi = 0xffffffffu;
    for (uint32_t c0 = g.cb; c0 < g.ce; c0 += NT * UNROLL) {
        float v[UNROLL][E];
        for (int u = 0; u < UNROLL; ++u) {
            g.load(a.logits, c0 + u * NT + tid, v[u]);
        }
        for (int u = 0; u < UNROLL; ++u) {
            const uint32_t c = c0 + u * NT + tid;
            for (int j = 0; j < E; ++j) {
                const uint32_t id = g.id_of(c, j);
                const bool inside = c < g.ce && id < g.vocab;  // id wraps for the pad
                const float x = v[u][j];
                if (inside && (x > bv || (x == bv && id < bi))) {
                    bv = x;
                    bi = id;
                }
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

template <int DT, bool EXCL, bool LSE>
__device__ void row_body(const RowArgs& a, const LaunchCfg& cfg, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    const uint32_t s = blockIdx.x, row = blockIdx.y, S = cfg.slices;
    const uint32_t vocab = cfg.vocab;
    const uint32_t step = a.step + cfg.step_delta;
    const bool want_lse = LSE && a.out_logprob != nullptr;
    uint64_t* cand = dyn_lds;
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
    } else if (a.flags & F_FORCED) {
        // Only the row's log-sum-exp is needed.
        LseAcc lse;
        lse.init();
        for (uint32_t id = g.id_lo + tid; id < g.id_hi; id += NT) {
            lse.add_one(pre_temperature_of<DT>(a, id), a.c2);
        }
        lse_reduce(sh, lse);
        if (tid == 0) {
            sh.n_cand = 0;
        }
        __syncthreads();
    } else {
        bool done = false;
        if (cfg.path != 1u) {
            const bool special = a.allow != nullptr || (a.flags & F_PEN) || a.n_bias != 0;
            if (EXCL || !special) {
                const bool two_pass = a.k > 64u || cfg.path == 2u;
                done = select_fast<DT, EXCL, LSE>(a, g, a.k, two_pass, cand, cfg.cand_cap, excl, sh, cfg,
                                                  sorted);
            }
        }
        if (!done) {
            __syncthreads();
            sorted = false;
            select_exhaustive<DT>(a, g.id_lo, g.id_hi, a.k, want_lse, cand, cfg.cand_cap, sh);
        }
    }

    uint32_t n = argmax ? 0u : min(sh.n_cand, cfg.cand_cap);
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
            for (uint32_t i = tid; i < n; i += NT) {
                store_through(&cfg.ws_cand[slot * cfg.ws_k + i], cand[i]);
            }
            if (tid == 0) {
                store_through(&cfg.ws_n[slot], n);
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
            // Gather every slice's candidates (absent slots read as 0 = invalid) and merge
            // the log-sum-exp partials, all slices at once.
            if (tid < S) {
                sh.hist[tid] = load_through(&cfg.ws_n[base + tid]);
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
            __syncthreads();
            const uint32_t slots = S * cfg.ws_k;
            for (uint32_t j = tid; j < slots; j += NT) {
                const uint32_t t = j / cfg.ws_k, i = j - t * cfg.ws_k;
                cand[j] = i < sh.hist[t] ? load_through(&cfg.ws_cand[(base + t) * cfg.ws_k + i]) : 0ull;
            }
            __syncthreads();
            n = slots;
            sorted = false;
            n = select_topk(cand, n, a.k, sh, sorted);
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
            write_logprob<DT>(a, sh, a.forced, vocab);
            emit(a, a.forced);
        }
        return;
    }
    tail<DT>(a, vocab, step, n, sorted, cand, sh);
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

template <int DT, bool EXCL, bool LSE>
__global__ __launch_bounds__(NT) void k_rows_inline(InlineRows rows, LaunchCfg cfg) {
    __shared__ Shared sh;
    __shared__ RowArgs a;
    // The row's arguments from the kernel-argument segment into LDS (a dynamic index into
    // the by-value array would copy all of it to scratch memory).
    for (int r = 0; r < INLINE_ROWS; ++r) {
        if (r == (int)blockIdx.y && threadIdx.x < sizeof(RowArgs) / 4) {
            reinterpret_cast<uint32_t*>(&a)[threadIdx.x] =
                reinterpret_cast<const uint32_t*>(&rows.r[r])[threadIdx.x];
        }
    }
    if (threadIdx.x == 0) {
        tail_arrays(sh);
    }
    __syncthreads();
    row_body<DT, EXCL, LSE>(a, cfg, sh);
}

template <int DT, bool EXCL, bool LSE>
__global__ __launch_bounds__(NT) void k_rows_table(LaunchCfg cfg) {
    __shared__ Shared sh;
    __shared__ RowArgs a;
    // One coalesced copy of the row's arguments into LDS.
    if (threadIdx.x < sizeof(RowArgs) / 4) {
        reinterpret_cast<uint32_t*>(&a)[threadIdx.x] =
            gload(reinterpret_cast<const uint32_t*>(&cfg.table[blockIdx.y]) + threadIdx.x);
    }
    if (threadIdx.x == 0) {
        tail_arrays(sh);
    }
    __syncthreads();
    row_body<DT, EXCL, LSE>(a, cfg, sh);
}

// ------------------------------------------------------------------ small kernels

__global__ void k_fill_u32(uint32_t* p, uint32_t n, uint32_t v) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

__global__ void k_add_history(uint32_t* counts, uint32_t* touched, uint32_t vocab,
                              const uint32_t* ids, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const uint32_t id = ids[i];
        if (id < vocab) {
            atomicAdd(&counts[id], 1u);
            atomicOr(&touched[id >> 5], 1u << (id & 31u));
        }
    }
}

__global__ void k_uncount(uint32_t* counts, uint32_t* touched, uint32_t vocab, uint32_t token) {
    if (blockIdx.x == 0 && threadIdx.x == 0 && token < vocab) {
        const uint32_t c = counts[token];
        if (c > 0u) {
            counts[token] = c - 1u;
            if (c == 1u) {
                touched[token >> 5] &= ~(1u << (token & 31u));
            }
        }
    }
}

// touched[w] = bits of the non-zero counts in word w (after counts were written whole).
__global__ void k_rebuild_touched(const uint32_t* counts, uint32_t* touched, uint32_t vocab) {
    const uint32_t w = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t words = (vocab + 31u) / 32u;
    if (w < words) {
        uint32_t bits = 0;
        for (uint32_t b = 0; b < 32u; ++b) {
            const uint32_t id = w * 32u + b;
            if (id < vocab && counts[id] != 0u) {
                bits |= 1u << b;
            }
        }
        touched[w] = bits;
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

template <int DT, bool EXCL, bool LSE>
static hipError_t launch_variant(hipStream_t stream, uint32_t rows, const LaunchCfg& cfg,
                                 const InlineRows* inline_rows, size_t dyn_bytes) {
    const dim3 grid(cfg.slices, rows), block(NT);
    if (inline_rows != nullptr) {
        hipLaunchKernelGGL((k_rows_inline<DT, EXCL, LSE>), grid, block, dyn_bytes, stream,
                           *inline_rows, cfg);
    } else {
        hipLaunchKernelGGL((k_rows_table<DT, EXCL, LSE>), grid, block, dyn_bytes, stream, cfg);
    }
    return hipGetLastError();
}

hipError_t launch_rows(hipStream_t stream, int dtype, bool excl, bool lse, uint32_t rows,
                       const LaunchCfg& cfg, const InlineRows* inline_rows, size_t dyn_bytes) {
#define LILY_DISPATCH(DT)                                                                      \
    if (excl) {                                                                                \
        return lse ? launch_variant<DT, true, true>(stream, rows, cfg, inline_rows, dyn_bytes)  \
                   : launch_variant<DT, true, false>(stream, rows, cfg, inline_rows, dyn_bytes); \
    }                                                                                          \
    return lse ? launch_variant<DT, false, true>(stream, rows, cfg, inline_rows, dyn_bytes)     \
               : launch_variant<DT, false, false>(stream, rows, cfg, inline_rows, dyn_bytes);
    if (dtype == LILY_BF16) {
        LILY_DISPATCH(LILY_BF16)
    }
    LILY_DISPATCH(LILY_F32)
#undef LILY_DISPATCH
}

hipError_t launch_fill_u32(hipStream_t stream, uint32_t* p, uint32_t n, uint32_t v) {
    if (n == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(k_fill_u32, dim3((n + 255) / 256), dim3(256), 0, stream, p, n, v);
    return hipGetLastError();
}

hipError_t launch_add_history(hipStream_t stream, uint32_t* counts, uint32_t* touched,
                              uint32_t vocab, const uint32_t* ids, uint32_t n) {
    if (n == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(k_add_history, dim3((n + 255) / 256), dim3(256), 0, stream, counts, touched,
                       vocab, ids, n);
    return hipGetLastError();
}

hipError_t launch_uncount(hipStream_t stream, uint32_t* counts, uint32_t* touched, uint32_t vocab,
                          uint32_t token) {
    hipLaunchKernelGGL(k_uncount, dim3(1), dim3(64), 0, stream, counts, touched, vocab, token);
    return hipGetLastError();
}

hipError_t launch_rebuild_touched(hipStream_t stream, const uint32_t* counts, uint32_t* touched,
                                  uint32_t vocab) {
    const uint32_t words = (vocab + 31u) / 32u;
    hipLaunchKernelGGL(k_rebuild_touched, dim3((words + 255) / 256), dim3(256), 0, stream, counts,
                       touched, vocab);
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
