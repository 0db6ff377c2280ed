// sampler_kernels.hip - gfx950 kernels of the logits-to-token stage.
//
// One launch serves a batch of logits rows.  Row r is scanned by `slices`
// workgroups (grid = slices x rows); each finds the exact top-k of its slice
// as 64-bit composites (order key of the adjusted value << 32 | ~id, so a
// greater composite is a better candidate and the lowest id wins a tie).  With
// several slices the last workgroup to arrive (an atomic ticket, nobody waits)
// merges them.  That workgroup then runs the tail: sort, softmax over the
// candidates, the sequential top-p / min-p prefix, the draw, and for the
// speculative modes the export or the accept / residual draw.
//
// Arithmetic that decides a token id follows tests/unit/kernels/sample.rs:8-54
// of the reference operation for operation (IEEE division by the temperature,
// left-to-right f32 sums, lilym_expf); see include/lily_sampler_math.h.
#include <hip/hip_runtime.h>

#include "../../include/lily_sampler_math.h"
#include "row_args.h"

namespace lily {

constexpr int NT = 512;
constexpr int NWAVE = NT / 64;
constexpr uint32_t K_CAP = LILY_SAMPLE_K_CAP;
constexpr float LOG2E = 1.4426950408889634f;

#define NEG_INF (-__builtin_huge_valf())

// ------------------------------------------------------------------ small helpers

template <int DT>
__device__ __forceinline__ float load_logit(const void* p, uint32_t i) {
    if (DT == LILY_BF16) {
        return lilym_bits_f32((uint32_t) static_cast<const uint16_t*>(p)[i] << 16);
    }
    return static_cast<const float*>(p)[i];
}

__device__ __forceinline__ bool bit_of(const uint32_t* words, uint32_t id) {
    return (words[id >> 5] >> (id & 31u)) & 1u;
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

// The value before the temperature, exactly as the oracle's map: bias (list
// order), mask, penalties.
template <int DT>
__device__ float pre_temperature_of(const RowArgs& a, uint32_t id) {
    float l = load_logit<DT>(a.logits, id);
    for (uint32_t j = 0; j < a.n_bias; ++j) {
        const lily_bias b = a.bias[j];
        if (b.id == id) {
            l += b.delta;
        }
    }
    if (a.allow != nullptr && !bit_of(a.allow, id)) {
        return NEG_INF;
    }
    if ((a.flags & F_PEN) && bit_of(a.touched, id)) {
        const uint32_t c = a.counts[id];
        if (c > 0u) {
            l = l > 0.0f ? l / a.repetition : l * a.repetition;
            l -= a.presence + a.frequency * (float)c;
        }
    }
    return l;
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
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
    for (int o = 32; o > 0; o >>= 1) {
        const uint64_t w = __shfl_xor((unsigned long long)v, o);
        v = w > v ? w : v;
    }
    return v;
}

// ------------------------------------------------------------------ shared memory

struct Shared {
    uint64_t cand[CAND_CAP];   // candidates / sort area
    float prob[K_CAP];         // exp(adjusted - top) per sorted candidate
    float cum[K_CAP];          // inclusive prefix of the kept ones
    float res[K_CAP];          // residual of the speculative draw
    uint32_t hist[256];
    double red_d[NWAVE];
    float red_f[NWAVE];
    uint64_t red_u[NWAVE];
    uint64_t prefix;
    uint32_t n_cand;
    uint32_t need;
    uint32_t sel_bin;
    uint32_t all_taken;
    uint32_t n_keep;
    uint32_t pick;
    uint32_t last;
    float mass;
    float p_d;
    float q_d;
    float lse_m;               // row maximum of the adjusted values (log2 domain reference)
    double lse_s;              // sum of exp2((adjusted - lse_m) * log2e)
};

// Running (maximum, sum of 2^((x - maximum) * log2e)) of one thread.
struct Lse {
    float m;
    float s;
    __device__ void init() {
        m = NEG_INF;
        s = 0.0f;
    }
    __device__ void add(float adj) {
        if (!(adj > NEG_INF)) {
            return;
        }
        if (adj > m) {
            s = s * exp2f((m - adj) * LOG2E);
            m = adj;
        }
        s += exp2f((adj - m) * LOG2E);
    }
};

// Workgroup-wide merge of the threads' Lse into sh.lse_m / sh.lse_s.
__device__ void lse_reduce(Shared& sh, const Lse& l) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    float m = wave_max_f(l.m);
    if (lane == 0) {
        sh.red_f[w] = m;
    }
    __syncthreads();
    m = sh.red_f[0];
    for (int i = 1; i < NWAVE; ++i) {
        m = fmaxf(m, sh.red_f[i]);
    }
    double s = 0.0;
    if (l.m > NEG_INF) {
        s = (double)l.s * exp2((double)(l.m - m) * (double)LOG2E);
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
        sh.lse_m = m;
        sh.lse_s = t;
    }
    __syncthreads();
}

// ------------------------------------------------------------------ exhaustive select
//
// The exact top-k of elements [e0, e1) by a radix select on the composite:
// eight passes of 8 bits, each re-evaluating every element.  Slow and correct
// for any input (ties, masks, few finite values); the other paths fall back to
// it.  Leaves the winners (unsorted) in sh.cand[0 .. sh.n_cand).
template <int DT>
__device__ void select_exhaustive(const RowArgs& a, uint32_t e0, uint32_t e1, uint32_t k,
                                  bool want_lse, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    uint64_t prefix = 0, pmask = 0;
    uint32_t need = k;
    Lse lse;
    lse.init();
    bool take_all = false;
    for (int pass = 0; pass < 8 && !take_all; ++pass) {
        const int shift = 56 - 8 * pass;
        if (tid < 256) {
            sh.hist[tid] = 0;
        }
        __syncthreads();
        for (uint32_t id = e0 + tid; id < e1; id += NT) {
            const float adj = adjusted_of<DT>(a, id);
            if (pass == 0 && want_lse) {
                lse.add(adj);
            }
            const uint64_t c = composite_of(adj, id);
            if (c != 0 && (c & pmask) == prefix) {
                atomicAdd(&sh.hist[(uint32_t)(c >> shift) & 255u], 1u);
            }
        }
        __syncthreads();
        if (tid == 0) {
            uint32_t seen = 0, bin = 0;
            bool found = false;
            for (int b = 255; b >= 0; --b) {
                const uint32_t h = sh.hist[b];
                if (seen + h >= need) {
                    bin = (uint32_t)b;
                    found = true;
                    break;
                }
                seen += h;
            }
            // Fewer valid elements than asked for (only possible on the first
            // pass, where every valid element is counted): take them all.
            sh.all_taken = found ? 0u : 1u;
            sh.sel_bin = bin;
            sh.need = found ? need - seen : 0u;
        }
        __syncthreads();
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
            if (at < CAND_CAP) {
                sh.cand[at] = c;
            }
        }
    }
    __syncthreads();
}

// ------------------------------------------------------------------ sort

// Bitonic sort, descending, of sh.cand[0..n) padded with zeros to a power of two.
__device__ void sort_desc(Shared& sh, uint32_t n) {
    uint32_t p = 2;
    while (p < n) {
        p <<= 1;
    }
    for (uint32_t i = n + threadIdx.x; i < p; i += NT) {
        sh.cand[i] = 0;
    }
    __syncthreads();
    for (uint32_t size = 2; size <= p; size <<= 1) {
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
            for (uint32_t i = threadIdx.x; i < (p >> 1); i += NT) {
                const uint32_t pos = ((i / stride) * (stride << 1)) + (i % stride);
                const uint32_t partner = pos + stride;
                const bool desc = (pos & size) == 0;
                const uint64_t x = sh.cand[pos], y = sh.cand[partner];
                if (desc ? x < y : x > y) {
                    sh.cand[pos] = y;
                    sh.cand[partner] = x;
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

template <int DT>
__device__ void write_logprob(const RowArgs& a, const Shared& sh, uint32_t id, uint32_t vocab) {
    if (a.out_logprob == nullptr) {
        return;
    }
    float lp = NEG_INF;
    if (id < vocab) {
        const float adj = adjusted_of<DT>(a, id);
        if (adj > NEG_INF) {
            const double lse = (double)sh.lse_m + log(sh.lse_s);
            lp = (float)((double)adj - lse);
        }
    }
    *a.out_logprob = lp;
}

// sh.cand[0..n) holds the row's candidates (at least its top-k); finishes the row.
template <int DT>
__device__ void tail(const RowArgs& a, uint32_t vocab, uint32_t step, uint32_t n, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    if (n == 0) {
        // No finite value anywhere: the oracle's order then starts at id 0.
        if (tid == 0) {
            emit(a, 0);
            if (a.out_logprob) {
                *a.out_logprob = NEG_INF;
            }
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
    sort_desc(sh, n);
    const uint32_t k = min(a.k, n);
    const float top = composite_value(sh.cand[0]);
    for (uint32_t i = tid; i < k; i += NT) {
        const float p = lilym_expf(composite_value(sh.cand[i]) - top);
        sh.prob[i] = p;
        if (a.dbg_ids) {
            a.dbg_ids[i] = composite_id(sh.cand[i]);
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
            a.q_ids[i] = composite_id(sh.cand[i]);
            a.q_probs[i] = sh.prob[i] / mass;
        }
        if (tid == 0) {
            *a.q_n = n_keep;
        }
    }

    if (a.mode != MODE_SPEC) {
        if (tid == 0) {
            const uint32_t slot = pick_sequential(sh.cum, n_keep, u1 * mass);
            const uint32_t id = composite_id(sh.cand[slot]);
            write_logprob<DT>(a, sh, id, vocab);  // before the id is counted
            emit(a, id);
        }
        return;
    }

    // Speculative draw (sample.metal:596-658, cpu_spec at tests/unit/kernels/sample.rs:264-283).
    const uint32_t d = *a.draft;
    const uint32_t qn = min(*a.q_n, K_CAP);
    for (uint32_t i = tid; i < n_keep; i += NT) {
        if (composite_id(sh.cand[i]) == d) {
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
        const uint32_t id = composite_id(sh.cand[i]);
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
        const uint32_t id = composite_id(sh.cand[slot]);
        write_logprob<DT>(a, sh, id, vocab);
        emit(a, id);
    }
}

// ------------------------------------------------------------------ argmax

// First maximum under float comparison (NaN never wins, -0 == +0), lowest id on
// ties: elementwise.metal:145-150.  Result: the best composite of [e0, e1).
template <int DT>
__device__ uint64_t slice_argmax(const RowArgs& a, uint32_t e0, uint32_t e1, Shared& sh) {
    uint64_t best = 0;
    for (uint32_t id = e0 + threadIdx.x; id < e1; id += NT) {
        float v = load_logit<DT>(a.logits, id);
        uint64_t c;
        if (v != v) {
            c = (uint64_t)(uint32_t)(~id);  // below every number, lowest id first
        } else {
            v = v + 0.0f;  // -0 -> +0
            c = ((uint64_t)lilym_order_key(v) << 32) | (uint32_t)(~id);
        }
        best = c > best ? c : best;
    }
    best = wave_max_u64(best);
    if ((threadIdx.x & 63) == 0) {
        sh.red_u[threadIdx.x >> 6] = best;
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

template <int DT>
__device__ void row_body(const RowArgs& a, const LaunchCfg& cfg, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    const uint32_t s = blockIdx.x, row = blockIdx.y, S = cfg.slices;
    const uint32_t vocab = cfg.vocab;
    const uint32_t step = a.step + cfg.step_delta;
    const bool want_lse = a.out_logprob != nullptr;

    if ((a.flags & F_FORCED) && !want_lse) {
        if (s == 0 && tid == 0) {
            emit(a, a.forced);
        }
        return;
    }

    // Slice bounds in elements: equal slices, a multiple of 2048 long.
    uint32_t len = (vocab + S - 1) / S;
    len = (len + 2047u) & ~2047u;
    const uint32_t e0 = min(s * len, vocab);
    const uint32_t e1 = min(e0 + len, vocab);

    const bool argmax = a.mode == MODE_ARGMAX;
    uint64_t best = 0;
    if (argmax) {
        best = slice_argmax<DT>(a, e0, e1, sh);
    } else if (a.flags & F_FORCED) {
        // Only the row's log-sum-exp is needed.
        Lse lse;
        lse.init();
        for (uint32_t id = e0 + tid; id < e1; id += NT) {
            lse.add(adjusted_of<DT>(a, id));
        }
        lse_reduce(sh, lse);
        if (tid == 0) {
            sh.n_cand = 0;
        }
        __syncthreads();
    } else {
        select_exhaustive<DT>(a, e0, e1, a.k, want_lse, sh);
    }

    uint32_t n = argmax ? 0u : min(sh.n_cand, CAND_CAP);
    if (S > 1) {
        const size_t slot = (size_t)row * S + s;
        if (argmax) {
            if (tid == 0) {
                cfg.ws_cand[slot * cfg.ws_k] = best;
            }
        } else {
            for (uint32_t i = tid; i < n; i += NT) {
                cfg.ws_cand[slot * cfg.ws_k + i] = sh.cand[i];
            }
            if (tid == 0) {
                cfg.ws_n[slot] = n;
                cfg.ws_lse[2 * slot] = sh.lse_m;
                cfg.ws_lse[2 * slot + 1] = (float)sh.lse_s;
            }
        }
        __threadfence();
        __syncthreads();
        if (tid == 0) {
            const uint32_t t = __hip_atomic_fetch_add(&cfg.ws_ticket[row], 1u, __ATOMIC_ACQ_REL,
                                                      __HIP_MEMORY_SCOPE_AGENT);
            sh.last = (t == S - 1) ? 1u : 0u;
        }
        __syncthreads();
        if (sh.last == 0u) {
            return;
        }
        __threadfence();
        if (tid == 0) {
            cfg.ws_ticket[row] = 0;
        }
        const size_t base = (size_t)row * S;
        if (argmax) {
            best = 0;
            for (uint32_t t = tid; t < S; t += NT) {
                const uint64_t c = __builtin_nontemporal_load(&cfg.ws_cand[(base + t) * cfg.ws_k]);
                best = c > best ? c : best;
            }
            best = wave_max_u64(best);
            if ((tid & 63) == 0) {
                sh.red_u[tid >> 6] = best;
            }
            __syncthreads();
            best = sh.red_u[0];
            for (int i = 1; i < NWAVE; ++i) {
                best = sh.red_u[i] > best ? sh.red_u[i] : best;
            }
        } else {
            // Gather every slice's candidates; merge the log-sum-exp partials.
            uint32_t total = 0;
            for (uint32_t t = 0; t < S; ++t) {
                const uint32_t nt = __builtin_nontemporal_load(&cfg.ws_n[base + t]);
                for (uint32_t i = tid; i < nt; i += NT) {
                    sh.cand[total + i] =
                        __builtin_nontemporal_load(&cfg.ws_cand[(base + t) * cfg.ws_k + i]);
                }
                total += nt;
            }
            n = total;
            if (want_lse && tid == 0) {
                float m = NEG_INF;
                for (uint32_t t = 0; t < S; ++t) {
                    m = fmaxf(m, __builtin_nontemporal_load(&cfg.ws_lse[2 * (base + t)]));
                }
                double sum = 0.0;
                for (uint32_t t = 0; t < S; ++t) {
                    const float mt = __builtin_nontemporal_load(&cfg.ws_lse[2 * (base + t)]);
                    const float st = __builtin_nontemporal_load(&cfg.ws_lse[2 * (base + t) + 1]);
                    if (mt > NEG_INF) {
                        sum += (double)st * exp2((double)(mt - m) * (double)LOG2E);
                    }
                }
                sh.lse_m = m;
                sh.lse_s = sum;
            }
            __syncthreads();
        }
    }

    if (argmax) {
        if (tid == 0) {
            *a.out_id = composite_id(best);
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
    tail<DT>(a, vocab, step, n, sh);
}

template <int DT>
__global__ __launch_bounds__(NT) void k_rows_inline(InlineRows rows, LaunchCfg cfg) {
    __shared__ Shared sh;
    row_body<DT>(rows.r[blockIdx.y], cfg, sh);
}

template <int DT>
__global__ __launch_bounds__(NT) void k_rows_table(LaunchCfg cfg) {
    __shared__ Shared sh;
    __shared__ RowArgs a;
    // One coalesced copy of the row's arguments into LDS.
    if (threadIdx.x < sizeof(RowArgs) / 4) {
        reinterpret_cast<uint32_t*>(&a)[threadIdx.x] =
            reinterpret_cast<const uint32_t*>(&cfg.table[blockIdx.y])[threadIdx.x];
    }
    __syncthreads();
    row_body<DT>(a, cfg, sh);
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

hipError_t launch_rows(hipStream_t stream, int dtype, uint32_t rows, const LaunchCfg& cfg,
                       const InlineRows* inline_rows) {
    const dim3 grid(cfg.slices, rows), block(NT);
    if (inline_rows != nullptr) {
        if (dtype == LILY_BF16) {
            hipLaunchKernelGGL(k_rows_inline<LILY_BF16>, grid, block, 0, stream, *inline_rows, cfg);
        } else {
            hipLaunchKernelGGL(k_rows_inline<LILY_F32>, grid, block, 0, stream, *inline_rows, cfg);
        }
    } else {
        if (dtype == LILY_BF16) {
            hipLaunchKernelGGL(k_rows_table<LILY_BF16>, grid, block, 0, stream, cfg);
        } else {
            hipLaunchKernelGGL(k_rows_table<LILY_F32>, grid, block, 0, stream, cfg);
        }
    }
    return hipGetLastError();
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
