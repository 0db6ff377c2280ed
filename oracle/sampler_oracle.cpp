// sampler_oracle.cpp - CPU restatement of the reference's sampler.
//
// TEST INFRASTRUCTURE ONLY.  Nothing in the product (the HIP library, its host
// mirror) may include, link or call this file; it is the checker that tests/,
// __graft_entry__.smoke() and bench.py's cpu_baseline leg run next to the GPU.
//
// Every function restates one piece of the reference (paths relative to the
// reference checkout):
//   lo_uniform_for      src/kernels/sample.rs:435-441
//   lo_is_greedy ...    src/kernels/sample.rs:47-95 (is_greedy, uses_penalties,
//                       validate, effective), :238-240 (samples)
//   lo_argmax_f32       src/kernels/metal/elementwise.metal:145-150 (argmax_merge)
//                       folded left to right as tests/unit/kernels/elementwise.rs:73-84
//   lo_sample           tests/unit/kernels/sample.rs:8-54 (cpu_sample)
//   lo_kept             tests/unit/kernels/sample.rs:251-260 (cpu_kept)
//   lo_spec             tests/unit/kernels/sample.rs:264-283 (cpu_spec)
//   lo_spec_accept      src/kernels/metal/spec.metal:14-38
//   lo_uncount          src/kernels/sample.rs:147-157
//   lo_host_accept      src/qwen4exp/spec.rs:194-199 (leading draw == draft count)
//
// What the reference does not have and this file defines (the GPU path follows
// the same definitions; the reference cannot pin them, closed forms and brute
// force in tests/ do): bf16 input (exact widening), a logit-bias list applied
// first in list order, an allow-bitmask that turns cleared ids into -inf, a
// forced token, an explicit uniform, and the chosen token's log-probability
// over the whole adjusted row in f64.
//
// Two exp() variants: EXP_LILY is lilym_expf from include/lily_sampler_math.h
// (bit-identical on the GPU), EXP_LIBM is the C library's expf, standing in
// for the reference's platform libm (f32::exp).
//
// Parity status of the restated functions: every function above is pinned by
// the reference's literal known-answer tests and by closed forms in
// tests/test_oracle_*.py.  The extension semantics are "parity unpinned" by
// the reference (it has no such feature); they are pinned by closed forms only.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <numeric>
#include <thread>
#include <vector>

#include "../include/lily_sampler_math.h"

extern "C" {

struct lo_params {
    float temperature;
    uint32_t top_k;
    float top_p;
    float min_p;
    float presence_penalty;
    float frequency_penalty;
    float repetition_penalty;
    uint32_t reserved;
    uint64_t seed;
};

struct lo_bias {
    uint32_t id;
    float delta;
};

enum { LO_F32 = 0, LO_BF16 = 1 };
enum { LO_EXP_LILY = 0, LO_EXP_LIBM = 1 };
enum { LO_SORT_PARTIAL = 0, LO_SORT_FULL = 1 };
enum { LO_K_CAP = 1024 };

// Extensions and options of one draw; zero-initialised means "reference behaviour".
struct lo_ext {
    const uint32_t* allow;   // packed bits, ceil(V/32) words, or null
    const lo_bias* bias;     // n_bias pairs or null
    uint32_t n_bias;
    uint32_t has_uniform;    // use `uniform` instead of uniform_for(seed, step)
    float uniform;
    uint32_t has_forced;     // emit `forced`, consume no draw
    uint32_t forced;
    uint32_t exp_mode;       // LO_EXP_*
    uint32_t sort_mode;      // LO_SORT_*
    uint32_t want_logprob;
};

struct lo_result {
    uint32_t chosen;
    uint32_t n_cand;
    uint32_t n_kept;
    float top;        // adjusted value of the best candidate
    float total;      // sum of candidate probabilities (unnormalised)
    float mass;       // cumulative probability of the last kept candidate
    float target;     // u * mass
    float uniform;    // the u that was used
    float gap;        // min_i |target - cum_i| / mass: distance to the nearest boundary
    uint32_t reserved;
    double logprob;   // chosen token, over the full adjusted row
};

float lo_uniform_for(uint64_t seed, uint32_t step) { return lilym_uniform_for(seed, step); }
uint32_t lo_draft_step(uint32_t step) { return lilym_draft_step(step); }
float lo_expf(float x) { return lilym_expf(x); }

int lo_is_greedy(const lo_params* p) { return p->temperature <= 0.0f || p->top_k == 1; }

int lo_uses_penalties(const lo_params* p) {
    return p->presence_penalty != 0.0f || p->frequency_penalty != 0.0f ||
           p->repetition_penalty != 1.0f;
}

int lo_samples(const lo_params* p) { return !lo_is_greedy(p) || lo_uses_penalties(p); }

// 0 when valid, else the number of the first failed rule (1..5).
int lo_validate(const lo_params* p) {
    if (!(std::isfinite(p->temperature) && p->temperature >= 0.0f)) return 1;
    if (!(std::isfinite(p->top_p) && p->top_p > 0.0f && p->top_p <= 1.0f)) return 2;
    if (!(std::isfinite(p->min_p) && p->min_p >= 0.0f && p->min_p <= 1.0f)) return 3;
    if (!(std::isfinite(p->repetition_penalty) && p->repetition_penalty > 0.0f)) return 4;
    if (!(std::isfinite(p->presence_penalty) && std::isfinite(p->frequency_penalty))) return 5;
    return 0;
}

void lo_effective(const lo_params* p, float* temperature, uint32_t* k) {
    if (lo_is_greedy(p)) {
        *temperature = 1.0f;
        *k = 1;
    } else {
        *temperature = p->temperature;
        *k = p->top_k == 0 ? (uint32_t)LO_K_CAP : std::min<uint32_t>(p->top_k, LO_K_CAP);
    }
}

void lo_draft_params(const lo_params* p, lo_params* out) {
    *out = *p;
    out->presence_penalty = 0.0f;
    out->frequency_penalty = 0.0f;
    out->repetition_penalty = 1.0f;
}

static inline float load_logit(const void* logits, int dtype, size_t i) {
    if (dtype == LO_BF16) {
        return lilym_bf16_to_f32(static_cast<const uint16_t*>(logits)[i]);
    }
    return static_cast<const float*>(logits)[i];
}

uint32_t lo_argmax(const void* x, int dtype, size_t n) {
    float bv = -std::numeric_limits<float>::infinity();
    uint32_t bi = 0;
    for (size_t i = 0; i < n; ++i) {
        const float v = load_logit(x, dtype, i);
        if (v > bv || (v == bv && (uint32_t)i < bi)) {
            bv = v;
            bi = (uint32_t)i;
        }
    }
    return bi;
}

// The adjusted logits of cpu_sample's first map, with the extensions in front.
void lo_adjust(const void* logits, int dtype, size_t v, const uint32_t* counts,
               const lo_params* p, const lo_ext* ext, float* adjusted) {
    float temperature;
    uint32_t k;
    lo_effective(p, &temperature, &k);
    const bool pen = lo_uses_penalties(p) && counts != nullptr;
    for (size_t i = 0; i < v; ++i) {
        adjusted[i] = load_logit(logits, dtype, i);
    }
    if (ext && ext->bias) {
        for (uint32_t j = 0; j < ext->n_bias; ++j) {
            if (ext->bias[j].id < v) {
                adjusted[ext->bias[j].id] += ext->bias[j].delta;
            }
        }
    }
    if (ext && ext->allow) {
        for (size_t i = 0; i < v; ++i) {
            if (!((ext->allow[i >> 5] >> (i & 31)) & 1u)) {
                adjusted[i] = -std::numeric_limits<float>::infinity();
            }
        }
    }
    for (size_t i = 0; i < v; ++i) {
        float l = adjusted[i];
        if (pen && counts[i] > 0) {
            l = l > 0.0f ? l / p->repetition_penalty : l * p->repetition_penalty;
            l -= p->presence_penalty + p->frequency_penalty * (float)counts[i];
        }
        adjusted[i] = l / temperature;
    }
}

static double full_row_logprob(const float* adjusted, size_t v, uint32_t id) {
    double m = -std::numeric_limits<double>::infinity();
    for (size_t i = 0; i < v; ++i) m = std::max(m, (double)adjusted[i]);
    double s = 0.0;
    for (size_t i = 0; i < v; ++i) s += std::exp((double)adjusted[i] - m);
    return (double)adjusted[id] - m - std::log(s);
}

// cpu_sample.  Outputs (any may be null): cand_ids/cand_adj/cand_prob hold the
// n_cand best candidates in order; kept_cum the inclusive prefix sums of the
// kept ones.  If `counts` is given and penalties are on, the emitted id is
// counted, as the kernel does (sample.metal:508-511).
int lo_sample(const void* logits, int dtype, size_t v, uint32_t* counts, const lo_params* p,
              uint32_t step, const lo_ext* ext, lo_result* res, uint32_t* cand_ids,
              float* cand_adj, float* cand_prob, float* kept_cum) {
    if (v == 0) return -1;
    float temperature;
    uint32_t k;
    lo_effective(p, &temperature, &k);
    std::vector<float> adjusted(v);
    lo_adjust(logits, dtype, v, counts, p, ext, adjusted.data());

    const size_t n = std::min<size_t>(k, v);
    std::vector<uint32_t> order(v);
    std::iota(order.begin(), order.end(), 0u);
    auto before = [&](uint32_t a, uint32_t b) {
        const uint32_t ka = lilym_order_key(adjusted[a]);
        const uint32_t kb = lilym_order_key(adjusted[b]);
        return ka != kb ? ka > kb : a < b;
    };
    if (ext && ext->sort_mode == LO_SORT_FULL) {
        std::sort(order.begin(), order.end(), before);
    } else {
        std::partial_sort(order.begin(), order.begin() + n, order.end(), before);
    }
    const bool libm = ext && ext->exp_mode == LO_EXP_LIBM;
    const float top = adjusted[order[0]];
    std::vector<float> probs(n);
    for (size_t i = 0; i < n; ++i) {
        const float d = adjusted[order[i]] - top;
        probs[i] = libm ? std::exp(d) : lilym_expf(d);
    }
    float total = 0.0f;
    for (size_t i = 0; i < n; ++i) total += probs[i];
    std::vector<float> cums;
    float cum = 0.0f;
    for (size_t rank = 0; rank < n; ++rank) {
        if (rank > 0 && !(cum < p->top_p * total && probs[rank] >= p->min_p)) break;
        cum += probs[rank];
        cums.push_back(cum);
    }
    const float mass = cums.back();
    const float u = (ext && ext->has_uniform) ? ext->uniform : lilym_uniform_for(p->seed, step);
    const float target = u * mass;
    uint32_t chosen = order[cums.size() - 1];
    for (size_t i = 0; i < cums.size(); ++i) {
        if (target < cums[i]) {
            chosen = order[i];
            break;
        }
    }
    float gap = std::numeric_limits<float>::infinity();
    for (size_t i = 0; i + 1 < cums.size(); ++i) {
        gap = std::min(gap, std::fabs(target - cums[i]) / mass);
    }
    if (ext && ext->has_forced) chosen = ext->forced;

    if (res) {
        res->chosen = chosen;
        res->n_cand = (uint32_t)n;
        res->n_kept = (uint32_t)cums.size();
        res->top = top;
        res->total = total;
        res->mass = mass;
        res->target = target;
        res->uniform = u;
        res->gap = gap;
        res->reserved = 0;
        res->logprob = (ext && ext->want_logprob && chosen < v)
                           ? full_row_logprob(adjusted.data(), v, chosen)
                           : 0.0;
    }
    for (size_t i = 0; i < n; ++i) {
        if (cand_ids) cand_ids[i] = order[i];
        if (cand_adj) cand_adj[i] = adjusted[order[i]];
        if (cand_prob) cand_prob[i] = probs[i];
    }
    if (kept_cum) std::copy(cums.begin(), cums.end(), kept_cum);
    if (counts && lo_uses_penalties(p) && chosen < v) counts[chosen] += 1;
    return 0;
}

// cpu_kept: the kept candidates of a draw with no penalty counts at step 0,
// probabilities recomputed from the raw logits and normalised over the kept
// mass.  Returns the kept count.
uint32_t lo_kept(const void* logits, int dtype, size_t v, const lo_params* p, uint32_t exp_mode,
                 uint32_t* ids, float* probs) {
    lo_ext ext;
    std::memset(&ext, 0, sizeof ext);
    ext.exp_mode = exp_mode;
    lo_result res;
    std::vector<uint32_t> cand(LO_K_CAP);
    lo_sample(logits, dtype, v, nullptr, p, 0, &ext, &res, cand.data(), nullptr, nullptr, nullptr);
    float temperature;
    uint32_t k;
    lo_effective(p, &temperature, &k);
    const float top = load_logit(logits, dtype, cand[0]) / temperature;
    std::vector<float> w(res.n_kept);
    for (uint32_t i = 0; i < res.n_kept; ++i) {
        const float d = load_logit(logits, dtype, cand[i]) / temperature - top;
        w[i] = exp_mode == LO_EXP_LIBM ? std::exp(d) : lilym_expf(d);
    }
    float mass = 0.0f;
    for (float x : w) mass += x;
    for (uint32_t i = 0; i < res.n_kept; ++i) {
        ids[i] = cand[i];
        probs[i] = w[i] / mass;
    }
    return res.n_kept;
}

static float dist_at(const uint32_t* ids, const float* probs, uint32_t n, uint32_t id) {
    for (uint32_t i = 0; i < n; ++i) {
        if (ids[i] == id) return probs[i];
    }
    return 0.0f;
}

// cpu_spec.  `u1`/`u2` override the two uniforms when has_u is set.  *accepted
// receives 1 when the proposal was taken on the first uniform; *zero_residual
// 1 when the residual had no mass (the reference test then returns p's last id,
// the reference kernel draws plainly from p: sample.metal:650-651).
uint32_t lo_spec(const uint32_t* p_ids, const float* p_probs, uint32_t pn, const uint32_t* q_ids,
                 const float* q_probs, uint32_t qn, uint32_t d, uint64_t seed, uint32_t step,
                 uint32_t has_u, float u1_in, float u2_in, uint32_t* accepted,
                 uint32_t* zero_residual, float* gap) {
    const float p_d = dist_at(p_ids, p_probs, pn, d);
    const float q_d = dist_at(q_ids, q_probs, qn, d);
    const float u1 = has_u ? u1_in : lilym_uniform_for(seed, step);
    if (accepted) *accepted = 0;
    if (zero_residual) *zero_residual = 0;
    if (gap) *gap = std::numeric_limits<float>::infinity();
    if (u1 * q_d < p_d) {
        if (accepted) *accepted = 1;
        return d;
    }
    std::vector<float> r(pn);
    for (uint32_t i = 0; i < pn; ++i) {
        r[i] = std::max(p_probs[i] - dist_at(q_ids, q_probs, qn, p_ids[i]), 0.0f);
    }
    float total = 0.0f;
    for (float x : r) total += x;
    const float u2 = has_u ? u2_in : lilym_uniform_for(seed, lilym_residual_step(step));
    const float target = u2 * total;
    if (zero_residual && !(total > 0.0f)) *zero_residual = 1;
    float cum = 0.0f;
    uint32_t out = p_ids[pn - 1];
    bool found = false;
    for (uint32_t i = 0; i < pn; ++i) {
        cum += r[i];
        if (!found && target < cum) {
            out = p_ids[i];
            found = true;
        }
        if (gap && total > 0.0f && i + 1 < pn) {
            *gap = std::min(*gap, std::fabs(target - cum) / total);
        }
    }
    return out;
}

// spec_accept: the accepted count and the control block.
void lo_spec_accept(const uint32_t* draws, const uint32_t* ids, uint32_t m, uint32_t pos0,
                    uint32_t ratio, uint32_t chain, uint32_t stride, uint32_t* ctrl) {
    uint32_t a = 0;
    while (a + 1 < m && draws[a] == ids[a + 1]) ++a;
    ctrl[0] = a;
    ctrl[stride] = a + 1;
    for (uint32_t i = 0; i < chain; ++i) {
        const uint32_t p = pos0 + a + 1 + i;
        ctrl[(2 + 3 * i) * stride] = p;
        ctrl[(3 + 3 * i) * stride] = p / ratio;
        ctrl[(4 + 3 * i) * stride] = ((p + 1) % ratio == 0) ? 1u : 0u;
    }
}

// The host's view of the same count: leading rows whose draw equals the draft after them.
uint32_t lo_host_accept(const uint32_t* sampled, const uint32_t* tokens, uint32_t m) {
    uint32_t a = 0;
    while (a + 1 < m && sampled[a] == tokens[a + 1]) ++a;
    return a;
}

void lo_uncount(uint32_t* counts, size_t v, uint32_t token) {
    if (token >= v) return;
    if (counts[token] > 0) counts[token] -= 1;
}

// Many independent rows over `threads` host threads (the CPU baseline leg).
// Rows are `row_stride` elements apart; counts (if any) are per row, V each.
// ids/logprobs receive one value per row.
int lo_sample_rows(const void* logits, int dtype, size_t v, size_t row_stride, uint32_t rows,
                   uint32_t* counts, const lo_params* params, const uint32_t* steps,
                   const lo_ext* exts, uint32_t threads, uint32_t* ids, double* logprobs) {
    if (threads == 0) threads = 1;
    const size_t es = dtype == LO_BF16 ? 2 : 4;
    auto work = [&](uint32_t t) {
        for (uint32_t r = t; r < rows; r += threads) {
            const char* row = static_cast<const char*>(logits) + (size_t)r * row_stride * es;
            lo_result res;
            lo_sample(row, dtype, v, counts ? counts + (size_t)r * v : nullptr, &params[r],
                      steps ? steps[r] : 0, exts ? &exts[r] : nullptr, &res, nullptr, nullptr,
                      nullptr, nullptr);
            ids[r] = res.chosen;
            if (logprobs) logprobs[r] = res.logprob;
        }
    };
    if (threads == 1) {
        work(0);
        return 0;
    }
    std::vector<std::thread> pool;
    for (uint32_t t = 0; t < threads; ++t) pool.emplace_back(work, t);
    for (auto& th : pool) th.join();
    return 0;
}

}  // extern "C"
