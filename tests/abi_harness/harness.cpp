// A caller of liblily_sampler_hip.so written against include/lily_sampler.h alone (plus the HIP
// runtime for device memory): what a host other than the Python tests sees.
//
//   harness cpu              host helpers only (no GPU): prints "cpu ok"
//   harness time ROWS V N    N calls of lily_sample_rows over ROWS x V bf16 logits with host
//                            descriptors every call (params, steps, scratches, penalties, logprobs):
//                            prints the host time a call takes to return and the time per call
//                            on the device (HIP events around the N calls)
//   harness head ROWS D V    the logits' producer on ROWS x D hidden states and V x D weights
//                            (bf16, from the hash below), once by this library's own kernel
//                            (LILY_SAMPLER_HEAD=own) and once the default way, which for a batch
//                            is the platform's GEMM library opened by name - in a program that
//                            has loaded no copy of it: prints "head library_calls N maxdiff X
//                            maxdiff_max Y maxdiff_sum Z" (the two ways' logits and summaries
//                            against each other, differences relative to 1 + |value|).
//   harness gpu V SEED       two draws through lily_sample_f32, two rows through
//                            lily_sample_rows and the same rows through a plan; prints
//                            "ids a b c d e f" - the Python side reproduces the inputs and
//                            checks the ids against the oracle.
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "lily_sampler.h"

#define CHECK(x)                                                                          \
    do {                                                                                  \
        int rc_ = (x);                                                                    \
        if (rc_ != 0) {                                                                   \
            std::fprintf(stderr, "%s -> %d: %s\n", #x, rc_, lily_last_error());            \
            return 1;                                                                     \
        }                                                                                 \
    } while (0)
#define HIP(x)                                                                            \
    do {                                                                                  \
        hipError_t e_ = (x);                                                              \
        if (e_ != hipSuccess) {                                                           \
            std::fprintf(stderr, "%s -> %s\n", #x, hipGetErrorString(e_));                 \
            return 1;                                                                     \
        }                                                                                 \
    } while (0)

// The inputs, reproducible anywhere: a 32-bit multiplicative hash of the index.
static float logit_of(uint32_t i, uint32_t seed) {
    uint32_t h = (i + 1u) * 2654435761u + seed * 40503u;
    h ^= h >> 15;
    h *= 2246822519u;
    h ^= h >> 13;
    return (float)(h >> 8) * (16.0f / 16777216.0f) - 8.0f;   // [-8, 8), a multiple of 2^-20
}

static int cpu_mode() {
    lily_sampling_params p;
    lily_params_greedy(&p);
    if (!lily_params_is_greedy(&p) || lily_params_uses_penalties(&p) || lily_params_validate(&p) != LILY_OK) {
        std::fprintf(stderr, "greedy defaults\n");
        return 1;
    }
    p.temperature = 0.7f;
    p.top_k = 5000;
    p.repetition_penalty = 1.1f;
    float t = 0.0f;
    uint32_t k = 0;
    lily_params_effective(&p, &t, &k);
    if (t != 0.7f || k != LILY_SAMPLE_K_CAP || !lily_params_uses_penalties(&p)) {
        std::fprintf(stderr, "effective: %g %u\n", t, k);
        return 1;
    }
    p.top_p = 0.0f;
    if (lily_params_validate(&p) != LILY_ERR_PARAMS || std::strlen(lily_last_error()) == 0) {
        std::fprintf(stderr, "top_p 0 must be rejected with a message\n");
        return 1;
    }
    const float u = lily_uniform_for(1234, 7);
    if (!(u >= 0.0f && u < 1.0f) || lily_uniform_for(1234, 7) != u || lily_uniform_for(1234, 8) == u) {
        std::fprintf(stderr, "uniform_for\n");
        return 1;
    }
    if (lily_draft_step(5) == 5 || lily_ctrl_words(2) < LILY_CTRL_STRIDE * 2) {
        std::fprintf(stderr, "draft_step / ctrl_words\n");
        return 1;
    }
    // the insertions queue (host state only) and the producer's shapes
    lily_insertions_t* q = nullptr;
    const uint32_t ids[2] = {10, 11};
    uint32_t forced[2] = {0, 0};
    if (lily_insertions_create(2, &q) != LILY_OK ||
        lily_insertions_push(q, 1, LILY_INSERT_BEFORE, 9, ids, 2, nullptr) != LILY_OK ||
        lily_insertions_pending(q, 1) != 3 || lily_insertions_next(q, forced) != 1 ||
        forced[0] != LILY_NO_TOKEN || forced[1] != 10) {
        std::fprintf(stderr, "insertions: %s\n", lily_last_error());
        return 1;
    }
    lily_insertions_destroy(q);
    if (lily_lm_head_tiles(151936) != 1187 || lily_lm_head_tiles(129) != 2) {
        std::fprintf(stderr, "lm_head_tiles\n");
        return 1;
    }
    // (the sizes a compiler gives the structs: the Python mirror's must be the same)
    std::printf("cpu ok uniform %.9g draft_step %u ctrl_words %u sizes %zu %zu %zu %zu\n", u, lily_draft_step(5),
                lily_ctrl_words(2), sizeof(lily_sampling_params), sizeof(lily_rows), sizeof(lily_lm_head),
                sizeof(lily_draft_dist));
    return 0;
}

static int gpu_mode(uint32_t vocab, uint32_t seed) {
    std::vector<float> x(2 * (size_t)vocab);
    for (uint32_t r = 0; r < 2; ++r) {
        for (uint32_t i = 0; i < vocab; ++i) {
            x[(size_t)r * vocab + i] = logit_of(i, seed + r);
        }
    }
    std::vector<uint32_t> hist(512);
    for (uint32_t i = 0; i < hist.size(); ++i) {
        hist[i] = (i * 7919u + seed) % vocab;
    }
    float* x_dev = nullptr;
    uint32_t *hist_dev = nullptr, *out_dev = nullptr;
    HIP(hipSetDevice(0));
    HIP(hipMalloc((void**)&x_dev, x.size() * 4));
    HIP(hipMalloc((void**)&hist_dev, hist.size() * 4));
    HIP(hipMalloc((void**)&out_dev, 8 * 4));
    HIP(hipMemcpy(x_dev, x.data(), x.size() * 4, hipMemcpyHostToDevice));
    HIP(hipMemcpy(hist_dev, hist.data(), hist.size() * 4, hipMemcpyHostToDevice));
    HIP(hipMemset(out_dev, 0xff, 8 * 4));

    hipStream_t stream;
    HIP(hipStreamCreate(&stream));
    lily_sampler_t* s = nullptr;
    CHECK(lily_sampler_create(0, stream, &s));
    lily_scratch_t* sc[2] = {nullptr, nullptr};
    for (int r = 0; r < 2; ++r) {
        CHECK(lily_scratch_create(s, vocab, &sc[r]));
        CHECK(lily_scratch_add_history(sc[r], hist_dev, (uint32_t)hist.size()));
    }
    lily_sampling_params p;
    lily_params_greedy(&p);
    p.temperature = 0.9f;
    p.top_k = 50;
    p.top_p = 0.95f;
    p.repetition_penalty = 1.2f;
    p.presence_penalty = 0.1f;
    p.frequency_penalty = 0.05f;
    p.seed = 77;
    // two draws of the reference's call shape (row 0, steps 0 and 1)
    CHECK(lily_sample_f32(s, x_dev, vocab, sc[0], &p, 0, out_dev + 0));
    CHECK(lily_sample_f32(s, x_dev, vocab, sc[0], &p, 1, out_dev + 1));
    // both rows in one call (steps 2, 2): row 0 sees the two draws above in its counts
    lily_sampling_params ps[2] = {p, p};
    ps[1].seed = 78;
    const uint32_t steps[2] = {2, 2};
    lily_rows b;
    std::memset(&b, 0, sizeof b);
    b.rows = 2;
    b.vocab = vocab;
    b.dtype = LILY_F32;
    b.logits_dev = x_dev;
    b.row_stride = vocab;
    b.params = ps;
    b.steps = steps;
    b.scratch = sc;
    b.out_ids_dev = out_dev + 2;
    CHECK(lily_sample_rows(s, &b));
    // and once more through a resident plan (steps 2 + 1)
    lily_plan_t* plan = nullptr;
    CHECK(lily_plan_create(s, 2, &plan));
    b.out_ids_dev = out_dev + 4;
    CHECK(lily_plan_set(plan, &b));
    CHECK(lily_plan_run(plan, 1));
    CHECK(lily_sampler_synchronize(s));
    uint32_t out[8];
    HIP(hipMemcpy(out, out_dev, sizeof out, hipMemcpyDeviceToHost));
    std::printf("ids %u %u %u %u %u %u\n", out[0], out[1], out[2], out[3], out[4], out[5]);
    // a scratch of another vocabulary is refused before anything is enqueued
    if (lily_sample_f32(s, x_dev, vocab - 1, sc[0], &p, 9, out_dev + 6) != LILY_ERR_VOCAB) {
        std::fprintf(stderr, "vocab mismatch must be LILY_ERR_VOCAB\n");
        return 1;
    }
    lily_plan_destroy(plan);
    lily_scratch_destroy(sc[0]);
    lily_scratch_destroy(sc[1]);
    lily_sampler_destroy(s);
    HIP(hipStreamDestroy(stream));
    HIP(hipFree(x_dev));
    HIP(hipFree(hist_dev));
    HIP(hipFree(out_dev));
    return 0;
}

static int time_mode(uint32_t rows, uint32_t vocab, uint32_t n) {
    HIP(hipSetDevice(0));
    hipStream_t stream;
    HIP(hipStreamCreate(&stream));
    lily_sampler_t* s = nullptr;
    CHECK(lily_sampler_create(0, stream, &s));
    // bf16 logits shaped like a language model's: a bulk in [-2, 2) and one id in about a
    // thousand raised by 12 to 36; every row is a rotation of one such row (distinct rows, cheap
    // to make)
    std::vector<uint16_t> one(2 * (size_t)vocab);
    for (uint32_t i = 0; i < 2 * vocab; ++i) {
        const uint32_t j = i % vocab;
        float v = 0.25f * logit_of(j, 3);
        if ((j * 2654435761u >> 12) % 1021u == 0u) {
            v += 12.0f + 1.5f * (logit_of(j, 9) + 8.0f);
        }
        uint32_t bits;
        std::memcpy(&bits, &v, 4);
        one[i] = (uint16_t)(bits >> 16);
    }
    uint16_t* x_dev = nullptr;
    HIP(hipMalloc((void**)&x_dev, (size_t)rows * vocab * 2));
    for (uint32_t r = 0; r < rows; ++r) {
        HIP(hipMemcpy(x_dev + (size_t)r * vocab, one.data() + (r * 97u) % vocab, (size_t)vocab * 2,
                      hipMemcpyHostToDevice));
    }
    std::vector<uint32_t> hist(vocab < 4096u ? vocab / 8u + 1u : 512u);
    for (uint32_t i = 0; i < hist.size(); ++i) {
        hist[i] = (i * 7919u + 11u) % vocab;
    }
    uint32_t *hist_dev = nullptr, *out_dev = nullptr;
    float* lp_dev = nullptr;
    HIP(hipMalloc((void**)&hist_dev, hist.size() * 4));
    HIP(hipMemcpy(hist_dev, hist.data(), hist.size() * 4, hipMemcpyHostToDevice));
    HIP(hipMalloc((void**)&out_dev, (size_t)rows * 4));
    HIP(hipMalloc((void**)&lp_dev, (size_t)rows * 4));
    std::vector<lily_scratch_t*> sc(rows);
    std::vector<lily_sampling_params> ps(rows);
    std::vector<uint32_t> steps(rows);
    for (uint32_t r = 0; r < rows; ++r) {
        CHECK(lily_scratch_create(s, vocab, &sc[r]));
        CHECK(lily_scratch_add_history(sc[r], hist_dev, (uint32_t)hist.size()));
        lily_params_greedy(&ps[r]);
        ps[r].temperature = 0.8f;
        ps[r].top_k = 64;
        ps[r].top_p = 0.9f;
        ps[r].repetition_penalty = 1.1f;
        ps[r].presence_penalty = 0.2f;
        ps[r].frequency_penalty = 0.1f;
        ps[r].seed = 5000 + r;
    }
    lily_rows b;
    std::memset(&b, 0, sizeof b);
    b.rows = rows;
    b.vocab = vocab;
    b.dtype = LILY_BF16;
    b.logits_dev = x_dev;
    b.row_stride = vocab;
    b.params = ps.data();
    b.steps = steps.data();
    b.scratch = sc.data();
    b.out_ids_dev = out_dev;
    b.out_logprobs_dev = lp_dev;
    for (uint32_t w = 0; w < 5; ++w) {
        CHECK(lily_sample_rows(s, &b));
    }
    CHECK(lily_sampler_synchronize(s));
    hipEvent_t e0, e1;
    HIP(hipEventCreate(&e0));
    HIP(hipEventCreate(&e1));
    double host_us = 0.0;
    HIP(hipEventRecord(e0, stream));
    for (uint32_t i = 0; i < n; ++i) {
        for (uint32_t r = 0; r < rows; ++r) {
            steps[r] = 5 + i;
        }
        const auto t0 = std::chrono::steady_clock::now();
        CHECK(lily_sample_rows(s, &b));
        host_us += std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
    }
    HIP(hipEventRecord(e1, stream));
    HIP(hipEventSynchronize(e1));
    float ms = 0.0f;
    HIP(hipEventElapsedTime(&ms, e0, e1));
    // the same call with the stream drained before each one: what the call itself costs the host
    double alone_us = 0.0;
    for (uint32_t i = 0; i < n; ++i) {
        CHECK(lily_sampler_synchronize(s));
        const auto t0 = std::chrono::steady_clock::now();
        CHECK(lily_sample_rows(s, &b));
        alone_us += std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
    }
    CHECK(lily_sampler_synchronize(s));
    // which selects served one more call (workgroups: streaming, sparse or bitmap, exhaustive;
    // and the reasons the streaming select gave up, as bits)
    uint32_t* stats_dev = nullptr;
    uint32_t stats[4] = {0, 0, 0, 0};
    HIP(hipMalloc((void**)&stats_dev, sizeof stats));
    HIP(hipMemcpy(stats_dev, stats, sizeof stats, hipMemcpyHostToDevice));
    CHECK(lily_sampler_set_path_stats(s, stats_dev));
    CHECK(lily_sample_rows(s, &b));
    CHECK(lily_sampler_synchronize(s));
    CHECK(lily_sampler_set_path_stats(s, nullptr));
    HIP(hipMemcpy(stats, stats_dev, sizeof stats, hipMemcpyDeviceToHost));
    HIP(hipFree(stats_dev));
    std::printf("time rows %u vocab %u calls %u host_us_per_call %.1f device_us_per_call %.1f "
                "host_us_per_call_idle_stream %.1f served_by %u %u %u gave_up_bits %u\n",
                rows, vocab, n, host_us / n, ms * 1000.0 / n, alone_us / n, stats[0], stats[1], stats[2],
                stats[3]);
    for (uint32_t r = 0; r < rows; ++r) {
        lily_scratch_destroy(sc[r]);
    }
    lily_sampler_destroy(s);
    HIP(hipStreamDestroy(stream));
    HIP(hipFree(x_dev));
    HIP(hipFree(hist_dev));
    HIP(hipFree(out_dev));
    HIP(hipFree(lp_dev));
    return 0;
}

static uint16_t bf16_of(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

static float f32_of(uint16_t b) {
    const uint32_t u = (uint32_t)b << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

static int head_mode(uint32_t rows, uint32_t d, uint32_t vocab) {
    HIP(hipSetDevice(0));
    hipStream_t stream;
    HIP(hipStreamCreate(&stream));
    const uint32_t tiles = lily_lm_head_tiles(vocab);
    std::vector<uint16_t> hidden((size_t)rows * d), weight((size_t)vocab * d);
    for (size_t i = 0; i < hidden.size(); ++i) {
        hidden[i] = bf16_of(0.125f * logit_of((uint32_t)i, 5));
    }
    const float scale = 0.25f / std::sqrt((float)d);
    for (size_t i = 0; i < weight.size(); ++i) {
        weight[i] = bf16_of(scale * logit_of((uint32_t)i, 9));
    }
    void *h_dev, *w_dev;
    HIP(hipMalloc(&h_dev, hidden.size() * 2));
    HIP(hipMalloc(&w_dev, weight.size() * 2));
    HIP(hipMemcpy(h_dev, hidden.data(), hidden.size() * 2, hipMemcpyHostToDevice));
    HIP(hipMemcpy(w_dev, weight.data(), weight.size() * 2, hipMemcpyHostToDevice));
    std::vector<float> temps(rows, 0.8f);
    std::vector<uint16_t> logits[2];
    std::vector<float> tmax[2], tsum[2];
    unsigned long long calls = 0;
    for (int way = 0; way < 2; ++way) {
        if (way == 0) {
            setenv("LILY_SAMPLER_HEAD", "own", 1);
        } else {
            unsetenv("LILY_SAMPLER_HEAD");
        }
        lily_sampler_t* s = nullptr;
        CHECK(lily_sampler_create(0, stream, &s));
        void *l_dev, *m_dev, *s_dev;
        HIP(hipMalloc(&l_dev, (size_t)rows * vocab * 2));
        HIP(hipMalloc(&m_dev, (size_t)rows * tiles * 4));
        HIP(hipMalloc(&s_dev, (size_t)rows * tiles * 4));
        lily_lm_head head;
        std::memset(&head, 0, sizeof(head));
        head.hidden_dev = h_dev;
        head.hidden_stride = d;
        head.weight_dev = w_dev;
        head.weight_stride = d;
        head.d = d;
        head.tile_max_dev = static_cast<float*>(m_dev);
        head.tile_sum_dev = static_cast<float*>(s_dev);
        CHECK(lily_lm_head_bf16(s, &head, rows, vocab, temps.data(), l_dev, vocab));
        HIP(hipStreamSynchronize(stream));
        logits[way].resize((size_t)rows * vocab);
        tmax[way].resize((size_t)rows * tiles);
        tsum[way].resize((size_t)rows * tiles);
        HIP(hipMemcpy(logits[way].data(), l_dev, logits[way].size() * 2, hipMemcpyDeviceToHost));
        HIP(hipMemcpy(tmax[way].data(), m_dev, tmax[way].size() * 4, hipMemcpyDeviceToHost));
        HIP(hipMemcpy(tsum[way].data(), s_dev, tsum[way].size() * 4, hipMemcpyDeviceToHost));
        if (way == 1) {
            calls = lily_lm_head_library_calls(s);
        } else if (lily_lm_head_library_calls(s) != 0) {
            std::fprintf(stderr, "the own kernel was asked for\n");
            return 1;
        }
        lily_sampler_destroy(s);
        HIP(hipFree(l_dev));
        HIP(hipFree(m_dev));
        HIP(hipFree(s_dev));
    }
    double diff = 0.0, diff_max = 0.0, diff_sum = 0.0;
    for (size_t i = 0; i < logits[0].size(); ++i) {
        const double a = f32_of(logits[0][i]), b = f32_of(logits[1][i]);
        diff = std::fmax(diff, std::fabs(a - b) / (1.0 + std::fabs(a)));
    }
    for (size_t i = 0; i < tmax[0].size(); ++i) {
        diff_max = std::fmax(diff_max, std::fabs((double)tmax[0][i] - tmax[1][i]) / (1.0 + std::fabs((double)tmax[0][i])));
        diff_sum = std::fmax(diff_sum, std::fabs((double)tsum[0][i] - tsum[1][i]) / (1.0 + std::fabs((double)tsum[0][i])));
    }
    std::printf("head library_calls %llu maxdiff %.6f maxdiff_max %.6f maxdiff_sum %.6f\n", calls, diff, diff_max,
                diff_sum);
    HIP(hipFree(h_dev));
    HIP(hipFree(w_dev));
    HIP(hipStreamDestroy(stream));
    return 0;
}

int main(int argc, char** argv) {
    if (argc >= 5 && std::strcmp(argv[1], "head") == 0) {
        return head_mode((uint32_t)std::atoi(argv[2]), (uint32_t)std::atoi(argv[3]), (uint32_t)std::atoi(argv[4]));
    }
    if (argc >= 2 && std::strcmp(argv[1], "cpu") == 0) {
        return cpu_mode();
    }
    if (argc >= 4 && std::strcmp(argv[1], "gpu") == 0) {
        return gpu_mode((uint32_t)std::atoi(argv[2]), (uint32_t)std::atoi(argv[3]));
    }
    if (argc >= 5 && std::strcmp(argv[1], "time") == 0) {
        return time_mode((uint32_t)std::atoi(argv[2]), (uint32_t)std::atoi(argv[3]), (uint32_t)std::atoi(argv[4]));
    }
    std::fprintf(stderr, "usage: harness cpu | harness gpu VOCAB SEED | harness time ROWS VOCAB CALLS | harness head ROWS D VOCAB\n");
    return 2;
}
