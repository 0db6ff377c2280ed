// rows_tiles.hip - the draw of rows whose logits came with the producer's summaries (the largest
// value and the sum of exponentials of every LILY_TILE_COLS columns): the row is not read,
// only the summaries and the few tiles that can hold one of its k largest values.
#include <algorithm>

#include "row_kernel.h"

namespace lily {

constexpr uint32_t TILES_PER_THREAD = 8;
constexpr uint32_t TILES_MAX = NT * TILES_PER_THREAD;    // summaries of a row
constexpr uint32_t TILE_CAND_CAP = 2048;                 // candidates gathered from the tiles
constexpr uint32_t TILES_DECLINE = 256;                  // a penalised row that needs more tiles is declined,
constexpr uint32_t SUMMED_DECLINE = 96;                  // or more tiles summed element by element
constexpr uint32_t REF_CAP = 2048;                       // pieces evaluated element by element

// One workgroup per row (rows without mask, at most STREAM_BIAS_CAP bias pairs, penalties only
// of the kind that can but lower a value, k <= STREAM_K_MAX; bf16 or f32 logits, rows at
// multiples of 16 bytes).
//   * The row's largest value is the largest summary; with at least k summaries at or above
//     x, at least k values are: the k-th largest summary bounds the k-th largest value from
//     below, and only tiles whose summary reaches it are read (16 bytes a lane: 16 lanes a tile
//     of bf16 logits, 32 of f32); their values at or above the bound are the candidates.
//   * The row's sum of exponentials is the summaries' sums brought to the row's reference.
//   * Under penalties the bound is the k-th largest summary as the worst penalty would leave it
//     (more tiles are read), values of listed ids are evaluated with their counts, and the tiles
//     that matter to the row's sum are summed element by element instead of by their summaries.
//   * A bias list (logit += delta before everything else, pairs of one id adding up in list
//     order): a summary says nothing about a biased id.  The tiles that hold one are always
//     read, every value of theirs evaluated (and, for the row's sum, summed one by one instead
//     of by the summary); a tile's largest value may belong to an id with a negative bias, so
//     the bound is the (k + pairs)-th largest summary - k of those tiles keep their largest.
//   * An allow-mask (a barred id counts as -inf): a tile none of whose ids is allowed drops out
//     with its summary; a tile that is allowed in part has a summary that says too much - its
//     values are tested one by one against the mask, it enters the row's sum value by value,
//     and the bound counts on k / 2 + 8 tiles more.  That is a guess, so the row checks it: with
//     fewer than k candidates at or above the bound it is left to the launch that follows, as is
//     a row with more than SUMMED_DECLINE partly allowed tiles to sum.
//   * More candidates than the buffer holds (ties by the thousand): the exhaustive select
//     over the whole row takes over.
// `tile_row[r]` is the row of the summaries that belongs to row r of the table; `served[r]` is
// written for rows under penalties or a mask: 1 = drawn here, 0 = left to the launch that follows.
// EXTRA: rows with a bias list or a mask are among the launch's (the kernel without them keeps the
// row's descriptor in fewer scalar registers, which the other spills).
template <int DT, bool LSE, bool EXTRA>
__global__ __launch_bounds__(NT, 4) void k_rows_tiles(LaunchCfg cfg, const float* tile_max,
                                                      const float* tile_sum, uint32_t tiles,
                                                      const uint32_t* tile_row, uint32_t* served) {
    __shared__ Shared sh;
    __shared__ uint16_t listed[TILES_MAX];   // tiles to read; bit 15: summed element by element
    __shared__ uint32_t refs[REF_CAP];       // pieces to evaluate: first id; bit 31: summed
    __shared__ uint32_t n_listed, n_refs, n_summed;
    __shared__ uint32_t bias_id[STREAM_BIAS_CAP];
    __shared__ float bias_delta[STREAM_BIAS_CAP];
    __shared__ uint32_t bias_tiles[TILES_MAX / 32u];   // bit t: tile t holds a biased id
    constexpr uint32_t E = (uint32_t)Geo<DT>::E;          // values in a piece of 16 bytes
    constexpr uint32_t ELEM = DT == LILY_BF16 ? 2u : 4u;  // bytes a value
    const LILY_CONST RowArgs* table = (const LILY_CONST RowArgs*)cfg.table;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    if (tid == 0) {
        tail_arrays(sh);
        n_listed = 0;
        n_refs = 0;
        n_summed = 0;
    }
    RowArgs a;
    load_row_args(a, table + blockIdx.y);
    const uint32_t vocab = cfg.vocab;
    const uint32_t step = a.step + cfg.step_delta;
    const bool want_lse = LSE && a.out_logprob != nullptr;
    uint64_t* cand = dyn_lds;
    const bool forced = (a.flags & F_FORCED) != 0;
    if (forced && !want_lse) {
        if (tid == 0) {
            emit(a, a.forced, vocab);
        }
        return;
    }
    const uint32_t n_bias = EXTRA ? min(a.n_bias, STREAM_BIAS_CAP) : 0u;   // (the host serves no longer lists here)
    if (n_bias != 0u) {
        if (tid < TILES_MAX / 32u) {
            bias_tiles[tid] = 0u;
        }
        if (tid < n_bias) {
            bias_id[tid] = gload(&a.bias[tid].id);
            bias_delta[tid] = gload(&a.bias[tid].delta);
        }
    }
    const size_t srow = (size_t)gload(tile_row + blockIdx.y) * tiles;
    // the summaries: both arrays asked for at once (clamped, so that no load hangs on a test)
    float ms[TILES_PER_THREAD], ss[TILES_PER_THREAD];
    float best = NEG_INF;
#pragma unroll
    for (uint32_t j = 0; j < TILES_PER_THREAD; ++j) {
        const uint32_t t = min(tid + j * NT, tiles - 1u);
        ms[j] = gload(tile_max + srow + t);
        ss[j] = gload(tile_sum + srow + t);
    }
    // The mask's four words of every tile: a tile with no allowed id drops out, one allowed in
    // part is marked (bit j of `partly`).
    const bool masked = EXTRA && a.allow != nullptr;
    const uint32_t words = (vocab + 31u) / 32u;
    uint32_t partly = 0;
    if (masked) {
        uint32_t mw[TILES_PER_THREAD][4];
#pragma unroll
        for (uint32_t j = 0; j < TILES_PER_THREAD; ++j) {
#pragma unroll
            for (uint32_t q = 0; q < 4u; ++q) {
                mw[j][q] = gload(a.allow + min((tid + j * NT) * 4u + q, words - 1u));
            }
        }
#pragma unroll
        for (uint32_t j = 0; j < TILES_PER_THREAD; ++j) {
            bool any = false, all = true;
#pragma unroll
            for (uint32_t q = 0; q < 4u; ++q) {
                const uint32_t first = ((tid + j * NT) * 4u + q) * 32u;   // the word's first id
                const uint32_t in_row = first >= vocab ? 0u : (vocab - first >= 32u ? 0xffffffffu : (1u << (vocab - first)) - 1u);
                any = any || (mw[j][q] & in_row) != 0u;
                all = all && (mw[j][q] & in_row) == in_row;
            }
            if (!any) {
                ms[j] = NEG_INF;
            } else if (!all) {
                partly |= 1u << j;
            }
        }
    }
#pragma unroll
    for (uint32_t j = 0; j < TILES_PER_THREAD; ++j) {
        if (tid + j * NT >= tiles) {
            ms[j] = NEG_INF;
        }
        best = fmaxf(best, ms[j]);
    }
    best = wave_max_f(best);
    if (lane == 0) {
        sh.red_f[w] = best;
    }
    __syncthreads();
    float top = sh.red_f[0];
    for (int i = 1; i < NWAVE; ++i) {
        top = fmaxf(top, sh.red_f[i]);
    }
    if (tid < n_bias && bias_id[tid] < vocab) {
        const uint32_t t = bias_id[tid] / LILY_TILE_COLS;
        atomicOr(&bias_tiles[t >> 5], 1u << (t & 31u));
    }
    __syncthreads();
    phase(cfg, 1);
    auto holds_bias = [&](uint32_t tile) -> bool {
        return n_bias != 0u && ((bias_tiles[tile >> 5] >> (tile & 31u)) & 1u) != 0u;
    };
    // (pairs of one id add up in list order, as the row kernels add them)
    auto with_bias = [&](uint32_t id, float x) -> float {
        for (uint32_t j = 0; j < n_bias; ++j) {
            if (bias_id[j] == id) {
                x += bias_delta[j];
            }
        }
        return x == x ? x : NEG_INF;
    };

    if (a.mode == MODE_ARGMAX && !forced) {
        // The first of the largest values: the lowest tile that holds it, its lowest column.
        uint32_t first = 0xffffffffu;
#pragma unroll
        for (uint32_t j = 0; j < TILES_PER_THREAD; ++j) {
            if (ms[j] == top && top > NEG_INF) {
                first = min(first, tid + j * NT);
            }
        }
        first = wave_min_u32(first);
        if (lane == 0) {
            sh.red_i[w] = first;
        }
        __syncthreads();
        first = min(min(sh.red_i[0], sh.red_i[1]), min(sh.red_i[2], sh.red_i[3]));
        if (w == 0) {
            uint32_t id = 0xffffffffu;
            if (first != 0xffffffffu) {
#pragma unroll
                for (uint32_t h = 0; h < LILY_TILE_COLS / 64u; ++h) {
                    const uint32_t col = first * LILY_TILE_COLS + h * 64u + lane;
                    if (col < vocab && load_logit<DT>(a.logits, col) == top) {
                        id = min(id, col);
                    }
                }
            }
            id = wave_min_u32(id);
            if (lane == 0) {
                *a.out_id = id == 0xffffffffu ? 0u : id;
            }
        }
        return;
    }

    // Rows under penalties that can only lower a value (the host serves no others here): a
    // summary describes raw values and bounds true ones from above.  `lowered(x)`: what a raw
    // value x is worth at least (the penalty of an id with the scratch's largest count).
    const bool pen = (a.flags & F_PEN) != 0;
    const uint32_t max_count = pen ? *(const LILY_CONST uint32_t*)(a.touched + words) : 0u;
    auto lowered = [&](float m) -> float {
        if (pen && m > NEG_INF) {
            float t = m > 0.0f ? m / a.repetition : m * a.repetition;
            t -= a.presence + a.frequency * (float)max_count;
            return t;
        }
        return m;
    };
    auto true_value = [&](uint32_t id, float raw) -> float {
        uint32_t cnt = gload(a.counts + id);
        asm volatile("" : "+v"(cnt));   // waited for here, inside the caller's branch
        float t = raw;
        if (cnt > 0u) {
            t = t > 0.0f ? t / a.repetition : t * a.repetition;
            t -= a.presence + a.frequency * (float)cnt;
        }
        return t;
    };
    // The summaries' part of the row's sum: every tile below the cut that holds no biased id and
    // no barred one.
    LseAcc lse;
    lse.init();
    auto add_summaries = [&](float below) {
#pragma unroll
        for (uint32_t j = 0; j < TILES_PER_THREAD; ++j) {
            const uint32_t t = tid + j * NT;
            if (t < tiles && ms[j] > NEG_INF && (!pen || ms[j] < below) && !holds_bias(t) &&
                ((partly >> j) & 1u) == 0u) {
                // the tile's sum has the reference tile_max * c2
                const float safe = lse.rebase(ms[j], a.c2);
                lse.s += ss[j] * __builtin_amdgcn_exp2f(ms[j] * a.c2 - safe);
            }
        }
    };
    if (forced) {   // (not under penalties, no bias list: the host keeps such rows off this kernel)
        if (want_lse) {
            add_summaries(0.0f);
            lse_reduce(sh, lse);
        }
        if (tid == 0) {
            finish_token<DT>(a, sh, a.forced, vocab);
        }
        return;
    }

    // The sum's cut: tiles whose summary lies below it are summed as their summaries give them
    // (their listed ids' raw terms stand for the true ones: each is below 2^-(log2 V + 21) of
    // the row's largest term), tiles at or above it element by element.  It hangs from a lower
    // bound of the row's largest TRUE value: the lowered largest summary (with a bias list or a
    // mask the lowered k-th, which k tiles reach with values that carry no bias; under a mask
    // that is a guess, which the row's check below - k candidates at or above it - confirms as
    // a floor of the largest true value as well) or, better where a sequence keeps coming back
    // to one token, the true value of the scratch's most-counted id.
    float cut = -__builtin_huge_valf();
    auto cut_below = [&](float floor_v) -> float {
        const uint32_t heavy = *(const LILY_CONST uint32_t*)(a.touched + words + 1u);
        const bool heavy_allowed =
            !masked || heavy >= vocab || ((gload(a.allow + (heavy >> 5)) >> (heavy & 31u)) & 1u) != 0u;
        if (heavy < vocab && max_count != 0u && heavy_allowed) {
            const float raw = load_logit<DT>(a.logits, heavy);
            const float biased = with_bias(heavy, raw == raw ? raw : NEG_INF);
            if (biased > NEG_INF) {
                floor_v = fmaxf(floor_v, true_value(heavy, biased));
            }
        }
        return floor_v - (log2f((float)vocab) + 21.0f) * (a.temperature * 0.6931471805599453f);
    };
    // A row without bias list and mask knows its cut from the largest summary alone: it forms
    // it, and the summaries' part of its sum, before the search for the bound, whose barriers
    // the loads behind the cut then wait out; the other rows need the bound first.
    const bool cut_first = n_bias == 0u && !masked;
    if (cut_first) {
        if (want_lse && pen) {
            cut = cut_below(lowered(top));
        }
        if (want_lse) {
            add_summaries(cut);
        }
    }
    // (with a bias list: n_bias tiles more, whose largest values may be the biased ones; under a
    // mask: a guess at how many of the best tiles owe their summaries to barred ids)
    const uint32_t k = a.k, k_tiles = a.k + n_bias + (masked ? a.k / 2u + 8u : 0u);
    // with at least k summaries at or above x, at least k raw values are, and their true values
    // are at or above lowered(x)
    // (a lower bound of the k-th largest summary, as the streaming select takes it: each wave's
    // ceil(k / NWAVE)-th largest of its lanes' best summaries - a 16-step search by ballots on the
    // top half of the order key -, the minimum over the waves; F32_LOWEST when a wave holds fewer)
    float lane_best = NEG_INF;
#pragma unroll
    for (uint32_t j = 0; j < TILES_PER_THREAD; ++j) {
        lane_best = fmaxf(lane_best, ms[j]);
    }
    float kth;
    if (tiles >= NT) {
        const uint32_t kw = (k_tiles + NWAVE - 1u) / NWAVE;
        const uint32_t key16 = lane_best > NEG_INF ? (lilym_order_key(lane_best) >> 16) : 0u;
        const uint32_t P = wave_kth_key16(key16, kw);
        if (lane == 0) {
            sh.red_f[w] = P != 0u ? lilym_key_value(P << 16) : F32_LOWEST;
        }
        __syncthreads();
        kth = sh.red_f[0];
        for (int i = 1; i < NWAVE; ++i) {
            kth = fminf(kth, sh.red_f[i]);
        }
        __syncthreads();
    } else {
        // a short row leaves whole waves without a summary: the exact k-th largest instead
        kth = wg_kth_largest(ms, k_tiles, sh);
    }
    if (!cut_first) {
        if (want_lse && pen) {
            cut = cut_below(lowered(kth));
        }
        if (want_lse) {
            add_summaries(cut);
        }
    }
    const float bound = lowered(kth);
    const float reach = (want_lse && pen) ? fminf(bound, cut) : bound;   // tiles read
    phase(cfg, 2);
    if (tid == 0) {
        sh.n_cand = 0;
    }
#pragma unroll
    for (uint32_t j = 0; j < TILES_PER_THREAD; ++j) {
        const uint32_t t = tid + j * NT;
        const bool biased = t < tiles && holds_bias(t);
        // (a tile allowed in part matters to the sum whatever its summary says; to the candidates
        // only where the summary reaches the bound)
        const bool part = ((partly >> j) & 1u) != 0u && ms[j] > NEG_INF;
        if ((ms[j] >= reach && ms[j] > NEG_INF) || biased || (part && want_lse)) {
            // (bit 15: every value of the tile is evaluated, and taken into the row's sum one by
            // one where there is a sum - the summaries' part leaves these tiles out)
            const bool sum_it = want_lse && ((pen && ms[j] >= cut && ms[j] > NEG_INF) || part);
            listed[atomicAdd(&n_listed, 1u)] = (uint16_t)(t | (sum_it || biased ? 0x8000u : 0u));
            if (sum_it) {
                atomicAdd(&n_summed, 1u);
            }
        }
    }
    __syncthreads();
    const uint32_t n_t = n_listed;
    phase(cfg, 8);
    // A row under penalties or a mask whose bound, cut or partly allowed tiles reach a large part
    // of its tiles is read faster as a whole: it is left to the launch that follows (`served`
    // stays 0).
    if (pen || masked) {
        const bool decline = n_t > TILES_DECLINE || n_summed > SUMMED_DECLINE;
        if (tid == 0) {
            served[blockIdx.y] = decline ? 0u : 1u;
        }
        if (decline) {
            return;
        }
    }
    // First the tiles are read, 16 lanes a tile and 16 bytes a lane, ROUNDS rounds of loads asked
    // for before the first is used; all a lane does with a piece is compare its largest value
    // with the bound: a piece that reaches it (or belongs to a summed tile) is put on a list.
    // (Evaluating such pieces on the spot keeps one or two lanes of a wave busy while the
    // others wait, eight times per round: that was most of the kernel's time.)
    constexpr uint32_t LANES = LILY_TILE_COLS / E, PER_ROUND = NT / LANES;
    const uint32_t sub = tid % LANES, slot = tid / LANES;
    constexpr int ROUNDS = 8;
    for (uint32_t r0 = 0; r0 < n_t; r0 += (uint32_t)ROUNDS * PER_ROUND) {
        u32x4 q[ROUNDS];
        uint32_t col0[ROUNDS];
#pragma unroll
        for (int u = 0; u < ROUNDS; ++u) {
            const uint32_t i = min(r0 + (uint32_t)u * PER_ROUND + slot, n_t - 1u);
            const uint32_t t = listed[i];
            const uint32_t c = (t & 0x7fffu) * LILY_TILE_COLS + sub * E;
            col0[u] = (r0 + (uint32_t)u * PER_ROUND + slot < n_t && c < vocab) ? (c | ((t & 0x8000u) << 16))
                                                                              : 0xffffffffu;
            // A row starts at a multiple of 16 bytes (the host checks), so these pieces do too:
            // one that holds a valid column lies inside the row's pages, and the others are
            // replaced by the row's last such piece.
            const uint32_t cc = min(c, (vocab - 1u) & ~(E - 1u));
            q[u] = gload(reinterpret_cast<const u32x4*>(static_cast<const char*>(a.logits) + (size_t)cc * ELEM));
        }
#pragma unroll
        for (int u = 0; u < ROUNDS; ++u) {
            // (true values are raw ones or lower: a piece whose largest raw value stays below the
            // bound holds no candidate)
            const bool want = col0[u] != 0xffffffffu &&
                              ((col0[u] >> 31) != 0u || chunk_max<DT>(q[u]) >= bound);
            const uint64_t votes = __ballot(want);
            if (votes != 0ull) {
                uint32_t base = 0;
                if (lane == 0) {
                    base = atomicAdd(&n_refs, (uint32_t)__popcll(votes));
                }
                base = (uint32_t)__shfl((int)base, 0);
                const uint32_t at = base + (uint32_t)__popcll(votes & ((1ull << lane) - 1ull));
                if (want && at < REF_CAP) {
                    refs[at] = col0[u];
                }
            }
        }
    }
    __syncthreads();
    // Then the listed pieces, a thread per value, four pieces' loads in flight per thread.
    const uint32_t n_r = n_refs;   // (beyond the list's capacity: the exhaustive select below)
    const uint32_t e_of = tid % E;
    for (uint32_t p0 = 0; p0 < min(n_r, REF_CAP); p0 += 4u * (NT / E)) {
        uint32_t ref[4], word[4], mword[4];
        float raw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t p = p0 + (uint32_t)u * (NT / E) + tid / E;
            ref[u] = p < min(n_r, REF_CAP) ? refs[p] : 0xffffffffu;
            const uint32_t id = min((ref[u] & 0x7fffffffu) + e_of, vocab - 1u);
            raw[u] = load_logit<DT>(a.logits, id);
            // (the word of the scratch's bitmap that covers the id; the summaries' first word
            // when there is no scratch to ask: the load stays unconditional)
            word[u] = gload((pen ? a.touched : reinterpret_cast<const uint32_t*>(tile_max)) + (pen ? (id >> 5) : 0u));
            mword[u] = masked ? gload(a.allow + (id >> 5)) : 0xffffffffu;   // (the same choice in every thread)
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint32_t id = (ref[u] & 0x7fffffffu) + e_of;
            if (ref[u] == 0xffffffffu || id >= vocab) {
                continue;
            }
            const bool summed = (ref[u] >> 31) != 0u;
            float x = raw[u] == raw[u] ? raw[u] : NEG_INF;
            if (summed && holds_bias(id / LILY_TILE_COLS)) {
                x = with_bias(id, x);
            }
            if (masked && ((mword[u] >> (id & 31u)) & 1u) == 0u) {
                x = NEG_INF;
            }
            if (pen && ((word[u] >> (id & 31u)) & 1u) != 0u && x > NEG_INF && (x >= bound || summed)) {
                x = true_value(id, x);
            }
            if (summed) {
                lse.add_one(x, a.c2);
            }
            if (x >= bound && x > NEG_INF) {
                const uint32_t at = atomicAdd(&sh.n_cand, 1u);
                if (at < TILE_CAND_CAP) {
                    cand[at] = composite_of(x / a.temperature, id);
                }
            }
        }
    }
    if (n_r > REF_CAP && tid == 0) {
        sh.n_cand = TILE_CAND_CAP + 1u;   // too many pieces: as with too many candidates
    }
    if (want_lse) {
        lse_reduce(sh, lse);
    }
    __syncthreads();
    phase(cfg, 3);
    uint32_t n = sh.n_cand;
    __syncthreads();
    // Under a mask the bound was a guess: it stands if k allowed values reach it.  (A row that
    // has fewer allowed values altogether is drawn by the launch that follows.)
    if (masked && n < k) {
        if (tid == 0) {
            served[blockIdx.y] = 0u;
        }
        return;
    }
    bool sorted = false;
    uint32_t took = 0;
    if (n > TILE_CAND_CAP) {
        took = 2;
        select_exhaustive<DT>(a, 0, vocab, k, want_lse, cand, cfg.cand_cap, sh);
        n = min(sh.n_cand, cfg.cand_cap);
    } else {
        n = select_topk(cand, n, k, sh, sorted);
    }
    if (cfg.path_stats != nullptr && tid == 0) {
        atomicAdd(&cfg.path_stats[took], 1u);
    }
    phase(cfg, 6);
    tail<DT, false>(a, vocab, step, n, sorted, cand, sh, cfg);
    phase(cfg, 7);
}

hipError_t launch_rows_tiles(hipStream_t stream, int dtype, bool lse, bool extra, uint32_t rows,
                             const LaunchCfg& cfg_in, const float* tile_max, const float* tile_sum,
                             uint32_t tiles, const uint32_t* tile_row, uint32_t* served) {
    if (tiles == 0 || tiles > TILES_MAX) {
        return hipErrorInvalidValue;
    }
    LaunchCfg cfg = cfg_in;
    cfg.slices = 1;
    cfg.cand_cap = TILE_CAND_CAP;
    const size_t tail_bytes = (size_t)LILY_SAMPLE_K_CAP * 8 + 3 * (size_t)LILY_SAMPLE_K_CAP * 4;
    const size_t dyn_bytes = std::max(tail_bytes, (size_t)TILE_CAND_CAP * 8);
    cfg.dyn_slots = (uint32_t)(dyn_bytes / 8);
    const dim3 grid(1, rows), block(NT);
#define LILY_TILES(DT, LSE)                                                                       \
    do {                                                                                          \
        if (extra) {                                                                              \
            hipLaunchKernelGGL((k_rows_tiles<DT, LSE, true>), grid, block, dyn_bytes, stream, cfg, tile_max,  \
                               tile_sum, tiles, tile_row, served);                                \
        } else {                                                                                  \
            hipLaunchKernelGGL((k_rows_tiles<DT, LSE, false>), grid, block, dyn_bytes, stream, cfg, tile_max, \
                               tile_sum, tiles, tile_row, served);                                \
        }                                                                                         \
    } while (0)
    if (dtype == LILY_BF16) {
        if (lse) {
            LILY_TILES(LILY_BF16, true);
        } else {
            LILY_TILES(LILY_BF16, false);
        }
    } else if (lse) {
        LILY_TILES(LILY_F32, true);
    } else {
        LILY_TILES(LILY_F32, false);
    }
#undef LILY_TILES
    return hipGetLastError();
}

}  // namespace lily
