// select_stream.h - the one-pass streaming select (k <= 64).
#pragma once

#include <type_traits>

#include "device_common.h"

namespace lily {

// ------------------------------------------------------------------ streaming select
//
// The select of rows with k <= STREAM_K_MAX.  One pass, every 16-byte chunk read from memory
// once, a barrier every fourth block of NT x STREAM_UNROLL chunks:
//
//   * Bound.  Each lane keeps the maximum of what it has seen; each wave takes the kw-th
//     largest of its 64 lane maxima (kw = ceil(k' / NWAVE), a 16-step ballot search on the
//     top half of the order key).  At least k' distinct elements are at or above the
//     minimum of the waves' values, so that minimum is a lower bound of the k'-th largest
//     value; it is the same in every wave while a block is processed, which makes the run
//     reproducible.
//   * Owner side.  A lane whose chunk holds a value at or above the bound appends the whole
//     chunk (16 raw bytes + its index) to its wave's queue and leaves it out of the running
//     sum of exponentials; all other chunks only feed the lane maximum and the sum.
//   * Listed ids (ids a scratch ever counted: their true value differs from the raw one) are
//     bits of the scratch's bitmap.  Where a row needs them beside its chunks, each wave reads
//     the words that cover its own chunks of a block (64 bytes per load of 64 bf16 chunks), so
//     a lane knows which of its elements are listed without anybody gathering anything.  When
//     penalties can only lower a value, a listed element matters only if its chunk is queued
//     (it is then evaluated exactly when the queue is expanded, its count gathered from the
//     dense histogram) or summed (its raw term is booked and its true term added); otherwise
//     every listed element is evaluated on the spot.  Which rows read bits during the scan and
//     which look them up afterwards is described where the scan's modes are chosen.  Barred
//     ids of a masked row are bits of the same kind and are replaced by -inf as the chunk
//     arrives.
//   * The sum's cut is measured against a lower bound of the row's largest TRUE value: with
//     penalties that only lower, the image of the largest raw value under the penalty an id
//     with the scratch's largest count would get.
//   * The bias list's ids (at most STREAM_BIAS_CAP) are streamed as they are; after the scan
//     one thread per id looks its chunk up again, redoes the owner's tests with the bound and
//     the cut its block was scanned with, books the raw term and offers the true value.
//   * After the scan the queued chunks are expanded: their elements add their term and, at or
//     above the final bound, become candidates.
//
// Values are compared before the division by the temperature; candidates are divided
// exactly and the final check (k-th candidate strictly above anything a value below the
// bound can map to) decides whether the result stands.  Any overflow returns false.

struct StreamLds {
    u32x4* qraw;
    uint32_t* qidx;
    uint16_t* noted;    // [NWAVE][S_CAP / NWAVE] numbers (within the slice) of summed chunks
    uint32_t* win;      // [NWAVE][2][WIN_WORDS]
    float* blk_bound;   // [MAX_BLOCKS] the bound block b was filtered with
    float* blk_cut;     // [MAX_BLOCKS] the sum's cut of block b
    uint32_t* blk_flag; // [MAX_BLOCKS] 1 = chunk maxima of block b were the non-negative kind
    uint32_t* bias_id;
    float* bias_delta;
    uint64_t* fc;
    __device__ __forceinline__ void init() {
        char* b = reinterpret_cast<char*>(dyn_lds);
        qraw = reinterpret_cast<u32x4*>(b + OFF_QRAW);
        qidx = reinterpret_cast<uint32_t*>(b + OFF_QIDX);
        noted = reinterpret_cast<uint16_t*>(b + OFF_NOTED);
        win = reinterpret_cast<uint32_t*>(b + OFF_WIN);
        blk_bound = reinterpret_cast<float*>(b + OFF_BLK);
        blk_cut = reinterpret_cast<float*>(b + OFF_BLK + MAX_BLOCKS * 4);
        blk_flag = reinterpret_cast<uint32_t*>(b + OFF_BLK + MAX_BLOCKS * 8);
        bias_id = reinterpret_cast<uint32_t*>(b + OFF_BIAS);
        bias_delta = reinterpret_cast<float*>(b + OFF_BIAS + STREAM_BIAS_CAP * 4);
        fc = reinterpret_cast<uint64_t*>(b + OFF_FC);
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
    constexpr uint32_t SSEG = S_CAP / NWAVE;
    constexpr uint32_t NONE = 0xffffffffu;
    constexpr uint32_t EMASK = (1u << E) - 1u;
    constexpr uint32_t WPP = 64u * E / 32u;   // bitmap words that hold the bits of a wave's 64 chunks
    constexpr uint32_t PIECE = WPP + 1u;      // + one for rows whose chunks start inside a word
    static_assert(PIECE <= WIN_PIECE_MAX && U == 4, "window layout");
    const uint32_t tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    const uint32_t nchunks = g.ce - g.cb;
    const uint32_t nblocks = (nchunks + BLOCK - 1) / BLOCK;
    const bool pen = (a.flags & F_PEN) != 0;
    const bool masked = MASKS && a.allow != nullptr;
    const uint32_t n_bias = a.n_bias;
    const bool want_lse = LSE && a.out_logprob != nullptr;
    const float c2 = a.c2;
    const uint32_t row_words = (g.vocab + 31u) / 32u;
    if (nblocks > MAX_BLOCKS || n_bias > STREAM_BIAS_CAP) {
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
    // The first block is asked for before anything else.  (Asking for the second and third here
    // as well - twelve loads a thread in flight across the row's preparations - made the launch of
    // 1 024 rows 8 us longer per extra block.)
    u32x4 buf_a[U], buf_b[U], buf_c[U];
    if (nblocks > 0) {
        fetch(buf_a, 0);
    }
    if (tid == 0) {
        sh.n_fc = 0;
        sh.fail = 0;
        sh.n_pairs = 0;
    }
    for (uint32_t i = tid; i < n_bias; i += NT) {
        L.bias_id[i] = gload(&a.bias[i].id);
        L.bias_delta[i] = gload(&a.bias[i].delta);
    }
    __syncthreads();
    phase(cfg, 13);
    if (masked) {
        // A row whose mask admits few ids is left to the select that reads only those.
        const uint32_t w_lo = g.id_lo >> 5, w_hi = (g.id_hi + 31u) >> 5;
        uint32_t mine = 0;
        for (uint32_t i = w_lo + tid; i < w_hi; i += NT) {
            mine += (uint32_t)__popc(gload(a.allow + i) & range32_at(g.id_lo, g.id_hi, (int64_t)i * 32));
        }
        for (int o = 32; o > 0; o >>= 1) {
            mine += __shfl_xor(mine, o);
        }
        if (lane == 0) {
            sh.red_i[w] = mine;
        }
        __syncthreads();
        uint32_t n_allowed = 0;
        for (int i = 0; i < NWAVE; ++i) {
            n_allowed += sh.red_i[i];
        }
        __syncthreads();
        if (n_allowed <= min(cfg.dyn_slots, MERGE_CAP) && n_allowed <= (g.id_hi - g.id_lo) / 4u) {
            return false;  // not a failure: the sparse select takes the row
        }
    }
    // Penalties with a repetition factor of at least 1 and non-negative presence and frequency
    // terms can only lower a value.  `lowering`: no listed id's true value exceeds its raw one
    // (ids the bias list names are dealt with apart, after the scan, listed or not).
    const bool lowering = a.repetition >= 1.0f && a.presence >= 0.0f && a.frequency >= 0.0f;
    // How a row's chunks are scanned:
    //   * without bits (mode 0): rows without penalties or masks, and rows whose listed ids can
    //     only be lowered and that want no row sum - a listed id then matters in queued chunks
    //     only, and the expansion looks their bits up itself;
    //   * with bits (mode 1): every block's bits arrive beside its values - masked rows, rows
    //     whose listed ids may rise, rows with a row sum and listed ids.  A chunk above the sum's
    //     cut is summed as it arrives and the listed ids among its elements corrected on the spot;
    //   * noting (mode 2), for rows with a row sum whose listed ids can only be lowered (no
    //     mask, no bias list): scanned without bits.  A chunk above the cut is summed as it is
    //     and its number noted in a list (16 bits an entry, a segment per wave); after the scan
    //     one thread per entry looks the chunk's bits up and, for the few chunks that hold a
    //     listed id, takes the raw term off and adds the true one.  Rows with a dominant value
    //     note a few dozen chunks, or a few hundred before that value has been seen.  A flat row
    //     fills its list within a few blocks: the refresh of the bound that finds a segment
    //     three quarters full hands the blocks after the current one to mode 1 (chunks that a
    //     full segment cannot note are corrected on the spot from bits fetched there and then).
    const bool noting = pen && lowering && want_lse && !masked && n_bias == 0u;
    const bool special = masked || (pen && (!lowering || want_lse));
    // The largest count any id of the scratch ever had (kept in the first spare word behind
    // the bitmap) bounds how far penalties can lower a value.
    const uint32_t max_count = pen ? *(const LILY_CONST uint32_t*)(a.touched + row_words) : 0u;
    // Whether id is named by the bias list (its true value then comes from the pass after the scan).
    auto biased = [&](uint32_t id) -> bool {
        bool hit = false;
        for (uint32_t j = 0; j < n_bias; ++j) {
            hit = hit || L.bias_id[j] == id;
        }
        return hit;
    };
    // A listed id's true value before the temperature from its raw one: bias in list order,
    // then penalties with the count gathered from the dense histogram.  (A barred id never
    // gets here: its raw value was replaced by -inf when its chunk arrived.)
    auto true_value = [&](uint32_t id, float raw) -> float {
        uint32_t cnt = 0;
        if (pen) {
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
        return t;
    };
    // Any id's true value bounds the row's largest from below, wherever in the row it lies (in
    // another slice, too).  One id is worth the look: the one the scratch counted most often.
    // Where a sequence keeps coming back to a token its raw value is among the row's largest, and
    // the sum's cut then stands from the first block on, however late the row's largest values
    // arrive; and no other id's true value is overstated more by the penalty the cut otherwise
    // assumes (that of the largest count).
    // Its logit, count and mask bit are the same for every thread: they come by scalar loads, whose
    // results are waited for apart from the vector loads - the row's first blocks, requested above,
    // stay in flight meanwhile (a vector load here would be waited for behind all of them).
    float row_floor = NEG_INF;
    if (want_lse && pen && lowering) {
        const uint32_t heavy = *(const LILY_CONST uint32_t*)(a.touched + row_words + 1u);
        if (heavy < g.vocab && max_count != 0u) {
            const uint32_t cnt = *(const LILY_CONST uint32_t*)(a.counts + heavy);
            float raw;
            if (DT == LILY_BF16) {
                const uintptr_t at = reinterpret_cast<uintptr_t>(a.logits) + (uintptr_t)heavy * 2u;
                const uint32_t word = *(const LILY_CONST uint32_t*)(at & ~(uintptr_t)3u);
                raw = lilym_bits_f32(((at & 2u) ? word >> 16 : word & 0xffffu) << 16);
            } else {
                raw = lilym_bits_f32(*(const LILY_CONST uint32_t*)(static_cast<const uint32_t*>(a.logits) + heavy));
            }
            bool allowed = true;
            if (masked) {
                allowed = ((*(const LILY_CONST uint32_t*)(a.allow + (heavy >> 5)) >> (heavy & 31u)) & 1u) != 0u;
            }
            if (allowed) {
                float t = raw;
                for (uint32_t j = 0; j < n_bias; ++j) {
                    if (L.bias_id[j] == heavy) {
                        t += L.bias_delta[j];
                    }
                }
                if (cnt > 0u) {
                    t = t > 0.0f ? t / a.repetition : t * a.repetition;
                    t -= a.presence + a.frequency * (float)cnt;
                }
                row_floor = t;
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
    float skip_b = NEG_INF;     // the block's cut: chunks whose maximum is not above it are not summed
    uint32_t wq = 0;            // this wave's queue fill
    bool give_up = false;       // a wave's queue segment overflowed (the same in every thread)
    bool stop = false;          // mode 2 ends with block `resume` - 1 (the same in every thread)
    uint32_t resume = 0;
    float own_max = NEG_INF;    // mode 2: what this wave's own lanes bound the row's largest value by
    uint32_t sfill = 0;         // this wave's noted chunks
    uint32_t note_max = 0;      // the fullest segment of noted chunks, as of the last refresh
    WaveLse wl;
    wl.init();
    double acc_t = 0.0, acc_r = 0.0;   // true terms added one by one; raw terms to take off
    constexpr int UP_UNSET = INT_MIN;
    int up = UP_UNSET;          // this thread's double sums are relative to ref_s + up
    uint32_t parity = 0;
    // One term 2^(v*c2 - ref_s - up) of a double sum.  The exponent is formed in double: a
    // row's largest value may lie hundreds of units above the reference (fixed after the
    // first block), where an f32 difference is good to 1e-5 only.  The thread's own
    // reference ref_s + up starts at its first term and moves up (its two sums scaled down
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
            // moves to the term (the two sums, if any, scaled down by the same power of two).
            double e = (double)v * c2d - (double)ref_s;
            e = e < 1.0e9 ? (e > -1.0e9 ? e : -1.0e9) : 1.0e9;
            const int now = (int)__builtin_floor(e);
            if (up != UP_UNSET) {
                const int step = now - up;
                acc_t = __builtin_ldexp(acc_t, -step);
                acc_r = __builtin_ldexp(acc_r, -step);
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

    // What a raw value is worth at least after penalties that can only lower (the penalty of an id
    // with the scratch's largest count); the value itself for all other rows, whose floor
    // refresh_bound forms apart.
    auto lowered = [&](float m) -> float {
        if (pen && lowering && m > NEG_INF) {
            float t = m > 0.0f ? m / a.repetition : m * a.repetition;
            t -= a.presence + a.frequency * (float)max_count;
            return t;
        }
        return m;
    };
    // Brings T up to date with everything the lanes have seen, the current block included.
    auto refresh_bound = [&](bool first, bool maxima) {
        const uint32_t key16 = lane_max > NEG_INF ? (lilym_order_key(lane_max) >> 16) : 0u;
        const uint32_t P = wave_kth_key16(key16, kw);
        const float mine = P != 0u ? lilym_key_value(P << 16) : F32_LOWEST;
        const float wm = maxima ? wave_max_dpp(lane_max) : 0.0f;
        if (lane == 0) {
            sh.bound[parity][w] = mine;
            sh.wfill[parity][w] = wq;
            sh.wnote[parity][w] = sfill;
            if (maxima) {
                sh.wmax[parity][w] = wm;
            }
        }
        __syncthreads();
        float t = sh.bound[parity][0];
        for (int i = 1; i < NWAVE; ++i) {
            t = fminf(t, sh.bound[parity][i]);
        }
        T = fmaxf(T, lower_by_slack(t));
        // A wave's queue segment is full: the row gives up at once (every thread sees it).
        note_max = 0;
        for (int i = 0; i < NWAVE; ++i) {
            give_up = give_up || sh.wfill[parity][i] > QSEG;
            note_max = max(note_max, sh.wnote[parity][i]);
        }
        if (maxima) {
            float m = sh.wmax[parity][0];
            for (int i = 1; i < NWAVE; ++i) {
                m = fmaxf(m, sh.wmax[parity][i]);
            }
            // A lower bound of the row's largest TRUE value.  The largest raw value may belong
            // to a listed id: penalties that can only lower take at most what they take from an
            // id with the scratch's largest count, and that map is monotone, so the image of the
            // largest raw value bounds the largest true value from below.  (Barred ids are -inf
            // before any maximum is taken; bias ids are few and only the sum's cut depends on
            // this bound, so a positive bias on the row's best id merely cuts less.)
            row_max = fmaxf(lowered(m), row_floor);
            if (pen && !lowering && m > NEG_INF) {
                // Penalties of either sign: a listed id's value is linear in its count, so what
                // they leave of the largest raw value at the least is the least of the value
                // itself (its id may not be listed) and its images at a count of 1 and at the
                // scratch's largest count - a frequency term that lowers can outweigh a presence
                // term that raises.  Monotone in the raw value, so this bounds the largest true
                // value from below.
                const float scaled = m > 0.0f ? m / a.repetition : m * a.repetition;
                const float off = a.presence + a.frequency * fmaxf(1.0f, (float)max_count);
                const float off1 = a.presence + a.frequency;
                row_max = fminf(m, scaled - fmaxf(off, off1));
            }
            if (first) {
                // Finite and far from overflow: every term is formed as 2^(v*c2 - ref_s).
                ref_s = m > NEG_INF ? fminf(fmaxf(m * c2, -1.0e30f), 1.0e30f) : 0.0f;
            }
        }
        parity ^= 1u;
    };

    // Element j of a chunk: one compare picks the 8-byte half, one 64-bit shift the element.
    auto elem_of = [&](const u32x4& q, uint32_t j) -> float {
        const bool upper = (j & (uint32_t)(E / 2)) != 0u;
        const uint64_t half = upper ? (((uint64_t)q.w << 32) | q.z) : (((uint64_t)q.y << 32) | q.x);
        if (E == 8) {
            return lilym_bits_f32((uint32_t)(half >> ((j & 3u) * 16u)) << 16);
        }
        return lilym_bits_f32((uint32_t)(half >> ((j & 1u) * 32u)));
    };
    // The chunk with the elements of `bits` replaced by -inf.
    auto without = [&](const u32x4& q, uint32_t bits) -> u32x4 {
        u32x4 r = q;
        if (E == 8) {
            auto fix = [](uint32_t v, uint32_t two) -> uint32_t {
                const uint32_t m = ((two & 1u) ? 0x0000ffffu : 0u) | ((two & 2u) ? 0xffff0000u : 0u);
                return (v & ~m) | (0xff80ff80u & m);
            };
            r.x = fix(q.x, bits);
            r.y = fix(q.y, bits >> 2);
            r.z = fix(q.z, bits >> 4);
            r.w = fix(q.w, bits >> 6);
        } else {
            r.x = (bits & 1u) ? 0xff800000u : q.x;
            r.y = (bits & 2u) ? 0xff800000u : q.y;
            r.z = (bits & 4u) ? 0xff800000u : q.z;
            r.w = (bits & 8u) ? 0xff800000u : q.w;
        }
        return r;
    };

    // ---- the bits of a block's chunks
    // Load u of a block brings the wave 64 consecutive chunks, whose ids' bits fill WPP
    // consecutive words of a bitmap (one more when the first chunk starts inside a word): lane
    // u * WPP + q requests word q of piece u, the first four lanes the pieces' extra words.
    // Words before or after the bitmap are replaced by its first or last word: they belong to
    // chunks that are not streamed, whose bits nobody looks at.
    const uint32_t win_sh = (g.cb * (uint32_t)E - g.pad) & 31u;   // a piece's first bit inside its first word
    struct Bits {
        uint32_t t, tx;   // listed ids: this lane's word, this lane's extra word
        uint32_t m, mx;   // allowed ids (masked rows)
    };
    const uint32_t* t_words = pen ? a.touched : reinterpret_cast<const uint32_t*>(g.base);
    const uint32_t* m_words = masked ? a.allow : reinterpret_cast<const uint32_t*>(g.base);
    auto piece_word0 = [&](uint32_t u) -> int32_t {   // in block 0
        const int32_t first = (int32_t)((g.cb + u * NT + w * 64u) * (uint32_t)E) - (int32_t)g.pad;
        return first >> 5;  // arithmetic: ids before the row lie in "word -1"
    };
    // This lane's two words of block 0's window; a block's chunks cover BLOCK * E / 32 words.
    const int32_t win_w0 = piece_word0(min(lane / WPP, 3u)) + (int32_t)(lane % WPP);
    const int32_t win_w1 = piece_word0(lane & 3u) + (int32_t)WPP;
    const int32_t win_hi = (int32_t)row_words - 1;
    auto bits_request = [&](Bits& d, uint32_t b) {
        const int32_t step = (int32_t)(b * (BLOCK * (uint32_t)E / 32u));
        const uint32_t i0 = (uint32_t)min(max(win_w0 + step, 0), win_hi);
        const uint32_t i1 = (uint32_t)min(max(win_w1 + step, 0), win_hi);
        d.t = gload(t_words + i0);
        d.tx = gload(t_words + i1);
        if (MASKS) {
            d.m = gload(m_words + i0);
            d.mx = gload(m_words + i1);
        }
    };
    // The wave passes its words through its own piece of LDS (its own writes and reads only:
    // LDS serves a wave's operations in order, so no barrier is needed) and every lane takes
    // the E bits of each of its four chunks.
    auto bits_take = [&](const Bits& d, uint32_t& tb_all, uint32_t (&mb)[U]) {
        uint32_t* mine = L.win + w * (2u * WIN_WORDS);
        const uint32_t u = lane / WPP, q = lane % WPP;
        if (u < 4u) {
            mine[u * PIECE + q] = d.t;
            if (MASKS) {
                mine[WIN_WORDS + u * PIECE + q] = d.m;
            }
        }
        if (lane < 4u) {
            mine[lane * PIECE + WPP] = d.tx;
            if (MASKS) {
                mine[WIN_WORDS + lane * PIECE + WPP] = d.mx;
            }
        }
        // (Nothing for the hardware to do; the compiler must not move the reads above the writes
        // of other lanes.)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        const uint32_t off = win_sh + lane * (uint32_t)E;
#pragma unroll
        for (int v = 0; v < U; ++v) {
            const uint32_t at = (uint32_t)v * PIECE + (off >> 5);
            const uint64_t two = ((uint64_t)mine[at + 1u] << 32) | mine[at];
            tb_all |= pen ? ((uint32_t)(two >> (off & 31u)) & EMASK) << (8 * v) : 0u;
            if (MASKS) {
                const uint64_t mtwo = ((uint64_t)mine[WIN_WORDS + at + 1u] << 32) | mine[WIN_WORDS + at];
                mb[v] = masked ? ~(uint32_t)(mtwo >> (off & 31u)) & EMASK : 0u;   // 1 = barred
            } else {
                mb[v] = 0u;
            }
        }
        __builtin_amdgcn_wave_barrier();
    };

    // Listed ids of a block's chunks that are not queued, on the spot.  `todo`: a byte per chunk
    // of the block, bit j = element j is a listed id that matters.  One loop for the whole
    // block: the lanes take their first such element together, so the gathers of its counts
    // are in flight together and waited for once.
    //   * Rows without a row sum whose listed ids may rise: the true value is offered as a
    //     candidate.  (With a row sum such chunks are queued instead.)
    //   * Rows with a row sum whose listed ids can only be lowered, chunks whose raw terms went
    //     into the running sum: the raw term is taken off again and the true term (never the
    //     larger one, so it fits the same reference) added, in the lane's own f32 sum.
    auto fix_listed = [&](const u32x4 (&cur)[U], uint32_t b, uint32_t todo) {
        while (todo != 0u) {
            const uint32_t i = (uint32_t)__builtin_ctz(todo);
            todo &= todo - 1u;
            const uint32_t u = i >> 3, j = i & 7u;
            u32x4 q = cur[0];
            q = u == 1u ? cur[1] : q;
            q = u == 2u ? cur[2] : q;
            q = u == 3u ? cur[3] : q;
            const float raw = elem_of(q, j);
            if (!(raw > NEG_INF)) {
                continue;  // barred as well, or -inf to begin with: no term, no candidate
            }
            const uint32_t id = g.id_of(g.cb + (b * U + u) * NT + tid, (int)j);
            if (n_bias != 0u && biased(id)) {
                continue;  // the pass after the scan speaks for it
            }
            const float t = true_value(id, raw);
            if (lowering) {
                const float off = __builtin_amdgcn_exp2f(__builtin_fmaf(raw, c2, -wl.ref));
                const float on = t > skip_b ? __builtin_amdgcn_exp2f(__builtin_fmaf(t, c2, -wl.ref)) : 0.0f;
                wl.s += on - off;
                wl.booked += off;
            } else if (t >= T && t > NEG_INF) {
                const uint32_t at = atomicAdd(&sh.n_fc, 1u);
                if (at < FC_CAP) {
                    L.fc[at] = composite_of(t / a.temperature, id);
                }
            }
        }
    };

    // The exact terms of one chunk of the slice, one by one in double: every element whose value
    // (the true one for the listed ids of `dm`) lies above `cut`.
    auto chunk_terms = [&](const u32x4& q, uint32_t c, uint32_t dm, float cut, auto&& add_term) {
#pragma unroll 1
        for (uint32_t j = 0; j < (uint32_t)E; ++j) {
            float x = elem_of(q, j);
            if (!(x > cut)) {
                continue;   // (penalties that only lower: a listed id below the cut stays below it)
            }
            if ((dm >> j) & 1u) {
                x = true_value(g.id_of(c, (int)j), x);
            }
            if (x > cut) {
                add_term(x);
            }
        }
    };

    // Blocks b + 1 and b + 2 are on their way while block b is worked on (three register
    // buffers that swap roles): one block in flight per wave leaves the memory idle whenever
    // a wave's arithmetic outlasts its load.
    const float lse_cut = (log2f((float)g.vocab) + 21.0f) * (a.temperature * 0.6931471805599453f);
    // The scan is compiled twice, for rows whose chunks come with bits and for rows without:
    // left as a test inside the loop, the bits' loads would be loads that may be skipped, and
    // every wait behind them would drain the blocks requested ahead.
    auto scan = [&](auto with_bits, auto queueing, uint32_t b_first) {
        constexpr bool SP = decltype(with_bits)::value;
        constexpr bool QM = LSE && decltype(queueing)::value;   // mode 2
        Bits bits_a = {}, bits_b = {}, bits_c = {};
        auto work = [&](u32x4 (&cur)[U], const Bits& bcur, uint32_t b) {
            if (give_up || stop || b >= nblocks) {
                return;
            }
            // A wave that has further to go asks to be issued first, so that the workgroups that
            // share a compute unit advance together instead of in the order they arrived (the
            // arbiter otherwise favours the oldest wave, and the rows dispatched last scan alone at
            // the end).  Four levels: the quarter of the way the wave has come, rows dispatched
            // earlier counted as two blocks further on per generation.
            {
                const uint32_t gen = min((blockIdx.y * 4u) / max(gridDim.y, 1u), 3u);
                const uint32_t q = min(((b + 2u * (3u - gen)) * 4u) / (nblocks + 6u), 3u);
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
            // tb_all: a byte per chunk of the block, bit j = element j is a listed id.
            uint32_t tb_all = 0u, mb[U] = {0u, 0u, 0u, 0u};
            if (SP) {
                bits_take(bcur, tb_all, mb);
            }
            if (!full_block(b)) {
                const uint32_t ninf = DT == LILY_BF16 ? 0xff80ff80u : 0xff800000u;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint32_t c = g.cb + (b * U + u) * NT + tid;
                    if (c < g.main_lo || c >= g.main_hi) {
                        cur[u] = u32x4{ninf, ninf, ninf, ninf};
                        tb_all &= ~(0xffu << (8 * u));
                        mb[u] = 0u;
                    }
                }
            }
            if (MASKS && masked) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    cur[u] = without(cur[u], mb[u]);
                }
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
                if (__ballot(bm > 0x7f800000) != 0ull) {
                    // A positive NaN among the block's values (its pattern lies above +inf's):
                    // the block's maxima are taken again the way that ignores NaNs.
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        m8[u] = chunk_max<DT>(cur[u]);
                        block_max = max2_raw(block_max, m8[u]);
                    }
                    lane_max = max2_raw(lane_max, block_max);
                } else {
                    block_max = lilym_bits_f32((uint32_t)bm);
                    lane_max = lilym_bits_f32((uint32_t)max((int)lilym_f32_bits(lane_max), bm));
                }
            } else {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    m8[u] = chunk_max<DT>(cur[u]);
                    block_max = max2_raw(block_max, m8[u]);
                }
                lane_max = max2_raw(lane_max, block_max);
            }
            // Rows with a row sum whose listed ids may rise: a chunk that holds a listed id is
            // queued whatever its values (the queue's expansion evaluates every element exactly).
            uint32_t forced = 0u;   // bit u: chunk u is queued for its listed ids
            if (SP && LSE && want_lse && !lowering) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    forced |= ((tb_all >> (8 * u)) & 0xffu) != 0u ? 1u << u : 0u;
                }
            }
            uint32_t fix = 0u;   // a byte per chunk: its listed ids that are evaluated on the spot
            // Mode 2: a lane whose chunk lies above the cut without being queued notes the chunk's
            // number; its terms are formed after the scan, against the row's final cut (most of
            // what a stale cut lets through is dropped there without a single exponential).  A
            // lane whose wave's segment is full forms its chunk's terms on the spot instead.
            auto note_chunk = [&](int u, bool wanted) {
                const uint64_t mask = __ballot(wanted);
                if (mask != 0ull) {
                    const uint32_t rank = __builtin_amdgcn_mbcnt_hi(
                        (uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
                    const uint32_t at = sfill + rank;
                    if (wanted && at < SSEG) {
                        L.noted[w * SSEG + at] = (uint16_t)((b * U + (uint32_t)u) * NT + tid);
                    }
                    if (sfill + (uint32_t)__popcll(mask) > SSEG) {
                        if (wanted && at >= SSEG) {
                            const uint32_t c = g.cb + (b * U + (uint32_t)u) * NT + tid;
                            if (c >= g.main_lo && c < g.main_hi) {
                                // Every element's count, asked for whatever the element is worth
                                // and waited for here, inside the branch: a fixed number of loads
                                // and no loop around them, so that the waits of the scan's own
                                // loads keep counting past this branch.
                                uint32_t cnt[E];
#pragma unroll
                                for (int j = 0; j < E; ++j) {
                                    cnt[j] = gload(a.counts + g.id_of(c, j));
                                }
#pragma unroll
                                for (int j = 0; j < E; ++j) {
                                    asm volatile("" : "+v"(cnt[j]));
                                }
#pragma unroll
                                for (int j = 0; j < E; ++j) {
                                    float x = elem_of(cur[u], (uint32_t)j);
                                    if (cnt[j] > 0u) {
                                        x = x > 0.0f ? x / a.repetition : x * a.repetition;
                                        x -= a.presence + a.frequency * (float)cnt[j];
                                    }
                                    if (x > skip_b) {
                                        acc_t += term_d(x);
                                    }
                                }
                            }
                        }
                    }
                    sfill = min(sfill + (uint32_t)__popcll(mask), SSEG);
                }
            };
            bool some = false;
            if (LSE && want_lse) {
                // A term 2^(v*c2) below 2^-21 / vocab of the largest one seen cannot move the row
                // sum by more than 2^-21 of it, even with every element of the row at that level:
                // such chunks are left out, by a rule every thread of the block can evaluate.
                skip_b = fmaxf(row_max, own_max) - lse_cut;
                wl.skip_below = skip_b;
                // Rows with a dominant value skip nearly every block as a whole.
                some = __ballot(block_max > skip_b) != 0ull;
                if (QM && some) {
                    // Between two refreshes of the row's maxima the wave's own lanes may have seen
                    // more than the row knew then: what they saw bounds the row's largest value
                    // just as well, and spares a row whose largest value comes late the noting of
                    // chunk after chunk against a cut that is out of date.
                    own_max = lowered(wave_max_dpp(lane_max));
                    skip_b = fmaxf(row_max, own_max) - lse_cut;
                    wl.skip_below = skip_b;
                    some = __ballot(block_max > skip_b) != 0ull;
                }
                if (!QM && some) {
                    wl.prepare(block_max < T_prev ? block_max : T_prev, c2);  // nothing above T_prev is added
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const bool sum_it = !(m8[u] >= T_prev) && ((forced >> u) & 1u) == 0u;
                        wl.template add_prepared<DT>(cur[u], m8[u], c2, sum_it);
                    }
                }
            }
            // The bound moves most in the first blocks: refresh it for each of them, then for
            // every fourth block (each refresh is a ballot search and a barrier).  The row's
            // maxima behind the sum's cut follow with every other of those.
            if (b < 4u || (b & 3u) == 0u) {
                refresh_bound(b == 0, b == 0 || (LSE && want_lse && (b < 4u || (b & 7u) == 0u)));
                if (LSE && want_lse) {
                    // The cut follows at once: what is summed from here on (all of block 0, whose
                    // chunks were held back above for want of a bound) is measured against the
                    // largest value known now.  Terms between the old cut and the new one that
                    // were summed already are as negligible as those that were not.
                    skip_b = fmaxf(row_max, own_max) - lse_cut;
                    wl.skip_below = skip_b;
                    if (QM && some) {
                        some = __ballot(block_max > skip_b) != 0ull;
                    }
                }
                if (QM && note_max >= SSEG * 3u / 4u) {
                    stop = true;
                    resume = b + 1u;   // this block is still finished here
                }
            }
            if (n_bias != 0u && tid == 0) {
                L.blk_bound[b] = T;
                L.blk_cut[b] = skip_b;
                L.blk_flag[b] = nonneg ? 1u : 0u;
            }
            const bool any_late = !QM && LSE && want_lse && T != T_prev &&
                                  __ballot(block_max >= T_prev && block_max > skip_b) != 0ull;
            // When values can only be lowered, a listed id in a chunk that was neither queued nor
            // summed is below the bound and below the sum's cut with its true value too: nothing
            // of it is evaluated (most chunks of most rows; rows with a dominant value sum next
            // to nothing, and their waves skip even the test).
            const bool fix_any = SP && (!lowering || (LSE && want_lse && __ballot(block_max > skip_b) != 0ull));
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t c = g.cb + (b * U + u) * NT + tid;
                const bool pass = m8[u] >= T || ((forced >> u) & 1u) != 0u;
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
                if (QM && some) {
                    note_chunk(u, !pass && m8[u] > skip_b);
                }
                if (SP && fix_any) {
                    const uint32_t tb = (tb_all >> (8 * u)) & 0xffu;
                    const bool matters = !lowering || (LSE && want_lse && m8[u] > skip_b);
                    fix |= (tb != 0u && !pass && matters) ? tb << (8 * u) : 0u;
                }
            }
            if (SP && fix != 0u) {
                fix_listed(cur, b, fix);
            }
        };
        // A request past the last block asks for the last block again (its lines are in the
        // cache and nothing uses the result): with the same loads in flight on every path the
        // wait for a block's data leaves the blocks requested after it in flight, where a request
        // that may be skipped makes that wait count as if it had been.
        auto request = [&](u32x4 (&dst)[U], Bits& bdst, uint32_t b) {
            const uint32_t bb = min(b, nblocks - 1u);
            if (SP) {
                bits_request(bdst, bb);
            }
            fetch(dst, bb);
        };
        if (nblocks == 0) {
            refresh_bound(true, true);  // the same barriers in every workgroup
        } else if (b_first < nblocks) {
            if (b_first != 0u) {
                fetch(buf_a, b_first);   // (block 0 was requested at the very start)
            }
            if (SP) {
                bits_request(bits_a, b_first);
            }
            request(buf_b, bits_b, b_first + 1u);
            for (uint32_t b = b_first; b < nblocks && !give_up && !stop; b += 3) {
                request(buf_c, bits_c, b + 2);
                work(buf_a, bits_a, b);
                if (b + 1 < nblocks) {
                    request(buf_a, bits_a, b + 3);
                    work(buf_b, bits_b, b + 1);
                    if (b + 2 < nblocks) {
                        request(buf_b, bits_b, b + 4);
                        work(buf_c, bits_c, b + 2);
                    }
                }
            }
        }
    };
    if (noting) {
        scan(std::false_type{}, std::true_type{}, 0u);
        if (stop && !give_up) {
            stop = false;
            scan(std::true_type{}, std::false_type{}, resume);
        }
    } else if (special) {
        scan(std::true_type{}, std::false_type{}, 0u);
    } else {
        scan(std::false_type{}, std::false_type{}, 0u);
    }
    phase(cfg, 2);

    // ---- after the scan
    const float wave_top = (LSE && noting) ? wave_max_dpp(lane_max) : 0.0f;
    if (lane == 0) {
        sh.qfill[w] = wq;
        sh.nfill[w] = sfill;
        sh.wmax[parity][w] = wave_top;
    }
    __syncthreads();
    phase(cfg, 14);
    // Mode 2 forms its terms after the scan, when the row's largest streamed value is known:
    // they are relative to that value's exponent (none of them exceeds 1: penalties only lower)
    // and add up in `acc_p`.
    double ref_p = 0.0, acc_p = 0.0;
    bool simple_p = false;   // the same in every thread
    if (LSE && noting) {
        // The row's cut as the whole scan leaves it: what follows forms no term below it.
        float m = sh.wmax[parity][0];
        for (int i = 1; i < NWAVE; ++i) {
            m = fmaxf(m, sh.wmax[parity][i]);
        }
        const float true_low = fmaxf(lowered(m), row_floor);   // the largest true value is not below this
        skip_b = fmaxf(skip_b, true_low - lse_cut);
        // One reference serves when every term above the cut is a double relative to it: the
        // largest raw value may lie far above what the penalties leave of it, and a temperature
        // near 0 stretches that distance beyond a double's range (such rows keep the references
        // that move, term_d).
        simple_p = m > NEG_INF && (m - true_low) * c2 <= 900.0f;
        ref_p = simple_p ? (double)m * c2d : 0.0;
        ref_p = ref_p < 1.0e30 ? (ref_p > -1.0e30 ? ref_p : -1.0e30) : 1.0e30;
    }
    auto term_p = [&](float v) -> double {
        const double d = __builtin_fma((double)v, c2d, -ref_p);
        return d > -1000.0 ? pow2_d(d < 1000.0 ? d : 1000.0) : 0.0;   // (-inf and NaN: nothing)
    };
    const float filt = T;
    {
        bool overflow = give_up;
        for (int i = 0; i < NWAVE; ++i) {
            overflow = overflow || sh.qfill[i] > QSEG;
        }
        if (overflow) {
            return stream_fail(cfg, 4u);
        }
    }
    auto offer = [&](float u, uint32_t id) {
        if (u >= filt && u > NEG_INF) {
            const uint32_t at = atomicAdd(&sh.n_fc, 1u);
            if (at < FC_CAP) {
                L.fc[at] = composite_of(u / a.temperature, id);
            }
        }
    };
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
    {
        uint32_t seg_end[NWAVE], total = 0;
#pragma unroll
        for (int i = 0; i < NWAVE; ++i) {
            total += sh.qfill[i];
            seg_end[i] = total;
        }
        auto queue_slot = [&](uint32_t ch) -> uint32_t {
            uint32_t ww = 0, before = 0;
#pragma unroll
            for (int i = 0; i + 1 < NWAVE; ++i) {
                if (ch >= seg_end[i]) {
                    ww = (uint32_t)i + 1u;
                    before = seg_end[i];
                }
            }
            return ww * QSEG + (ch - before);
        };
        // Mode 2's noted chunks: their 16 bytes and their bits of the scratch's bitmap are asked
        // for first, four chunks a thread, and looked at behind the queue's listing below, which
        // touches LDS only.
        uint32_t n_seg_end[NWAVE], n_total = 0;
#pragma unroll
        for (int i = 0; i < NWAVE; ++i) {
            n_total += (LSE && noting) ? sh.nfill[i] : 0u;
            n_seg_end[i] = n_total;
        }
        auto noted_at = [&](uint32_t e) -> uint32_t {
            uint32_t ww = 0, before = 0;
#pragma unroll
            for (int i = 0; i + 1 < NWAVE; ++i) {
                if (e >= n_seg_end[i]) {
                    ww = (uint32_t)i + 1u;
                    before = n_seg_end[i];
                }
            }
            return (uint32_t)L.noted[ww * SSEG + (e - before)];
        };
        uint32_t n_cc[4] = {0u, 0u, 0u, 0u}, n_dm[4] = {0u, 0u, 0u, 0u};
        u32x4 n_q[4] = {};
        bool n_ok[4] = {false, false, false, false};
        auto noted_request = [&](uint32_t e0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t e = e0 + (uint32_t)i * NT;
                const uint32_t c = g.cb + noted_at(min(e, n_total - 1u));
                // (A chunk outside the slice was scanned as -inf throughout, and is noted where
                // chunk maxima are the kind that reports +0 for it.)
                n_ok[i] = e < n_total && c >= g.main_lo && c < g.main_hi;
                n_cc[i] = min(c, c_last);
                n_q[i] = gload(reinterpret_cast<const u32x4*>(g.base + (n_cc[i] << 4)));
                n_dm[i] = bits32_at(a.touched, row_words, (int64_t)g.id_of(n_cc[i], 0)) & EMASK;
            }
        };
        // A chunk whose largest value lies above the final cut adds its terms (listed ids with
        // their true values); the others - all that a cut which was out of date while the row's
        // largest values had yet to come let through - are dropped.
        auto noted_consume = [&]() {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (n_ok[i] && chunk_max<DT>(n_q[i]) > skip_b) {
                    chunk_terms(n_q[i], n_cc[i], n_dm[i], skip_b, [&](float x) {
                        if (simple_p) {
                            acc_p += term_p(x);
                        } else {
                            acc_t += term_d(x);
                        }
                    });
                }
            }
        };
        if (n_total != 0u) {
            noted_request(tid);
        }
        // Rows under penalties that only lower (the common kind): every element of a queued chunk
        // that matters by its raw value - at or above the bound, or above the sum's cut - is
        // listed as an (id, raw value) pair, wave by wave; then one thread per pair gathers the
        // id's count, so that all of the row's gathers are one round trip to memory.  (A listed
        // id's true value is not above its raw one: what does not matter raw does not matter.)
        uint64_t* pairs = L.fc;   // the candidates' place: they arrive once the pairs are in registers
        const bool pair_path = pen && lowering;
        if (pair_path) {
            for (uint32_t ch0 = 0; ch0 < total; ch0 += NT) {
                const uint32_t ch = ch0 + tid;
                uint32_t todo = 0, c = 0;
                u32x4 q = {};
                if (ch < total) {
                    const uint32_t slot = queue_slot(ch);
                    q = L.qraw[slot];
                    c = L.qidx[slot];
                    float v[E];
                    unpack<DT>(q, v);
#pragma unroll
                    for (int j = 0; j < E; ++j) {
                        const bool term = want_lse && v[j] > skip_b;
                        const bool cand = v[j] >= filt && v[j] > NEG_INF;
                        todo |= (term || cand) ? 1u << j : 0u;
                    }
                }
                while (__ballot(todo != 0u) != 0ull) {
                    const bool has = todo != 0u;
                    const uint32_t j = has ? (uint32_t)__builtin_ctz(todo) : 0u;
                    todo &= todo - 1u;   // (0 stays 0)
                    const uint32_t id = g.id_of(c, (int)j);
                    const bool push = has && !(n_bias != 0u && biased(id));
                    const uint64_t mask = __ballot(push);
                    if (mask != 0ull) {
                        const uint32_t rank = __builtin_amdgcn_mbcnt_hi(
                            (uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
                        uint32_t first = 0;
                        if (rank == 0u && push) {
                            first = atomicAdd(&sh.n_pairs, (uint32_t)__popcll(mask));
                        }
                        first = (uint32_t)__builtin_amdgcn_readlane((int)first, __builtin_ctzll(mask));
                        if (push && first + rank < FC_CAP) {
                            pairs[first + rank] = ((uint64_t)lilym_f32_bits(elem_of(q, j)) << 32) | id;
                        }
                    }
                }
            }
        }
        if (n_total != 0u) {
            noted_consume();
            for (uint32_t e0 = tid + 4u * NT; e0 < n_total + tid; e0 += 4u * NT) {   // (the same trips in every thread)
                noted_request(e0);
                noted_consume();
            }
        }
        bool paired = false;
        if (pair_path) {
            __syncthreads();
            paired = sh.n_pairs <= FC_CAP;
        }
        if (paired) {
            const uint32_t n_pairs = sh.n_pairs;
            uint64_t pr[4];
            uint32_t cnt[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t at = tid + (uint32_t)i * NT;
                pr[i] = at < n_pairs ? pairs[at] : 0ull;
                cnt[i] = gload(a.counts + (uint32_t)pr[i]);   // (id 0 for an empty place)
            }
            __syncthreads();   // every pair is in a register: the candidates may take their place
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool valid = tid + (uint32_t)i * NT < n_pairs;
                const uint32_t id = (uint32_t)pr[i];
                float x = lilym_bits_f32((uint32_t)(pr[i] >> 32));
                if (cnt[i] > 0u) {
                    x = x > 0.0f ? x / a.repetition : x * a.repetition;
                    x -= a.presence + a.frequency * (float)cnt[i];
                }
                if (valid && want_lse && x > skip_b) {
                    if (simple_p) {
                        acc_p += term_p(x);
                    } else {
                        acc_t += term_d(x);
                    }
                }
                const bool cand = valid && x >= filt && x > NEG_INF;
                const uint64_t mask = __ballot(cand);
                if (mask != 0ull) {
                    const uint32_t rank = __builtin_amdgcn_mbcnt_hi(
                        (uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
                    uint32_t first = 0;
                    if (rank == 0u && cand) {
                        first = atomicAdd(&sh.n_fc, (uint32_t)__popcll(mask));
                    }
                    first = (uint32_t)__builtin_amdgcn_readlane((int)first, __builtin_ctzll(mask));
                    if (cand && first + rank < FC_CAP) {
                        L.fc[first + rank] = composite_of(x / a.temperature, id);
                    }
                }
            }
        }
        // Every other row (and a row whose pairs outgrew their place): one thread per queued
        // chunk (the waves' segments counted through in order): its elements add their term and
        // are offered - listed ones with their true value, ids of the bias list not at all (the
        // pass below speaks for them).
        for (uint32_t ch = tid; !paired && ch < total; ch += NT) {
            const uint32_t slot = queue_slot(ch);
            const u32x4 q = L.qraw[slot];
            const uint32_t c = L.qidx[slot];
            // Its listed elements, from the scratch's bitmap (barred ids are -inf already).
            const uint32_t dm =
                pen ? bits32_at(a.touched, row_words, (int64_t)g.id_of(c, 0)) & EMASK : 0u;
            float v[E];
            unpack<DT>(q, v);
            // Few elements of a queued chunk matter (usually the one that got it queued):
            // they are marked first and then taken one at a time, in ascending order, instead
            // of eight branches that some lane of the wave enters every time.  A listed element
            // whose value can only be lowered matters under the same conditions as any other.
            uint32_t todo = 0, finite = 0;
#pragma unroll
            for (int j = 0; j < E; ++j) {
                const bool term = want_lse && v[j] > skip_b;  // the cut of the streamed terms
                const bool cand = v[j] >= filt && v[j] > NEG_INF;
                todo |= (term || cand) ? 1u << j : 0u;
                finite |= v[j] > NEG_INF ? 1u << j : 0u;
            }
            todo = (todo & ~dm) | (dm & (lowering ? todo : finite));
            while (todo != 0u) {
                const uint32_t j = (uint32_t)__builtin_ctz(todo);
                todo &= todo - 1u;
                float x = elem_of(q, j);
                const uint32_t id = g.id_of(c, (int)j);
                if (n_bias != 0u && biased(id)) {
                    continue;
                }
                if ((dm >> j) & 1u) {
                    x = true_value(id, x);
                }
                if (want_lse && x > skip_b) {
                    acc_t += term_d(x);
                }
                offer(x, id);
            }
        }
    }
    phase(cfg, 8);
    if (n_bias != 0u) {
        // The bias list's ids were streamed with their raw values and left alone by everything
        // above.  One thread per id - the first entry that names it - looks the chunk up again
        // and redoes its owner's tests with the bound, the cut and the kind of maximum its block
        // was scanned with: a summed chunk's raw term is booked, the true term (bias in list
        // order, then penalties) added and the true value offered.
        for (uint32_t i = tid; i < n_bias; i += NT) {
            const uint32_t id = L.bias_id[i];
            bool first = true;
            for (uint32_t j = 0; j < i; ++j) {
                first = first && L.bias_id[j] != id;
            }
            const uint32_t b = block_of(id);
            if (!first || b == NONE || (masked && !bit_of(a.allow, id))) {
                continue;  // an edge id, or a barred id (streamed as -inf)
            }
            const uint32_t c = (id + g.pad) / E;
            u32x4 q = gload(reinterpret_cast<const u32x4*>(g.base + (c << 4)));
            if (masked) {
                q = without(q, ~bits32_at(a.allow, row_words, (int64_t)g.id_of(c, 0)) & EMASK);
            }
            float cm = L.blk_flag[b] != 0u ? chunk_max_nonneg<DT>(q) : chunk_max<DT>(q);
            if (lilym_f32_bits(cm) > 0x7f800000u && !(cm < 0.0f)) {
                cm = chunk_max<DT>(q);   // a NaN in the chunk: as its owner did
            }
            const float cut = L.blk_cut[b];
            bool queued = cm >= L.blk_bound[b];
            if (LSE && want_lse && pen && !lowering) {
                // (a row with a sum whose listed ids may rise queued every chunk that holds a
                // listed id, whatever its values: none of that chunk's raw terms was summed)
                queued = queued || (bits32_at(a.touched, row_words, (int64_t)g.id_of(c, 0)) & EMASK) != 0u;
            }
            const bool summed = !queued && cm > cut;
            const float raw = elem_of(q, (id + g.pad) % E);
            const float t = true_value(id, raw);
            if (want_lse) {
                if (summed) {
                    acc_r += term_d(raw);
                }
                if (t > cut) {
                    acc_t += term_d(t);
                }
            }
            offer(t, id);
        }
    }
    // Ids of partial 16-byte chunks at the row's ends were not streamed: exact, one by one.
    for (int side = 0; side < 2; ++side) {
        const uint32_t lo = side == 0 ? g.id_lo : g.edge_hi_begin;
        const uint32_t hi = side == 0 ? g.edge_lo_end : g.id_hi;
        for (uint32_t id = lo + tid; id < hi; id += NT) {
            const float u = pre_temperature_of<DT>(a, id);
            if (want_lse) {
                acc_t += term_d(u);
            }
            offer(u, id);
        }
    }
    phase(cfg, 9);
    if (want_lse) {
        // Mode 2 as a rule holds nothing but its post-scan terms, all relative to one reference:
        // the waves' sums meet in LDS behind one barrier.  A thread with a sum of another kind
        // (terms formed during the scan, edge ids, a scan that went on with bits beside the
        // chunks) sends the row the long way below.
        const bool other_sums = up != UP_UNSET || !(wl.s == 0.0f) || !(wl.booked == 0.0f);
        const double p_wave = wave_sum_d_dpp(acc_p);
        if (lane == 0) {
            sh.red_d[w] = p_wave;
        }
        const bool long_way = __syncthreads_or((!simple_p || other_sums) ? 1 : 0) != 0;
        double p_all = 0.0;
        for (int i = 0; i < NWAVE; ++i) {
            p_all += sh.red_d[i];
        }
        if (!long_way) {
            phase(cfg, 10);
            if (tid == 0) {
                sh.lse_mc = ref_p;
                sh.lse_s = p_all;
            }
        } else {
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
            double part[4];
            {
                double d = stream_at - (double)ref_w;  // <= 1 where there is a sum
                d = d < -1000.0 ? -1000.0 : d;
                const double scale = pow2_d(d);
                part[0] = wl.s > 0.0f ? (double)wl.s * scale : 0.0;
                part[3] = wl.booked > 0.0f ? (double)wl.booked * scale : 0.0;
            }
            part[1] = __builtin_ldexp(acc_r, down);
            part[2] = __builtin_ldexp(acc_t, down);
    #pragma unroll
            for (int i = 0; i < 4; ++i) {
                part[i] = wave_sum_d(part[i]);
                if (lane == 0) {
                    sh.red3[i][w] = part[i];
                }
            }
            if (lane == 0) {
                sh.red_i[w] = (uint32_t)ref_w;
            }
            // A NaN logit in a summed chunk leaves its wave's running sum a NaN: such a logit is
            // worth -inf, and the row's sum is formed again from every value.
            const bool poisoned = __syncthreads_or(wl.s != wl.s ? 1 : 0) != 0;
            int ref_all = (int)sh.red_i[0];
            for (int i = 1; i < NWAVE; ++i) {
                ref_all = max(ref_all, (int)sh.red_i[i]);
            }
    #pragma unroll
            for (int i = 0; i < 4; ++i) {
                part[i] = 0.0;
                for (int ww = 0; ww < NWAVE; ++ww) {
                    const int at = (int)sh.red_i[ww];
                    part[i] += at == UP_UNSET ? 0.0 : __builtin_ldexp(sh.red3[i][ww], at - ref_all);
                }
            }
            if (ref_all == UP_UNSET) {
                ref_all = 0;  // no term anywhere: the sums are zero
            }
            // part[0]: the running sums, the listed ids' raw terms of part[3] already taken off (and
            // their true terms added); part[1]: raw terms still to take off; part[2]: terms added
            // one by one.
            const double streamed = part[0], booked = part[1], exact = part[2], taken = part[3];
            const double rest = streamed - booked;
            // The streamed sums are f32: taking the listed ids' raw terms off again leaves an error of
            // about 1e-6 of what was streamed.  Where that is more than 20 times the row's sum (listed
            // ids held nearly everything that was streamed, and nothing larger was added exactly) the
            // difference is too coarse.
            const bool coarse = poisoned ||
                                (booked + taken > 0.0 &&
                                 !((rest > 0.0 ? rest : 0.0) + exact > 0.05 * (streamed + taken)));
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
                double mc = (double)ref_s + (double)ref_all;
                double sum = (rest > 0.0 ? rest : 0.0) + exact;
                if (p_all > 0.0) {
                    // Mode 2's post-scan terms have a reference of their own: the higher of the
                    // two serves both (what lies 2^1000 below the other adds nothing).
                    if (!(sum > 0.0)) {
                        mc = ref_p;
                        sum = p_all;
                    } else {
                        const double top = mc > ref_p ? mc : ref_p;
                        const double d0 = mc - top, d1 = ref_p - top;
                        sum = sum * pow2_d(d0 < -1000.0 ? -1000.0 : d0) +
                              p_all * pow2_d(d1 < -1000.0 ? -1000.0 : d1);
                        mc = top;
                    }
                }
                sh.lse_mc = mc;
                sh.lse_s = sum;
            }
    
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
