// lm_head_codes.hip - the language-model head over the reference's affine codes for a decode
// step: up to 16 hidden rows against 4- or 8-bit weights, read once at the speed of memory.
//
// The reference's form for few rows (gemv_q4_bf16_f32out / gemv_q8_bf16_f32out,
// src/kernels/metal/quant.metal:8-60 and 130-176): the codes are never turned into weights; a
// group's part of a logit is  scale * sum(q * x) + bias * sum(x)  with f32 sums.  Here sum(q * x)
// and sum(x) of a group of 64 come out of the matrix cores - the codes as bf16 integers (exact),
// a block of ones beside them - and the scale and bias meet the sums once per group and column.
#include <hip/hip_runtime.h>

#include "launch.h"

namespace lily {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t w32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t w32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr int CB = LILY_TILE_COLS / 32;   // blocks of 16 columns a wave multiplies: half a tile's
constexpr int THREADS = 512;              // eight waves: two halves of the columns x four shares of d
constexpr int AHEAD = 4;                  // stages asked from memory ahead of the one being multiplied
constexpr int NBUF = 2;                   // stages of codes in LDS: one multiplied, one being written
constexpr int STAGE_BYTES = LILY_TILE_COLS * 128;   // 128 bytes (one line of memory) of every row
constexpr int PART_CB = 4 * 64 + 16;      // floats of one block's partial sums (padded: two blocks
                                          // read side by side then lie in different banks)
constexpr int PART_SHARE = 2 * CB * PART_CB;   // one share of d: all 128 columns
// (the partial sums reuse the stages' place)
constexpr int RING_BYTES = NBUF * STAGE_BYTES > 4 * PART_SHARE * 4 ? NBUF * STAGE_BYTES : 4 * PART_SHARE * 4;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __builtin_bit_cast(float, b << 16); }

// The product instruction: 16 x 16 outputs over 32 values of d.  Lane l gives row (or column)
// l % 16, the 8 values of d from 8 * (l / 16) on; it receives column l % 16, rows 4 * (l / 16) + v.
__device__ __forceinline__ f32x4 product(const w32x4& a, const w32x4& b, const f32x4& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                   c, 0, 0, 0);
}

// Bytes of LDS a launch needs: the stages, then every scale and bias of the tile's 128 columns.
inline size_t codes_lds_bytes(uint32_t groups) { return (size_t)RING_BYTES + (size_t)LILY_TILE_COLS * groups * 4u; }

}  // namespace

// One workgroup of eight waves per 128 columns (one summary).  The codes pass through LDS as
// they lie in memory: a stage is 128 bytes - one line - of each of the 128 rows, brought by 16
// loads of 1 KB (two a wave, eight whole lines each), AHEAD stages on their way in registers,
// written to LDS one pass before they are multiplied.  (A lane's own operand would be 8 bytes of
// each of 16 rows: the 64 lines such a load touches, not its bytes, bounded an earlier form at a
// seventh of the memory's speed.  Loads that write LDS themselves keep only what LDS holds in
// flight, which is too little here.)  The stage's 256 (4-bit) or 128 (8-bit) values of d are
// split among four waves, the 128 columns between two; the four partial tiles are added through
// LDS at the end.  The scales and biases of the whole tile are brought into LDS once, ahead of
// the first stage.
//
// 4-bit codes become bf16 without arithmetic: 0x4300 | q is the bf16 128 + q, two codes a
// register by one and-or ((word >> 4p) & 0x000f000f | 0x43004300: codes p and p + 4, so the
// hidden values are put in that order too), and the 128 is taken off with the bias (bias - 128
// * scale meets the same sum of x).  8-bit codes go through the byte-to-f32 conversion, whose
// upper half is the bf16.
template <int WBITS>
__global__ void __launch_bounds__(THREADS, 4)   // (four waves a SIMD: two workgroups a compute unit)
k_lm_head_codes(const uint16_t* __restrict__ hidden, uint64_t hidden_stride, const uint32_t* __restrict__ codes,
                uint64_t weight_stride, uint32_t rows, uint32_t d, uint32_t vocab,
                const float* __restrict__ c2_of_row, float* __restrict__ logits, uint64_t logits_stride,
                float* __restrict__ tile_max, float* __restrict__ tile_sum, uint32_t tiles_per_row,
                const uint16_t* __restrict__ scales, const uint16_t* __restrict__ biases, uint32_t group_shift,
                unsigned long long* trace) {
    // Diagnostic stamps, compiled in with -DLILY_HEAD_TRACE: [workgroup][8] device-clock values
    // (0 start, 1 scales and first stage written, 2 past the barrier, 3 loop done, 4 end).
#ifdef LILY_HEAD_TRACE
#define HEAD_MARK(i) do { if (trace != nullptr && threadIdx.x == 0) { trace[(size_t)blockIdx.x * 8 + (i)] = wall_clock64(); } } while (0)
#else
#define HEAD_MARK(i)
#endif
    HEAD_MARK(0);
    constexpr int STEPS = WBITS == 4 ? 2 : 1;          // products over 32 values a wave makes per stage and block
    constexpr uint32_t STAGE_K = 128u * 8u / WBITS;    // values of d in a stage
    constexpr uint32_t WAVE_K = STAGE_K / 4u;          // ... of which a wave multiplies these
    extern __shared__ __align__(16) char lds[];
    float* part = reinterpret_cast<float*>(lds);       // [4 shares][2 * CB][4 v x 64 lanes, padded], at the end
    uint32_t* sz = reinterpret_cast<uint32_t*>(lds + RING_BYTES);   // scales, then biases
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t share = wave & 3u, half = wave >> 2;
    const uint32_t c = lane & 15u, kq = lane >> 4;
    const uint32_t n_tile = blockIdx.x, n0 = n_tile * LILY_TILE_COLS;
    const uint32_t nstages = d / STAGE_K, groups = d >> group_shift, pairs = groups >> 1;
    // Each tile walks d from a place of its own and wraps round: rows lie a power of two apart
    // for the usual d, and tiles that all start at column 0 and advance in step queue up at one
    // memory channel after the other.
    const uint32_t rot = (n_tile * 5u) % nstages;
    auto place = [&](uint32_t stage_no) -> uint32_t {
        uint32_t at = min(stage_no, nstages - 1u) + rot;
        return at >= nstages ? at - nstages : at;
    };

    // ---- who brings what.  Load i of a wave is the 1 KB block 2 * wave + i of a stage: the
    // lines of 8 columns, lane l the 16 bytes that belong at l * 16 - piece (l % 8) ^ (l / 8) of
    // column l / 8 (the pieces of a line change places by the column's number: 16 columns'
    // operands are then read out of all banks).
    const char* from_c[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t col = 8u * (2u * wave + (uint32_t)i) + (lane >> 3), q = (lane & 7u) ^ (lane >> 3);
        from_c[i] = reinterpret_cast<const char*>(codes) + (uint64_t)min(n0 + col, vocab - 1u) * weight_stride * 4u + q * 16u;
    }
    // A lane's hidden values: row c (the last one again past `rows`), the wave's share of the
    // stage, 8 values a product from 8 * kq on (two neighbouring eights for 4-bit codes).
    const char* from_a = reinterpret_cast<const char*>(hidden) + (uint64_t)min(c, rows - 1u) * hidden_stride * 2u +
                         (share * WAVE_K + kq * 8u * STEPS) * 2u;
    // (every load unconditional, past the end of d the last stage again: the compiler then
    // counts the loads in flight and waits for the oldest only)
    auto fetch_codes = [&](w32x4 (&l)[2], uint32_t stage_no) {
        const uint32_t at = place(stage_no);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            l[i] = *reinterpret_cast<const w32x4*>(from_c[i] + at * 128u);
        }
    };
    auto fetch_hidden = [&](w32x4 (&l)[STEPS], uint32_t stage_no) {
        const char* p = from_a + (uint64_t)place(stage_no) * (STAGE_K * 2u);
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            l[t] = *reinterpret_cast<const w32x4*>(p + 16 * t);
        }
    };
    auto stage = [&](const w32x4 (&l)[2], uint32_t buf) {
        char* base = lds + buf * STAGE_BYTES + wave * 2048u + lane * 16u;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            *reinterpret_cast<w32x4*>(base + i * 1024) = l[i];
        }
    };
    // where a lane's codes lie in a stage (block cb: column 64 * half + 16 * cb + c; the wave's
    // share of the line is its pieces 2 * share and the next, 8 bytes a lane) and its scales in sz
    uint32_t code_at[CB], scale_at[CB], turn[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        const uint32_t col = 64u * half + 16u * (uint32_t)cb + c, q = 2u * share + (kq >> 1);
        code_at[cb] = (col >> 3) * 1024u + ((col & 7u) * 8u + (q ^ (col & 7u))) * 16u + (kq & 1u) * 8u;
        scale_at[cb] = col * pairs;
        turn[cb] = col % pairs;
    }

    f32x4 total[CB];
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        total[cb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const w32x4 ONES = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
    const f32x4 ZERO = {0.0f, 0.0f, 0.0f, 0.0f};

    auto multiply = [&](const w32x4 (&hid)[STEPS], uint32_t stage_no, uint32_t buf, bool real) {
        const uint32_t keep = real ? 0xffffffffu : 0u;
        w32x4 a[STEPS];
#pragma unroll
        for (int t = 0; t < STEPS; ++t) {
            const w32x4 h = hid[t] & keep;
            if constexpr (WBITS == 4) {
                // values 0..7 in the order 0 4 1 5 2 6 3 7 of the codes' registers
                a[t].x = __builtin_amdgcn_perm(h.z, h.x, 0x05040100u);
                a[t].y = __builtin_amdgcn_perm(h.z, h.x, 0x07060302u);
                a[t].z = __builtin_amdgcn_perm(h.w, h.y, 0x05040100u);
                a[t].w = __builtin_amdgcn_perm(h.w, h.y, 0x07060302u);
            } else {
                a[t] = h;
            }
        }
        // the sums of the hidden values themselves, where the products' sums will lie
        f32x4 xs = product(a[0], ONES, ZERO);
        if constexpr (STEPS == 2) {
            xs = product(a[1], ONES, xs);
        }
        // the wave's values of this stage lie in one group (64 values, or 32 of one)
        const uint32_t g = (place(stage_no) * STAGE_K + share * WAVE_K) >> group_shift, w = g >> 1, odd = (g & 1u) * 16u;
        const char* codes_in = lds + buf * STAGE_BYTES;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            const w32x2 raw = *reinterpret_cast<const w32x2*>(codes_in + code_at[cb]);
            w32x4 b[STEPS];
            if constexpr (WBITS == 4) {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const uint32_t word = raw[t];
                    b[t].x = (word & 0x000f000fu) | 0x43004300u;
                    b[t].y = ((word >> 4) & 0x000f000fu) | 0x43004300u;
                    b[t].z = ((word >> 8) & 0x000f000fu) | 0x43004300u;
                    b[t].w = ((word >> 12) & 0x000f000fu) | 0x43004300u;
                }
            } else {
                uint32_t out[4];
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const uint32_t word = raw[p >> 1];
                    const float lo = (float)((word >> (16 * (p & 1))) & 0xffu);
                    const float hi = (float)((word >> (16 * (p & 1) + 8)) & 0xffu);
                    out[p] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, hi), __builtin_bit_cast(uint32_t, lo),
                                                   0x07060302u);
                }
                b[0] = w32x4{out[0], out[1], out[2], out[3]};
            }
            f32x4 qx = product(a[0], b[0], ZERO);
            if constexpr (STEPS == 2) {
                qx = product(a[1], b[1], qx);
            }
            uint32_t at = w + turn[cb];
            at = at >= pairs ? at - pairs : at;
            const float s = bf16_bits_to_f32((sz[scale_at[cb] + at] >> odd) & 0xffffu);
            float z = bf16_bits_to_f32((sz[LILY_TILE_COLS * pairs + scale_at[cb] + at] >> odd) & 0xffffu);
            if constexpr (WBITS == 4) {
                z = __builtin_fmaf(-128.0f, s, z);
            }
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                total[cb][v] = __builtin_fmaf(s, qx[v], __builtin_fmaf(z, xs[v], total[cb][v]));
            }
        }
    };

    // ---- the stages.  Two rings of registers hold the loads on their way, AHEAD stages deep:
    // in pass s codes[j] holds the codes of stage s + 1 and hid[j] the hidden values of stage s.
    // Every pass multiplies the stage that lies in one half of LDS, writes the next one's codes
    // into the other half (nobody reads it: the barrier that closed the pass before saw to
    // that), asks for the codes and the hidden values AHEAD further on into the registers just
    // freed, and meets the other waves.
    w32x4 codes_ring[AHEAD][2], hid[AHEAD][STEPS];
    fetch_codes(codes_ring[0], 0u);
    stage(codes_ring[0], 0u);
#pragma unroll
    for (int j = 0; j < AHEAD; ++j) {
        fetch_hidden(hid[j], (uint32_t)j);
        fetch_codes(codes_ring[j], (uint32_t)j + 1u);
        __builtin_amdgcn_sched_barrier(0);   // (in this order: the loop waits for the oldest only)
    }
    // (the first stages are on their way while the scales are brought)
    // ---- the tile's scales and biases, two groups (one word) at a time: word w of column col
    // at sz[col * pairs + (w + col) % pairs] (turned by the column's number: the 16 columns a
    // product reads at once then lie in different banks), the biases behind all the scales.
    {
        const uint32_t words = LILY_TILE_COLS * pairs;
        // (unconditional loads, the last word again past the end: eight in flight a thread)
        for (uint32_t base = 0; base < 2u * words; base += 8u * THREADS) {
            uint32_t got[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const uint32_t i = min(base + (uint32_t)u * THREADS + tid, 2u * words - 1u);
                const uint32_t arr = i >= words ? 1u : 0u, j = i - arr * words, col = j / pairs, w = j - col * pairs;
                const uint16_t* src = (arr != 0u ? biases : scales) + (uint64_t)min(n0 + col, vocab - 1u) * groups + 2u * w;
                got[u] = *reinterpret_cast<const uint32_t*>(src);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const uint32_t i = min(base + (uint32_t)u * THREADS + tid, 2u * words - 1u);
                const uint32_t arr = i >= words ? 1u : 0u, j = i - arr * words, col = j / pairs, w = j - col * pairs;
                sz[arr * words + col * pairs + (w + col) % pairs] = got[u];   // (the last word by several: the same value)
            }
        }
    }
    HEAD_MARK(1);
    __syncthreads();   // (the scales and stage 0 are written)
    HEAD_MARK(2);
    const uint32_t padded = (nstages + AHEAD - 1u) / AHEAD * AHEAD;
    static_assert(AHEAD % 2 == 0, "the halves of LDS alternate within a trip");
    for (uint32_t s0 = 0; s0 < padded; s0 += AHEAD) {
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) {
            const uint32_t s = s0 + (uint32_t)j, buf = (uint32_t)j & 1u;
            multiply(hid[j], s, buf, s < nstages);
            stage(codes_ring[j], buf ^ 1u);
            // (nor may the compiler move the requests down to where their values are used)
            __builtin_amdgcn_sched_barrier(0);
            fetch_hidden(hid[j], s + AHEAD);
            fetch_codes(codes_ring[j], s + 1u + AHEAD);
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
        }
    }
    __syncthreads();

    HEAD_MARK(3);
    // ---- the four partial tiles, added; thread t then holds column t % 128 of the rows
    // 4 * (t / 128) .. + 3.
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            part[share * PART_SHARE + (half * CB + cb) * PART_CB + v * 64 + lane] = total[cb][v];
        }
    }
    __syncthreads();
    const uint32_t col_in = tid & 127u, rq = tid >> 7;   // (a wave's threads share rq)
    const uint32_t col = n0 + col_in;
    const float NEG = -__builtin_huge_valf();
    float x[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t r = 4u * rq + (uint32_t)j;
        const uint32_t at = (col_in >> 4) * PART_CB + (uint32_t)j * 64u + rq * 16u + (col_in & 15u);
        x[j] = (part[at] + part[PART_SHARE + at]) + (part[2 * PART_SHARE + at] + part[3 * PART_SHARE + at]);
        if (r < rows && col < vocab) {
            logits[(uint64_t)r * logits_stride + col] = x[j];
        }
        // what a stored value counts for: a NaN and a column outside the vocabulary count as -inf
        x[j] = (col < vocab && x[j] == x[j]) ? x[j] : NEG;
    }
    __syncthreads();
    // each row's largest value and sum of exponentials over the 128 columns (two waves a row)
    float* red = part;            // [8 waves][4]
    float* row_max = part + 32;   // [16]
    auto across = [&](float v, auto op) -> float {
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) {
            v = op(v, __shfl_xor(v, o));
        }
        return v;
    };
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float m = across(x[j], [](float p, float q) { return fmaxf(p, q); });
        if (lane == 0u) {
            red[wave * 4u + (uint32_t)j] = m;
        }
    }
    __syncthreads();
    // (row r: waves 2 * (r / 4) and the next, entry r % 4 of each)
    if (tid < 16u) {
        const uint32_t w0 = 2u * (tid >> 2);
        row_max[tid] = fmaxf(red[w0 * 4u + (tid & 3u)], red[(w0 + 1u) * 4u + (tid & 3u)]);
    }
    __syncthreads();
    float e[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t r = 4u * rq + (uint32_t)j;
        const float cc = c2_of_row[min(r, rows - 1u)], top = row_max[r] * cc;
        e[j] = x[j] > NEG ? __builtin_amdgcn_exp2f(__builtin_fmaf(x[j], cc, -top)) : 0.0f;
    }
    // (red is free again: its readers passed the barrier above)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float sum = across(e[j], [](float p, float q) { return p + q; });
        if (lane == 0u) {
            red[wave * 4u + (uint32_t)j] = sum;
        }
    }
    __syncthreads();
    if (tid < 16u && tid < rows) {
        const uint32_t w0 = 2u * (tid >> 2);
        const float sum = red[w0 * 4u + (tid & 3u)] + red[(w0 + 1u) * 4u + (tid & 3u)];
        const size_t at = (size_t)tid * tiles_per_row + n_tile;
        const float keep_max = row_max[tid];
        tile_max[at] = keep_max;
        tile_sum[at] = keep_max > NEG ? sum : 0.0f;
    }
    HEAD_MARK(4);
}

template <int WBITS>
static hipError_t launch_codes(hipStream_t stream, const void* hidden, uint64_t hidden_stride, const void* weight,
                               uint64_t weight_stride, uint32_t rows, uint32_t d, uint32_t vocab,
                               const float* c2_of_row, void* logits, uint64_t logits_stride, float* tile_max,
                               float* tile_sum, const HeadWeights& wq) {
    const uint32_t tiles_per_row = (vocab + LILY_TILE_COLS - 1u) / LILY_TILE_COLS;
    const size_t lds = codes_lds_bytes(d >> wq.group_shift);
    // (more than the 64 KB a kernel may have without asking: said once per device and size)
    static size_t sized[64] = {};
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) {
        return e;
    }
    if (device < 0 || device >= 64 || sized[device] < lds) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(k_lm_head_codes<WBITS>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            return e;
        }
        if (device >= 0 && device < 64) {
            sized[device] = lds;
        }
    }
    hipLaunchKernelGGL((k_lm_head_codes<WBITS>), dim3(tiles_per_row), dim3(THREADS), lds, stream,
                       static_cast<const uint16_t*>(hidden), hidden_stride, static_cast<const uint32_t*>(weight),
                       weight_stride, rows, d, vocab, c2_of_row, static_cast<float*>(logits), logits_stride,
                       tile_max, tile_sum, tiles_per_row, static_cast<const uint16_t*>(wq.scales),
                       static_cast<const uint16_t*>(wq.biases), wq.group_shift,
                       wq.trace_words >= (unsigned long long)tiles_per_row * 8u ? wq.trace : nullptr);
    return hipGetLastError();
}

bool lm_head_codes_serves(uint32_t rows, uint32_t d, uint32_t vocab, uint64_t hidden_stride, uint64_t weight_stride,
                          const HeadWeights& wq) {
    if ((wq.bits != 4u && wq.bits != 8u) || rows < 1u || rows > 16u || wq.group_shift < 6u) {
        return false;
    }
    // whole stages (128 bytes of codes a row), an even number of groups a row (their scales are
    // read two at a time), all the tile's scales in LDS beside the stages
    const uint32_t stage_k = 128u * 8u / wq.bits, groups = d >> wq.group_shift;
    return d >= stage_k && d % stage_k == 0u && groups % 2u == 0u && (groups << wq.group_shift) == d &&
           codes_lds_bytes(groups) <= 160u * 1024u;
}

hipError_t launch_lm_head_codes(hipStream_t stream, const void* hidden, uint64_t hidden_stride, const void* weight,
                                uint64_t weight_stride, uint32_t rows, uint32_t d, uint32_t vocab,
                                const float* c2_of_row, void* logits, uint64_t logits_stride, float* tile_max,
                                float* tile_sum, const HeadWeights& wq) {
    if (!lm_head_codes_serves(rows, d, vocab, hidden_stride, weight_stride, wq)) {
        return hipErrorInvalidValue;
    }
    if (wq.bits == 4u) {
        return launch_codes<4>(stream, hidden, hidden_stride, weight, weight_stride, rows, d, vocab, c2_of_row,
                               logits, logits_stride, tile_max, tile_sum, wq);
    }
    return launch_codes<8>(stream, hidden, hidden_stride, weight, weight_stride, rows, d, vocab, c2_of_row, logits,
                           logits_stride, tile_max, tile_sum, wq);
}

}  // namespace lily
