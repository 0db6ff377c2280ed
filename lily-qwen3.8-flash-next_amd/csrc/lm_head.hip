// lm_head.hip - the producer of the logits: hidden[rows, d] x weight[vocab, d]^T in bf16 on the
// matrix cores, with an epilogue that leaves beside the bf16 logits what the draw needs of
// every tile of 128 columns: its largest value and the sum of its exponentials.
//
// The call sites this stands in for: the language-model head in front of the per-row draws
// (src/qwen4exp/batch.rs:573-582, src/qwen4exp/model.rs:2959-2966 and 4157-4164).
#include <hip/hip_runtime.h>

#include "launch.h"

namespace lily {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t w32x4 __attribute__((ext_vector_type(4)));

namespace head {
constexpr int BM = 128;              // rows of a workgroup's tile
constexpr int BN = LILY_TILE_COLS;   // columns of a workgroup's tile = the width of a summary
constexpr int BK = 64;               // depth of one staged piece
constexpr int ROW_BYTES = BK * 2 + 16;   // a staged row and its padding: rows 8 apart share banks
constexpr int OPERAND_BYTES = BM * ROW_BYTES;
constexpr int STAGE_BYTES = 2 * OPERAND_BYTES;     // hidden rows, then weight rows
constexpr int LDS_BYTES = 2 * STAGE_BYTES;         // two stages
static_assert(BM == BN, "one loader serves both operands");
static_assert(LDS_BYTES >= 4 * BM * 4 + BM * 4, "the epilogue's reductions reuse the stages");
}  // namespace head

// One workgroup of 256 threads per 128 x 128 tile of the logits; its four waves take a
// quarter each (64 x 64: 2 x 2 products of 32 x 32 x 16).  Both operands are contiguous along
// d, which is how a lane of the matrix instruction wants its 8 values: rows are staged in
// LDS 64 columns of d at a time (16-byte loads from memory one stage ahead of the
// arithmetic, 16-byte reads out of LDS, rows padded so that 8 rows cover all banks).
//
// Workgroups are numbered so that the tiles over one block of 128 weight rows - one per 128
// rows of the batch - run on the same XCD one after the other: the weight rows, the large
// operand, are then fetched from memory once and served to the other tiles by that XCD's L2.
__global__ void __launch_bounds__(256)
k_lm_head_bf16(const uint16_t* __restrict__ hidden, uint64_t hidden_stride,
               const uint16_t* __restrict__ weight, uint64_t weight_stride, uint32_t rows,
               uint32_t d, uint32_t vocab, const float* __restrict__ c2_of_row,
               uint16_t* __restrict__ logits, uint64_t logits_stride, float* __restrict__ tile_max,
               float* __restrict__ tile_sum, uint32_t tiles_per_row, uint32_t m_tiles) {
    using namespace head;
    extern __shared__ __align__(16) char lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
    const uint32_t n_tile = (slot / m_tiles) * 8u + xcd, m_tile = slot % m_tiles;
    if (n_tile >= tiles_per_row) {
        return;
    }
    const uint32_t m0 = m_tile * BM, n0 = n_tile * BN;
    const uint32_t wm = wave >> 1, wn = wave & 1u;

    // The loader: thread t brings pieces t, t + 256, ... of 16 bytes; a staged row has 8.
    const uint16_t* src_h[4];
    const uint16_t* src_w[4];
    uint32_t dst[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t piece = tid + 256u * (uint32_t)i, r = piece >> 3, kc = piece & 7u;
        const uint32_t hr = min(m0 + r, rows - 1u), wr = min(n0 + r, vocab - 1u);
        src_h[i] = hidden + (uint64_t)hr * hidden_stride + kc * 8u;
        src_w[i] = weight + (uint64_t)wr * weight_stride + kc * 8u;
        dst[i] = r * ROW_BYTES + kc * 16u;
    }
    w32x4 next_h[4], next_w[4];
    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            next_h[i] = *reinterpret_cast<const w32x4*>(src_h[i] + k0);
            next_w[i] = *reinterpret_cast<const w32x4*>(src_w[i] + k0);
        }
    };
    auto stage = [&](uint32_t buf) {
        char* base = lds + buf * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<w32x4*>(base + dst[i]) = next_h[i];
            *reinterpret_cast<w32x4*>(base + OPERAND_BYTES + dst[i]) = next_w[i];
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                acc[mi][ni][v] = 0.0f;
            }
        }
    }
    // A lane's operand values: row lane % 32 of the 32, 8 values of d from (lane / 32) * 8 on.
    const uint32_t frag = (lane & 31u) * ROW_BYTES + (lane >> 5) * 16u;
    const uint32_t a_at = wm * 64u * ROW_BYTES + frag;
    const uint32_t b_at = OPERAND_BYTES + wn * 64u * ROW_BYTES + frag;

    fetch(0);
    stage(0);
    __syncthreads();
    const uint32_t steps = d / BK;
    for (uint32_t s = 0; s < steps; ++s) {
        const uint32_t buf = s & 1u;
        if (s + 1u < steps) {
            fetch((s + 1u) * BK);
        }
        const char* base = lds + buf * STAGE_BYTES;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            bf16x8 a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                a[i] = *reinterpret_cast<const bf16x8*>(base + a_at + i * 32 * ROW_BYTES + kk * 32);
                b[i] = *reinterpret_cast<const bf16x8*>(base + b_at + i * 32 * ROW_BYTES + kk * 32);
            }
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
                for (int ni = 0; ni < 2; ++ni) {
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mi], b[ni], acc[mi][ni], 0, 0, 0);
                }
            }
        }
        if (s + 1u < steps) {
            stage(buf ^ 1u);   // nobody reads that stage: the barrier below closed the step before
        }
        __syncthreads();
    }

    // ---- epilogue.  Element v of a lane's 16 sits in row 8 * (v / 4) + 4 * (lane / 32) + v % 4
    // of its 32 x 32 product, column lane % 32.  Values are rounded to bf16 first: the maximum
    // and the sum describe the logits as they are stored.
    float* red = reinterpret_cast<float*>(lds);              // [2][BM] by column half
    float* row_max = red + 2 * BM;                           // [BM]
    float* row_c2 = row_max + BM;                            // [BM]
    if (tid < (uint32_t)BM) {
        row_c2[tid] = c2_of_row[min(m0 + tid, rows - 1u)];
    }
    const float NEG = -__builtin_huge_valf();
    uint32_t bits[2][2][16];
    float val[2][2][16];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const bool in_vocab = n0 + wn * 64u + (uint32_t)ni * 32u + (lane & 31u) < vocab;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float f = acc[mi][ni][v];   // (a bit_cast of the element itself reads element 0)
                const uint32_t u = __builtin_bit_cast(uint32_t, f);
                // round to nearest even; a NaN stays one (quiet), and counts as -inf below
                const uint32_t r = (u & 0x7fffffffu) > 0x7f800000u ? ((u >> 16) | 0x40u)
                                                                   : ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
                bits[mi][ni][v] = r;
                const float x = __builtin_bit_cast(float, r << 16);
                val[mi][ni][v] = (in_vocab && x == x) ? x : NEG;
            }
        }
    }
    auto across32 = [&](float x, auto op) -> float {
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) {
            x = op(x, __shfl_xor(x, o));
        }
        return x;
    };
    auto row_of = [&](int mi, int v) -> uint32_t {
        return wm * 64u + (uint32_t)mi * 32u + 8u * (uint32_t)(v >> 2) + 4u * (lane >> 5) + (uint32_t)(v & 3);
    };
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float m = across32(fmaxf(val[mi][0][v], val[mi][1][v]),
                                     [](float p, float q) { return fmaxf(p, q); });
            if ((lane & 31u) == 0u) {
                red[wn * BM + row_of(mi, v)] = m;
            }
        }
    }
    __syncthreads();
    if (tid < (uint32_t)BM) {
        row_max[tid] = fmaxf(red[tid], red[BM + tid]);
    }
    __syncthreads();
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t r = row_of(mi, v);
            const float c = row_c2[r], top = row_max[r] * c;
            float e = 0.0f;
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                const float x = val[mi][ni][v];
                e += x > NEG ? __builtin_amdgcn_exp2f(__builtin_fmaf(x, c, -top)) : 0.0f;
            }
            e = across32(e, [](float p, float q) { return p + q; });
            if ((lane & 31u) == 0u) {
                red[wn * BM + r] = e;
            }
        }
    }
    __syncthreads();
    if (tid < (uint32_t)BM && m0 + tid < rows) {
        const size_t at = (size_t)(m0 + tid) * tiles_per_row + n_tile;
        tile_max[at] = row_max[tid];
        tile_sum[at] = row_max[tid] > NEG ? red[tid] + red[BM + tid] : 0.0f;
    }
    // the logits themselves
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            const uint32_t col = n0 + wn * 64u + (uint32_t)ni * 32u + (lane & 31u);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t r = m0 + row_of(mi, v);
                if (r < rows && col < vocab) {
                    logits[(uint64_t)r * logits_stride + col] = (uint16_t)bits[mi][ni][v];
                }
            }
        }
    }
}

hipError_t launch_lm_head_bf16(hipStream_t stream, const void* hidden, uint64_t hidden_stride,
                               const void* weight, uint64_t weight_stride, uint32_t rows, uint32_t d,
                               uint32_t vocab, const float* c2_of_row, void* logits,
                               uint64_t logits_stride, float* tile_max, float* tile_sum) {
    using namespace head;
    static bool sized = false;
    if (!sized) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(k_lm_head_bf16),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        if (e != hipSuccess) {
            return e;
        }
        sized = true;
    }
    const uint32_t tiles_per_row = (vocab + BN - 1u) / BN, m_tiles = (rows + BM - 1u) / BM;
    const uint32_t groups = (tiles_per_row + 7u) / 8u;
    hipLaunchKernelGGL(k_lm_head_bf16, dim3(8u * groups * m_tiles), dim3(256), LDS_BYTES, stream,
                       reinterpret_cast<const uint16_t*>(hidden), hidden_stride,
                       reinterpret_cast<const uint16_t*>(weight), weight_stride, rows, d, vocab,
                       c2_of_row, reinterpret_cast<uint16_t*>(logits), logits_stride, tile_max, tile_sum,
                       tiles_per_row, m_tiles);
    return hipGetLastError();
}

}  // namespace lily
