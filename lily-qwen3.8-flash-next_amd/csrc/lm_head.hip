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

// x as the lane CTRL names holds it (DPP controls: 0x120 + n = rotate right by n within each
// row of 16 lanes).
template <int CTRL>
__device__ __forceinline__ float rotated(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}

// A workgroup's tile and how its four waves share it.  WAVES_M x (4 / WAVES_M) waves, each
// MI x NI products of 32 x 32; the tile is WAVES_M * MI * 32 rows by 128 columns (the width of a
// summary), staged BK columns of d at a time, AHEAD stages of loads in flight (what is in flight
// has to cover the memory's latency at the rate the tiles consume it).
template <int WAVES_M_, int MI_, int NI_, int BK_, int AHEAD_, int RESIDENT_, bool DIRECT_ = false>
struct HeadTile {
    // DIRECT: the loads write LDS themselves (global_load_lds_dwordx4, a wave's 64 pieces side by
    // side), AHEAD + 1 stages in LDS; otherwise they pass through registers into two stages.
    static constexpr bool DIRECT = DIRECT_;
    static constexpr int RESIDENT = RESIDENT_;   // workgroups a compute unit is to hold (bounds the registers)
    static constexpr int WAVES_M = WAVES_M_, WAVES_N = 4 / WAVES_M_, MI = MI_, NI = NI_, BK = BK_;
    static constexpr int AHEAD = AHEAD_;   // stages asked from memory ahead of the one being multiplied
    static constexpr int BM = WAVES_M * MI * 32;
    static constexpr int BN = WAVES_N * NI * 32;
    static constexpr int PIECES = BK / 8;                  // 16-byte pieces of a staged row
    // A staged row: 128 bytes of d and 16 of padding (8 rows then cover all banks), or 64 bytes
    // without padding whose four 16-byte pieces change places by the row's number (piece ^
    // (row / 4) % 4): rows r, r + 4, r + 8 and r + 12 start in the same bank, so the pieces of
    // one column that 16 lanes read from 16 rows in a row lie in 16 different groups of banks.
    static constexpr bool SWIZZLED = BK == 32;
    static constexpr int ROW_BYTES = SWIZZLED ? BK * 2 : BK * 2 + 16;
    static constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;  // hidden rows, then weight rows
    static constexpr int LDS_BYTES = (DIRECT ? AHEAD + 1 : 2) * STAGE_BYTES;
    static constexpr int A_PER = BM * PIECES / 256, B_PER = BN * PIECES / 256;   // pieces a thread brings
    static_assert(BN == LILY_TILE_COLS, "a workgroup's columns are one summary");
    static_assert(BM * PIECES % 256 == 0 && BN * PIECES % 256 == 0 && A_PER >= 1, "whole pieces per thread");
    static_assert(!DIRECT || SWIZZLED, "the direct loads fill 64-byte rows");
    static_assert(LDS_BYTES >= (WAVES_N + 2) * BM * 4, "the epilogue's reductions reuse the stages");
};

// One workgroup of 256 threads per tile of the logits.  Both operands are contiguous along d,
// which is how a lane of the matrix instruction wants its 8 values: rows are staged in LDS BK
// columns of d at a time (16-byte loads from memory several stages ahead of the arithmetic,
// 16-byte reads out of LDS).  The shapes: 32 rows for a decode step of a few sequences (the weights are
// then read once at the speed of memory and the matrix cores idle), 256 rows - each wave 128 x
// 64, six operand reads out of LDS for eight products, loads that write LDS themselves - for a
// batch, whose bound is the matrix cores and, just behind, the bandwidth of LDS.
//
// Workgroups are numbered so that an XCD's L2 holds the hidden rows its workgroups share (see
// the numbering at the top of the kernel).
//
// OUT_F32: the logits are stored as the f32 sums they are (the reference's sampler reads F32
// logits, src/kernels/sample.rs:263), the summaries describe those; otherwise rounded to bf16.
// WBITS 4 / 8: the weights are the reference's affine codes (QuantWeights, src/weights.rs:27-36:
// u32 words of eight 4-bit or four 8-bit codes, low code first, a bf16 scale and bias per group
// of a row), turned into bf16 as dequant_q4_bf16 / dequant_q8_bf16 turn them (w = q * scale +
// bias in f32 - here one fused operation -, rounded to bf16: src/kernels/metal/quant.metal:179-233)
// on their way into LDS;
// `weight` then points at the codes, weight_stride counts words, and a row has
// (d >> group_shift) groups.  (Tiles whose loads pass through registers only.)
struct HeadQuant {
    const uint16_t* scales;   // bf16 [vocab][d >> group_shift]
    const uint16_t* biases;
    uint32_t group_shift;
};

template <class T, bool OUT_F32, int WBITS>
__global__ void __launch_bounds__(256, T::RESIDENT)
k_lm_head_bf16(const uint16_t* __restrict__ hidden, uint64_t hidden_stride,
               const uint16_t* __restrict__ weight, uint64_t weight_stride, uint32_t rows,
               uint32_t d, uint32_t vocab, const float* __restrict__ c2_of_row,
               void* __restrict__ logits_out, uint64_t logits_stride, float* __restrict__ tile_max,
               float* __restrict__ tile_sum, uint32_t tiles_per_row, uint32_t m_tiles, HeadQuant quant) {
    static_assert(WBITS == 0 || !T::DIRECT, "codes pass through registers");
    constexpr int BM = T::BM, BN = T::BN, BK = T::BK, MI = T::MI, NI = T::NI, ROW_BYTES = T::ROW_BYTES;
    extern __shared__ __align__(16) char lds[];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    // Which tile: consecutive workgroups go to consecutive XCDs (eight of them, an L2 each).  An
    // XCD keeps to one block of BM hidden rows for as long as it can - that block (BM x d x 2
    // bytes) then stays in its L2 and is shared by all its workgroups, which stream different
    // blocks of weight rows past it; the XCDs that hold other blocks of hidden rows stream the
    // same weights at about the same time and find them in the memory-side cache.  With up to 8
    // blocks of hidden rows the XCDs are divided among the blocks and split the weights' blocks
    // between them; with more, an XCD takes every eighth block in turn.
    const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
    uint32_t m_tile, n_tile;
    if (m_tiles <= 8u) {
        m_tile = xcd % m_tiles;
        const uint32_t rank = xcd / m_tiles, sharers = (8u - m_tile + m_tiles - 1u) / m_tiles;
        n_tile = rank + slot * sharers;
        if (n_tile >= tiles_per_row) {
            return;
        }
    } else {
        m_tile = xcd + 8u * (slot / tiles_per_row);
        n_tile = slot % tiles_per_row;
        if (m_tile >= m_tiles) {
            return;
        }
    }
    const uint32_t m0 = m_tile * BM, n0 = n_tile * BN;
    const uint32_t wm = wave / T::WAVES_N, wn = wave % T::WAVES_N;

    // The loader: thread t brings pieces t, t + 256, ... of 16 bytes of either operand.
    const uint16_t* src_h[T::A_PER];
    const uint16_t* src_w[T::B_PER];
    uint32_t dst_h[T::A_PER], dst_w[T::B_PER];
#pragma unroll
    for (int i = 0; i < T::A_PER; ++i) {
        const uint32_t piece = tid + 256u * (uint32_t)i, r = piece / T::PIECES, kc = piece % T::PIECES;
        src_h[i] = hidden + (uint64_t)min(m0 + r, rows - 1u) * hidden_stride + kc * 8u;
        dst_h[i] = r * ROW_BYTES + (T::SWIZZLED ? (kc ^ ((r >> 2) & 3u)) : kc) * 16u;
    }
    // (codes: the row's words, the piece's eight codes at word (k0 + kc * 8) * WBITS / 32; the
    // row's scales and biases, the piece's group at (k0 + kc * 8) >> group_shift)
    const uint16_t* src_s[T::B_PER];
    const uint16_t* src_b[T::B_PER];
    uint32_t k_in[T::B_PER];
#pragma unroll
    for (int i = 0; i < T::B_PER; ++i) {
        const uint32_t piece = tid + 256u * (uint32_t)i, r = piece / T::PIECES, kc = piece % T::PIECES;
        const uint64_t row = min(n0 + r, vocab - 1u);
        if constexpr (WBITS == 0) {
            src_w[i] = weight + row * weight_stride + kc * 8u;
        } else {
            src_w[i] = weight + (row * weight_stride + kc * (8u * WBITS / 32u)) * 2u;   // (counted in 16-bit units)
            src_s[i] = quant.scales + row * (uint64_t)(d >> quant.group_shift);
            src_b[i] = quant.biases + row * (uint64_t)(d >> quant.group_shift);
            k_in[i] = kc * 8u;
        }
        dst_w[i] = T::A_BYTES + r * ROW_BYTES + (T::SWIZZLED ? (kc ^ ((r >> 2) & 3u)) : kc) * 16u;
    }
    // ring[j]: the loads of a stage on their way (registers), written to LDS one step before use
    w32x4 ring_h[T::AHEAD][T::A_PER], ring_w[T::AHEAD][T::B_PER];
    auto fetch = [&](w32x4 (&h)[T::A_PER], w32x4 (&w)[T::B_PER], uint32_t k0) {
#pragma unroll
        for (int i = 0; i < T::A_PER; ++i) {
            h[i] = *reinterpret_cast<const w32x4*>(src_h[i] + k0);
        }
#pragma unroll
        for (int i = 0; i < T::B_PER; ++i) {
            if constexpr (WBITS == 0) {
                w[i] = *reinterpret_cast<const w32x4*>(src_w[i] + k0);
            } else {
                // the piece's codes (8 or 4 bytes), its group's scale and bias
                const uint32_t* codes = reinterpret_cast<const uint32_t*>(src_w[i]) + k0 * WBITS / 32u;
                const uint32_t g = (k0 + k_in[i]) >> quant.group_shift;
                w[i].x = codes[0];
                w[i].y = WBITS == 8 ? codes[1] : 0u;
                w[i].z = (uint32_t)src_s[i][g] | ((uint32_t)src_b[i][g] << 16);
                w[i].w = 0u;
            }
        }
    };
    // eight codes and their group's (scale, bias) as eight bf16 weights: q * scale + bias as one
    // fused f32 operation (the exact value rounded once), then to bf16 (nearest even) two at a
    // time by the hardware's conversion
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    auto dequantised = [&](const w32x4& c) -> w32x4 {
        const float sc = __builtin_bit_cast(float, c.z << 16), bi = __builtin_bit_cast(float, c.z & 0xffff0000u);
        uint32_t out[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            f32x2 f;
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int j = 2 * p + e;
                const uint32_t q = WBITS == 8 ? (((j < 4 ? c.x : c.y) >> (8 * (j & 3))) & 0xffu) : ((c.x >> (4 * j)) & 0xfu);
                f[e] = __builtin_fmaf((float)q, sc, bi);
            }
            out[p] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
        }
        return w32x4{out[0], out[1], out[2], out[3]};
    };
    // (`real` false: a step past the end of d, run so that every pass of the loop is alike -
    // the hidden rows are staged as zeros and add nothing)
    auto stage = [&](const w32x4 (&h)[T::A_PER], const w32x4 (&w)[T::B_PER], uint32_t buf, bool real) {
        char* base = lds + buf * T::STAGE_BYTES;
        const uint32_t keep = real ? 0xffffffffu : 0u;
#pragma unroll
        for (int i = 0; i < T::A_PER; ++i) {
            *reinterpret_cast<w32x4*>(base + dst_h[i]) = h[i] & keep;
        }
#pragma unroll
        for (int i = 0; i < T::B_PER; ++i) {
            if constexpr (WBITS == 0) {
                *reinterpret_cast<w32x4*>(base + dst_w[i]) = w[i];
            } else {
                *reinterpret_cast<w32x4*>(base + dst_w[i]) = dequantised(w[i]);
            }
        }
    };

    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                acc[mi][ni][v] = 0.0f;
            }
        }
    }
    // A lane's operand values: row lane % 32 of the 32, 8 values of d from (lane / 32) * 8 on.
    // (piece (lane / 32) + 2 * kk of the row; its place in a swizzled row depends on the row's
    // number, which is the lane's within every block of 32 rows)
    uint32_t piece_at[BK / 16];
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
        const uint32_t piece = (lane >> 5) + 2u * (uint32_t)kk;
        piece_at[kk] = (T::SWIZZLED ? (piece ^ ((lane >> 2) & 3u)) : piece) * 16u;
    }
    const uint32_t a_at = (wm * (MI * 32u) + (lane & 31u)) * ROW_BYTES;
    const uint32_t b_at = T::A_BYTES + (wn * (NI * 32u) + (lane & 31u)) * ROW_BYTES;

    if constexpr (T::DIRECT) {
        // Loads that write LDS themselves.  One instruction of a wave fills 1 KB of LDS, lane
        // after lane: 16 staged rows of 64 bytes; a lane asks memory for the piece that belongs
        // in its place (the pieces of a row change places by the row's number, see HeadTile).
        // Every step: wait until this step's own loads have landed (those of the steps asked for
        // later may still be on their way), meet the other waves - their loads have landed too,
        // and nobody reads the stage of the step before any more -, ask for the step AHEAD
        // steps on into that stage, multiply.  All loads are unconditional (past the end of d
        // the last step is asked for again, into a stage nobody will read).
        const uint32_t steps = d / BK;
        const uint32_t rot = (n_tile * 5u + m_tile * 3u) % steps;
        auto k_of = [&](uint32_t stage_no) -> uint32_t {
            uint32_t at = min(stage_no, steps - 1u) + rot;
            at = at >= steps ? at - steps : at;
            return at * BK;
        };
        constexpr int A_LOADS = T::A_BYTES / 4096, B_LOADS = T::B_BYTES / 4096;   // per wave and stage
        static_assert(T::A_BYTES % 4096 == 0 && T::B_BYTES % 4096 == 0, "whole 1 KB blocks per wave");
        const uint16_t* from_h[A_LOADS];
        const uint16_t* from_w[B_LOADS];
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const uint32_t r = ((uint32_t)i * 4u + wave) * 16u + (lane >> 2);
            const uint32_t kc = (lane & 3u) ^ ((r >> 2) & 3u);
            from_h[i] = hidden + (uint64_t)min(m0 + r, rows - 1u) * hidden_stride + kc * 8u;
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            const uint32_t r = ((uint32_t)i * 4u + wave) * 16u + (lane >> 2);
            const uint32_t kc = (lane & 3u) ^ ((r >> 2) & 3u);
            from_w[i] = weight + (uint64_t)min(n0 + r, vocab - 1u) * weight_stride + kc * 8u;
        }
        typedef __attribute__((address_space(1))) const void* gptr;
        typedef __attribute__((address_space(3))) void* lptr;
        auto ask = [&](uint32_t stage_no, uint32_t buf) {
            const uint32_t k0 = k_of(stage_no);
            char* base = lds + buf * T::STAGE_BYTES + wave * 1024u;
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) {
                __builtin_amdgcn_global_load_lds((gptr)(from_h[i] + k0), (lptr)(base + i * 4096), 16, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < B_LOADS; ++i) {
                __builtin_amdgcn_global_load_lds((gptr)(from_w[i] + k0), (lptr)(base + T::A_BYTES + i * 4096), 16, 0, 0);
            }
        };
        // NBUF stages in LDS, all asked for before the first product.  The loop works in half
        // steps (BK = 32 is two operands of 16 along d): while the products of one half run,
        // the operands of the next half are on their way from LDS into the other set of
        // registers.  The barrier sits between the halves: before it a wave has read all it
        // wants of stage s, behind it stage s + 1 has landed for everybody, stage s's place
        // is asked for stage s + NBUF, and the second half's products run over the reads of
        // stage s + 1's first operands.
        constexpr int NBUF = T::AHEAD + 1;
        static_assert(BK == 32, "two halves a step");
#pragma unroll
        for (int j = 0; j < NBUF; ++j) {
            ask((uint32_t)j, (uint32_t)j);
        }
        auto operands = [&](bf16x8 (&a)[MI], bf16x8 (&b)[NI], uint32_t from, int kk) {
            const char* base = lds + from * T::STAGE_BYTES;
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                b[i] = *reinterpret_cast<const bf16x8*>(base + b_at + i * 32 * ROW_BYTES + piece_at[kk]);
            }
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                a[i] = *reinterpret_cast<const bf16x8*>(base + a_at + i * 32 * ROW_BYTES + piece_at[kk]);
            }
        };
        auto products = [&](const bf16x8 (&a)[MI], const bf16x8 (&b)[NI]) {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mi], b[ni], acc[mi][ni], 0, 0, 0);
                }
            }
        };
        // stage 0 has landed when all but the loads of the NBUF - 1 later stages have
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NBUF - 1) * (A_LOADS + B_LOADS)) : "memory");
        bf16x8 a0[MI], b0[NI], a1[MI], b1[NI];
        operands(a0, b0, 0, 0);
        uint32_t buf = 0;
        for (uint32_t s = 0; s < steps; ++s) {
            const uint32_t after = buf + 1u == (uint32_t)NBUF ? 0u : buf + 1u;
            // This half's operands have had eight products' time to arrive.  Said here, as an
            // instruction the compiler counts, before the reads of the next half are issued:
            // left to itself it waits behind them, for all of them.
            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
            __builtin_amdgcn_sched_barrier(0);
            operands(a1, b1, buf, 1);
            __builtin_amdgcn_sched_barrier(0);
            products(a0, b0);
            __builtin_amdgcn_sched_barrier(0);
            // (the barrier as an instruction: __syncthreads() carries a fence that would wait for
            // every load in flight, the ones asked ahead included)
            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): this wave has read what it wants of stage s
            asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NBUF - 2) * (A_LOADS + B_LOADS)) : "memory");
            ask(s + (uint32_t)NBUF, buf);
            operands(a0, b0, after, 0);
            __builtin_amdgcn_sched_barrier(0);
            products(a1, b1);
            __builtin_amdgcn_sched_barrier(0);
            buf = after;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the loads asked past the end
        __syncthreads();
    } else {
    // Every load and every write to LDS below is unconditional (past the end of d the last
    // stage is asked for again): the compiler then counts the loads in flight and waits for
    // the oldest only; with a branch around any of them it waits for all.
    const uint32_t steps = d / BK, padded = (steps + T::AHEAD - 1u) / T::AHEAD * T::AHEAD;
    // Each tile walks d from a place of its own (and wraps round): rows of either operand lie
    // d x 2 bytes apart, a power of two for the usual d, so the same 64 or 128 bytes of every
    // row sit behind the same memory channel; tiles that all start at column 0 and advance in
    // step would queue up at one channel after the other.
    const uint32_t rot = (n_tile * 5u + m_tile * 3u) % steps;
    auto k_of = [&](uint32_t stage_no) -> uint32_t {
        uint32_t at = min(stage_no, steps - 1u) + rot;
        at = at >= steps ? at - steps : at;
        return at * BK;
    };
    fetch(ring_h[0], ring_w[0], k_of(0));
    stage(ring_h[0], ring_w[0], 0, true);
#pragma unroll
    for (int j = 0; j < T::AHEAD; ++j) {
        fetch(ring_h[j], ring_w[j], k_of((uint32_t)j + 1u));   // ring[j] <- stage j + 1
    }
    __syncthreads();
    for (uint32_t s0 = 0; s0 < padded; s0 += T::AHEAD) {
#pragma unroll
        for (int j = 0; j < T::AHEAD; ++j) {
            const uint32_t s = s0 + (uint32_t)j;
            const uint32_t buf = s & 1u;
            const char* base = lds + buf * T::STAGE_BYTES;
#pragma unroll
            for (int kk = 0; kk < BK / 16; ++kk) {
                bf16x8 a[MI], b[NI];
#pragma unroll
                for (int i = 0; i < MI; ++i) {
                    a[i] = *reinterpret_cast<const bf16x8*>(base + a_at + i * 32 * ROW_BYTES + piece_at[kk]);
                }
#pragma unroll
                for (int i = 0; i < NI; ++i) {
                    b[i] = *reinterpret_cast<const bf16x8*>(base + b_at + i * 32 * ROW_BYTES + piece_at[kk]);
                }
#pragma unroll
                for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) {
                        acc[mi][ni] =
                            __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mi], b[ni], acc[mi][ni], 0, 0, 0);
                    }
                }
            }
            // ring[j] holds stage s + 1: into the other LDS stage (nobody reads it: the barrier
            // that closed step s - 1 saw to that), and the registers ask for stage s + 1 + AHEAD.
            // Behind the products, so that a wave that must wait for its loads waits while the
            // matrix pipe works.
            stage(ring_h[j], ring_w[j], buf ^ 1u, s + 1u < steps);
            fetch(ring_h[j], ring_w[j], k_of(s + 1u + T::AHEAD));
            __syncthreads();
        }
    }

    }

    // ---- epilogue.  Element v of a lane's 16 sits in row 8 * (v / 4) + 4 * (lane / 32) + v % 4
    // of its 32 x 32 product, column lane % 32.  Values are rounded to bf16 first, in place: the
    // maximum and the sum describe the logits as they are stored.
    float* red = reinterpret_cast<float*>(lds);              // [WAVES_N][BM] by column group
    float* row_max = red + T::WAVES_N * BM;                  // [BM]
    float* row_c2 = row_max + BM;                            // [BM]
    if (tid < (uint32_t)BM) {
        row_c2[tid] = c2_of_row[min(m0 + tid, rows - 1u)];
    }
    const float NEG = -__builtin_huge_valf();
    bool in_vocab[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        in_vocab[ni] = n0 + wn * (NI * 32u) + (uint32_t)ni * 32u + (lane & 31u) < vocab;
    }
    if constexpr (!OUT_F32) {
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float f = acc[mi][ni][v];   // (a bit_cast of the element itself reads element 0)
                    const uint32_t u = __builtin_bit_cast(uint32_t, f);
                    // round to nearest even; a NaN stays one (quiet)
                    const uint32_t r = (u & 0x7fffffffu) > 0x7f800000u ? ((u >> 16) | 0x40u)
                                                                       : ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
                    acc[mi][ni][v] = __builtin_bit_cast(float, r << 16);
                }
            }
        }
    }
    // what a stored value counts for: a NaN and a column outside the vocabulary count as -inf
    auto worth = [&](int mi, int ni, int v) -> float {
        const float x = acc[mi][ni][v];
        return (in_vocab[ni] && x == x) ? x : NEG;
    };
    // A reduction over the 32 lanes that hold one row's columns: rotations by 8, 4, 2 and 1 within
    // each row of 16 lanes (DPP operands of the arithmetic itself), then one exchange between the
    // two rows.  (Five exchanges through the LDS crossbar per value, as __shfl_xor compiles, made
    // the epilogue as long as the products at 1024 rows.)
    auto across32 = [&](float x, auto op) -> float {
        x = op(x, rotated<0x128>(x));
        x = op(x, rotated<0x124>(x));
        x = op(x, rotated<0x122>(x));
        x = op(x, rotated<0x121>(x));
        return op(x, __shfl_xor(x, 16));
    };
    auto row_of = [&](int mi, int v) -> uint32_t {
        return wm * (MI * 32u) + (uint32_t)mi * 32u + 8u * (uint32_t)(v >> 2) + 4u * (lane >> 5) +
               (uint32_t)(v & 3);
    };
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            float m = NEG;
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
                m = fmaxf(m, worth(mi, ni, v));
            }
            m = across32(m, [](float p, float q) { return fmaxf(p, q); });
            if ((lane & 31u) == 0u) {
                red[wn * BM + row_of(mi, v)] = m;
            }
        }
    }
    __syncthreads();
    if (tid < (uint32_t)BM) {
        float m = red[tid];
#pragma unroll
        for (int g = 1; g < T::WAVES_N; ++g) {
            m = fmaxf(m, red[g * BM + tid]);
        }
        row_max[tid] = m;
    }
    __syncthreads();
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t r = row_of(mi, v);
            const float c = row_c2[r], top = row_max[r] * c;
            float e = 0.0f;
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
                const float x = worth(mi, ni, v);
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
        float e = red[tid];
#pragma unroll
        for (int g = 1; g < T::WAVES_N; ++g) {
            e += red[g * BM + tid];
        }
        tile_max[at] = row_max[tid];
        tile_sum[at] = row_max[tid] > NEG ? e : 0.0f;
    }
    // the logits themselves
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
            const uint32_t col = n0 + wn * (NI * 32u) + (uint32_t)ni * 32u + (lane & 31u);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t r = m0 + row_of(mi, v);
                if (r < rows && col < vocab) {
                    const float f = acc[mi][ni][v];
                    if constexpr (OUT_F32) {
                        static_cast<float*>(logits_out)[(uint64_t)r * logits_stride + col] = f;
                    } else {
                        static_cast<uint16_t*>(logits_out)[(uint64_t)r * logits_stride + col] =
                            (uint16_t)(__builtin_bit_cast(uint32_t, f) >> 16);
                    }
                }
            }
        }
    }
}

template <class T, bool OUT_F32, int WBITS>
static hipError_t launch_head_shape(hipStream_t stream, const void* hidden, uint64_t hidden_stride,
                                    const void* weight, uint64_t weight_stride, uint32_t rows, uint32_t d,
                                    uint32_t vocab, const float* c2_of_row, void* logits,
                                    uint64_t logits_stride, float* tile_max, float* tile_sum,
                                    const HeadQuant& quant) {
    static bool sized[64] = {};
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) {
        return e;
    }
    if (device < 0 || device >= 64 || !sized[device]) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(k_lm_head_bf16<T, OUT_F32, WBITS>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
        if (e != hipSuccess) {
            return e;
        }
        if (device >= 0 && device < 64) {
            sized[device] = true;
        }
    }
    const uint32_t tiles_per_row = (vocab + T::BN - 1u) / T::BN, m_tiles = (rows + T::BM - 1u) / T::BM;
    // slots an XCD needs at most (see the kernel's numbering)
    const uint32_t slots = m_tiles <= 8u ? (tiles_per_row + (8u / m_tiles) - 1u) / (8u / m_tiles)
                                         : ((m_tiles + 7u) / 8u) * tiles_per_row;
    hipLaunchKernelGGL((k_lm_head_bf16<T, OUT_F32, WBITS>), dim3(8u * slots), dim3(256), T::LDS_BYTES, stream,
                       reinterpret_cast<const uint16_t*>(hidden), hidden_stride,
                       reinterpret_cast<const uint16_t*>(weight), weight_stride, rows, d, vocab,
                       c2_of_row, logits, logits_stride, tile_max, tile_sum, tiles_per_row, m_tiles, quant);
    return hipGetLastError();
}

hipError_t launch_lm_head_bf16(hipStream_t stream, const void* hidden, uint64_t hidden_stride,
                               const void* weight, uint64_t weight_stride, uint32_t rows, uint32_t d,
                               uint32_t vocab, const float* c2_of_row, void* logits,
                               uint64_t logits_stride, float* tile_max, float* tile_sum, bool out_f32,
                               const HeadWeights& wq) {
    HeadQuant quant;
    quant.scales = static_cast<const uint16_t*>(wq.scales);
    quant.biases = static_cast<const uint16_t*>(wq.biases);
    quant.group_shift = wq.group_shift;
#define LILY_HEAD_ARGS                                                                              \
    stream, hidden, hidden_stride, weight, weight_stride, rows, d, vocab, c2_of_row, logits,        \
        logits_stride, tile_max, tile_sum, quant
    typedef HeadTile<1, 1, 1, 64, 4, 3> Tile32;
    typedef HeadTile<1, 2, 1, 64, 3, 3> Tile64;
    typedef HeadTile<2, 2, 2, 64, 3, 2> Tile128;
    typedef HeadTile<2, 4, 2, 32, 2, 2, true> Tile256;
    // (the pass over the stored logits reads 16-byte pieces: rows that start at multiples of 16 bytes)
    const bool rows_aligned = (reinterpret_cast<uintptr_t>(logits) & 15u) == 0u &&
                              (logits_stride * (out_f32 ? 4u : 2u)) % 16u == 0u;
    if (wq.library_rows != 0u && rows >= wq.library_rows && (wq.bits == 0u || out_f32) && rows_aligned &&
        (vocab + LILY_TILE_COLS - 1u) / LILY_TILE_COLS <= HEAD_LIBRARY_MAX_TILES) {
        const hipError_t e = launch_head_library(stream, hidden, hidden_stride, weight, weight_stride, rows, d, vocab,
                                                 logits, logits_stride, out_f32, wq);
        if (e == hipSuccess) {
            if (wq.library_calls != nullptr) {
                ++*wq.library_calls;
            }
            return launch_head_summaries(stream, logits, logits_stride, rows, vocab, c2_of_row, tile_max, tile_sum,
                                         out_f32);
        }
        if (e != hipErrorNotSupported) {
            return e;
        }
    }
    if (wq.bits != 0u) {
        // codes: f32 logits only (what the reference's quantised head produces), and the tiles
        // whose loads pass through registers, whatever the number of rows
        if (!out_f32 || (wq.bits != 4u && wq.bits != 8u)) {
            return hipErrorInvalidValue;
        }
        if (lm_head_codes_serves(rows, d, vocab, hidden_stride, weight_stride, wq)) {
            return launch_lm_head_codes(stream, hidden, hidden_stride, weight, weight_stride, rows, d, vocab,
                                        c2_of_row, logits, logits_stride, tile_max, tile_sum, wq);
        }
#define LILY_HEAD_Q(TILE)                                                                           \
    (wq.bits == 8u ? launch_head_shape<TILE, true, 8>(LILY_HEAD_ARGS)                               \
                   : launch_head_shape<TILE, true, 4>(LILY_HEAD_ARGS))
        if (rows <= 32u) {
            return LILY_HEAD_Q(Tile32);
        }
        if (rows <= 64u) {
            return LILY_HEAD_Q(Tile64);
        }
        return LILY_HEAD_Q(Tile128);
#undef LILY_HEAD_Q
    }
#define LILY_HEAD_B(TILE)                                                                           \
    (out_f32 ? launch_head_shape<TILE, true, 0>(LILY_HEAD_ARGS) : launch_head_shape<TILE, false, 0>(LILY_HEAD_ARGS))
    if (rows <= 32u) {
        return LILY_HEAD_B(Tile32);
    }
    if (rows <= 64u) {
        return LILY_HEAD_B(Tile64);
    }
    if (rows <= 128u) {
        return LILY_HEAD_B(Tile128);
    }
    return LILY_HEAD_B(Tile256);
#undef LILY_HEAD_B
#undef LILY_HEAD_ARGS
}

}  // namespace lily
