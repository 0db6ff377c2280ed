// launch.h - host-callable launchers defined in sampler_kernels.hip.
#pragma once

#include <hip/hip_runtime_api.h>

#include "row_args.h"

namespace lily {

// `kind`: 0 = no row has a mask, penalties or a bias list, 1 = some row has, 2 = every sampled
// row takes the streaming select; `lse`: some row wants a log-probability.
// `dyn_bytes`: dynamic LDS (see shape_of in sampler_api.cpp).
hipError_t launch_rows(hipStream_t stream, int dtype, int kind, bool lse, uint32_t rows,
                       const LaunchCfg& cfg, const InlineRows* inline_rows, size_t dyn_bytes);
hipError_t launch_fill_u32(hipStream_t stream, uint32_t* p, uint32_t n, uint32_t v);
hipError_t launch_add_history(hipStream_t stream, const ScratchView& sc, const uint32_t* ids,
                              uint32_t n);
hipError_t launch_uncount(hipStream_t stream, const ScratchView& sc, uint32_t token);
hipError_t launch_uncount_after(hipStream_t stream, const ScratchView& sc, const uint32_t* draws,
                                uint32_t m, const uint32_t* accepted, uint32_t cap);
// touched = the ids with a non-zero count.
hipError_t launch_rebuild_listed(hipStream_t stream, const ScratchView& sc);
hipError_t launch_spec_accept(hipStream_t stream, const uint32_t* draws, const uint32_t* ids,
                              uint32_t* ctrl, uint32_t m, uint32_t pos0, uint32_t ratio,
                              uint32_t chain);
// logits[rows, vocab] = hidden[rows, d] x weight[vocab, d]^T (bf16, strides in elements, d a
// multiple of 64), with the largest value and the sum of 2^((x - largest) * c2_of_row[row]) of
// every LILY_TILE_COLS columns in tile_max / tile_sum [rows, ceil(vocab / LILY_TILE_COLS)].
// out_f32: the logits are f32 [rows, logits_stride] instead of bf16.  wq.bits 4 / 8: `weight` points
// at the reference's affine codes (u32 words, weight_stride words a row), wq.scales / wq.biases at
// bf16 [vocab, d >> wq.group_shift]; f32 logits only.
struct HeadWeights {
    uint32_t bits = 0;          // 0 = bf16 weights
    const void* scales = nullptr;
    const void* biases = nullptr;
    uint32_t group_shift = 6;   // log2 of the group size
    unsigned long long* trace = nullptr;   // diagnostic stamps, [workgroups][8] (builds with -DLILY_HEAD_TRACE)
    unsigned long long trace_words = 0;
    // batches of at least this many rows go through the vendor's GEMM library where it is present
    // and takes the shape, followed by the pass that forms the summaries (0: never)
    uint32_t library_rows = 0;
    unsigned long long* library_calls = nullptr;   // counts the calls that went that way
};
hipError_t launch_lm_head_bf16(hipStream_t stream, const void* hidden, uint64_t hidden_stride,
                               const void* weight, uint64_t weight_stride, uint32_t rows, uint32_t d,
                               uint32_t vocab, const float* c2_of_row, void* logits,
                               uint64_t logits_stride, float* tile_max, float* tile_sum, bool out_f32,
                               const HeadWeights& wq);
// The same over codes for up to 16 rows in the reference's form for few rows (the codes are not
// turned into weights: scale * sum(q * x) + bias * sum(x) per group, f32 logits); `serves` says
// whether a shape can take it (groups of 64 or more, operands within 4 GB).
bool lm_head_codes_serves(uint32_t rows, uint32_t d, uint32_t vocab, uint64_t hidden_stride, uint64_t weight_stride,
                          const HeadWeights& wq);
hipError_t launch_lm_head_codes(hipStream_t stream, const void* hidden, uint64_t hidden_stride, const void* weight,
                                uint64_t weight_stride, uint32_t rows, uint32_t d, uint32_t vocab,
                                const float* c2_of_row, void* logits, uint64_t logits_stride, float* tile_max,
                                float* tile_sum, const HeadWeights& wq);
// The batch form through the vendor's GEMM library, opened by name at run time: the product alone
// (codes are turned into bf16 weights first, in memory this call keeps per device and stream);
// hipErrorNotSupported where the library is absent or has no algorithm for the shape - the
// caller then runs its own kernel.  launch_head_summaries: tile_max / tile_sum of stored logits.
constexpr uint32_t HEAD_LIBRARY_MAX_TILES = 2048;   // summaries a row that launch_head_summaries takes
bool head_library_present();
hipError_t launch_head_library(hipStream_t stream, const void* hidden, uint64_t hidden_stride, const void* weight,
                               uint64_t weight_stride, uint32_t rows, uint32_t d, uint32_t vocab, void* logits,
                               uint64_t logits_stride, bool out_f32, const HeadWeights& wq);
hipError_t launch_head_summaries(hipStream_t stream, const void* logits, uint64_t logits_stride, uint32_t rows,
                                 uint32_t vocab, const float* c2_of_row, float* tile_max, float* tile_sum,
                                 bool f32);
// The draw of `rows` rows of cfg.table from the summaries ([.., tiles] each) and the few tiles of
// the logits (bf16 or f32) that matter; tile_row[r] = the summaries' row of table row r; served[r] is set
// for rows under penalties or a mask (1 = drawn, 0 = declined: the row is better read whole).
// `extra`: some row carries a bias list or a mask.
hipError_t launch_rows_tiles(hipStream_t stream, int dtype, bool lse, bool extra, uint32_t rows,
                             const LaunchCfg& cfg, const float* tile_max, const float* tile_sum,
                             uint32_t tiles, const uint32_t* tile_row, uint32_t* served);
// Rows that draw among many candidates (k > 64), spread over cfg.slices workgroups a row: two
// launches (the row's bound, then the values that reach it, merge, select, tail).
// lane_max [rows][slices][256], bound [rows], count [rows][slices].
hipError_t launch_rows_wide(hipStream_t stream, int dtype, bool lse, uint32_t rows, const LaunchCfg& cfg,
                            const InlineRows* inline_rows, float* lane_max, uint32_t* count);
hipError_t launch_copy_pieces(hipStream_t stream, const void* src, void* dst, size_t bytes);
hipError_t launch_probe_read(hipStream_t stream, const void* base, uint32_t rows, uint64_t row_bytes,
                             uint64_t stride_bytes, uint32_t* out);
hipError_t launch_copy_row(hipStream_t stream, const uint32_t* src, uint32_t* dst, uint32_t words,
                           uint32_t rows, const uint32_t* row_dev);

}  // namespace lily
