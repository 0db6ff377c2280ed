// row_args.h - what one logits row's workgroups receive, and the launch-wide settings.
// Shared by the kernels and the C-ABI layer that packs it.
#pragma once

#include <stdint.h>

#include "../../include/lily_sampler.h"

namespace lily {

enum Mode : uint32_t {
    MODE_ARGMAX = 0,  // exact first-max over the raw row (greedy, nothing else asked)
    MODE_PLAIN = 1,   // sample_f32
    MODE_DRAFT = 2,   // sample_draft_f32: also exports the kept distribution
    MODE_SPEC = 3,    // sample_spec_f32: accept/reject against an exported distribution
};

enum : uint32_t {
    F_PEN = 1u,      // penalties on: read counts, count the emitted id
    F_UNIFORM = 2u,  // use `uniform` (and `uniform2`) instead of the seeded draws
    F_FORCED = 4u,   // emit `forced`
};

struct alignas(16) RowArgs {
    const void* logits;        // this row's first element
    const uint32_t* allow;     // packed allow bits or null
    uint32_t* counts;          // dense emission histogram or null
    uint32_t* touched;         // bit per id with counts[id] != 0, or null
    const lily_bias* bias;     // n_bias pairs or null
    uint32_t* out_id;
    float* out_logprob;        // or null
    uint32_t* q_ids;           // draft export (MODE_DRAFT writes, MODE_SPEC reads)
    float* q_probs;
    uint32_t* q_n;
    const uint32_t* draft;     // MODE_SPEC proposal
    uint32_t* dbg_ids;         // diagnostics or null
    float* dbg_probs;
    uint32_t* dbg_counts;
    uint64_t seed;
    uint32_t step;
    uint32_t n_bias;
    uint32_t k;                // effective candidate count (1..1024)
    uint32_t mode;
    uint32_t flags;
    uint32_t forced;
    float temperature;         // effective
    float c2;                  // log2(e) / temperature
    float top_p;
    float min_p;
    float presence;
    float frequency;
    float repetition;
    float uniform;
    float uniform2;
    float pad;
};
static_assert(sizeof(RowArgs) == 192, "RowArgs layout");

constexpr int INLINE_ROWS = 8;
struct InlineRows {
    RowArgs r[INLINE_ROWS];
};

// Launch-wide settings and the workspace of rows that span several workgroups.
struct LaunchCfg {
    const RowArgs* table;   // device row table, or null when rows travel inline
    uint32_t vocab;
    uint32_t slices;        // workgroups per row
    uint32_t step_delta;    // added to every row's step
    uint32_t ws_k;          // candidate slots per (row, slice) in ws_cand
    uint64_t* ws_cand;      // [rows][slices][ws_k] (value key << 32 | ~id)
    uint32_t* ws_n;         // [rows][slices] candidates written
    double* ws_lse;         // [rows][slices][2] log2-domain reference, sum of 2^(x - reference)
    uint32_t* ws_ticket;    // [rows] arrival counter, left at 0
    uint32_t path;          // 0 = automatic, 1 = exhaustive select only, 2 = two-pass select only
    uint32_t cand_cap;      // candidate slots at the start of dynamic LDS (the bitmap follows)
    uint64_t* phase_trace;  // null, or [rows][slices][PHASE_SLOTS] 100 MHz timestamps
    uint32_t excl_words;    // words reserved for the slice bitmap (the specials' id list follows)
    uint32_t pad;
};

constexpr uint32_t PHASE_SLOTS = 8;

constexpr uint32_t CAND_CAP = 2048;   // candidates a workgroup collects while scanning
constexpr uint32_t MERGE_CAP = 4096;  // candidates the merging workgroup gathers (slices x k)
constexpr uint32_t MAX_SLICES = 64;
constexpr uint32_t SPECIAL_LIST_CAP = 2048;  // ids of penalised / biased tokens gathered per batch

}  // namespace lily
