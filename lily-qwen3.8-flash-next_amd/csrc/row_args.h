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
    F_STREAM = 8u,   // eligible for the streaming select (k <= 64, no allow-mask, short bias list)
    F_SORT_FIRST = 16u,  // host only: this row's list is due for sorting before the launch
};

// One entry of a scratch's list of the ids that were ever counted: the id in the low
// LIST_ID_BITS bits, min(count, LIST_COUNT_MAX) above them (a saturated entry sends the reader
// to the dense counts).
typedef uint32_t ListEntry;
constexpr uint32_t LIST_ID_BITS = 20;
constexpr uint32_t LIST_COUNT_MAX = 4095;
__host__ __device__ inline ListEntry list_entry(uint32_t id, uint32_t count) {
    return id | ((count < LIST_COUNT_MAX ? count : LIST_COUNT_MAX) << LIST_ID_BITS);
}

struct alignas(16) RowArgs {
    const void* logits;        // this row's first element
    const uint32_t* allow;     // packed allow bits or null
    uint32_t* counts;          // dense emission histogram or null
    uint32_t* touched;         // bit per id that is in `pairs` (set with the first count), or null
    ListEntry* pairs;          // the listed ids with their counts (a count may have gone back to 0):
                               // [0, n_sorted) in ascending id order, and the ids first counted
                               // since the list was last sorted at [pairs_cap - n_tail, pairs_cap),
                               // newest lowest
    uint32_t* list_hdr;        // [LIST_HDR_WORDS + buckets + 1]: n_sorted, n_tail, two spare words,
                               // then start[b] = entries of the sorted part whose id is below
                               // b << SORT_SHIFT (n_sorted + n_tail above pairs_cap: the list is unusable)
    uint32_t* pos;             // [vocab] pairs index of a listed id
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
    uint32_t pairs_cap;
    uint32_t tail_hint;        // host's upper bound of n_tail when the row was packed (saves loads only)
    uint32_t pad;
};
static_assert(sizeof(RowArgs) == 224, "RowArgs layout");

// The sorted part of a scratch's list is indexed by buckets of 1 << SORT_SHIFT ids.
constexpr uint32_t SORT_SHIFT = 8;
constexpr uint32_t LIST_HDR_WORDS = 4;   // n_sorted, n_tail, two spare words; the bucket starts follow
constexpr uint32_t HDR_SORTED = 0, HDR_TAIL = 1;
// Draws append to the unsorted tail; the host has the list sorted again (one launch over the
// batch's scratches) before its bound of the tail's length passes this.
constexpr uint32_t TAIL_SORT_AT = 256;

// A scratch's device state as the small maintenance kernels take it.
struct ScratchView {
    uint32_t* counts;    // [vocab]
    uint32_t* touched;   // [ceil(vocab / 32) + 4]
    ListEntry* pairs;    // [pairs_cap]
    uint32_t* list_hdr;  // [LIST_HDR_WORDS + ceil(vocab >> SORT_SHIFT) + 1]
    uint32_t* pos;       // [vocab]
    uint32_t vocab;
    uint32_t pairs_cap;
};

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
    double* ws_lse;         // [rows][slices][2] log2-domain reference, sum of 2^(x - reference)
    uint32_t* ws_ticket;    // [rows] arrival counter, left at 0
    uint32_t path;          // 0 = automatic, 1 = exhaustive select only, 2 = two-pass select only,
                            // 3 = no streaming select
    uint32_t cand_cap;      // candidate slots at the start of dynamic LDS (the bitmap follows)
    uint64_t* phase_trace;  // null, or [rows][slices][PHASE_SLOTS] 100 MHz timestamps
    uint32_t excl_words;    // words reserved for the slice bitmap (the specials' id list follows)
    uint32_t list_cap;      // ids the specials' list holds
    uint32_t bitmap_layout;    // dynamic LDS holds cand_cap candidates + the bitmap + the id list
    uint32_t hint_growth;   // added to every row's tail_hint (draws since the table was packed)
    uint32_t hint_replace;  // the lists were sorted since: hint_growth alone bounds the tails
    uint32_t dyn_slots;     // 64-bit slots of dynamic LDS in all
    uint32_t* path_stats;   // null, or [4] counters: slices finished by the streaming select, the
                            // bitmap select, the exhaustive select; [3] unused
};

constexpr uint32_t PHASE_SLOTS = 16;

constexpr uint32_t CAND_CAP = 2048;   // candidates a workgroup collects while scanning
constexpr uint32_t MERGE_CAP = 4096;  // candidates the merging workgroup gathers (slices x k)
constexpr uint32_t MAX_SLICES = 64;
constexpr uint32_t SPECIAL_LIST_CAP = 2048;  // ids of penalised / biased tokens gathered per batch

// Streaming select (k <= STREAM_K_MAX, no allow-mask): dynamic LDS layout in bytes.
constexpr uint32_t STREAM_K_MAX = 64;
constexpr uint32_t STREAM_UNROLL = 4;      // 16-byte chunks per thread per block
constexpr uint32_t Q_CAP = 768;            // queued chunks (those holding a value at or above the bound)
constexpr uint32_t SPEC_CAP = 3072;        // penalised / biased ids of one slice
constexpr uint32_t FC_CAP = 1024;          // final candidates
constexpr uint32_t DROP_CAP = 128;         // penalised / biased ids found inside queued chunks
constexpr uint32_t MAX_BUCKETS = 64;       // blocks of one slice
constexpr uint32_t STREAM_BIAS_CAP = 64;   // bias pairs kept in LDS
constexpr uint32_t SPEC_ID_BITS = LIST_ID_BITS;  // an LDS bucket entry has the list's own format
constexpr uint32_t OFF_QRAW = 0;
constexpr uint32_t OFF_QIDX = OFF_QRAW + Q_CAP * 16;
constexpr uint32_t OFF_SPEC = OFF_QIDX + Q_CAP * 4;
constexpr uint32_t OFF_FC = OFF_SPEC + SPEC_CAP * 4;
constexpr uint32_t OFF_DROP = OFF_FC + FC_CAP * 8;
constexpr uint32_t OFF_DMASK = OFF_DROP + DROP_CAP * 4;       // a byte per queue slot
constexpr uint32_t OFF_BKT = OFF_DMASK + Q_CAP;               // [MAX_BUCKETS + 1] offsets
constexpr uint32_t OFF_BFILL = OFF_BKT + (MAX_BUCKETS + 4) * 4;   // [MAX_BUCKETS] fill counters
constexpr uint32_t OFF_BIAS = OFF_BFILL + MAX_BUCKETS * 4;    // ids then deltas
constexpr uint32_t OFF_HSEG = OFF_BIAS + STREAM_BIAS_CAP * 8; // [MAX_BUCKETS] (first, end) of each block's
                                                              // entries in the sorted part of the list
constexpr uint32_t STREAM_LDS_BYTES = OFF_HSEG + MAX_BUCKETS * 8;
static_assert(OFF_FC % 8 == 0 && STREAM_LDS_BYTES % 16 == 0, "stream LDS layout");

}  // namespace lily
