// row_args.h - what one logits row's workgroups receive, and the launch-wide settings.
// Shared by the kernels and the C-ABI layer that packs it.
#pragma once

#include <stdint.h>

#include "../../include/lily_sampler.h"

namespace lily {

// Columns of the logits that one summary (largest value, sum of exponentials) of the
// logits' producer covers.
#define LILY_TILE_COLS 128   // = LILY_LOGIT_TILE_COLS of the public header


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
};

struct alignas(16) RowArgs {
    const void* logits;        // this row's first element
    const uint32_t* allow;     // packed allow bits or null
    uint32_t* counts;          // dense emission histogram or null
    uint32_t* touched;         // bit per id that was ever counted (a count may have gone back to
                               // 0), or null
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
    uint32_t k_draw;           // rows of a chained launch: the draw's own candidate count (k is
                               // then what the select collects); 0 otherwise
    uint32_t sel_rows;         // rows behind `logits` that sel_row may pick from
    uint32_t pad;
    // A draw whose row and step a kernel before it chose (words of the speculative control
    // block, typically): the row is logits + min(*sel_row, sel_rows - 1) * sel_stride bytes and
    // the step is step + *sel_step.  Null pointers: the row and the step as given.
    const uint32_t* sel_row;
    const uint32_t* sel_step;
    uint64_t sel_stride;
    uint64_t pad2;
};
static_assert(sizeof(RowArgs) == 224, "RowArgs layout");

// A scratch's device state as the small maintenance kernels take it.
struct ScratchView {
    uint32_t* counts;    // [vocab]
    uint32_t* touched;   // [ceil(vocab / 32) + 4]
    uint32_t vocab;
};

constexpr int INLINE_ROWS = 8;
struct InlineRows {
    RowArgs r[INLINE_ROWS];
};

// Device memory that one workgroup writes and another reads after taking a ticket.  The type has
// no indexing and no dereference: kernels reach it through handed_store() / handed_load()
// (device_common.h) only, which go through to memory and read past the caches - the hand-over
// depends on every access being of that kind.
template <class T>
struct Handed {
    T* p;
};

// Launch-wide settings and the workspace of rows that span several workgroups.
struct LaunchCfg {
    const RowArgs* table;   // device row table, or null when rows travel inline
    uint32_t vocab;
    uint32_t slices;        // workgroups per row
    uint32_t step_delta;    // added to every row's step
    uint32_t ws_k;          // candidate slots per (row, slice) in ws_cand
    Handed<uint64_t> ws_cand;   // [rows][slices][ws_k] (value key << 32 | ~id)
    Handed<double> ws_lse;  // [rows][slices][2] log2-domain reference, sum of 2^(x - reference)
    uint32_t* ws_ticket;    // [rows] arrival counter, left at 0
    uint32_t path;          // 0 = automatic, 1 = exhaustive select only, 2 = two-pass select only,
                            // 3 = no streaming select
    uint32_t cand_cap;      // candidate slots at the start of dynamic LDS (the bitmap follows)
    uint64_t* phase_trace;  // null, or [rows][slices][PHASE_SLOTS] 100 MHz timestamps
    uint32_t excl_words;    // words reserved for the slice bitmap (the specials' id list follows)
    uint32_t list_cap;      // ids the specials' list holds
    uint32_t bitmap_layout;    // dynamic LDS holds cand_cap candidates + the bitmap + the id list
    uint32_t dyn_slots;     // 64-bit slots of dynamic LDS in all
    uint32_t* path_stats;   // null, or [4] counters: slices finished by the streaming select, the
                            // bitmap select, the exhaustive select; [3] a bit per reason the
                            // streaming select gave a slice up
    // A chained launch (rows that share one scratch and must draw in order, each seeing the
    // counts the rows before it left): every row's candidates are collected against the counts
    // as they stood, published here, and the workgroup that finishes last draws row after row.
    uint32_t chain_rows;    // 0 = the rows are independent
    Handed<uint64_t> chain_cand;   // [chain_rows][CHAIN_CAP]
    Handed<uint32_t> chain_n;      // [chain_rows] candidates published
    uint32_t* chain_ticket; // [1] rows that have published, left at 0
    // spec_accept by the same workgroup once the last row has drawn (null: not asked for)
    uint32_t* accept_ctrl;
    const uint32_t* accept_ids;   // [chain_rows] the pass's input ids (ids[j + 1] = proposal j)
    uint32_t accept_pos0;
    uint32_t accept_ratio;
    uint32_t accept_chain;
    // null, or [rows]: a row whose word is not 0 has been drawn by an earlier launch of the same
    // call (from the producer's summaries) and is left alone
    const uint32_t* served;
    // 1 = the slices' hand-over in its relaxed form (last_to_arrive() in device_common.h)
    uint32_t relaxed_handover;
    uint32_t pad_cfg;
};

constexpr uint32_t CHAIN_CAP = LILY_SAMPLE_K_CAP;   // candidates a chained row publishes
// Where the workgroup that draws the rows keeps what it requested ahead: behind the sorted
// candidates and the tail's three float arrays, 16 bytes for each of a row's first 64 candidates
// and 8 for each of the first 64 entries of its draft distribution.
constexpr uint32_t CHAIN_LDS_OFFSET = LILY_SAMPLE_K_CAP * 8 + 3 * LILY_SAMPLE_K_CAP * 4;
constexpr uint32_t CHAIN_LDS_BYTES = CHAIN_LDS_OFFSET + LILY_MAX_VERIFY_ROWS * 64 * 24;

constexpr uint32_t PHASE_SLOTS = 16;

constexpr uint32_t CAND_CAP = 2048;   // candidates a workgroup collects while scanning
constexpr uint32_t MERGE_CAP = 4096;  // candidates the merging workgroup gathers (slices x k)
constexpr uint32_t MAX_SLICES = 64;
constexpr uint32_t SPECIAL_LIST_CAP = 2048;  // ids of penalised / biased tokens gathered per batch

// Streaming select (k <= STREAM_K_MAX): dynamic LDS layout in bytes.
constexpr uint32_t STREAM_K_MAX = 64;
constexpr uint32_t STREAM_UNROLL = 4;      // 16-byte chunks per thread per block
constexpr uint32_t Q_CAP = 768;            // queued chunks (those holding a value at or above the bound)
constexpr uint32_t S_CAP = 4096;           // noted chunks (summed before their listed ids were looked at)
constexpr uint32_t FC_CAP = 1024;          // final candidates
constexpr uint32_t MAX_BLOCKS = 64;        // blocks of one slice
constexpr uint32_t STREAM_BIAS_CAP = 64;   // bias pairs kept in LDS
// A wave's window into a bitmap of the row's ids (listed ids, barred ids): for each of the block's
// four loads the words that hold the bits of the wave's 64 chunks, one more for rows whose chunks
// do not start on a word of the bitmap.
constexpr uint32_t WIN_PIECE_MAX = 64 * 8 / 32 + 1;           // bf16: 64 chunks of 8 ids
constexpr uint32_t WIN_WORDS = STREAM_UNROLL * WIN_PIECE_MAX; // per wave and bitmap
constexpr uint32_t OFF_QRAW = 0;
constexpr uint32_t OFF_QIDX = OFF_QRAW + Q_CAP * 16;
constexpr uint32_t OFF_NOTED = OFF_QIDX + Q_CAP * 4;          // [4 waves][S_CAP / 4] x 16 bits
constexpr uint32_t OFF_WIN = OFF_NOTED + S_CAP * 2;           // [4 waves][2 bitmaps][WIN_WORDS]
constexpr uint32_t OFF_BLK = OFF_WIN + 4 * 2 * WIN_WORDS * 4; // [MAX_BLOCKS] x (bound, cut, flags)
constexpr uint32_t OFF_BIAS = OFF_BLK + MAX_BLOCKS * 12;      // ids then deltas
// The final candidates lie above everything the tail and the merge use (the sorted candidates
// and the tail's three float arrays: K_CAP * 8 + 3 * K_CAP * 4 bytes from the start).
constexpr uint32_t OFF_FC = (OFF_BIAS + STREAM_BIAS_CAP * 8 + 15u) / 16u * 16u;
constexpr uint32_t STREAM_LDS_BYTES = OFF_FC + FC_CAP * 8;
static_assert(OFF_FC >= 20480, "stream LDS layout");
static_assert(OFF_FC % 8 == 0 && OFF_WIN % 4 == 0 && STREAM_LDS_BYTES % 16 == 0, "stream LDS layout");

}  // namespace lily
