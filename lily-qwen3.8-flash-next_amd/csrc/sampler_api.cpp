// sampler_api.cpp - the C ABI of include/lily_sampler.h over the HIP kernels.
//
// Host-side work per draw is validation and packing one RowArgs per row; up to
// INLINE_ROWS rows travel as kernel arguments, larger batches go through a pinned
// staging ring and one asynchronous copy into the sampler's device row table.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <algorithm>
#include <vector>

#include "../../include/lily_sampler.h"
#include "../../include/lily_sampler_math.h"
#include "api_internal.h"
#include "launch.h"

using namespace lily;

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    return fail(LILY_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(call)                      \
    do {                                   \
        hipError_t e_ = (call);            \
        if (e_ != hipSuccess) {            \
            return hip_fail(e_, #call);    \
        }                                  \
    } while (0)

// Makes `device` the calling thread's current device for the rest of the enclosing scope and
// puts the caller's own choice back on the way out: a library call must not leave the host
// thread on another GPU than it came with.
struct DeviceScope {
    int before = -1;
    bool switched = false;
    hipError_t err = hipSuccess;
    explicit DeviceScope(int device) {
        err = hipGetDevice(&before);
        if (err == hipSuccess && before != device) {
            err = hipSetDevice(device);
            switched = err == hipSuccess;
        }
    }
    ~DeviceScope() {
        if (switched) {
            DeviceScope device_scope_(before);
        }
    }
    DeviceScope(const DeviceScope&) = delete;
    DeviceScope& operator=(const DeviceScope&) = delete;
};
#define ON_DEVICE(device)                 \
    DeviceScope device_scope_(device);    \
    HIP_TRY(device_scope_.err)

constexpr uint32_t WS_ROWS = 4096;      // rows that may span several workgroups
// Batches of the logits' producer from this many rows on go through the vendor's GEMM library
// where it is present (below, this library's own tiles are as fast or faster; over codes the
// library's way begins with a pass that turns all of them into bf16 weights).
constexpr uint32_t HEAD_LIBRARY_ROWS = 129, HEAD_LIBRARY_ROWS_CODES = 256;
constexpr uint32_t WS_SLOTS = 1u << 22; // candidate slots of the workspace (rows x slices x k)
constexpr uint32_t STAGE_SLOTS = 4;
constexpr size_t STAGE_ROW_BYTES = sizeof(RowArgs) + 16;   // a staged row: descriptor + three words + slack
constexpr uint32_t TARGET_GROUPS = 512;  // workgroups a small batch is spread over
constexpr uint32_t WIDE_FLOATS = 1u << 20;   // lane maxima the wide rows' workspace holds

}  // namespace

struct lily_sampler {
    int device = 0;
    hipStream_t stream = nullptr;
    uint64_t* ws_cand = nullptr;
    double* ws_lse = nullptr;
    uint32_t* ws_ticket = nullptr;
    uint64_t* chain_cand = nullptr;   // [LILY_MAX_VERIFY_ROWS][CHAIN_CAP], then the rows' counts and
    uint32_t* chain_n = nullptr;      // the ticket of a chained launch
    uint32_t* chain_ticket = nullptr;
    // rows that draw among many candidates (rows_wide.hip): null in a view without them
    float* wide_max = nullptr;     // [WIDE_FLOATS] lane maxima, rows x slices x 256
    uint32_t* wide_count = nullptr;  // [WS_ROWS] candidates listed so far, 0 between launches
    uint32_t ws_rows = WS_ROWS;    // rows that may span several workgroups
    uint32_t ws_slots = WS_SLOTS;  // candidate slots behind ws_cand
    // Row table of lily_sample_rows batches above INLINE_ROWS.
    RowArgs* table_dev = nullptr;
    uint32_t table_cap = 0;
    RowArgs* stage[STAGE_SLOTS] = {};
    hipEvent_t stage_done[STAGE_SLOTS] = {};
    bool stage_used[STAGE_SLOTS] = {};
    uint32_t stage_cap = 0;
    uint32_t stage_next = 0;
    uint32_t force_path = 0;
    uint32_t force_slices = 0;
    bool no_wide = false;   // LILY_SAMPLER_WIDE=0: rows of many candidates go the other kernels' way
    // LILY_SAMPLER_HEAD: batches of this many rows or more are produced through the vendor's GEMM
    // library ("own": never, "library": every batch it takes, a number: from that many rows on)
    uint32_t head_library_rows = HEAD_LIBRARY_ROWS, head_library_rows_codes = HEAD_LIBRARY_ROWS_CODES;
    unsigned long long head_library_calls = 0;   // producer calls that went through the vendor's library
    uint32_t handover = 0;  // LILY_SAMPLER_HANDOVER: 0 = by the launch's size, 1 = strict, 2 = relaxed
    // What the last lily_lm_head_bf16 call of this sampler left: where, and with which exponent
    // scale per row (tile_sum is only good for a log-probability at that scale).
    const float* head_sum = nullptr;
    std::vector<float> head_c2;
    uint64_t* phase_trace = nullptr;
    uint64_t phase_words = 0;
    uint32_t* path_stats = nullptr;
};

struct lily_scratch {
    lily_sampler* s = nullptr;
    uint32_t vocab = 0;
    uint32_t words = 0;
    uint32_t* counts = nullptr;   // [vocab]; the one allocation, the bitmap follows it
    uint32_t* touched = nullptr;  // [words + 4] bit per id that was ever counted, then the largest
                                  // count any id has reached
};

struct lily_draft_dists {
    lily_sampler* s = nullptr;
    uint32_t slots = 0;
    uint32_t* ids = nullptr;
    float* probs = nullptr;
    uint32_t* counts = nullptr;
};

struct lily_token_slots {
    lily_sampler* s = nullptr;
    uint32_t slots = 0, words = 0;
    uint32_t* dev = nullptr;    // [slots][words]
    uint32_t* host = nullptr;   // pinned mirror, [slots][words]
    hipEvent_t* done = nullptr; // [slots] recorded behind each slot's copy to the mirror
    bool* published = nullptr;  // [slots] an event has been recorded since the slot was last read
};

// One launch over consecutive rows of a packed table.
struct LaunchPart {
    uint32_t first = 0;
    uint32_t rows = 0;
    uint32_t slices = 1;
    uint32_t ws_k = 0;
    int kind = 0;
    bool lse = false;
    size_t dyn_bytes = 0;
    uint32_t excl_words = 0;
    bool bitmap_layout = false;
    uint32_t cand_cap = 0;
    bool wide = false;   // every row draws among many candidates: the two launches of rows_wide.hip
};

struct lily_plan {
    lily_sampler* s = nullptr;
    uint32_t max_rows = 0;
    RowArgs* table_dev = nullptr;
    uint32_t rows = 0;
    uint32_t vocab = 0;
    uint32_t dtype = 0;
    LaunchPart parts[2];                     // the batch's one or two launches
    uint32_t n_parts = 0;
    uint32_t runs = 0;                       // launches since the table was packed
};

namespace {

ScratchView view_of(const lily_scratch* sc) {
    ScratchView v;
    v.counts = sc->counts;
    v.touched = sc->touched;
    v.vocab = sc->vocab;
    return v;
}

bool samples(const lily_sampling_params* p) {
    return !lily_params_is_greedy(p) || lily_params_uses_penalties(p);
}

struct RowExtras {
    const uint32_t* allow = nullptr;
    const lily_bias* bias = nullptr;
    uint32_t n_bias = 0;
    uint32_t forced = LILY_NO_TOKEN;
    bool has_uniform = false;
    float uniform = 0.0f, uniform2 = 0.0f;
    float* out_logprob = nullptr;
    uint32_t* dbg_ids = nullptr;
    float* dbg_probs = nullptr;
    uint32_t* dbg_counts = nullptr;
    // a row and a step left to the device (lily_sample_f32_at)
    const uint32_t* sel_row = nullptr;
    const uint32_t* sel_step = nullptr;
    uint32_t sel_rows = 0;
    uint64_t sel_stride = 0;   // bytes
};

// Validates one row and packs it.  `mode` is the draw the caller asked for.
int pack_row(RowArgs* out, const void* logits, uint32_t vocab, lily_scratch* scratch,
             const lily_sampling_params* params, uint32_t step, uint32_t mode, uint32_t* out_id,
             const lily_draft_dist* dist, const uint32_t* draft, const RowExtras& x) {
    if (logits == nullptr || vocab == 0) {
        return fail(LILY_ERR_INVALID_ARG, "logits must be [V] with V > 0");
    }
    if (out_id == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "out must be U32 [1]");
    }
    if (params == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "params is null");
    }
    if (int rc = lily_params_validate(params)) {
        return rc;
    }
    const bool pen = lily_params_uses_penalties(params) != 0;
    if (scratch != nullptr && scratch->vocab != vocab) {
        return fail(LILY_ERR_VOCAB, "sampler scratch sized for a different vocabulary");
    }
    if (pen && scratch == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "penalties need a sampler scratch");
    }
    if (x.forced != LILY_NO_TOKEN && x.forced >= vocab) {
        return fail(LILY_ERR_RANGE, "forced token %u outside the vocabulary", x.forced);
    }
    std::memset(out, 0, sizeof *out);
    float temperature;
    uint32_t k;
    lily_params_effective(params, &temperature, &k);
    const bool extended = x.allow != nullptr || x.n_bias != 0 || x.out_logprob != nullptr ||
                          x.forced != LILY_NO_TOKEN;
    if (!samples(params) && !extended) {
        mode = MODE_ARGMAX;  // sample.rs:382-385, :404-406, :428-430
    } else if (!samples(params)) {
        mode = MODE_PLAIN;   // greedy over the masked / biased row: a top-1 draw
    }
    if (mode == MODE_DRAFT || mode == MODE_SPEC) {
        if (dist == nullptr || dist->ids_dev == nullptr || dist->probs_dev == nullptr ||
            dist->count_dev == nullptr) {
            return fail(LILY_ERR_INVALID_ARG, "draft distribution slot is null");
        }
        out->q_ids = dist->ids_dev;
        out->q_probs = dist->probs_dev;
        out->q_n = dist->count_dev;
    }
    if (mode == MODE_SPEC) {
        if (draft == nullptr) {
            return fail(LILY_ERR_INVALID_ARG, "draft must be U32 [1]");
        }
        out->draft = draft;
    }
    out->logits = logits;
    out->allow = x.allow;
    out->bias = x.n_bias ? x.bias : nullptr;
    out->n_bias = x.bias ? x.n_bias : 0;
    if (pen) {
        out->counts = scratch->counts;
        out->touched = scratch->touched;
        out->flags |= F_PEN;
    }
    if (x.has_uniform) {
        out->flags |= F_UNIFORM;
        out->uniform = x.uniform;
        out->uniform2 = x.uniform2;
    }
    if (x.forced != LILY_NO_TOKEN) {
        out->flags |= F_FORCED;
        out->forced = x.forced;
    }
    out->sel_row = x.sel_row;
    out->sel_step = x.sel_step;
    out->sel_rows = x.sel_rows;
    out->sel_stride = x.sel_stride;
    out->out_id = out_id;
    out->out_logprob = x.out_logprob;
    out->dbg_ids = x.dbg_ids;
    out->dbg_probs = x.dbg_probs;
    out->dbg_counts = x.dbg_counts;
    out->seed = params->seed;
    out->step = step;
    out->k = k;
    out->mode = mode;
    out->temperature = temperature;
    out->c2 = (float)(1.4426950408889634 / (double)temperature);
    out->top_p = params->top_p;
    out->min_p = params->min_p;
    out->presence = params->presence_penalty;
    out->frequency = params->frequency_penalty;
    out->repetition = params->repetition_penalty;
    if (mode != MODE_ARGMAX && k <= STREAM_K_MAX && out->n_bias <= STREAM_BIAS_CAP) {
        out->flags |= F_STREAM;
    }
    return LILY_OK;
}

// Workgroups per row for a batch of `rows` whose largest candidate count is kmax.
uint32_t choose_slices(const lily_sampler* s, uint32_t rows, uint32_t kmax, uint32_t vocab,
                       int dtype) {
    if (rows > s->ws_rows) {
        return 1;
    }
    uint32_t sl = s->force_slices ? s->force_slices : (TARGET_GROUPS + rows - 1) / rows;
    if (!s->force_slices) {
        // No finer than one block of 256 x 4 chunks per slice: below that a slice saves no
        // time and every further workgroup costs the merge a partial to gather.
        const uint32_t e = dtype == LILY_BF16 ? 8 : 4;
        const uint32_t nch = (vocab + 2 * (e - 1)) / e + 1;
        const uint32_t by_block = (nch + 256u * STREAM_UNROLL - 1) / (256u * STREAM_UNROLL);
        sl = sl > by_block ? by_block : sl;
    }
    sl = sl < 1 ? 1 : sl;
    sl = sl > MAX_SLICES ? MAX_SLICES : sl;
    const uint32_t by_k = MERGE_CAP / (kmax ? kmax : 1);
    sl = sl > by_k ? by_k : sl;
    const uint32_t by_len = (vocab + 2047u) / 2048u;
    sl = sl > by_len ? by_len : sl;
    const uint64_t by_ws = (uint64_t)s->ws_slots / ((uint64_t)rows * (kmax ? kmax : 1));
    sl = sl > by_ws ? (uint32_t)by_ws : sl;
    return sl < 1 ? 1 : sl;
}

// Launches of more than this many workgroups hand their slices over in the relaxed form (see
// last_to_arrive() in device_common.h): there the release / acquire pair costs most (14 us of the
// 72 that 64 rows of 1 024 candidates take over 2 x 1 024 workgroups; 1.2 us of a 4-row step).
constexpr uint32_t RELAXED_MIN_GROUPS = 256;

void fill_cfg(const lily_sampler* s, LaunchCfg* cfg, uint32_t rows, uint32_t vocab, uint32_t slices,
              uint32_t kmax, uint32_t step_delta, const RowArgs* table) {
    std::memset(cfg, 0, sizeof *cfg);
    cfg->relaxed_handover = s->handover == 2u || (s->handover == 0u && (uint64_t)rows * slices > RELAXED_MIN_GROUPS)
                                ? 1u : 0u;
    cfg->table = table;
    cfg->vocab = vocab;
    cfg->slices = slices;
    cfg->step_delta = step_delta;
    cfg->ws_k = kmax ? kmax : 1;
    cfg->ws_cand = Handed<uint64_t>{s->ws_cand};
    cfg->ws_lse = Handed<double>{s->ws_lse};
    cfg->ws_ticket = s->ws_ticket;
    cfg->path = s->force_path;
    cfg->cand_cap = CAND_CAP;
    cfg->path_stats = s->path_stats;
    cfg->list_cap = SPECIAL_LIST_CAP;
}

// Whether a launch over `rows` goes the way of rows that draw among many candidates, and over how
// many workgroups a row then: every row a plain draw (not forced, given as it is or selected on
// the device) without mask or bias list, penalties none or of the kind that only lowers (the
// second launch passes over chunks whose raw values stay below the bound), some row with
// k > STREAM_K_MAX, and at least two workgroups a row.  0 = no.
uint32_t wide_slices(const lily_sampler* s, const RowArgs* rows, uint32_t n, int dtype, uint32_t vocab) {
    if (s->wide_max == nullptr || s->no_wide || s->force_path != 0 || n > s->ws_rows) {
        return 0;
    }
    uint32_t kmax = 0;
    for (uint32_t i = 0; i < n; ++i) {
        const RowArgs& r = rows[i];
        if (r.mode != MODE_PLAIN || (r.flags & F_FORCED) || r.allow != nullptr || r.n_bias != 0) {
            return 0;
        }
        if (r.flags & F_PEN) {
            const bool lowering = r.repetition >= 1.0f && r.presence >= 0.0f && r.frequency >= 0.0f;
            if (!lowering) {
                return 0;
            }
        }
        kmax = r.k > kmax ? r.k : kmax;
    }
    if (kmax <= STREAM_K_MAX) {
        return 0;
    }
    // (twice the workgroups of the other kernels: what runs long here is the one workgroup a
    // row that finishes each launch, and the others have left the CUs by then)
    uint32_t sl = s->force_slices ? s->force_slices : (2 * TARGET_GROUPS + n - 1) / n;
    const uint32_t e = dtype == LILY_BF16 ? 8 : 4;
    const uint32_t nch = (vocab + 2 * (e - 1)) / e + 1;
    const uint32_t by_block = (nch + 256u * STREAM_UNROLL - 1) / (256u * STREAM_UNROLL);
    sl = sl > by_block ? by_block : sl;
    sl = sl > MAX_SLICES ? MAX_SLICES : sl;
    if ((uint64_t)n * MERGE_CAP > s->ws_slots) {   // a row's list of candidates: MERGE_CAP slots
        return 0;
    }
    const uint64_t by_max = (uint64_t)WIDE_FLOATS / ((uint64_t)n * 257u);   // 256 lane maxima and one value a slice
    sl = sl > by_max ? (uint32_t)by_max : sl;
    // the bound is the k-th largest of slices x 256 lane maxima: with twice k of them it is the
    // median of the lanes' maxima, which about 1.4 k values reach on rows of Gaussian logits
    if (sl < 2 || (uint64_t)sl * 256u < 2ull * kmax) {
        return 0;
    }
    return sl;
}

// Attaches the phase trace when the launch fits the caller's buffer.
void attach_trace(const lily_sampler* s, LaunchCfg* cfg, uint32_t rows) {
    if (s->phase_trace != nullptr &&
        (uint64_t)rows * cfg->slices * PHASE_SLOTS <= s->phase_words) {
        cfg->phase_trace = s->phase_trace;
    }
}

// What a launch over `rows` needs beyond the configuration: which kernel variant and
// how much dynamic LDS (candidate slots, then the widest slice's exclusion bitmap; the
// merging workgroup reuses both for up to slices x k gathered candidates).
struct LaunchShape {
    bool excl = false;
    bool lse = false;
    bool bitmap_layout = false;
    size_t dyn_bytes = 0;
    uint32_t excl_words = 0;
    uint32_t cand_cap = 0;
    int kind() const { return bitmap_layout ? (excl ? 1 : 0) : 2; }
};

LaunchShape shape_of(const lily_sampler* s, const RowArgs* rows, uint32_t n, int dtype,
                     uint32_t vocab, uint32_t slices, uint32_t kmax) {
    LaunchShape sh;
    bool any_stream = false, any_old = false, masked = false;
    for (uint32_t i = 0; i < n; ++i) {
        sh.excl = sh.excl || rows[i].allow != nullptr || (rows[i].flags & F_PEN) || rows[i].n_bias;
        sh.lse = sh.lse || rows[i].out_logprob != nullptr;
        if (rows[i].mode == MODE_ARGMAX) {
            continue;
        }
        const bool stream = (rows[i].flags & F_STREAM) && s->force_path == 0;
        any_stream = any_stream || stream;
        // A masked row may be streamed (dense masks), but decides that on the device.
        any_old = any_old || !stream || rows[i].allow != nullptr;
        masked = masked || rows[i].allow != nullptr;
    }
    // Rows outside the streaming select need the candidate buffer, the id list and (rows with
    // an allow-mask) the slice bitmap; a launch of streaming rows only falls back to the
    // exhaustive select.
    sh.bitmap_layout = any_old;
    if (any_old) {
        const uint32_t e = dtype == LILY_BF16 ? 8 : 4;
        const uint32_t nch = (vocab + 2 * (e - 1)) / e + 1;
        const uint32_t per = (nch + slices - 1) / slices;
        sh.excl_words = masked ? (per * e + 31) / 32 + 2 : 0;
        const size_t extra = sh.excl ? ((size_t)sh.excl_words + SPECIAL_LIST_CAP) * 4 : 0;
        sh.dyn_bytes = (size_t)CAND_CAP * 8 + extra;
    }
    if (any_stream && STREAM_LDS_BYTES > sh.dyn_bytes) {
        sh.dyn_bytes = STREAM_LDS_BYTES;
    }
    const size_t tail = (size_t)LILY_SAMPLE_K_CAP * 8 + 3 * (size_t)LILY_SAMPLE_K_CAP * 4;
    if (tail > sh.dyn_bytes) {
        sh.dyn_bytes = tail;
    }
    const size_t merge = slices > 1 ? (size_t)slices * kmax * 8 : 0;
    if (merge > sh.dyn_bytes) {
        sh.dyn_bytes = merge;
    }
    const size_t cap = sh.dyn_bytes / 8;
    sh.cand_cap = any_old ? CAND_CAP : (uint32_t)(cap < CAND_CAP ? cap : CAND_CAP);
    return sh;
}

uint32_t max_k(const RowArgs* rows, uint32_t n) {
    uint32_t k = 1;
    for (uint32_t i = 0; i < n; ++i) {
        if (rows[i].mode != MODE_ARGMAX && rows[i].k > k) {
            k = rows[i].k;
        }
    }
    return k;
}

// Rows that need the kernel holding every select: not streamable, or carrying an allow-mask.
bool heavy_row(const lily_sampler* s, const RowArgs& r) {
    if (r.mode == MODE_ARGMAX) {
        return false;
    }
    return s->force_path != 0 || !(r.flags & F_STREAM) || r.allow != nullptr;
}

constexpr uint32_t SPLIT_MIN_LIGHT = 64;  // streamable rows worth a launch of their own

// Describes the launch(es) of a packed table.  A few rows that need the kernel with every
// select would drag a large batch of streamable rows into it (three workgroups per compute
// unit, more LDS each): the table is then reordered - every row carries its own output
// pointers - and launched in two parts, streamable rows first.
uint32_t plan_parts(const lily_sampler* s, RowArgs* table, uint32_t rows, int dtype, uint32_t vocab,
                    LaunchPart* parts) {
    uint32_t heavy = 0;
    for (uint32_t i = 0; i < rows; ++i) {
        heavy += heavy_row(s, table[i]) ? 1u : 0u;
    }
    const bool split = heavy != 0 && rows - heavy >= SPLIT_MIN_LIGHT;
    if (split) {
        std::stable_partition(table, table + rows,
                              [s](const RowArgs& r) { return !heavy_row(s, r); });
    }
    const uint32_t n_parts = split ? 2u : 1u;
    for (uint32_t q = 0; q < n_parts; ++q) {
        LaunchPart& part = parts[q];
        part.first = q == 0 ? 0u : rows - heavy;
        part.rows = !split ? rows : (q == 0 ? rows - heavy : heavy);
        const RowArgs* sub = table + part.first;
        part.ws_k = max_k(sub, part.rows);
        part.slices = choose_slices(s, part.rows, part.ws_k, vocab, dtype);
        if (const uint32_t ws = wide_slices(s, sub, part.rows, dtype, vocab)) {
            part.wide = true;
            part.slices = ws;
        }
        const LaunchShape shp = shape_of(s, sub, part.rows, dtype, vocab, part.slices, part.ws_k);
        part.kind = shp.kind();
        part.lse = shp.lse;
        part.dyn_bytes = shp.dyn_bytes;
        part.excl_words = shp.excl_words;
        part.bitmap_layout = shp.bitmap_layout;
        part.cand_cap = shp.cand_cap;
    }
    return n_parts;
}

int launch_part(lily_sampler* s, const LaunchPart& part, const RowArgs* table_dev, int dtype,
                uint32_t vocab, uint32_t step_delta, bool traced, const uint32_t* served = nullptr) {
    LaunchCfg cfg;
    fill_cfg(s, &cfg, part.rows, vocab, part.slices, part.ws_k, step_delta, table_dev + part.first);
    cfg.served = served != nullptr ? served + part.first : nullptr;
    if (traced) {
        attach_trace(s, &cfg, part.rows);
    }
    cfg.excl_words = part.excl_words;
    cfg.bitmap_layout = part.bitmap_layout ? 1u : 0u;
    cfg.cand_cap = part.cand_cap;
    if (part.wide) {
        HIP_TRY(launch_rows_wide(s->stream, dtype, part.lse, part.rows, cfg, nullptr, s->wide_max,
                                 s->wide_count));
        return LILY_OK;
    }
    HIP_TRY(launch_rows(s->stream, dtype, part.kind, part.lse, part.rows, cfg, nullptr, part.dyn_bytes));
    return LILY_OK;
}

// What spec_accept needs when the launch that draws the rows in order also runs it.
struct AcceptArgs {
    uint32_t* ctrl = nullptr;
    const uint32_t* ids = nullptr;
    uint32_t pos0 = 0, ratio = 1, chain = 0;
};

int launch_inline(lily_sampler* s, int dtype, uint32_t vocab, const InlineRows& rows, uint32_t n,
                  bool chained = false, const AcceptArgs& accept = AcceptArgs()) {
    ON_DEVICE(s->device);
    const uint32_t kmax = max_k(rows.r, n);
    LaunchCfg cfg;
    if (!chained) {
        if (const uint32_t ws = wide_slices(s, rows.r, n, dtype, vocab)) {
            fill_cfg(s, &cfg, n, vocab, ws, kmax, 0, nullptr);
            bool lse = false;
            for (uint32_t i = 0; i < n; ++i) {
                lse = lse || rows.r[i].out_logprob != nullptr;
            }
            HIP_TRY(launch_rows_wide(s->stream, dtype, lse, n, cfg, &rows, s->wide_max, s->wide_count));
            return LILY_OK;
        }
    }
    const uint32_t slices = choose_slices(s, n, kmax, vocab, dtype);
    fill_cfg(s, &cfg, n, vocab, slices, kmax, 0, nullptr);
    if (chained) {
        // Rows that draw in order count what the rows before them drew into one histogram: the
        // kernel's bookkeeping (an id drawn j times so far has its count raised by j) holds for
        // rows of one scratch under one kind of penalty only.
        for (uint32_t i = 1; i < n; ++i) {
            if (rows.r[i].counts != rows.r[0].counts || rows.r[i].touched != rows.r[0].touched ||
                ((rows.r[i].flags ^ rows.r[0].flags) & F_PEN) != 0u) {
                return fail(LILY_ERR_INVALID_ARG, "rows that draw in order share one scratch (row %u differs)", i);
            }
        }
        cfg.chain_rows = n;
        cfg.chain_cand = Handed<uint64_t>{s->chain_cand};
        cfg.chain_n = Handed<uint32_t>{s->chain_n};
        cfg.chain_ticket = s->chain_ticket;
        cfg.accept_ctrl = accept.ctrl;
        cfg.accept_ids = accept.ids;
        cfg.accept_pos0 = accept.pos0;
        cfg.accept_ratio = accept.ratio;
        cfg.accept_chain = accept.chain;
    }
    attach_trace(s, &cfg, n);
    const LaunchShape shp = shape_of(s, rows.r, n, dtype, vocab, slices, kmax);
    cfg.excl_words = shp.excl_words;
    cfg.bitmap_layout = shp.bitmap_layout ? 1u : 0u;
    cfg.cand_cap = shp.cand_cap;
    const size_t dyn = chained && shp.dyn_bytes < CHAIN_LDS_BYTES ? (size_t)CHAIN_LDS_BYTES : shp.dyn_bytes;
    HIP_TRY(launch_rows(s->stream, dtype, shp.kind(), shp.lse, n, cfg, &rows, dyn));
    return LILY_OK;
}

int one_row(lily_sampler* s, const void* logits, int dtype, uint32_t vocab, lily_scratch* scratch,
            const lily_sampling_params* params, uint32_t step, uint32_t mode, uint32_t* out,
            const lily_draft_dist* dist, const uint32_t* draft, const RowExtras& x = RowExtras()) {
    if (s == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "sampler is null");
    }
    InlineRows rows;
    if (int rc = pack_row(&rows.r[0], logits, vocab, scratch, params, step, mode, out, dist, draft, x)) {
        return rc;
    }
    return launch_inline(s, dtype, vocab, rows, 1);
}

// Packs a lily_rows batch into `table[0..rows)`.
int pack_batch(const lily_rows* b, RowArgs* table) {
    if (b == nullptr || b->rows == 0) {
        return fail(LILY_ERR_INVALID_ARG, "empty batch");
    }
    if (b->dtype != LILY_F32 && b->dtype != LILY_BF16) {
        return fail(LILY_ERR_INVALID_ARG, "dtype must be LILY_F32 or LILY_BF16");
    }
    if (b->logits_dev == nullptr || b->params == nullptr || b->out_ids_dev == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "logits, params and out_ids are required");
    }
    if (b->row_stride < b->vocab) {
        return fail(LILY_ERR_INVALID_ARG, "row_stride is shorter than the vocabulary");
    }
    if (b->bias_dev != nullptr && b->bias_offsets == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "bias needs bias_offsets");
    }
    const size_t es = b->dtype == LILY_BF16 ? 2 : 4;
    const uint32_t words = (b->vocab + 31u) / 32u;
    if (b->scratch != nullptr) {
        // No row under penalties may share its scratch with an earlier row: the rows of a launch
        // run side by side.  Sorted by scratch, sharers are neighbours.
        static thread_local std::vector<std::pair<uintptr_t, uint32_t>> owners;
        owners.clear();
        for (uint32_t r = 0; r < b->rows; ++r) {
            if (b->scratch[r] != nullptr) {
                owners.emplace_back(reinterpret_cast<uintptr_t>(b->scratch[r]), r);
            }
        }
        // (scratches made one after the other usually arrive in ascending order already)
        if (!std::is_sorted(owners.begin(), owners.end())) {
            std::sort(owners.begin(), owners.end());
        }
        // Rows without penalties never touch their scratch: among the rows that name one scratch
        // at most one may use penalties (two would count into one histogram at once).
        for (size_t lo = 0; lo < owners.size();) {
            size_t hi = lo + 1;
            while (hi < owners.size() && owners[hi].first == owners[lo].first) {
                ++hi;
            }
            uint32_t first_pen = 0, n_pen = 0;
            for (size_t i = lo; i < hi && hi - lo > 1; ++i) {
                if (lily_params_uses_penalties(&b->params[owners[i].second])) {
                    if (n_pen++ != 0) {
                        return fail(LILY_ERR_INVALID_ARG, "rows %u and %u use penalties and share a scratch",
                                    first_pen, owners[i].second);
                    }
                    first_pen = owners[i].second;
                }
            }
            lo = hi;
        }
    }
    for (uint32_t r = 0; r < b->rows; ++r) {
        RowExtras x;
        if (b->allow_dev != nullptr) {
            x.allow = b->allow_dev + (size_t)r * b->allow_stride;
            if (b->allow_stride != 0 && b->allow_stride < words) {
                return fail(LILY_ERR_INVALID_ARG, "allow_stride is shorter than the mask");
            }
        }
        if (b->bias_dev != nullptr) {
            const uint32_t lo = b->bias_offsets[r], hi = b->bias_offsets[r + 1];
            if (hi < lo) {
                return fail(LILY_ERR_INVALID_ARG, "bias_offsets must not decrease");
            }
            x.bias = b->bias_dev + lo;
            x.n_bias = hi - lo;
        }
        if (b->forced != nullptr) {
            x.forced = b->forced[r];
        }
        if (b->uniforms != nullptr && !std::isnan(b->uniforms[r])) {
            x.has_uniform = true;
            x.uniform = b->uniforms[r];
            x.uniform2 = b->uniforms[r];
        }
        if (b->out_logprobs_dev != nullptr) {
            x.out_logprob = b->out_logprobs_dev + r;
        }
        if (b->dbg_ids_dev != nullptr) {
            x.dbg_ids = b->dbg_ids_dev + (size_t)r * LILY_SAMPLE_K_CAP;
        }
        if (b->dbg_probs_dev != nullptr) {
            x.dbg_probs = b->dbg_probs_dev + (size_t)r * LILY_SAMPLE_K_CAP;
        }
        if (b->dbg_counts_dev != nullptr) {
            x.dbg_counts = b->dbg_counts_dev + (size_t)r * 2;
        }
        const char* row = static_cast<const char*>(b->logits_dev) + (size_t)r * b->row_stride * es;
        lily_scratch* sc = b->scratch ? b->scratch[r] : nullptr;
        if (int rc = pack_row(&table[r], row, b->vocab, sc, &b->params[r],
                              b->steps ? b->steps[r] : 0, MODE_PLAIN, b->out_ids_dev + r, nullptr,
                              nullptr, x)) {
            return rc;
        }
    }
    return LILY_OK;
}

int ensure_table(lily_sampler* s, uint32_t rows) {
    if (rows <= s->table_cap && rows <= s->stage_cap) {
        return LILY_OK;
    }
    // Growing is rare (first large batch); drain the stream so nothing reads the old buffers.
    HIP_TRY(hipStreamSynchronize(s->stream));
    uint32_t cap = 1024;
    while (cap < rows) {
        cap <<= 1;
    }
    if (s->table_dev) {
        (void)hipFree(s->table_dev);
        s->table_dev = nullptr;
    }
    for (uint32_t i = 0; i < STAGE_SLOTS; ++i) {
        if (s->stage[i]) {
            (void)hipHostFree(s->stage[i]);
            s->stage[i] = nullptr;
        }
        s->stage_used[i] = false;
    }
    s->table_cap = s->stage_cap = 0;
    // (behind the descriptors: three words a row for the calls that draw from summaries)
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&s->table_dev), (size_t)cap * STAGE_ROW_BYTES));
    for (uint32_t i = 0; i < STAGE_SLOTS; ++i) {
        HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&s->stage[i]), (size_t)cap * STAGE_ROW_BYTES,
                              hipHostMallocDefault));
    }
    s->table_cap = s->stage_cap = cap;
    return LILY_OK;
}

}  // namespace

namespace lily {

int api_fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return code;
}

int scratch_device(const lily_scratch_t* sc) { return sc->s->device; }

int sample_row_with_workspace(int device, hipStream_t stream, const Workspace& ws, const float* logits,
                              uint32_t vocab, lily_scratch_t* scratch,
                              const lily_sampling_params* params, uint32_t step, uint32_t* out) {
    lily_sampler s;  // a view for this one launch: owns nothing, is never destroyed
    s.device = device;
    s.stream = stream;
    s.ws_cand = ws.cand;
    s.ws_lse = ws.lse;
    s.ws_ticket = ws.ticket;
    s.ws_rows = ws.rows;
    s.ws_slots = ws.slots;
    return one_row(&s, logits, LILY_F32, vocab, scratch, params, step, MODE_PLAIN, out, nullptr,
                   nullptr);
}

}  // namespace lily

extern "C" {

const char* lily_last_error(void) { return g_error; }

// ---- pure host helpers

void lily_params_greedy(lily_sampling_params* out) {
    out->temperature = 0.0f;
    out->top_k = 1;
    out->top_p = 1.0f;
    out->min_p = 0.0f;
    out->presence_penalty = 0.0f;
    out->frequency_penalty = 0.0f;
    out->repetition_penalty = 1.0f;
    out->reserved = 0;
    out->seed = 0;
}

int lily_params_is_greedy(const lily_sampling_params* p) {
    return p->temperature <= 0.0f || p->top_k == 1;
}

int lily_params_uses_penalties(const lily_sampling_params* p) {
    return p->presence_penalty != 0.0f || p->frequency_penalty != 0.0f ||
           p->repetition_penalty != 1.0f;
}

int lily_params_validate(const lily_sampling_params* p) {
    if (!(std::isfinite(p->temperature) && p->temperature >= 0.0f)) {
        return fail(LILY_ERR_PARAMS, "temperature must be a finite number >= 0");
    }
    if (!(std::isfinite(p->top_p) && p->top_p > 0.0f && p->top_p <= 1.0f)) {
        return fail(LILY_ERR_PARAMS, "top_p must be in (0, 1]");
    }
    if (!(std::isfinite(p->min_p) && p->min_p >= 0.0f && p->min_p <= 1.0f)) {
        return fail(LILY_ERR_PARAMS, "min_p must be in [0, 1]");
    }
    if (!(std::isfinite(p->repetition_penalty) && p->repetition_penalty > 0.0f)) {
        return fail(LILY_ERR_PARAMS, "repetition_penalty must be > 0");
    }
    if (!(std::isfinite(p->presence_penalty) && std::isfinite(p->frequency_penalty))) {
        return fail(LILY_ERR_PARAMS, "penalties must be finite");
    }
    return LILY_OK;
}

int lily_params_resolve(const lily_sampling_fields* f, const lily_sampling_params* d,
                        uint64_t fresh_seed, lily_sampling_params* out) {
    if (f == nullptr || d == nullptr || out == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "resolve needs fields, defaults and out");
    }
    lily_sampling_params p = *d;
    p.reserved = 0;
    if (f->has & LILY_HAS_TEMPERATURE) p.temperature = f->temperature;
    if (f->has & LILY_HAS_TOP_P) p.top_p = f->top_p;
    if (f->has & LILY_HAS_MIN_P) p.min_p = f->min_p;
    if (f->has & LILY_HAS_PRESENCE) p.presence_penalty = f->presence_penalty;
    if (f->has & LILY_HAS_FREQUENCY) p.frequency_penalty = f->frequency_penalty;
    if (f->has & LILY_HAS_REPETITION) p.repetition_penalty = f->repetition_penalty;
    if (f->has & LILY_HAS_TOP_K) {
        // api.rs:803-807: a negative k is "off"; beyond u32 the cap applies anyway.
        p.top_k = f->top_k < 0 ? 0u : (f->top_k > 0xffffffffll ? 0xffffffffu : (uint32_t)f->top_k);
    }
    p.seed = (f->has & LILY_HAS_SEED) ? (uint64_t)f->seed : fresh_seed;
    *out = p;
    return lily_params_validate(out);
}

void lily_params_effective(const lily_sampling_params* p, float* temperature, uint32_t* top_k) {
    if (lily_params_is_greedy(p)) {
        *temperature = 1.0f;
        *top_k = 1;
    } else {
        *temperature = p->temperature;
        *top_k = p->top_k == 0 ? LILY_SAMPLE_K_CAP
                               : (p->top_k < LILY_SAMPLE_K_CAP ? p->top_k : LILY_SAMPLE_K_CAP);
    }
}

void lily_draft_params(const lily_sampling_params* p, lily_sampling_params* out) {
    *out = *p;
    out->presence_penalty = 0.0f;
    out->frequency_penalty = 0.0f;
    out->repetition_penalty = 1.0f;
}

uint32_t lily_draft_step(uint32_t step) { return lilym_draft_step(step); }
float lily_uniform_for(uint64_t seed, uint32_t step) { return lilym_uniform_for(seed, step); }
uint32_t lily_slot_pos(uint32_t i) { return 2 + 3 * i; }
uint32_t lily_slot_block(uint32_t i) { return 3 + 3 * i; }
uint32_t lily_slot_count(uint32_t i) { return 4 + 3 * i; }
uint32_t lily_ctrl_words(uint32_t chain) { return (2 + 3 * chain) * LILY_CTRL_STRIDE; }

// ---- sampler

int lily_sampler_create(int device, void* hip_stream, lily_sampler_t** out) {
    if (out == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "out is null");
    }
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0) {
        return fail(LILY_ERR_HIP, "no HIP device: %s", hipGetErrorString(e));
    }
    if (device < 0 || device >= n) {
        return fail(LILY_ERR_RANGE, "device %d of %d", device, n);
    }
    ON_DEVICE(device);
    lily_sampler* s = new (std::nothrow) lily_sampler;
    if (s == nullptr) {
        return fail(LILY_ERR_NOMEM, "out of host memory");
    }
    s->device = device;
    s->stream = static_cast<hipStream_t>(hip_stream);
    if (const char* p = std::getenv("LILY_SAMPLER_PATH")) {
        s->force_path = (uint32_t)std::atoi(p);
    }
    if (const char* p = std::getenv("LILY_SAMPLER_SLICES")) {
        s->force_slices = (uint32_t)std::atoi(p);
    }
    if (const char* p = std::getenv("LILY_SAMPLER_WIDE")) {
        s->no_wide = std::atoi(p) == 0;
    }
    if (const char* p = std::getenv("LILY_SAMPLER_HEAD")) {
        s->head_library_rows = std::strcmp(p, "own") == 0 ? 0u : std::strcmp(p, "library") == 0 ? 1u : (uint32_t)std::atoi(p);
        s->head_library_rows_codes = s->head_library_rows;
    }
    if (const char* p = std::getenv("LILY_SAMPLER_HANDOVER")) {
        s->handover = std::strcmp(p, "strict") == 0 ? 1u : std::strcmp(p, "relaxed") == 0 ? 2u : 0u;
    }
    const size_t slots = (size_t)WS_ROWS * MAX_SLICES;
    hipError_t err = hipMalloc(reinterpret_cast<void**>(&s->ws_cand),
                               (size_t)WS_SLOTS * sizeof(uint64_t));
    if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void**>(&s->ws_lse), slots * 16);
    if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void**>(&s->ws_ticket), WS_ROWS * 4);
    if (err == hipSuccess) err = hipMemset(s->ws_ticket, 0, WS_ROWS * 4);
    if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void**>(&s->wide_max), (size_t)WIDE_FLOATS * 4);
    if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void**>(&s->wide_count), WS_ROWS * 4);
    if (err == hipSuccess) err = hipMemset(s->wide_count, 0, WS_ROWS * 4);
    const size_t chain_bytes = (size_t)LILY_MAX_VERIFY_ROWS * CHAIN_CAP * 8 + (LILY_MAX_VERIFY_ROWS + 1) * 4;
    if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void**>(&s->chain_cand), chain_bytes);
    if (err == hipSuccess) err = hipMemset(s->chain_cand, 0, chain_bytes);
    if (err == hipSuccess) {
        s->chain_n = reinterpret_cast<uint32_t*>(s->chain_cand + (size_t)LILY_MAX_VERIFY_ROWS * CHAIN_CAP);
        s->chain_ticket = s->chain_n + LILY_MAX_VERIFY_ROWS;
    }
    for (uint32_t i = 0; i < STAGE_SLOTS && err == hipSuccess; ++i) {
        err = hipEventCreateWithFlags(&s->stage_done[i], hipEventDisableTiming | hipEventReleaseToDevice);
    }
    if (err != hipSuccess) {
        lily_sampler_destroy(s);
        return hip_fail(err, "sampler workspace");
    }
    if (int rc = static_scratch_init(device)) {
        lily_sampler_destroy(s);
        return rc;
    }
    *out = s;
    return LILY_OK;
}

void lily_sampler_destroy(lily_sampler_t* s) {
    if (s == nullptr) {
        return;
    }
    DeviceScope device_scope_(s->device);
    (void)hipStreamSynchronize(s->stream);
    (void)hipFree(s->ws_cand);
    (void)hipFree(s->ws_lse);
    (void)hipFree(s->ws_ticket);
    (void)hipFree(s->wide_max);
    (void)hipFree(s->wide_count);
    (void)hipFree(s->chain_cand);
    (void)hipFree(s->table_dev);
    for (uint32_t i = 0; i < STAGE_SLOTS; ++i) {
        if (s->stage[i]) (void)hipHostFree(s->stage[i]);
        if (s->stage_done[i]) (void)hipEventDestroy(s->stage_done[i]);
    }
    delete s;
}

int lily_sampler_set_phase_trace(lily_sampler_t* s, uint64_t* trace_dev, uint64_t capacity_words) {
    if (s == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "sampler is null");
    }
    s->phase_trace = trace_dev;
    s->phase_words = trace_dev ? capacity_words : 0;
    return LILY_OK;
}

int lily_sampler_set_path_stats(lily_sampler_t* s, uint32_t* stats_dev) {
    if (s == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "sampler is null");
    }
    s->path_stats = stats_dev;
    return LILY_OK;
}

uint32_t lily_sampler_slices_for(const lily_sampler_t* s, uint32_t rows, uint32_t k, uint32_t vocab,
                                 lily_dtype dtype) {
    if (s == nullptr || rows == 0) {
        return 0;
    }
    return choose_slices(s, rows, k ? k : 1, vocab, (int)dtype);
}

int lily_sampler_synchronize(lily_sampler_t* s) {
    if (s == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "sampler is null");
    }
    HIP_TRY(hipStreamSynchronize(s->stream));
    return LILY_OK;
}

// ---- scratch

int lily_scratch_create(lily_sampler_t* s, uint32_t vocab, lily_scratch_t** out) {
    if (s == nullptr || out == nullptr || vocab == 0) {
        return fail(LILY_ERR_INVALID_ARG, "scratch needs a sampler and a vocabulary > 0");
    }
    *out = nullptr;
    ON_DEVICE(s->device);
    lily_scratch* sc = new (std::nothrow) lily_scratch;
    if (sc == nullptr) {
        return fail(LILY_ERR_NOMEM, "out of host memory");
    }
    sc->s = s;
    sc->vocab = vocab;
    sc->words = (vocab + 31u) / 32u;
    // One allocation: the counts, then the bitmap (16-byte aligned, four spare words).
    const size_t dense = (((size_t)vocab * 4) + 15) & ~(size_t)15;
    const size_t bitmap = (((size_t)(sc->words + 4) * 4) + 15) & ~(size_t)15;
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&sc->counts), dense + bitmap);
    if (e != hipSuccess) {
        delete sc;
        return hip_fail(e, "scratch allocation");
    }
    sc->touched = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(sc->counts) + dense);
    *out = sc;
    return lily_scratch_reset_counts(sc);
}

void lily_scratch_destroy(lily_scratch_t* sc) {
    if (sc == nullptr) {
        return;
    }
    DeviceScope device_scope_(sc->s->device);
    (void)hipStreamSynchronize(sc->s->stream);
    (void)hipFree(sc->counts);
    delete sc;
}

uint32_t lily_scratch_vocab(const lily_scratch_t* sc) { return sc ? sc->vocab : 0; }

int lily_scratch_reset_counts(lily_scratch_t* sc) {
    if (sc == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "scratch is null");
    }
    ON_DEVICE(sc->s->device);
    HIP_TRY(launch_fill_u32(sc->s->stream, sc->counts, sc->vocab, 0));
    HIP_TRY(launch_fill_u32(sc->s->stream, sc->touched, sc->words + 4, 0));
    return LILY_OK;
}

int lily_scratch_uncount(lily_scratch_t* sc, uint32_t token) {
    if (sc == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "scratch is null");
    }
    if (token >= sc->vocab) {
        return LILY_OK;  // sample.rs:149-151
    }
    ON_DEVICE(sc->s->device);
    HIP_TRY(launch_uncount(sc->s->stream, view_of(sc), token));
    return LILY_OK;
}

int lily_scratch_uncount_after(lily_scratch_t* sc, const uint32_t* draws_dev, uint32_t m,
                               const uint32_t* accepted_dev, uint32_t accepted_cap) {
    if (sc == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "scratch is null");
    }
    if (draws_dev == nullptr || accepted_dev == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "draws or accepted row is null");
    }
    if (m == 0 || m > LILY_MAX_VERIFY_ROWS) {
        return fail(LILY_ERR_RANGE, "rollback over %u rows (1..%u)", m, (unsigned)LILY_MAX_VERIFY_ROWS);
    }
    ON_DEVICE(sc->s->device);
    HIP_TRY(launch_uncount_after(sc->s->stream, view_of(sc), draws_dev, m, accepted_dev, accepted_cap));
    return LILY_OK;
}

int lily_scratch_copy_counts_from(lily_scratch_t* dst, const lily_scratch_t* src) {
    if (dst == nullptr || src == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "scratch is null");
    }
    if (dst->vocab != src->vocab) {
        return fail(LILY_ERR_VOCAB, "sampler scratches for different vocabularies");
    }
    ON_DEVICE(dst->s->device);
    HIP_TRY(hipMemcpyAsync(dst->counts, src->counts, (size_t)src->vocab * 4, hipMemcpyDeviceToDevice,
                           dst->s->stream));
    // (the bitmap and the largest count behind it)
    HIP_TRY(hipMemcpyAsync(dst->touched, src->touched, (size_t)(src->words + 2) * 4,
                           hipMemcpyDeviceToDevice, dst->s->stream));
    return LILY_OK;
}

int lily_scratch_add_history(lily_scratch_t* sc, const uint32_t* ids_dev, uint32_t n) {
    if (sc == nullptr || (ids_dev == nullptr && n != 0)) {
        return fail(LILY_ERR_INVALID_ARG, "scratch or ids is null");
    }
    ON_DEVICE(sc->s->device);
    HIP_TRY(launch_add_history(sc->s->stream, view_of(sc), ids_dev, n));
    return LILY_OK;
}

int lily_scratch_write_counts(lily_scratch_t* sc, const uint32_t* host_counts) {
    if (sc == nullptr || host_counts == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "scratch or counts is null");
    }
    ON_DEVICE(sc->s->device);
    HIP_TRY(hipStreamSynchronize(sc->s->stream));
    HIP_TRY(hipMemcpy(sc->counts, host_counts, (size_t)sc->vocab * 4, hipMemcpyHostToDevice));
    HIP_TRY(launch_rebuild_listed(sc->s->stream, view_of(sc)));
    HIP_TRY(hipStreamSynchronize(sc->s->stream));
    return LILY_OK;
}

int lily_scratch_read_counts(lily_scratch_t* sc, uint32_t* host_counts) {
    if (sc == nullptr || host_counts == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "scratch or counts is null");
    }
    ON_DEVICE(sc->s->device);
    HIP_TRY(hipStreamSynchronize(sc->s->stream));
    HIP_TRY(hipMemcpy(host_counts, sc->counts, (size_t)sc->vocab * 4, hipMemcpyDeviceToHost));
    return LILY_OK;
}

// ---- draft distributions

int lily_draft_dists_create(lily_sampler_t* s, uint32_t slots, lily_draft_dists_t** out) {
    if (s == nullptr || out == nullptr || slots == 0) {
        return fail(LILY_ERR_INVALID_ARG, "draft dists need a sampler and slots > 0");
    }
    *out = nullptr;
    ON_DEVICE(s->device);
    lily_draft_dists* d = new (std::nothrow) lily_draft_dists;
    if (d == nullptr) {
        return fail(LILY_ERR_NOMEM, "out of host memory");
    }
    d->s = s;
    d->slots = slots;
    const size_t n = (size_t)slots * LILY_SAMPLE_K_CAP;
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&d->ids), n * 8 + (size_t)slots * 4);
    if (e != hipSuccess) {
        delete d;
        return hip_fail(e, "draft dists allocation");
    }
    d->probs = reinterpret_cast<float*>(d->ids + n);
    d->counts = reinterpret_cast<uint32_t*>(d->probs + n);
    e = hipMemsetAsync(d->ids, 0, n * 8 + (size_t)slots * 4, s->stream);
    if (e != hipSuccess) {
        (void)hipFree(d->ids);
        delete d;
        return hip_fail(e, "draft dists clear");
    }
    *out = d;
    return LILY_OK;
}

void lily_draft_dists_destroy(lily_draft_dists_t* d) {
    if (d == nullptr) {
        return;
    }
    DeviceScope device_scope_(d->s->device);
    (void)hipStreamSynchronize(d->s->stream);
    (void)hipFree(d->ids);
    delete d;
}

// ---- token slots (the decode loop's ping-pong outputs)

int lily_token_slots_create(lily_sampler_t* s, uint32_t slots, uint32_t words, lily_token_slots_t** out) {
    if (s == nullptr || out == nullptr || slots == 0 || words == 0 || slots > 64 || words > (1u << 20)) {
        return fail(LILY_ERR_INVALID_ARG, "token slots need a sampler, 1..64 slots and 1..2^20 words");
    }
    *out = nullptr;
    ON_DEVICE(s->device);
    lily_token_slots* t = new (std::nothrow) lily_token_slots;
    if (t == nullptr) {
        return fail(LILY_ERR_NOMEM, "out of host memory");
    }
    t->s = s;
    t->slots = slots;
    t->words = words;
    t->done = new (std::nothrow) hipEvent_t[slots]();
    t->published = new (std::nothrow) bool[slots]();
    const size_t bytes = (size_t)slots * words * 4;
    hipError_t e = t->done && t->published ? hipSuccess : hipErrorOutOfMemory;
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&t->dev), bytes);
    if (e == hipSuccess) e = hipMemsetAsync(t->dev, 0xff, bytes, s->stream);
    if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void**>(&t->host), bytes, hipHostMallocDefault);
    for (uint32_t i = 0; e == hipSuccess && i < slots; ++i) {
        e = hipEventCreateWithFlags(&t->done[i], hipEventDisableTiming);
    }
    if (e != hipSuccess) {
        lily_token_slots_destroy(t);
        return hip_fail(e, "token slots allocation");
    }
    std::memset(t->host, 0xff, bytes);
    *out = t;
    return LILY_OK;
}

void lily_token_slots_destroy(lily_token_slots_t* t) {
    if (t == nullptr) {
        return;
    }
    DeviceScope device_scope_(t->s->device);
    (void)hipStreamSynchronize(t->s->stream);
    for (uint32_t i = 0; t->done != nullptr && i < t->slots; ++i) {
        if (t->done[i]) (void)hipEventDestroy(t->done[i]);
    }
    if (t->dev) (void)hipFree(t->dev);
    if (t->host) (void)hipHostFree(t->host);
    delete[] t->done;
    delete[] t->published;
    delete t;
}

uint32_t* lily_token_slots_device(const lily_token_slots_t* t, uint32_t slot) {
    if (t == nullptr || slot >= t->slots) {
        (void)fail(LILY_ERR_RANGE, "token slot out of range");
        return nullptr;
    }
    return t->dev + (size_t)slot * t->words;
}

int lily_token_slots_publish(lily_token_slots_t* t, uint32_t slot) {
    if (t == nullptr || slot >= t->slots) {
        return fail(LILY_ERR_RANGE, "token slot out of range");
    }
    ON_DEVICE(t->s->device);
    const size_t off = (size_t)slot * t->words;
    HIP_TRY(hipMemcpyAsync(t->host + off, t->dev + off, (size_t)t->words * 4, hipMemcpyDeviceToHost,
                           t->s->stream));
    HIP_TRY(hipEventRecord(t->done[slot], t->s->stream));
    t->published[slot] = true;
    return LILY_OK;
}

int lily_token_slots_poll(lily_token_slots_t* t, uint32_t slot, uint32_t* host_out, int* ready) {
    if (t == nullptr || slot >= t->slots || ready == nullptr) {
        return fail(LILY_ERR_RANGE, "token slot out of range, or ready is null");
    }
    *ready = 0;
    if (!t->published[slot]) {
        return fail(LILY_ERR_INVALID_ARG, "token slot %u was not published since it was last read", slot);
    }
    const hipError_t e = hipEventQuery(t->done[slot]);
    if (e == hipErrorNotReady) {
        return LILY_OK;
    }
    HIP_TRY(e);
    if (host_out != nullptr) {
        std::memcpy(host_out, t->host + (size_t)slot * t->words, (size_t)t->words * 4);
    }
    t->published[slot] = false;
    *ready = 1;
    return LILY_OK;
}

int lily_token_slots_wait_polled(lily_token_slots_t* t, uint32_t slot, uint32_t* host_out,
                                 uint64_t max_polls) {
    for (uint64_t i = 0; max_polls == 0 || i < max_polls; ++i) {
        int ready = 0;
        if (int rc = lily_token_slots_poll(t, slot, host_out, &ready)) {
            return rc;
        }
        if (ready) {
            return LILY_OK;
        }
    }
    return fail(LILY_ERR_RANGE, "token slot %u not ready after %llu polls", slot,
                (unsigned long long)max_polls);
}

int lily_scratch_move_counts(lily_scratch_t* from, lily_scratch_t* to) {
    if (from == nullptr || to == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "move_counts needs two scratches");
    }
    if (from == to) {
        return LILY_OK;   // batch.rs:147-149
    }
    return lily_scratch_copy_counts_from(to, from);
}

int lily_draft_dists_slot(const lily_draft_dists_t* d, uint32_t i, lily_draft_dist* out) {
    if (d == nullptr || out == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "draft dists or out is null");
    }
    if (i >= d->slots) {
        return fail(LILY_ERR_RANGE, "slot %u of %u", i, d->slots);
    }
    out->ids_dev = d->ids + (size_t)i * LILY_SAMPLE_K_CAP;
    out->probs_dev = d->probs + (size_t)i * LILY_SAMPLE_K_CAP;
    out->count_dev = d->counts + i;
    return LILY_OK;
}

// ---- single-row draws

int lily_sample_f32(lily_sampler_t* s, const float* logits_dev, uint32_t vocab,
                    lily_scratch_t* scratch, const lily_sampling_params* params, uint32_t step,
                    uint32_t* out_dev) {
    return one_row(s, logits_dev, LILY_F32, vocab, scratch, params, step, MODE_PLAIN, out_dev,
                   nullptr, nullptr);
}

int lily_sample_draft_f32(lily_sampler_t* s, const float* logits_dev, uint32_t vocab,
                          lily_scratch_t* scratch, const lily_sampling_params* params,
                          uint32_t step, uint32_t* out_dev, const lily_draft_dist* dist) {
    return one_row(s, logits_dev, LILY_F32, vocab, scratch, params, step, MODE_DRAFT, out_dev, dist,
                   nullptr);
}

namespace {

int selection(RowExtras* x, uint32_t vocab, uint64_t row_stride, uint32_t rows, const uint32_t* row_dev,
              const uint32_t* step_dev) {
    if (rows == 0 || row_stride < vocab) {
        return fail(LILY_ERR_INVALID_ARG, "logits must be [rows][row_stride] with rows > 0 and "
                                          "row_stride >= vocab");
    }
    x->sel_row = row_dev;
    x->sel_step = step_dev;
    x->sel_rows = rows;
    x->sel_stride = row_stride * 4;
    return LILY_OK;
}

}  // namespace

int lily_sample_f32_at(lily_sampler_t* s, const float* logits_dev, uint32_t vocab, uint64_t row_stride,
                       uint32_t rows, const uint32_t* row_dev, lily_scratch_t* scratch,
                       const lily_sampling_params* params, uint32_t step_base,
                       const uint32_t* step_dev, uint32_t* out_dev) {
    RowExtras x;
    if (int rc = selection(&x, vocab, row_stride, rows, row_dev, step_dev)) {
        return rc;
    }
    return one_row(s, logits_dev, LILY_F32, vocab, scratch, params, step_base, MODE_PLAIN, out_dev,
                   nullptr, nullptr, x);
}

int lily_sample_draft_f32_at(lily_sampler_t* s, const float* logits_dev, uint32_t vocab,
                             uint64_t row_stride, uint32_t rows, const uint32_t* row_dev,
                             lily_scratch_t* scratch, const lily_sampling_params* params,
                             uint32_t step_base, const uint32_t* step_dev, uint32_t* out_dev,
                             const lily_draft_dist* dist) {
    RowExtras x;
    if (int rc = selection(&x, vocab, row_stride, rows, row_dev, step_dev)) {
        return rc;
    }
    return one_row(s, logits_dev, LILY_F32, vocab, scratch, params, step_base, MODE_DRAFT, out_dev,
                   dist, nullptr, x);
}

int lily_sample_spec_f32(lily_sampler_t* s, const float* logits_dev, uint32_t vocab,
                         lily_scratch_t* scratch, const lily_sampling_params* params,
                         uint32_t step, const lily_draft_dist* dist, const uint32_t* draft_dev,
                         uint32_t* out_dev) {
    return one_row(s, logits_dev, LILY_F32, vocab, scratch, params, step, MODE_SPEC, out_dev, dist,
                   draft_dev);
}

// A draw's uniforms lie in [0, 1) like uniform_for's (sample.rs:435-441).
static int check_uniform(float u, const char* name) {
    if (!(u >= 0.0f && u < 1.0f)) {
        return fail(LILY_ERR_INVALID_ARG, "%s must lie in [0, 1)", name);
    }
    return LILY_OK;
}

int lily_sample_spec_f32_uniforms(lily_sampler_t* s, const float* logits_dev, uint32_t vocab,
                                  lily_scratch_t* scratch, const lily_sampling_params* params,
                                  uint32_t step, const lily_draft_dist* dist,
                                  const uint32_t* draft_dev, uint32_t* out_dev, float u1, float u2) {
    if (int rc = check_uniform(u1, "u1")) {
        return rc;
    }
    if (int rc = check_uniform(u2, "u2")) {
        return rc;
    }
    RowExtras x;
    x.has_uniform = true;
    x.uniform = u1;
    x.uniform2 = u2;
    return one_row(s, logits_dev, LILY_F32, vocab, scratch, params, step, MODE_SPEC, out_dev, dist,
                   draft_dev, x);
}

int lily_argmax_f32(lily_sampler_t* s, const float* x_dev, uint32_t n, uint32_t* out_dev) {
    lily_sampling_params g;
    lily_params_greedy(&g);
    if (n == 0) {
        return fail(LILY_ERR_INVALID_ARG, "empty argmax input");
    }
    return one_row(s, x_dev, LILY_F32, n, nullptr, &g, 0, MODE_PLAIN, out_dev, nullptr, nullptr);
}

// ---- speculative control

int lily_spec_accept(lily_sampler_t* s, const uint32_t* draws_dev, const uint32_t* ids_dev,
                     uint32_t m, uint32_t* ctrl_dev, uint32_t ctrl_words, uint32_t pos0,
                     uint32_t ratio, uint32_t chain) {
    if (s == nullptr || draws_dev == nullptr || ids_dev == nullptr || ctrl_dev == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "spec_accept works on U32 tensors");
    }
    if (m == 0) {
        return fail(LILY_ERR_INVALID_ARG, "draws and ids must both hold the verified rows");
    }
    if (ctrl_words < lily_ctrl_words(chain)) {
        return fail(LILY_ERR_RANGE, "control block too small for %u chain rows", chain);
    }
    if (ratio == 0) {
        return fail(LILY_ERR_INVALID_ARG, "indexer block ratio must be nonzero");
    }
    ON_DEVICE(s->device);
    HIP_TRY(launch_spec_accept(s->stream, draws_dev, ids_dev, ctrl_dev, m, pos0, ratio, chain));
    return LILY_OK;
}

int lily_copy_row_u32(lily_sampler_t* s, const uint32_t* src_dev, uint32_t rows, uint32_t words,
                      const uint32_t* row_dev, uint32_t* dst_dev) {
    if (s == nullptr || src_dev == nullptr || row_dev == nullptr || dst_dev == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "copy_row needs src, row and dst");
    }
    if (rows == 0 || words == 0) {
        return fail(LILY_ERR_INVALID_ARG, "src must be [rows, words] with both > 0");
    }
    ON_DEVICE(s->device);
    HIP_TRY(launch_copy_row(s->stream, src_dev, dst_dev, words, rows, row_dev));
    return LILY_OK;
}

int lily_probe_read(lily_sampler_t* s, const void* base_dev, uint32_t rows, uint64_t row_bytes,
                    uint64_t stride_bytes, uint32_t* out_dev) {
    if (s == nullptr || base_dev == nullptr || out_dev == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "probe_read needs base and out");
    }
    if (rows == 0 || row_bytes < 16 || row_bytes % 16 != 0 || stride_bytes % 16 != 0 ||
        stride_bytes < row_bytes || (reinterpret_cast<uintptr_t>(base_dev) & 15u) != 0) {
        return fail(LILY_ERR_INVALID_ARG,
                    "probe_read: rows > 0, 16-byte aligned base, row_bytes and stride_bytes multiples "
                    "of 16 with 16 <= row_bytes <= stride_bytes");
    }
    ON_DEVICE(s->device);
    HIP_TRY(launch_probe_read(s->stream, base_dev, rows, row_bytes, stride_bytes, out_dev));
    return LILY_OK;
}

int lily_spec_verify(lily_sampler_t* s, const void* logits_dev, lily_dtype dtype, uint32_t vocab,
                     uint64_t row_stride, uint32_t m, lily_scratch_t* scratch,
                     const lily_sampling_params* params, uint32_t step0,
                     const lily_draft_dists_t* dists, const uint32_t* ids_dev,
                     uint32_t* verify_tokens_dev, uint32_t* ctrl_dev, uint32_t ctrl_words,
                     uint32_t pos0, uint32_t ratio, uint32_t chain, const float* uniforms) {
    if (s == nullptr || logits_dev == nullptr || ids_dev == nullptr || verify_tokens_dev == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "verify needs logits, ids and verify_tokens");
    }
    if (m == 0 || m > LILY_MAX_VERIFY_ROWS) {
        return fail(LILY_ERR_RANGE, "verify rows %u outside 1..%u", m, LILY_MAX_VERIFY_ROWS);
    }
    if (dtype != LILY_F32 && dtype != LILY_BF16) {
        return fail(LILY_ERR_INVALID_ARG, "dtype must be LILY_F32 or LILY_BF16");
    }
    if (row_stride < vocab) {
        return fail(LILY_ERR_INVALID_ARG, "row_stride is shorter than the vocabulary");
    }
    if (params == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "params is null");
    }
    const bool sampled = samples(params);
    if (sampled && m > 1 && (dists == nullptr || dists->slots < m - 1)) {
        return fail(LILY_ERR_RANGE, "verify needs %u draft distribution slots", m - 1);
    }
    // Everything is validated before the first row is enqueued: an error leaves no draw counted.
    if (ctrl_dev != nullptr) {
        if (ctrl_words < lily_ctrl_words(chain)) {
            return fail(LILY_ERR_RANGE, "control block too small for %u chain rows", chain);
        }
        if (ratio == 0) {
            return fail(LILY_ERR_INVALID_ARG, "indexer block ratio must be nonzero");
        }
    }
    for (uint32_t j = 0; uniforms != nullptr && j < 2 * m; ++j) {
        if (int rc = check_uniform(uniforms[j], "verify uniforms")) {
            return rc;
        }
    }
    const size_t es = dtype == LILY_BF16 ? 2 : 4;
    // Under penalties row j must see the counts of the rows before it.  Where the penalties can
    // only lower a value, all rows share one launch whose last workgroup draws them in order
    // (each row collects m - 1 candidates more than it draws from, see row_body); otherwise one
    // launch per row.  Without penalties the rows are independent and share one launch.
    static_assert(LILY_MAX_VERIFY_ROWS <= (uint32_t)INLINE_ROWS, "verify rows travel inline");
    const bool pen = lily_params_uses_penalties(params) != 0;
    float t_eff;
    uint32_t k_eff;
    lily_params_effective(params, &t_eff, &k_eff);
    const bool in_order = pen && m > 1 && params->repetition_penalty >= 1.0f &&
                          params->presence_penalty >= 0.0f && params->frequency_penalty >= 0.0f &&
                          k_eff + m - 1 <= LILY_SAMPLE_K_CAP;
    const bool chained = pen && !in_order;
    InlineRows rows;
    for (uint32_t j = 0; j < m; ++j) {
        const char* row = static_cast<const char*>(logits_dev) + (size_t)j * row_stride * es;
        RowExtras x;
        if (uniforms != nullptr) {
            x.has_uniform = true;
            x.uniform = uniforms[2 * j];
            x.uniform2 = uniforms[2 * j + 1];
        }
        lily_draft_dist slot;
        const bool spec = j + 1 < m && sampled;
        if (spec) {
            if (int rc = lily_draft_dists_slot(dists, j, &slot)) {
                return rc;
            }
        }
        if (int rc = pack_row(&rows.r[chained ? 0 : j], row, vocab, scratch, params, step0 + j,
                              spec ? MODE_SPEC : MODE_PLAIN, verify_tokens_dev + j,
                              spec ? &slot : nullptr, spec ? ids_dev + j + 1 : nullptr, x)) {
            return rc;
        }
        if (chained) {
            if (int rc = launch_inline(s, dtype, vocab, rows, 1)) {
                return rc;
            }
        }
    }
    if (in_order) {
        for (uint32_t j = 0; j < m; ++j) {
            RowArgs& r = rows.r[j];
            r.k_draw = r.k;
            r.k = r.k + m - 1;
            if (r.k > STREAM_K_MAX) {
                r.flags &= ~(uint32_t)F_STREAM;
            }
        }
    }
    if (!chained) {
        AcceptArgs accept;
        if (in_order && ctrl_dev != nullptr) {
            accept.ctrl = ctrl_dev;
            accept.ids = ids_dev;
            accept.pos0 = pos0;
            accept.ratio = ratio;
            accept.chain = chain;
        }
        if (int rc = launch_inline(s, dtype, vocab, rows, m, in_order, accept)) {
            return rc;
        }
        if (accept.ctrl != nullptr) {
            return LILY_OK;   // the launch wrote the control block itself
        }
    }
    if (ctrl_dev != nullptr) {
        return lily_spec_accept(s, verify_tokens_dev, ids_dev, m, ctrl_dev, ctrl_words, pos0, ratio,
                                chain);
    }
    return LILY_OK;
}

// ---- batched rows

int lily_sample_rows(lily_sampler_t* s, const lily_rows* b) {
    if (s == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "sampler is null");
    }
    if (b != nullptr && b->rows != 0 && b->rows <= (uint32_t)INLINE_ROWS) {
        InlineRows rows;
        if (int rc = pack_batch(b, rows.r)) {
            return rc;
        }
        return launch_inline(s, (int)b->dtype, b->vocab, rows, b->rows);
    }
    if (b == nullptr || b->rows == 0) {
        return fail(LILY_ERR_INVALID_ARG, "empty batch");
    }
    ON_DEVICE(s->device);
    if (int rc = ensure_table(s, b->rows)) {
        return rc;
    }
    const uint32_t slot = s->stage_next;
    s->stage_next = (slot + 1) % STAGE_SLOTS;
    if (s->stage_used[slot]) {
        HIP_TRY(hipEventSynchronize(s->stage_done[slot]));
    }
    if (int rc = pack_batch(b, s->stage[slot])) {
        return rc;
    }
    LaunchPart parts[2];
    const uint32_t n_parts = plan_parts(s, s->stage[slot], b->rows, (int)b->dtype, b->vocab, parts);
    // A small kernel of the library's own carries the descriptors (224 bytes a row) from the
    // pinned memory they were packed in to the device, ahead of the row kernels in the same
    // stream.  (The copy engine's start-up costs about 100 us a call on this system; row kernels
    // that read the descriptors in place pay a trip across the bus for every field the compiler
    // chooses to load again, about 55 us on a launch of a thousand rows.)
    RowArgs* table_mapped = nullptr;
    HIP_TRY(hipHostGetDevicePointer(reinterpret_cast<void**>(&table_mapped), s->stage[slot], 0));
    HIP_TRY(launch_copy_pieces(s->stream, table_mapped, s->table_dev, (size_t)b->rows * sizeof(RowArgs)));
    HIP_TRY(hipEventRecord(s->stage_done[slot], s->stream));
    s->stage_used[slot] = true;
    for (uint32_t q = 0; q < n_parts; ++q) {
        if (int rc = launch_part(s, parts[q], s->table_dev, (int)b->dtype, b->vocab, 0, q == 0)) {
            return rc;
        }
    }
    return LILY_OK;
}

// ---- insertions (src/thinking.rs:485-608: Action::{Before, After, Replace})

struct lily_insertions {
    std::vector<std::vector<uint32_t>> pending;   // per row, next token first
    std::vector<size_t> head;                      // tokens of pending[row] already handed out
};

int lily_insertions_create(uint32_t rows, lily_insertions_t** out) {
    if (out == nullptr || rows == 0) {
        return fail(LILY_ERR_INVALID_ARG, "insertions need rows > 0");
    }
    *out = nullptr;
    lily_insertions* q = new (std::nothrow) lily_insertions;
    if (q == nullptr) {
        return fail(LILY_ERR_NOMEM, "out of host memory");
    }
    q->pending.resize(rows);
    q->head.assign(rows, 0);
    *out = q;
    return LILY_OK;
}

void lily_insertions_destroy(lily_insertions_t* q) { delete q; }

int lily_insertions_push(lily_insertions_t* q, uint32_t row, lily_insert_kind kind, uint32_t drawn,
                         const uint32_t* ids, uint32_t n, lily_scratch_t* scratch) {
    if (q == nullptr || row >= q->pending.size()) {
        return fail(LILY_ERR_INVALID_ARG, "row outside the insertions' rows");
    }
    if (n != 0 && ids == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "ids is null");
    }
    if (kind != LILY_INSERT_AFTER && kind != LILY_INSERT_BEFORE && kind != LILY_INSERT_REPLACE) {
        return fail(LILY_ERR_INVALID_ARG, "unknown kind of insertion");
    }
    for (uint32_t i = 0; i < n; ++i) {
        if (ids[i] == LILY_NO_TOKEN) {
            return fail(LILY_ERR_RANGE, "an inserted id cannot be LILY_NO_TOKEN");
        }
    }
    if (kind != LILY_INSERT_AFTER && scratch != nullptr) {
        // the draw counted `drawn`; BEFORE emits it again as a forced token (counted there),
        // REPLACE never emits it
        if (int rc = lily_scratch_uncount(scratch, drawn)) {
            return rc;
        }
    }
    std::vector<uint32_t>& p = q->pending[row];
    if (q->head[row] == p.size()) {
        p.clear();
        q->head[row] = 0;
    }
    p.insert(p.end(), ids, ids + n);
    if (kind == LILY_INSERT_BEFORE) {
        p.push_back(drawn);
    }
    return LILY_OK;
}

uint32_t lily_insertions_next(lily_insertions_t* q, uint32_t* forced_out) {
    if (q == nullptr || forced_out == nullptr) {
        return 0;
    }
    uint32_t forced = 0;
    for (size_t r = 0; r < q->pending.size(); ++r) {
        if (q->head[r] < q->pending[r].size()) {
            forced_out[r] = q->pending[r][q->head[r]++];
            ++forced;
        } else {
            forced_out[r] = LILY_NO_TOKEN;
        }
    }
    return forced;
}

uint32_t lily_insertions_pending(const lily_insertions_t* q, uint32_t row) {
    if (q == nullptr || row >= q->pending.size()) {
        return 0;
    }
    return (uint32_t)(q->pending[row].size() - q->head[row]);
}

void lily_insertions_clear(lily_insertions_t* q, uint32_t row) {
    if (q != nullptr && row < q->pending.size()) {
        q->pending[row].clear();
        q->head[row] = 0;
    }
}

// ---- the logits' producer and the draws from its summaries

namespace {

size_t round16(size_t n) { return (n + 15u) & ~(size_t)15u; }

// Takes the next staging buffer (waiting, if need be, for the call that used it four calls back).
int stage_acquire(lily_sampler* s, uint32_t rows, uint32_t* slot_out) {
    if (int rc = ensure_table(s, rows)) {
        return rc;
    }
    const uint32_t slot = s->stage_next;
    s->stage_next = (slot + 1) % STAGE_SLOTS;
    if (s->stage_used[slot]) {
        HIP_TRY(hipEventSynchronize(s->stage_done[slot]));
    }
    *slot_out = slot;
    return LILY_OK;
}

// Carries the first `bytes` of the staging buffer to the device (same offsets in table_dev).
int stage_commit(lily_sampler* s, uint32_t slot, size_t bytes) {
    void* mapped = nullptr;
    HIP_TRY(hipHostGetDevicePointer(&mapped, s->stage[slot], 0));
    HIP_TRY(launch_copy_pieces(s->stream, mapped, s->table_dev, round16(bytes)));
    HIP_TRY(hipEventRecord(s->stage_done[slot], s->stream));
    s->stage_used[slot] = true;
    return LILY_OK;
}

float c2_of_temperature(float t) {
    const float c = (float)(1.4426950408889634 / (double)t);
    return std::isfinite(c) ? c : 0.0f;
}

int check_head(const lily_lm_head* h, uint32_t rows, uint32_t vocab, const void* logits_dev,
               uint64_t row_stride) {
    if (h == nullptr || h->hidden_dev == nullptr || h->weight_dev == nullptr || h->tile_max_dev == nullptr ||
        h->tile_sum_dev == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "hidden, weight, tile_max and tile_sum are required");
    }
    if (rows == 0 || vocab == 0 || logits_dev == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "rows, vocab and the logits buffer are required");
    }
    if (h->d == 0 || h->d % 64u != 0) {
        return fail(LILY_ERR_INVALID_ARG, "d must be a positive multiple of 64");
    }
    if (h->hidden_stride < h->d || h->hidden_stride % 8u != 0 ||
        reinterpret_cast<uintptr_t>(h->hidden_dev) % 16u != 0 ||
        reinterpret_cast<uintptr_t>(h->weight_dev) % 16u != 0) {
        return fail(LILY_ERR_INVALID_ARG,
                    "hidden and weight rows must start at multiples of 16 bytes and hold d elements");
    }
    if (h->weight_bits == 0u) {
        if (h->weight_stride < h->d || h->weight_stride % 8u != 0) {
            return fail(LILY_ERR_INVALID_ARG,
                        "hidden and weight rows must start at multiples of 16 bytes and hold d elements");
        }
    } else {
        if (h->weight_bits != 4u && h->weight_bits != 8u) {
            return fail(LILY_ERR_INVALID_ARG, "weight_bits is 0 (bf16), 4 or 8");
        }
        const uint64_t words = (uint64_t)h->d * h->weight_bits / 32u;
        if (h->weight_stride < words || h->weight_stride % 4u != 0) {
            return fail(LILY_ERR_INVALID_ARG, "rows of codes hold d * bits / 32 words and start at multiples of 16 bytes");
        }
        const uint32_t gs = h->group_size;
        if (gs < 32u || (gs & (gs - 1u)) != 0u || h->d % gs != 0u) {
            return fail(LILY_ERR_INVALID_ARG, "group_size is a power of two from 32 on that divides d");
        }
        if (h->scales_dev == nullptr || h->biases_dev == nullptr) {
            return fail(LILY_ERR_INVALID_ARG, "codes come with scales and biases");
        }
        if (h->logits_f32 == 0u) {
            return fail(LILY_ERR_INVALID_ARG, "a head of codes produces f32 logits (logits_f32 = 1)");
        }
    }
    if (h->logits_f32 > 1u) {
        return fail(LILY_ERR_INVALID_ARG, "logits_f32 is 0 or 1");
    }
    if (row_stride < vocab) {
        return fail(LILY_ERR_INVALID_ARG, "row_stride is shorter than the vocabulary");
    }
    return LILY_OK;
}

struct HeadWeightsOf : HeadWeights {
    HeadWeightsOf(const lily_sampler* s, const lily_lm_head* h);
};
HeadWeightsOf::HeadWeightsOf(const lily_sampler* s, const lily_lm_head* h) {
    HeadWeights& w = *this;
    w.library_rows = h->weight_bits != 0u ? s->head_library_rows_codes : s->head_library_rows;
    w.library_calls = const_cast<unsigned long long*>(&s->head_library_calls);
    w.bits = h->weight_bits;
    w.scales = h->scales_dev;
    w.biases = h->biases_dev;
    uint32_t shift = 0;
    while (h->weight_bits != 0u && (1u << shift) < h->group_size) {
        ++shift;
    }
    w.group_shift = shift;
}

// Rows the summaries serve: penalties only of the lowering kind, the row given as it is, and a
// greedy row or a plain draw among at most STREAM_K_MAX candidates; a bias list of up to
// STREAM_BIAS_CAP pairs or an allow-mask on a row that draws and is not forced (a summary says
// nothing about the largest biased or the largest allowed value, which a greedy or a forced
// row's answer hangs on).  Rows under penalties or a mask may be declined on the device.
bool tiles_serve(const RowArgs& r) {
    if (r.sel_row != nullptr || r.n_bias > STREAM_BIAS_CAP) {
        return false;
    }
    if ((r.n_bias != 0 || r.allow != nullptr) && (r.mode == MODE_ARGMAX || (r.flags & F_FORCED))) {
        return false;
    }
    if (r.mode == MODE_ARGMAX) {
        return true;   // (a greedy row ignores penalties: sample.rs:382-385)
    }
    if (r.flags & F_PEN) {
        // summaries describe raw values: they bound true ones only where penalties lower
        const bool lowering = r.repetition >= 1.0f && r.presence >= 0.0f && r.frequency >= 0.0f;
        if (!lowering || (r.flags & F_FORCED)) {
            return false;
        }
    }
    return r.mode == MODE_PLAIN && r.k <= STREAM_K_MAX;
}

// The draws of batch `b` with the summaries of its logits at hand; with `h` set, the logits and
// the summaries are produced first, in the same stream.
int rows_with_tiles(lily_sampler* s, const lily_lm_head* h, const lily_rows* b, const float* tile_max,
                    const float* tile_sum) {
    if (b == nullptr || b->rows == 0) {
        return fail(LILY_ERR_INVALID_ARG, "empty batch");
    }
    if (b->dtype != LILY_BF16 && b->dtype != LILY_F32) {
        return fail(LILY_ERR_INVALID_ARG, "logits are bf16 or f32");
    }
    if (h != nullptr && (h->logits_f32 != 0u) != (b->dtype == LILY_F32)) {
        return fail(LILY_ERR_INVALID_ARG, "the head's logits_f32 and the batch's dtype disagree");
    }
    if (tile_max == nullptr || tile_sum == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "tile_max and tile_sum are required");
    }
    if (reinterpret_cast<uintptr_t>(b->logits_dev) % 16u != 0 ||
        (b->rows > 1 && b->row_stride % (b->dtype == LILY_BF16 ? 8u : 4u) != 0)) {
        return fail(LILY_ERR_INVALID_ARG, "rows of logits must start at multiples of 16 bytes");
    }
    const uint32_t rows = b->rows, tiles = lily_lm_head_tiles(b->vocab);
    if (tiles > 2048u) {
        return fail(LILY_ERR_INVALID_ARG, "vocabulary beyond 2048 summaries a row");
    }
    if (h != nullptr) {
        if (int rc = check_head(h, rows, b->vocab, b->logits_dev, b->row_stride)) {
            return rc;
        }
    }
    ON_DEVICE(s->device);
    uint32_t slot = 0;
    if (int rc = stage_acquire(s, rows, &slot)) {
        return rc;
    }
    static thread_local std::vector<RowArgs> packed;
    packed.resize(rows);
    if (int rc = pack_batch(b, packed.data())) {
        return rc;
    }
    // staged: the descriptors - rows the summaries serve for certain, then rows under penalties
    // (served from the summaries unless the kernel declines them: the launch of the remaining
    // rows covers them too and skips those already drawn), then the others -, each row's row of
    // the summaries, every row's exponent scale (the producer's), a word per row that says
    // whether the row has been drawn
    char* stage = reinterpret_cast<char*>(s->stage[slot]);
    RowArgs* table = reinterpret_cast<RowArgs*>(stage);
    const size_t idx_off = (size_t)rows * sizeof(RowArgs), c2_off = idx_off + round16((size_t)rows * 4);
    const size_t served_off = c2_off + round16((size_t)rows * 4);
    uint32_t* tile_row = reinterpret_cast<uint32_t*>(stage + idx_off);
    float* c2 = reinterpret_cast<float*>(stage + c2_off);
    uint32_t* served_flags = reinterpret_cast<uint32_t*>(stage + served_off);
    uint32_t certain = 0, maybe = 0;
    bool lse = false, extra = false;
    uint32_t at = 0;
    // Summaries this sampler's lily_lm_head_bf16 produced at another temperature than the row's
    // (or at none) would give the row a wrong log-probability with the right token: such a row
    // is drawn from its logits instead.  (Summaries of any other origin are taken on trust.)
    auto sum_at_other_scale = [&](uint32_t r) -> bool {
        if (h != nullptr || tile_sum != s->head_sum || packed[r].out_logprob == nullptr) {
            return false;
        }
        const float mine = std::isfinite(packed[r].c2) ? packed[r].c2 : 0.0f;
        return r >= s->head_c2.size() || s->head_c2[r] != mine;
    };
    for (int group = 0; group < 3; ++group) {
        for (uint32_t r = 0; r < rows; ++r) {
            const RowArgs& row = packed[r];
            const bool serve = tiles_serve(row) && !sum_at_other_scale(r);
            const bool pen = serve && row.mode != MODE_ARGMAX && ((row.flags & F_PEN) != 0 || row.allow != nullptr);
            const int g = !serve ? 2 : (pen ? 1 : 0);
            if (g != group) {
                continue;
            }
            if (serve) {
                lse = lse || row.out_logprob != nullptr;
                extra = extra || row.n_bias != 0 || row.allow != nullptr;
                tile_row[at] = r;
                certain += group == 0 ? 1u : 0u;
                maybe += group == 1 ? 1u : 0u;
            }
            served_flags[at] = 0u;
            table[at++] = row;
        }
    }
    for (uint32_t r = 0; r < rows; ++r) {
        c2[r] = std::isfinite(packed[r].c2) ? packed[r].c2 : 0.0f;
    }
    if (h != nullptr) {
        s->head_sum = h->tile_sum_dev;
        s->head_c2.assign(c2, c2 + rows);
    }
    const uint32_t served = certain + maybe;
    LaunchPart parts[2];
    const uint32_t n_parts =
        certain < rows ? plan_parts(s, table + certain, rows - certain, (int)b->dtype, b->vocab, parts) : 0u;
    if (int rc = stage_commit(s, slot, served_off + (size_t)rows * 4)) {
        return rc;
    }
    const char* dev = reinterpret_cast<const char*>(s->table_dev);
    if (h != nullptr) {
        HIP_TRY(launch_lm_head_bf16(s->stream, h->hidden_dev, h->hidden_stride, h->weight_dev,
                                    h->weight_stride, rows, h->d, b->vocab,
                                    reinterpret_cast<const float*>(dev + c2_off),
                                    const_cast<void*>(b->logits_dev), b->row_stride, h->tile_max_dev,
                                    h->tile_sum_dev, h->logits_f32 != 0u, HeadWeightsOf(s, h)));
    }
    uint32_t* served_dev = reinterpret_cast<uint32_t*>(const_cast<char*>(dev) + served_off);
    if (served != 0) {
        LaunchCfg cfg;
        fill_cfg(s, &cfg, served, b->vocab, 1, 1, 0, s->table_dev);
        attach_trace(s, &cfg, served);
        HIP_TRY(launch_rows_tiles(s->stream, (int)b->dtype, lse, extra, served, cfg, tile_max, tile_sum, tiles,
                                  reinterpret_cast<const uint32_t*>(dev + idx_off), served_dev));
    }
    for (uint32_t q = 0; q < n_parts; ++q) {
        if (int rc = launch_part(s, parts[q], s->table_dev + certain, (int)b->dtype, b->vocab, 0, false,
                                 maybe != 0 ? served_dev + certain : nullptr)) {
            return rc;
        }
    }
    return LILY_OK;
}

}  // namespace

static_assert(LILY_TILE_COLS == LILY_LOGIT_TILE_COLS, "the kernels' tile is the header's");

uint32_t lily_lm_head_tiles(uint32_t vocab) {
    return (vocab + LILY_LOGIT_TILE_COLS - 1u) / LILY_LOGIT_TILE_COLS;
}

uint64_t lily_lm_head_library_calls(const lily_sampler_t* s) {
    return s != nullptr ? s->head_library_calls : 0u;
}

int lily_lm_head_bf16(lily_sampler_t* s, const lily_lm_head* h, uint32_t rows, uint32_t vocab,
                      const float* temperatures, void* logits_dev, uint64_t row_stride) {
    if (s == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "sampler is null");
    }
    if (int rc = check_head(h, rows, vocab, logits_dev, row_stride)) {
        return rc;
    }
    ON_DEVICE(s->device);
    uint32_t slot = 0;
    if (int rc = stage_acquire(s, rows, &slot)) {
        return rc;
    }
    float* c2 = reinterpret_cast<float*>(s->stage[slot]);
    s->head_sum = h->tile_sum_dev;
    s->head_c2.resize(rows);
    for (uint32_t r = 0; r < rows; ++r) {
        c2[r] = temperatures != nullptr ? c2_of_temperature(temperatures[r]) : 0.0f;
        s->head_c2[r] = c2[r];
    }
    if (int rc = stage_commit(s, slot, (size_t)rows * 4)) {
        return rc;
    }
    HeadWeightsOf hw(s, h);
    hw.trace = reinterpret_cast<unsigned long long*>(s->phase_trace);
    hw.trace_words = s->phase_words;
    HIP_TRY(launch_lm_head_bf16(s->stream, h->hidden_dev, h->hidden_stride, h->weight_dev, h->weight_stride,
                                rows, h->d, vocab, reinterpret_cast<const float*>(s->table_dev), logits_dev,
                                row_stride, h->tile_max_dev, h->tile_sum_dev, h->logits_f32 != 0u, hw));
    return LILY_OK;
}

int lily_sample_rows_tiled(lily_sampler_t* s, const lily_rows* b, const float* tile_max_dev,
                           const float* tile_sum_dev) {
    if (s == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "sampler is null");
    }
    return rows_with_tiles(s, nullptr, b, tile_max_dev, tile_sum_dev);
}

int lily_lm_head_sample_rows(lily_sampler_t* s, const lily_lm_head* h, const lily_rows* b) {
    if (s == nullptr || h == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "sampler and head are required");
    }
    return rows_with_tiles(s, h, b, h->tile_max_dev, h->tile_sum_dev);
}

int lily_plan_create(lily_sampler_t* s, uint32_t max_rows, lily_plan_t** out) {
    if (s == nullptr || out == nullptr || max_rows == 0) {
        return fail(LILY_ERR_INVALID_ARG, "plan needs a sampler and max_rows > 0");
    }
    *out = nullptr;
    ON_DEVICE(s->device);
    lily_plan* p = new (std::nothrow) lily_plan;
    if (p == nullptr) {
        return fail(LILY_ERR_NOMEM, "out of host memory");
    }
    p->s = s;
    p->max_rows = max_rows;
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&p->table_dev),
                             (size_t)max_rows * sizeof(RowArgs));
    if (e != hipSuccess) {
        delete p;
        return hip_fail(e, "plan allocation");
    }
    *out = p;
    return LILY_OK;
}

void lily_plan_destroy(lily_plan_t* p) {
    if (p == nullptr) {
        return;
    }
    DeviceScope device_scope_(p->s->device);
    (void)hipStreamSynchronize(p->s->stream);
    (void)hipFree(p->table_dev);
    delete p;
}

int lily_plan_set(lily_plan_t* p, const lily_rows* b) {
    if (p == nullptr) {
        return fail(LILY_ERR_INVALID_ARG, "plan is null");
    }
    if (b == nullptr || b->rows == 0 || b->rows > p->max_rows) {
        return fail(LILY_ERR_RANGE, "batch rows outside 1..%u", p->max_rows);
    }
    std::vector<RowArgs> table(b->rows);
    if (int rc = pack_batch(b, table.data())) {
        return rc;
    }
    p->n_parts = plan_parts(p->s, table.data(), b->rows, (int)b->dtype, b->vocab, p->parts);
    ON_DEVICE(p->s->device);
    HIP_TRY(hipStreamSynchronize(p->s->stream));
    HIP_TRY(hipMemcpy(p->table_dev, table.data(), (size_t)b->rows * sizeof(RowArgs),
                      hipMemcpyHostToDevice));
    p->rows = b->rows;
    p->vocab = b->vocab;
    p->dtype = b->dtype;
    p->runs = 0;
    return LILY_OK;
}

int lily_plan_run(lily_plan_t* p, uint32_t step_delta) {
    if (p == nullptr || p->rows == 0) {
        return fail(LILY_ERR_INVALID_ARG, "plan is null or not set");
    }
    ON_DEVICE(p->s->device);
    for (uint32_t q = 0; q < p->n_parts; ++q) {
        if (int rc = launch_part(p->s, p->parts[q], p->table_dev, (int)p->dtype, p->vocab, step_delta,
                                 q == 0)) {
            return rc;
        }
    }
    p->runs += 1;
    return LILY_OK;
}

}  // extern "C"
