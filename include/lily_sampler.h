/*
 * lily_sampler.h - C ABI of the MI355X logits-to-token stage (liblily_sampler_hip.so).
 *
 * Every entry point states the reference interface it stands in for (paths relative
 * to the reference checkout).  The reference encodes work into a Metal pass and runs
 * it at commit; here every draw is ENQUEUED on the HIP stream the sampler was created
 * on and returns at once.  Results appear in the device buffers in stream order; the
 * caller synchronises the stream (or calls lily_sampler_synchronize) before reading.
 * Nothing here allocates on the draw calls, reads device memory on the host, or
 * synchronises, except where a function says so.
 *
 * Pointers named *_dev are device pointers borrowed for the duration of the enqueued
 * work (the reference's "a pass holds buffers by address only").  A sampler and the
 * objects made from it belong to one host thread at a time.
 *
 * Return value: 0 on success, a negative lily_status otherwise; lily_last_error()
 * returns the message of the calling thread's last failure.
 */
#ifndef LILY_SAMPLER_H
#define LILY_SAMPLER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LILY_SAMPLE_K_CAP 1024u          /* src/kernels/sample.rs:17 SAMPLE_K_CAP */
#define LILY_CTRL_STRIDE 4u              /* src/kernels/spec.rs:15 CTRL_STRIDE */
#define LILY_SLOT_ACCEPTED 0u            /* src/kernels/spec.rs:18 */
#define LILY_SLOT_KEEP 1u                /* src/kernels/spec.rs:20 */
#define LILY_NO_TOKEN 0xFFFFFFFFu        /* "no forced token" in lily_rows.forced */
#define LILY_MAX_VERIFY_ROWS 8u

typedef enum lily_status {
    LILY_OK = 0,
    LILY_ERR_INVALID_ARG = -1, /* null/misaligned pointer, zero size, bad enum */
    LILY_ERR_PARAMS = -2,      /* SamplingParams::validate failed (sample.rs:57-79) */
    LILY_ERR_VOCAB = -3,       /* scratch sized for a different vocabulary (sample.rs:264) */
    LILY_ERR_HIP = -4,         /* a HIP runtime call failed; message holds hipGetErrorString */
    LILY_ERR_NOMEM = -5,
    LILY_ERR_RANGE = -6        /* index or size beyond a stated limit */
} lily_status;

typedef enum lily_dtype { LILY_F32 = 0, LILY_BF16 = 1 } lily_dtype;

/* src/kernels/sample.rs:21-31 SamplingParams, field for field (top_k as u32). */
typedef struct lily_sampling_params {
    float temperature;        /* 0 = greedy */
    uint32_t top_k;           /* 0 = off (capped at LILY_SAMPLE_K_CAP) */
    float top_p;
    float min_p;
    float presence_penalty;
    float frequency_penalty;
    float repetition_penalty;
    uint32_t reserved;        /* must be 0 */
    uint64_t seed;
} lily_sampling_params;

typedef struct lily_bias {
    uint32_t id;
    float delta;
} lily_bias;

typedef struct lily_sampler lily_sampler_t;         /* MetalContext + ComputePass of the path */
typedef struct lily_scratch lily_scratch_t;         /* src/kernels/sample.rs:116-128 SamplerScratch */
typedef struct lily_draft_dists lily_draft_dists_t; /* src/kernels/sample.rs:186-190 DraftDists */

/* src/kernels/sample.rs:193-197 DraftDist: one slot's device arrays. */
typedef struct lily_draft_dist {
    uint32_t* ids_dev;   /* [LILY_SAMPLE_K_CAP] kept ids, best first */
    float* probs_dev;    /* [LILY_SAMPLE_K_CAP] probabilities over the kept mass */
    uint32_t* count_dev; /* [1] kept count */
} lily_draft_dist;

const char* lily_last_error(void);

/* ---- pure host helpers (no GPU) ---------------------------------------------------- */

/* src/kernels/sample.rs:34-45 SamplingParams::greedy() */
void lily_params_greedy(lily_sampling_params* out);
/* src/kernels/sample.rs:47-49 is_greedy */
int lily_params_is_greedy(const lily_sampling_params* p);
/* src/kernels/sample.rs:51-55 uses_penalties */
int lily_params_uses_penalties(const lily_sampling_params* p);
/* src/kernels/sample.rs:57-79 validate: LILY_OK or LILY_ERR_PARAMS with the rule's message */
int lily_params_validate(const lily_sampling_params* p);
/* src/kernels/sample.rs:83-94 effective: the temperature and candidate count the kernel uses */
void lily_params_effective(const lily_sampling_params* p, float* temperature, uint32_t* top_k);
/* A request's sampling fields over the server's defaults (resolve_sampling,
 * src/serve/api.rs:798-834; the fields are SamplingFields, :440-456): a field is taken when its
 * bit of `has` is set, else the default's; top_k < 0 means 0 (off); a request without a seed gets
 * `fresh_seed` (the reference draws it from the clock and the process id: the caller supplies
 * its own entropy here, which keeps the function pure).  The result is validated:
 * LILY_OK or LILY_ERR_PARAMS with the rule's message, `out` written either way. */
enum {
    LILY_HAS_TEMPERATURE = 1, LILY_HAS_TOP_P = 2, LILY_HAS_TOP_K = 4, LILY_HAS_MIN_P = 8,
    LILY_HAS_SEED = 16, LILY_HAS_PRESENCE = 32, LILY_HAS_FREQUENCY = 64, LILY_HAS_REPETITION = 128
};
typedef struct lily_sampling_fields {
    uint32_t has;             /* LILY_HAS_* bits */
    float temperature;
    float top_p;
    float min_p;
    int64_t top_k;
    int64_t seed;             /* taken as u64, as the reference's `s as u64` */
    float presence_penalty;
    float frequency_penalty;
    float repetition_penalty;
    uint32_t reserved;        /* must be 0 */
} lily_sampling_fields;
int lily_params_resolve(const lily_sampling_fields* fields, const lily_sampling_params* defaults,
                        uint64_t fresh_seed, lily_sampling_params* out);
/* src/kernels/sample.rs:227-234 draft_params */
void lily_draft_params(const lily_sampling_params* p, lily_sampling_params* out);
/* src/kernels/sample.rs:220-222 draft_step */
uint32_t lily_draft_step(uint32_t step);
/* src/kernels/sample.rs:435-441 uniform_for */
float lily_uniform_for(uint64_t seed, uint32_t step);
/* src/kernels/spec.rs:23-40 slot_pos / slot_block / slot_count / ctrl_words */
uint32_t lily_slot_pos(uint32_t i);
uint32_t lily_slot_block(uint32_t i);
uint32_t lily_slot_count(uint32_t i);
uint32_t lily_ctrl_words(uint32_t chain);

/* ---- sampler (context) --------------------------------------------------------------- */

/* MetalContext::new + ctx.begin (src/metal.rs:400, :618): binds `device` and an existing
 * hipStream_t (`hip_stream`; NULL = the device's default stream).  Allocates the
 * workspace the multi-workgroup rows use.  Fails loudly if no HIP device is present. */
int lily_sampler_create(int device, void* hip_stream, lily_sampler_t** out);
void lily_sampler_destroy(lily_sampler_t* s);
/* ComputePass::commit_wait (src/metal.rs:2290): blocks until the stream has drained. */
int lily_sampler_synchronize(lily_sampler_t* s);

/* Per-kernel profile transport of the reference (LILY_KERNEL_PROFILE, src/metal.rs:30-33,
 * :140-198) at a finer grain: while trace_dev is set, thread 0 of every workgroup of the row
 * kernels stores the 100 MHz device wall clock at up to 16 phase boundaries into
 * trace_dev[(row * slices + slice) * 16 + phase] (u64; 0 start, 1 scan about to start, 2 scan
 * done, 3 sums merged, 4 slice top-k done, 5 ticket taken, 6 slices merged, 7 row
 * done; 8-15 finer marks: 8 queue expanded, 9 edge ids done, 10-11 sum merge, 12 candidates
 * ranked, 13-15 inside phase 1).  capacity_words bounds rows * slices * 16; larger launches run
 * untraced.  NULL stops. */
int lily_sampler_set_phase_trace(lily_sampler_t* s, uint64_t* trace_dev, uint64_t capacity_words);
/* Diagnostics with no counterpart in the reference: while stats_dev (device, u32[4], cleared by
 * the caller) is set, every workgroup of a sampled row adds 1 to [0] when the streaming select
 * (k <= 64) produced its slice, [1] for the selects of sparsely masked rows and of k > 64
 * (sparse or bitmap), [2] for the exhaustive select; [3] collects a bit per reason the streaming
 * select gave a slice up.  A row of k > 64 that the two launches for rows of many candidates
 * draw (plain rows without mask or bias list, penalties none or lowering) adds 1 to [1], or to
 * [2], once, whatever the number of its workgroups.  NULL stops. */
int lily_sampler_set_path_stats(lily_sampler_t* s, uint32_t* stats_dev);
/* Measurement aid with no counterpart in the reference: one launch that only reads `rows` rows of
 * row_bytes bytes (stride_bytes apart) with the row kernel's shape - a workgroup of 256 threads a
 * row, 16-byte loads, three blocks requested ahead - and writes each row's largest 32-bit word
 * (as an unsigned integer, combined with atomicMax) to out_dev[rows].  Its rate is the ceiling a
 * row-per-workgroup launch of that size can reach on the device.  base_dev 16-byte aligned,
 * row_bytes and stride_bytes multiples of 16. */
int lily_probe_read(lily_sampler_t* s, const void* base_dev, uint32_t rows, uint64_t row_bytes,
                    uint64_t stride_bytes, uint32_t* out_dev);
/* Workgroups per row the next launch of `rows` rows with candidate count k would use. */
uint32_t lily_sampler_slices_for(const lily_sampler_t* s, uint32_t rows, uint32_t k, uint32_t vocab,
                                 lily_dtype dtype);

/* ---- SamplerScratch ------------------------------------------------------------------- */

/* SamplerScratch::new (sample.rs:131-143).  Device state: the emission histogram
 * counts[vocab] and a vocab-bit map of the ids whose count is non-zero. */
int lily_scratch_create(lily_sampler_t* s, uint32_t vocab, lily_scratch_t** out);
void lily_scratch_destroy(lily_scratch_t* sc);
/* SamplerScratch::vocab (sample.rs:176-178) */
uint32_t lily_scratch_vocab(const lily_scratch_t* sc);
/* SamplerScratch::reset_counts (sample.rs:161-163); stream-ordered. */
int lily_scratch_reset_counts(lily_scratch_t* sc);
/* SamplerScratch::uncount (sample.rs:147-157): saturating, out-of-range ignored; stream-ordered. */
int lily_scratch_uncount(lily_scratch_t* sc, uint32_t token);
/* The rollback of a verify step's rejected draws (finish_speculation,
 * src/qwen4exp/spec.rs:213-217: `for token in sampled[accepted + 1..] { uncount(token) }`)
 * without the host reading the accepted row: a = min(accepted_dev[0], accepted_cap) and
 * draws_dev[a + 1 .. m) are un-counted in order.  accepted_dev is typically the control
 * block's LILY_SLOT_ACCEPTED word; accepted_cap is where the engine stopped earlier (a stop
 * token among the accepted rows), UINT32_MAX when it did not.  Stream-ordered. */
int lily_scratch_uncount_after(lily_scratch_t* sc, const uint32_t* draws_dev, uint32_t m,
                               const uint32_t* accepted_dev, uint32_t accepted_cap);
/* SamplerScratch::copy_counts_from (sample.rs:168-174): LILY_ERR_VOCAB on a size mismatch. */
int lily_scratch_copy_counts_from(lily_scratch_t* dst, const lily_scratch_t* src);
/* move_sampler_counts (src/qwen4exp/batch.rs:138-162, engine slot <-> batch slot): `to` takes
 * `from`'s counts in stream order; from == to does nothing. */
int lily_scratch_move_counts(lily_scratch_t* from, lily_scratch_t* to);
/* No counterpart in the reference (its histogram only ever grows by the kernel's own
 * draws): counts[id] += multiplicity of id in ids_dev[0..n); ids >= vocab are ignored. */
int lily_scratch_add_history(lily_scratch_t* sc, const uint32_t* ids_dev, uint32_t n);
/* scratch.counts.write_bytes / to_u32 as the reference's tests use them
 * (tests/unit/kernels/sample.rs:66,166): host <-> device copies; both synchronise. */
int lily_scratch_write_counts(lily_scratch_t* sc, const uint32_t* host_counts);
int lily_scratch_read_counts(lily_scratch_t* sc, uint32_t* host_counts);

/* ---- DraftDists ----------------------------------------------------------------------- */

/* DraftDists::new (sample.rs:200-206) / slot (sample.rs:208-214) */
int lily_draft_dists_create(lily_sampler_t* s, uint32_t slots, lily_draft_dists_t** out);
void lily_draft_dists_destroy(lily_draft_dists_t* d);
int lily_draft_dists_slot(const lily_draft_dists_t* d, uint32_t i, lily_draft_dist* out);

/* ---- the decode loop's output slots ------------------------------------------------------ */

/* The ping-pong `next_token` slots of the decode loop and its polled completion
 * (src/generate.rs:776-891: a step reads slot_in and writes the other slot, the following step is
 * encoded while this one runs, `wait_polled` + `read_slot`).  `slots` device arrays of `words`
 * u32 each (one word per row of a batched step) with a pinned host mirror and an event per slot.
 * A draw is given lily_token_slots_device(t, i) as its out_dev / out_ids_dev; the next step's
 * kernels read the same address.  lily_token_slots_publish enqueues, behind the work already on
 * the sampler's stream, the slot's copy to the mirror and an event; lily_token_slots_poll
 * never blocks: ready = 1 and the slot's words in host_out once that event has passed.
 * lily_token_slots_wait_polled polls until then (max_polls = 0: without limit; else
 * LILY_ERR_RANGE after that many polls) - the host thread spins instead of sleeping in the
 * driver, which is what wakes it within microseconds of the step's end.  A slot must be read
 * (ready = 1) before it is published again. */
typedef struct lily_token_slots lily_token_slots_t;
int lily_token_slots_create(lily_sampler_t* s, uint32_t slots, uint32_t words, lily_token_slots_t** out);
void lily_token_slots_destroy(lily_token_slots_t* t);
uint32_t* lily_token_slots_device(const lily_token_slots_t* t, uint32_t slot);
int lily_token_slots_publish(lily_token_slots_t* t, uint32_t slot);
int lily_token_slots_poll(lily_token_slots_t* t, uint32_t slot, uint32_t* host_out, int* ready);
int lily_token_slots_wait_polled(lily_token_slots_t* t, uint32_t slot, uint32_t* host_out,
                                 uint64_t max_polls);

/* ---- single-row draws (the reference's call signature) --------------------------------- */

/* Logits are read in whole 16-byte aligned blocks: up to 15 bytes before a row's first and
 * after its last element are read and discarded (never beyond the aligned blocks the row
 * itself occupies).
 *
 * NaN logits (the reference states no rule: its kernels compare with <, which a NaN never wins;
 * its CPU twin sorts with total_cmp) are worth -inf in every draw: never a candidate, no term of
 * the row sum behind a log-probability.  A row that holds one forms that sum by a slower path.
 *
 * sample_f32 (sample.rs:373-387): one draw from logits_dev[vocab] into out_dev[0].
 * Greedy without penalties is the exact first-max argmax; otherwise penalties,
 * temperature, top-k, top-p/min-p and the inverse-CDF draw on uniform_for(seed, step).
 * Under penalties counts[out] += 1.  `scratch` may be NULL when params use no penalties. */
int lily_sample_f32(lily_sampler_t* s, const float* logits_dev, uint32_t vocab,
                    lily_scratch_t* scratch, const lily_sampling_params* params, uint32_t step,
                    uint32_t* out_dev);
/* sample_draft_f32 (sample.rs:394-408): as lily_sample_f32, and the kept distribution
 * goes to `dist`.  Greedy exports nothing. */
int lily_sample_draft_f32(lily_sampler_t* s, const float* logits_dev, uint32_t vocab,
                          lily_scratch_t* scratch, const lily_sampling_params* params,
                          uint32_t step, uint32_t* out_dev, const lily_draft_dist* dist);
/* sample_spec_f32 (sample.rs:417-432): speculative draw against `dist` and the proposal
 * draft_dev[0]; greedy is the plain argmax. */
int lily_sample_spec_f32(lily_sampler_t* s, const float* logits_dev, uint32_t vocab,
                         lily_scratch_t* scratch, const lily_sampling_params* params,
                         uint32_t step, const lily_draft_dist* dist, const uint32_t* draft_dev,
                         uint32_t* out_dev);
/* As lily_sample_spec_f32 with the two draws given instead of seeded: u1 stands in for
 * uniform_for(seed, step) (the accept test and, for a greedy-free plain row, the draw) and u2
 * for the residual draw's uniform_for(seed, step | 0x80000000) (sample.metal:626-651; the host
 * twin uniform_for exists "for tests and replay", sample.rs:434-441).  Both in [0, 1). */
int lily_sample_spec_f32_uniforms(lily_sampler_t* s, const float* logits_dev, uint32_t vocab,
                                  lily_scratch_t* scratch, const lily_sampling_params* params,
                                  uint32_t step, const lily_draft_dist* dist,
                                  const uint32_t* draft_dev, uint32_t* out_dev, float u1, float u2);
/* No counterpart in the reference.  lily_sample_f32 for callers that cannot allocate device
 * memory or own a sampler object: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  The draw is enqueued on `hip_stream` of the CURRENT device; the memory
 * a row spread over several workgroups needs (slices' candidates, partial sums, the arrival
 * ticket: 34 048 bytes) lives in a device array inside the library, one copy per GPU, kept
 * until the process ends.  The call allocates and frees nothing and does not synchronise.
 * Same results as lily_sample_f32.  Limits: one row of at most LILY_STATIC_MAX_VOCAB logits
 * (LILY_ERR_RANGE beyond); every call on a GPU shares that GPU's array, so two calls that may
 * overlap on one GPU (different streams, or graphs replayed concurrently) race - order them.
 * The first call on a device looks the array's address up (hipGetSymbolAddress, which may load
 * the library's code object): make one call outside any stream capture on each device before
 * capturing calls into a graph. */
#define LILY_STATIC_MAX_VOCAB 1048576u
int lily_sample_f32_static(void* hip_stream, const float* logits_dev, uint32_t vocab,
                           lily_scratch_t* scratch, const lily_sampling_params* params,
                           uint32_t step, uint32_t* out_dev);
/* Draws whose row and step a kernel before them chose - the device-side chaining of
 * src/qwen4exp/spec.rs:398-528, where the draft pass that follows a verify pass is encoded
 * before the host knows how many rows were accepted and its dispatches read the control block's
 * words as arguments (Arg::Gpu / Pos::gpu).  logits_dev is [rows][row_stride]; the draw reads row
 * min(row_dev[0], rows - 1) at step step_base + step_dev[0].  row_dev / step_dev are device
 * words written earlier on the stream (typically ctrl + LILY_SLOT_ACCEPTED * LILY_CTRL_STRIDE);
 * either may be NULL (row 0 / step_base).  Otherwise as lily_sample_f32 / lily_sample_draft_f32.
 * With lily_spec_verify, lily_scratch_uncount_after and lily_copy_row_u32 this lets
 * verify -> accept -> rollback -> the next draws be enqueued without a host read between. */
int lily_sample_f32_at(lily_sampler_t* s, const float* logits_dev, uint32_t vocab, uint64_t row_stride,
                       uint32_t rows, const uint32_t* row_dev, lily_scratch_t* scratch,
                       const lily_sampling_params* params, uint32_t step_base,
                       const uint32_t* step_dev, uint32_t* out_dev);
int lily_sample_draft_f32_at(lily_sampler_t* s, const float* logits_dev, uint32_t vocab,
                             uint64_t row_stride, uint32_t rows, const uint32_t* row_dev,
                             lily_scratch_t* scratch, const lily_sampling_params* params,
                             uint32_t step_base, const uint32_t* step_dev, uint32_t* out_dev,
                             const lily_draft_dist* dist);
/* argmax_f32 (src/kernels/elementwise.rs:297-308): first max, lowest index on ties.  The
 * reference's `partials` tensor (ARGMAX_GROUPS * 8 bytes of caller scratch between its two
 * dispatches) has no counterpart: the partial maxima of a row spread over several workgroups
 * live in the sampler's own workspace, and the call is one launch. */
int lily_argmax_f32(lily_sampler_t* s, const float* x_dev, uint32_t n, uint32_t* out_dev);

/* ---- speculative control --------------------------------------------------------------- */

/* spec_accept (src/kernels/spec.rs:52-91): a = leading draws[a] == ids[a+1]; writes the
 * control block (slots LILY_CTRL_STRIDE words apart). */
int lily_spec_accept(lily_sampler_t* s, const uint32_t* draws_dev, const uint32_t* ids_dev,
                     uint32_t m, uint32_t* ctrl_dev, uint32_t ctrl_words, uint32_t pos0,
                     uint32_t ratio, uint32_t chain);
/* copy_row (src/kernels/spec.rs:96-127) with a GPU-supplied row index: dst[0..words) =
 * src[row_dev[0]][0..words); copies nothing when the index is >= rows. */
int lily_copy_row_u32(lily_sampler_t* s, const uint32_t* src_dev, uint32_t rows, uint32_t words,
                      const uint32_t* row_dev, uint32_t* dst_dev);
/* The verify pass's draws (src/qwen4exp/model.rs:3008-3040) followed by spec_accept
 * (src/qwen4exp/spec.rs:414-424): rows j < m-1 are speculative draws against dists slot j
 * and proposal ids_dev[j+1] at step0+j, the last row a plain draw; row j sees the counts
 * of rows before it (one launch per row under penalties, one launch for all rows without).
 * verify_tokens_dev[m] receives the draws, ctrl_dev the control block (NULL: no spec_accept).
 * uniforms: NULL, or host [m][2] = (u1, u2) per row replacing the seeded draws (the last
 * row, a plain draw, uses its u1 only).  Every argument is validated before the first row is
 * enqueued, so an error return leaves the counts untouched. */
int lily_spec_verify(lily_sampler_t* s, const void* logits_dev, lily_dtype dtype, uint32_t vocab,
                     uint64_t row_stride, uint32_t m, lily_scratch_t* scratch,
                     const lily_sampling_params* params, uint32_t step0,
                     const lily_draft_dists_t* dists, const uint32_t* ids_dev,
                     uint32_t* verify_tokens_dev, uint32_t* ctrl_dev, uint32_t ctrl_words,
                     uint32_t pos0, uint32_t ratio, uint32_t chain, const float* uniforms);

/* ---- batched rows ---------------------------------------------------------------------- */

/* The per-row draw loop of a batched step (src/qwen4exp/batch.rs:583-593) as ONE launch:
 * row r draws from logits + r*row_stride with params[r], steps[r] and scratch[r].
 * Host arrays are read during the call; device arrays are borrowed until the work ran.
 * Beyond the reference: bf16 logits, a per-row allow-bitmask, a per-row logit-bias list,
 * a forced token, an explicit uniform and the chosen token's log-probability. */
typedef struct lily_rows {
    uint32_t rows;
    uint32_t vocab;
    uint32_t dtype;                      /* lily_dtype */
    uint32_t reserved;                   /* must be 0 */
    const void* logits_dev;              /* [rows][row_stride] */
    uint64_t row_stride;                 /* elements between rows */
    const lily_sampling_params* params;  /* host [rows] */
    const uint32_t* steps;               /* host [rows] */
    lily_scratch_t* const* scratch;      /* host [rows] or NULL; entries may be NULL.  A row
                                            touches its scratch only when its params use
                                            penalties: a scratch may stand in several rows of one
                                            call as long as at most one of them does */
    const uint32_t* allow_dev;           /* packed bits, bit id&31 of word id>>5, or NULL */
    uint64_t allow_stride;               /* words between rows; 0 = one mask for all rows */
    const lily_bias* bias_dev;           /* concatenated per-row lists or NULL */
    const uint32_t* bias_offsets;        /* host [rows+1] into bias_dev */
    const uint32_t* forced;              /* host [rows] or NULL; LILY_NO_TOKEN = draw */
    const float* uniforms;               /* host [rows] or NULL; NaN = uniform_for(seed, step) */
    uint32_t* out_ids_dev;               /* [rows] */
    float* out_logprobs_dev;             /* [rows] or NULL; a greedy row (exact argmax, no distribution
                                            is formed) leaves its entry as it was */
    /* diagnostics, any may be NULL: the sorted top-k candidates before truncation */
    uint32_t* dbg_ids_dev;               /* [rows][LILY_SAMPLE_K_CAP] */
    float* dbg_probs_dev;                /* [rows][LILY_SAMPLE_K_CAP] exp(adjusted - top) */
    uint32_t* dbg_counts_dev;            /* [rows][2] = candidates, kept */
} lily_rows;

/* Host cost and waits: up to 8 rows travel as kernel arguments.  Beyond that the call packs one
 * 224-byte descriptor per row into one of four pinned staging buffers, which a small kernel of
 * the library carries to the device ahead of the draws.  It blocks only (a) when the launch of the call four calls back has not finished,
 * (b) the first time `rows` exceeds every earlier call's (beyond 1024): the staging buffers are
 * reallocated, which drains the stream.  A caller that must never hit (b) mid-run issues one call
 * at its largest batch size first. */
int lily_sample_rows(lily_sampler_t* s, const lily_rows* batch);

/* A resident batch: the row table is packed and uploaded once (lily_plan_set, which
 * synchronises) and each lily_plan_run is a single launch with steps[r] + step_delta.
 * No counterpart in the reference, whose encode call re-sends its constants per draw. */
typedef struct lily_plan lily_plan_t;
int lily_plan_create(lily_sampler_t* s, uint32_t max_rows, lily_plan_t** out);
void lily_plan_destroy(lily_plan_t* p);
int lily_plan_set(lily_plan_t* p, const lily_rows* batch);
int lily_plan_run(lily_plan_t* p, uint32_t step_delta);

/* ---- Insertions: what the thinking control decides, as the `forced` input of the next steps.
 *
 * The reference's ThinkingControl::decide / decide_stop (src/thinking.rs:485-608) read decoded
 * text and stay on the host; each answers with an Action - Keep, Before(ids), After(ids),
 * Replace(ids) - about the token a step has just drawn.  This queue turns those answers into
 * per-row forced tokens of the steps that follow (lily_rows.forced), and does on the device,
 * in stream order, what the reference's TODO at thinking.rs:587-592 leaves undone: a replaced
 * draw leaves the row's penalty counts.
 *   AFTER   (drawn, ids): drawn stays emitted; the next steps are forced to ids[0..n).
 *   BEFORE  (drawn, ids): ids are emitted first, then drawn again as a forced token; its count
 *           from the draw is taken back so that it is counted once.
 *   REPLACE (drawn, ids): drawn is not emitted: its count is taken back; ids follow.
 * Host state only; the un-counting is lily_scratch_uncount on the row's scratch (NULL: none). */
typedef struct lily_insertions lily_insertions_t;
typedef enum lily_insert_kind {
    LILY_INSERT_AFTER = 0,
    LILY_INSERT_BEFORE = 1,
    LILY_INSERT_REPLACE = 2
} lily_insert_kind;
int lily_insertions_create(uint32_t rows, lily_insertions_t** out);
void lily_insertions_destroy(lily_insertions_t* q);
int lily_insertions_push(lily_insertions_t* q, uint32_t row, lily_insert_kind kind, uint32_t drawn,
                         const uint32_t* ids, uint32_t n, lily_scratch_t* scratch);
/* Fills forced_out[0..rows) for the next lily_sample_rows call (LILY_NO_TOKEN = the row draws)
 * and removes what it hands out.  Returns the number of rows that are forced. */
uint32_t lily_insertions_next(lily_insertions_t* q, uint32_t* forced_out);
/* Tokens still queued for `row` (0 for a row out of range). */
uint32_t lily_insertions_pending(const lily_insertions_t* q, uint32_t row);
/* Drops what is queued for `row` (a finished or cancelled request). */
void lily_insertions_clear(lily_insertions_t* q, uint32_t row);

/* ---- The producer of the logits and the draws from its summaries.
 *
 * Replaces the language-model head in front of the draws: `project_mat(mixed, lm_head, logits)`
 * followed by one `sample_f32` per row (src/qwen4exp/batch.rs:573-593) and the single-row
 * `gemv_quant(lm_head, mixed, logits)` + `sample_f32` (src/qwen4exp/model.rs:2959-2966,
 * 4157-4169).  The head is held in bf16 or in one of the reference's affine formats (4- or 8-bit
 * codes with a bf16 scale and bias per group of a row: QuantWeights, src/weights.rs:27-36; its
 * lm_head is 4 bits in groups of 64, or 8 under `--q8 head`).  Codes follow the reference's two
 * forms.  Up to 16 rows - a decode or verify step - take its form for few rows (gemv_q4_bf16 /
 * gemv_q8_bf16 and their _f32out kinds, src/kernels/metal/quant.metal:8-60 and 130-176): the
 * codes are not turned into weights, a group's part of a logit is scale * sum(q * x) + bias *
 * sum(x) with f32 sums, the weight is exactly q * scale + bias.  (Groups of 64 or more, an even
 * number of them a row, d a multiple of 256 (4 bits) or 128 (8 bits).)  Every other shape takes
 * its form for batches: the weights are what dequant_q4_bf16 / dequant_q8_bf16 make of the
 * codes (q * scale + bias in f32, rounded to bf16: src/kernels/metal/quant.metal:179-233), on
 * their way into the product.  logits[r][v] = sum_i hidden[r][i] * weight[v][i],
 * accumulated in f32 on the matrix cores and stored as f32 (what the reference's sampler reads,
 * src/kernels/sample.rs:263) or rounded to bf16 (nearest even).  Beside the logits the producer leaves,
 * for every LILY_LOGIT_TILE_COLS columns of every row, the largest value and the sum of
 * 2^((x - largest) * log2(e) / T[r]) over the tile - "summaries".  A row that is greedy or
 * draws among at most 64 candidates, under no penalties or under penalties that can only lower
 * a value (repetition >= 1, presence and frequency >= 0), is then drawn from the summaries and
 * the few tiles that can hold a candidate (about k tiles of 256 bytes instead of the row; a
 * penalised row whose values lie too close together for that is recognised on the device and
 * read whole).  A row that draws may carry a bias list of up to 64 pairs (the tiles that hold a
 * biased id are read besides) or an allow-mask (tiles the mask bars drop out, tiles allowed in
 * part are tested id by id; a row whose mask bars too many of its best values, or leaves too
 * many tiles allowed in part for its log-probability, is recognised on the device and read
 * whole); a greedy or forced row with either, and every other row of the batch, is drawn from
 * the logits as lily_sample_rows draws it.  Ids and log-probabilities are those of lily_sample_rows
 * on the same logits. */
#define LILY_LOGIT_TILE_COLS 128u

typedef struct lily_lm_head {
    const void* hidden_dev;   /* bf16 [rows][hidden_stride], d valid elements a row */
    uint64_t hidden_stride;   /* elements; a multiple of 8; rows start at multiples of 16 bytes */
    const void* weight_dev;   /* weight_bits 0: bf16 [vocab][weight_stride], row v the weights of id v;
                                 4 or 8: the codes, u32 [vocab][weight_stride] (d * bits / 32 words
                                 hold a row, the lowest code of a word first) */
    uint64_t weight_stride;   /* bf16 elements (a multiple of 8) or words of codes (a multiple of 4) */
    uint32_t d;               /* a multiple of 64 */
    uint32_t weight_bits;     /* 0 = bf16 weights; 4 or 8 = affine codes (f32 logits only) */
    float* tile_max_dev;      /* out [rows][lily_lm_head_tiles(vocab)] */
    float* tile_sum_dev;      /* out, same shape */
    const void* scales_dev;   /* weight_bits 4 / 8: bf16 [vocab][d / group_size]; else unused */
    const void* biases_dev;   /* same shape */
    uint32_t group_size;      /* weight_bits 4 / 8: a power of two from 32 on that divides d */
    uint32_t logits_f32;      /* 0 = the logits are bf16 [rows][row_stride], 1 = f32 */
} lily_lm_head;

/* Summaries a row: ceil(vocab / LILY_LOGIT_TILE_COLS); at most 2048 are supported. */
uint32_t lily_lm_head_tiles(uint32_t vocab);

/* The producer alone.  temperatures: host [rows], the temperature each row will be drawn at, as
 * lily_params_effective reports it (1 for a greedy row); NULL or an entry that is not a positive
 * finite number: the sums of that row are not to be used.
 * logits_dev: bf16 or f32 (head->logits_f32) [rows][row_stride]. */
int lily_lm_head_bf16(lily_sampler_t* s, const lily_lm_head* head, uint32_t rows, uint32_t vocab,
                      const float* temperatures, void* logits_dev, uint64_t row_stride);

/* A batch of many rows (from 129 on; from 256 on over codes) is a plain matrix product of the
 * kind the platform's GEMM library (hipBLASLt) is tuned for: where a program can open that library
 * by its name (libhipblaslt.so.1: it is opened at run time, never linked) and the library has an
 * algorithm for the shape, the producer forms the logits through it - codes are first turned
 * into bf16 weights, all of them, in memory the call keeps (vocab x d x 2 bytes a device and
 * stream; the reference does the same for a batch) - and the summaries by a pass over the stored
 * logits; otherwise, and for fewer rows, by this library's own kernels.  Same values to the
 * producer's bar either way (the order of the f32 additions differs).  The first call of a shape
 * allocates (workspace, descriptors): make it outside a stream capture.  Environment,
 * read at lily_sampler_create: LILY_SAMPLER_HEAD=own (never the library), =library (every
 * batch it takes) or a number of rows to begin at.  lily_lm_head_library_calls: how many of this
 * sampler's producer calls went through the library so far. */
uint64_t lily_lm_head_library_calls(const lily_sampler_t* s);

/* The draws alone: batch->logits_dev (bf16 or f32, rows at multiples of 16 bytes) and the summaries must
 * come from one producer call made with the temperatures of batch->params.  Where the summaries
 * are those of this sampler's last producer call, a row that asks for a log-probability at
 * another temperature than its sums were formed at is drawn from its logits instead (right
 * token, right log-probability); summaries of any other origin are taken on trust. */
int lily_sample_rows_tiled(lily_sampler_t* s, const lily_rows* batch, const float* tile_max_dev,
                           const float* tile_sum_dev);

/* Both, in the sampler's stream: batch->logits_dev is where the logits are written (it is
 * written to although the field is const), batch->vocab and batch->rows size the product. */
int lily_lm_head_sample_rows(lily_sampler_t* s, const lily_lm_head* head, const lily_rows* batch);

#ifdef __cplusplus
}
#endif

#endif /* LILY_SAMPLER_H */
