// api_internal.h - what the C-ABI layer's source files share with each other (not exported
// through include/lily_sampler.h).
#pragma once

#include <hip/hip_runtime_api.h>

#include "../../include/lily_sampler.h"

namespace lily {

// Records the calling thread's error message (what lily_last_error returns); returns `code`.
int api_fail(int code, const char* fmt, ...);

// Workspace of rows that span several workgroups, as the row kernel takes it.
struct Workspace {
    uint64_t* cand = nullptr;    // [slots] candidate composites
    double* lse = nullptr;       // [rows * MAX_SLICES][2]
    uint32_t* ticket = nullptr;  // [rows], zero between launches
    uint32_t rows = 0;           // rows that may span several workgroups
    uint32_t slots = 0;          // candidate slots (rows x slices x k)
};

// One plain draw (lily_sample_f32's work) on `stream` of `device` with the caller's workspace
// instead of a sampler's: validation, packing and one launch; allocates nothing.
int sample_row_with_workspace(int device, hipStream_t stream, const Workspace& ws, const float* logits,
                              uint32_t vocab, lily_scratch_t* scratch,
                              const lily_sampling_params* params, uint32_t step, uint32_t* out);

// Device and stream a scratch was created for.
int scratch_device(const lily_scratch_t* sc);

// Resolves the calling device's address of the static scratch array (once per device);
// LILY_OK or LILY_ERR_HIP.  Called by lily_sampler_create so that the first no-allocation
// draw finds it done.
int static_scratch_init(int device);

}  // namespace lily
