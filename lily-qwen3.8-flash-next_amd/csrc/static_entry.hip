// static_entry.hip - the draw that allocates nothing: lily_sample_f32_static.
//
// A row that spans several workgroups needs device memory beyond its inputs and outputs: every
// slice's candidates, its (reference, sum) pair and the row's arrival ticket.  The other entry
// points take it from the workspace lily_sampler_create allocates; this one takes it from a
// file-scope device array, so a caller that must not allocate (under HIP graph capture, in a
// serving loop, in a harness that forbids hipMalloc) needs no sampler object at all.  Each GPU
// the library runs on holds its own copy of the array until the process ends.
#include <hip/hip_runtime.h>

#include <mutex>

#include "api_internal.h"
#include "launch.h"

// One row: up to MERGE_CAP candidate slots (slices x k), MAX_SLICES (reference, sum) pairs, a ticket.
constexpr size_t CAND_BYTES = (size_t)lily::MERGE_CAP * sizeof(uint64_t);       // 32 768
constexpr size_t LSE_BYTES = (size_t)lily::MAX_SLICES * 2 * sizeof(double);     //  1 024
constexpr size_t TICKET_BYTES = 256;
constexpr size_t SCRATCH_BYTES = CAND_BYTES + LSE_BYTES + TICKET_BYTES;          // 34 048

// In host code this name is a stand-in, not a device address: everything below goes through
// the pointer hipGetSymbolAddress returns for the current device.
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
std::mutex g_lock;
unsigned char* g_ptr[MAX_DEVICES] = {};  // each device's own copy of the array

}  // namespace

namespace lily {

int static_scratch_init(int device) {
    if (device < 0 || device >= MAX_DEVICES) {
        return api_fail(LILY_ERR_RANGE, "device %d outside 0..%d", device, MAX_DEVICES - 1);
    }
    std::lock_guard<std::mutex> hold(g_lock);
    if (g_ptr[device] != nullptr) {
        return LILY_OK;
    }
    int current = -1;
    hipError_t e = hipGetDevice(&current);
    if (e == hipSuccess && current != device) {
        e = hipSetDevice(device);
    }
    void* p = nullptr;
    if (e == hipSuccess) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    }
    if (e == hipSuccess && current >= 0 && current != device) {
        e = hipSetDevice(current);
    }
    if (e != hipSuccess || p == nullptr) {
        return api_fail(LILY_ERR_HIP, "address of the static scratch on device %d: %s", device,
                        hipGetErrorString(e));
    }
    g_ptr[device] = static_cast<unsigned char*>(p);
    return LILY_OK;
}

}  // namespace lily

extern "C" int lily_sample_f32_static(void* hip_stream, const float* logits_dev, uint32_t vocab,
                                      lily_scratch_t* scratch_counts,
                                      const lily_sampling_params* params, uint32_t step,
                                      uint32_t* out_dev) {
    using namespace lily;
    if (vocab > LILY_STATIC_MAX_VOCAB) {
        return api_fail(LILY_ERR_RANGE, "lily_sample_f32_static draws from at most %u logits, got %u",
                        (unsigned)LILY_STATIC_MAX_VOCAB, vocab);
    }
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) {
        return api_fail(LILY_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
    }
    if (scratch_counts != nullptr && scratch_device(scratch_counts) != device) {
        return api_fail(LILY_ERR_INVALID_ARG, "the sampler scratch lives on device %d, the draw runs on %d",
                        scratch_device(scratch_counts), device);
    }
    if (int rc = static_scratch_init(device)) {  // first call on this device only
        return rc;
    }
    unsigned char* base = g_ptr[device];
    Workspace ws;
    ws.cand = reinterpret_cast<uint64_t*>(base);
    ws.lse = reinterpret_cast<double*>(base + CAND_BYTES);
    ws.ticket = reinterpret_cast<uint32_t*>(base + CAND_BYTES + LSE_BYTES);
    ws.rows = 1;
    ws.slots = MERGE_CAP;
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    // The array keeps the last call's contents.  Candidates and sums are written whole by every
    // slice before they are read; the ticket must start at zero (a fill kernel, not a memset
    // node, so that the call can be captured into a graph).
    e = launch_fill_u32(stream, ws.ticket, 1, 0);
    if (e != hipSuccess) {
        return api_fail(LILY_ERR_HIP, "clearing the ticket: %s", hipGetErrorString(e));
    }
    return sample_row_with_workspace(device, stream, ws, logits_dev, vocab, scratch_counts, params, step,
                                     out_dev);
}
