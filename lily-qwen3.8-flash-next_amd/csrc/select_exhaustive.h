// select_exhaustive.h - the radix select that is correct for any input.
#pragma once

#include "device_common.h"

namespace lily {

// ------------------------------------------------------------------ exhaustive select
//
// The exact top-k of ids [id_lo, id_hi) by a radix select on the composite: up to
// eight passes of 8 bits, each re-evaluating every element.  Slow and correct for
// any input (ties, masks, few finite values).  Leaves the winners (unsorted) in
// cand[0 .. sh.n_cand).
template <int DT>
__device__ __forceinline__ void select_exhaustive(const RowArgs& a, uint32_t e0, uint32_t e1, uint32_t k,
                                  bool want_lse, uint64_t* cand, uint32_t cap, Shared& sh) {
    const uint32_t tid = threadIdx.x;
    uint64_t prefix = 0, pmask = 0;
    uint32_t need = k;
    LseAcc lse;
    lse.init();
    bool take_all = false;
    for (int pass = 0; pass < 8 && !take_all; ++pass) {
        const int shift = 56 - 8 * pass;
        if (tid < 256) {
            sh.hist[tid] = 0;
        }
        __syncthreads();
        HistRun run;
        run.init();
        for (uint32_t id = e0 + tid; id < e1; id += NT) {
            const float u = pre_temperature_of<DT>(a, id);
            if (pass == 0 && want_lse) {
                lse.add_one(u, a.c2);
            }
            const uint64_t c = composite_of(u / a.temperature, id);
            run.add(sh.hist, (uint32_t)(c >> shift) & 255u, c != 0 && (c & pmask) == prefix);
        }
        run.flush(sh.hist);
        __syncthreads();
        find_bin(sh, need);
        take_all = sh.all_taken != 0u;
        if (!take_all) {
            prefix |= (uint64_t)sh.sel_bin << shift;
            pmask |= (uint64_t)255u << shift;
            need = sh.need;
        }
    }
    if (want_lse) {
        lse_reduce(sh, lse);
    }
    if (tid == 0) {
        sh.n_cand = 0;
    }
    __syncthreads();
    const uint64_t floor_c = take_all ? 1ull : prefix;
    for (uint32_t id = e0 + tid; id < e1; id += NT) {
        const uint64_t c = composite_of(adjusted_of<DT>(a, id), id);
        if (c >= floor_c && c != 0) {
            const uint32_t at = atomicAdd(&sh.n_cand, 1u);
            if (at < cap) {
                cand[at] = c;
            }
        }
    }
    __syncthreads();
}


}  // namespace lily
