// scratch_kernels.hip - the small kernels (scratch maintenance, speculative control) and the
// host-callable launchers, including the dispatch among the row kernel's variants.
#include <hip/hip_runtime.h>

#include "launch.h"

namespace lily {

// ------------------------------------------------------------------ small kernels

__global__ void k_fill_u32(uint32_t* p, uint32_t n, uint32_t v) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

// counts[id] += 1 per occurrence, the id's bit in `touched`, the largest count reached (the first
// spare word behind the bitmap) and an id that reached it (the second; a hint, see tail.h).
__global__ void k_add_history(ScratchView sc, const uint32_t* ids, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const uint32_t id = ids[i];
        if (id < sc.vocab) {
            const uint32_t before = atomicAdd(&sc.counts[id], 1u);
            atomicOr(&sc.touched[id >> 5], 1u << (id & 31u));
            const uint32_t words = (sc.vocab + 31u) / 32u;
            if (atomicMax(&sc.touched[words], before + 1u) <= before + 1u) {
                sc.touched[words + 1u] = id;
            }
        }
    }
}

// Saturating decrement; the id stays on the bitmap (with a count that may now be 0).
__device__ __forceinline__ void uncount_one(const ScratchView& sc, uint32_t token) {
    if (token >= sc.vocab) {
        return;
    }
    const uint32_t c = sc.counts[token];
    if (c > 0u) {
        sc.counts[token] = c - 1u;
    }
}

__global__ void k_uncount(ScratchView sc, uint32_t token) {
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        uncount_one(sc, token);
    }
}

// The rollback of the rejected rows' draws (src/qwen4exp/spec.rs:213-217) with the accepted
// row read on the device: draws[a + 1 .. m) are un-counted in order, a = min(accepted[0], cap).
__global__ void k_uncount_after(ScratchView sc, const uint32_t* draws, uint32_t m,
                                const uint32_t* accepted, uint32_t cap) {
    if (blockIdx.x != 0 || threadIdx.x != 0) {
        return;
    }
    const uint32_t a = min(accepted[0], cap);
    if (a >= m) {
        return;
    }
    for (uint32_t j = a + 1u; j < m; ++j) {
        uncount_one(sc, draws[j]);
    }
}

// After counts were written whole: touched[w] = bits of the non-zero counts in word w, and the
// largest count (the word behind the bitmap, cleared before the launch).
__global__ void k_touch_from_counts(ScratchView sc) {
    const uint32_t w = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t words = (sc.vocab + 31u) / 32u;
    if (w < words) {
        uint32_t bits = 0, most = 0, most_id = 0;
        for (uint32_t b = 0; b < 32u; ++b) {
            const uint32_t id = w * 32u + b;
            const uint32_t c = id < sc.vocab ? sc.counts[id] : 0u;
            if (c != 0u) {
                bits |= 1u << b;
                if (c > most) {
                    most = c;
                    most_id = id;
                }
            }
        }
        sc.touched[w] = bits;
        if (most != 0u && atomicMax(&sc.touched[words], most) <= most) {
            sc.touched[words + 1u] = most_id;
        }
    }
}

// spec.metal:14-38
__global__ void k_spec_accept(const uint32_t* draws, const uint32_t* ids, uint32_t* ctrl,
                              uint32_t m, uint32_t pos0, uint32_t ratio, uint32_t chain,
                              uint32_t stride) {
    if (blockIdx.x != 0 || threadIdx.x != 0) {
        return;
    }
    uint32_t a = 0;
    while (a + 1 < m && draws[a] == ids[a + 1]) {
        ++a;
    }
    ctrl[0] = a;
    ctrl[stride] = a + 1;
    for (uint32_t i = 0; i < chain; ++i) {
        const uint32_t p = pos0 + a + 1 + i;
        ctrl[(2 + 3 * i) * stride] = p;
        ctrl[(3 + 3 * i) * stride] = p / ratio;
        ctrl[(4 + 3 * i) * stride] = ((p + 1) % ratio == 0) ? 1u : 0u;
    }
}

// spec.metal:42-52
__global__ void k_copy_row_u32(const uint32_t* src, uint32_t* dst, uint32_t words, uint32_t rows,
                               const uint32_t* row_dev) {
    const uint32_t row = *row_dev;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows || i >= words) {
        return;
    }
    dst[i] = src[(size_t)row * words + i];
}

// n 16-byte pieces from src to dst (src may be pinned host memory mapped into the device).
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(256) k_copy_pieces(const u32x4* src, u32x4* dst, uint32_t n) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < n) {
        dst[i] = src[i];
    }
}

// The row kernel's access pattern with nothing else: one workgroup of 256 threads per row,
// 16-byte loads, three blocks of four loads per thread requested ahead, an integer maximum as
// the only arithmetic.  What this reaches is the ceiling a launch of the same shape can reach.
__global__ void __launch_bounds__(256) k_probe_read(const u32x4* base, uint64_t row_chunks,
                                                    uint64_t stride_chunks, uint32_t* out) {
    const u32x4* row = base + (uint64_t)blockIdx.x * stride_chunks;
    const uint64_t last = row_chunks - 1u;
    auto fetch = [&](u32x4 (&d)[4], uint64_t b) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const uint64_t c = b * 1024u + (uint64_t)u * 256u + threadIdx.x;
            d[u] = row[c < last ? c : last];
        }
    };
    auto fold = [](uint32_t m, const u32x4 (&d)[4]) -> uint32_t {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            m = max(max(m, d[u].x), max(max(d[u].y, d[u].z), d[u].w));
        }
        return m;
    };
    const uint64_t nblocks = (row_chunks + 1023u) / 1024u;
    u32x4 a[4], b[4], c[4];
    uint32_t m = 0;
    fetch(a, 0);
    fetch(b, 1 < nblocks ? 1 : nblocks - 1u);
    for (uint64_t i = 0; i < nblocks; i += 3) {
        fetch(c, i + 2 < nblocks ? i + 2 : nblocks - 1u);
        m = fold(m, a);
        if (i + 1 < nblocks) {
            fetch(a, i + 3 < nblocks ? i + 3 : nblocks - 1u);
            m = fold(m, b);
            if (i + 2 < nblocks) {
                fetch(b, i + 4 < nblocks ? i + 4 : nblocks - 1u);
                m = fold(m, c);
            }
        }
    }
    for (int o = 32; o > 0; o >>= 1) {
        m = max(m, (uint32_t)__shfl_xor((int)m, o));
    }
    if ((threadIdx.x & 63u) == 0) {
        atomicMax(out + blockIdx.x, m);
    }
}

// ------------------------------------------------------------------ launchers (host)

#define LILY_VARIANT(DT, KIND)                                                                   \
    hipError_t launch_rows_dt##DT##_kind##KIND(hipStream_t stream, bool lse, uint32_t rows,      \
                                               const LaunchCfg& cfg, const InlineRows* inline_rows, \
                                               size_t dyn_bytes);
LILY_VARIANT(0, 0)
LILY_VARIANT(0, 1)
LILY_VARIANT(0, 2)
LILY_VARIANT(1, 0)
LILY_VARIANT(1, 1)
LILY_VARIANT(1, 2)
#undef LILY_VARIANT

hipError_t launch_rows(hipStream_t stream, int dtype, int kind, bool lse, uint32_t rows,
                       const LaunchCfg& cfg_in, const InlineRows* inline_rows, size_t dyn_bytes) {
    LaunchCfg cfg = cfg_in;
    cfg.dyn_slots = (uint32_t)(dyn_bytes / 8);
    if (dtype == LILY_BF16) {
        switch (kind) {
            case 0: return launch_rows_dt1_kind0(stream, lse, rows, cfg, inline_rows, dyn_bytes);
            case 1: return launch_rows_dt1_kind1(stream, lse, rows, cfg, inline_rows, dyn_bytes);
            default: return launch_rows_dt1_kind2(stream, lse, rows, cfg, inline_rows, dyn_bytes);
        }
    }
    switch (kind) {
        case 0: return launch_rows_dt0_kind0(stream, lse, rows, cfg, inline_rows, dyn_bytes);
        case 1: return launch_rows_dt0_kind1(stream, lse, rows, cfg, inline_rows, dyn_bytes);
        default: return launch_rows_dt0_kind2(stream, lse, rows, cfg, inline_rows, dyn_bytes);
    }
}

hipError_t launch_fill_u32(hipStream_t stream, uint32_t* p, uint32_t n, uint32_t v) {
    if (n == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(k_fill_u32, dim3((n + 255) / 256), dim3(256), 0, stream, p, n, v);
    return hipGetLastError();
}

hipError_t launch_add_history(hipStream_t stream, const ScratchView& sc, const uint32_t* ids,
                              uint32_t n) {
    if (n == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(k_add_history, dim3((n + 255) / 256), dim3(256), 0, stream, sc, ids, n);
    return hipGetLastError();
}

hipError_t launch_uncount(hipStream_t stream, const ScratchView& sc, uint32_t token) {
    hipLaunchKernelGGL(k_uncount, dim3(1), dim3(64), 0, stream, sc, token);
    return hipGetLastError();
}

hipError_t launch_uncount_after(hipStream_t stream, const ScratchView& sc, const uint32_t* draws,
                                uint32_t m, const uint32_t* accepted, uint32_t cap) {
    hipLaunchKernelGGL(k_uncount_after, dim3(1), dim3(64), 0, stream, sc, draws, m, accepted, cap);
    return hipGetLastError();
}

hipError_t launch_rebuild_listed(hipStream_t stream, const ScratchView& sc) {
    const uint32_t words = (sc.vocab + 31u) / 32u;
    hipLaunchKernelGGL(k_fill_u32, dim3(1), dim3(64), 0, stream, sc.touched + words, 2u, 0u);
    hipLaunchKernelGGL(k_touch_from_counts, dim3((words + 255) / 256), dim3(256), 0, stream, sc);
    return hipGetLastError();
}

hipError_t launch_spec_accept(hipStream_t stream, const uint32_t* draws, const uint32_t* ids,
                              uint32_t* ctrl, uint32_t m, uint32_t pos0, uint32_t ratio,
                              uint32_t chain) {
    hipLaunchKernelGGL(k_spec_accept, dim3(1), dim3(64), 0, stream, draws, ids, ctrl, m, pos0, ratio,
                       chain, LILY_CTRL_STRIDE);
    return hipGetLastError();
}

hipError_t launch_copy_row(hipStream_t stream, const uint32_t* src, uint32_t* dst, uint32_t words,
                           uint32_t rows, const uint32_t* row_dev) {
    hipLaunchKernelGGL(k_copy_row_u32, dim3((words + 255) / 256), dim3(256), 0, stream, src, dst,
                       words, rows, row_dev);
    return hipGetLastError();
}

hipError_t launch_copy_pieces(hipStream_t stream, const void* src, void* dst, size_t bytes) {
    const uint32_t n = (uint32_t)(bytes / 16u);
    if (n == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(k_copy_pieces, dim3((n + 255u) / 256u), dim3(256), 0, stream,
                       reinterpret_cast<const u32x4*>(src), reinterpret_cast<u32x4*>(dst), n);
    return hipGetLastError();
}

hipError_t launch_probe_read(hipStream_t stream, const void* base, uint32_t rows, uint64_t row_bytes,
                             uint64_t stride_bytes, uint32_t* out) {
    hipLaunchKernelGGL(k_probe_read, dim3(rows), dim3(256), 0, stream,
                       reinterpret_cast<const u32x4*>(base), row_bytes / 16u, stride_bytes / 16u, out);
    return hipGetLastError();
}

}  // namespace lily
