// head_library.hip - the producer of the logits for a batch of rows through the vendor's GEMM
// library (hipBLASLt), and the pass over the stored logits that leaves what the producer's own
// epilogue leaves: every tile's largest value and the sum of its exponentials.
//
// A plain hidden[rows, d] x weight[vocab, d]^T of a few hundred rows is the work that library is
// tuned for (one persistent workgroup a compute unit, 256 x 256 tiles); this library's own kernel
// (lm_head.hip) holds the few-row shapes, where the weights stream once at the memory's speed,
// and stays the fallback wherever the vendor's library is absent or declines a shape.  The call
// sites this stands in for are lm_head.hip's (src/qwen4exp/batch.rs:573-582,
// src/qwen4exp/model.rs:2959-2966 and 4157-4164); codes (QuantWeights, src/weights.rs:27-36) are
// turned into bf16 weights first, as the reference does for a batch (dequant_q4_bf16 /
// dequant_q8_bf16 into a scratch matrix, then the GEMM: src/kernels/metal/quant.metal:179-233).
//
// The vendor's library is opened at run time by its name (the copy a host program has loaded
// already is the one that answers), never linked: without it every call here reports
// hipErrorNotSupported and the caller goes on with its own kernel.
#include <dlfcn.h>
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <type_traits>
#include <utility>
#include <vector>

#include "launch.h"

namespace lily {

namespace {

// x as the lane CTRL names holds it (0x120 + n: rotate right by n within each row of 16 lanes)
template <int CTRL>
__device__ __forceinline__ float rotated16(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// The summaries of stored logits.  One workgroup streams a slice of one row: 16 lanes a tile of
// 128 columns, 8 values a lane (one 16-byte piece of bf16, two of f32), blocks of four (bf16) or
// two (f32) tiles a thread with two blocks asked ahead of the one being reduced.  The arithmetic
// is what bounds it (a 64-wide vector instruction takes four clocks, an exponential sixteen), so
// it is kept short: the maximum skips a NaN by itself (IEEE maximum of a number and a NaN is the
// number), 2^(x * c2 - max * c2) of a column at -inf is 0 by itself, and a tile whose sum comes
// out as a NaN is summed again with every value tested.  What counts is what counts in the
// producer's epilogue: a NaN and a column outside the vocabulary are -inf.  (A row whose c2 is 0
// - its sums are not to be used - gets the count of its finite values, as there.)  The row's
// last tile, where the vocabulary ends inside it, is read value by value at the end.
template <bool F32>
__global__ void __launch_bounds__(256)
k_head_summaries(const void* __restrict__ logits, uint64_t stride, uint32_t vocab,
                 const float* __restrict__ c2_of_row, float* __restrict__ tile_max,
                 float* __restrict__ tile_sum, uint32_t tiles_per_row, uint32_t blocks_per_slice) {
    constexpr uint32_t ELEM = F32 ? 4u : 2u, PIECES = F32 ? 2u : 1u;
    constexpr uint32_t LOADS = F32 ? 2u : 4u, PER_BLOCK = LOADS * 16u;   // tiles a thread / a workgroup takes per block
    typedef typename std::conditional<F32, f32x4, u32x4>::type piece_t;
    struct Got {
        piece_t p[PIECES];
    };
    const uint32_t row = blockIdx.x, sub = threadIdx.x & 15u, mine = threadIdx.x >> 4;
    const float NEG = -__builtin_huge_valf();
    const float c = c2_of_row[row];
    const uint32_t full = vocab / 128u;   // whole tiles
    const uint32_t all_blocks = (full + PER_BLOCK - 1u) / PER_BLOCK;
    const uint32_t b0 = blockIdx.y * blocks_per_slice;
    const uint32_t b1 = b0 + blocks_per_slice < all_blocks ? b0 + blocks_per_slice : all_blocks;
    const char* base = static_cast<const char*>(logits) + (uint64_t)row * stride * ELEM;
    float* out_max = tile_max + (size_t)row * tiles_per_row;
    float* out_sum = tile_sum + (size_t)row * tiles_per_row;
    // Results wait in LDS until the slice is read: a store to memory inside the loop would be
    // counted with the loads in flight, and the loop would wait for all of them every pass.
    __shared__ float stash_max[HEAD_LIBRARY_MAX_TILES + 64], stash_sum[HEAD_LIBRARY_MAX_TILES + 64];
    const uint32_t first_tile = b0 * PER_BLOCK;
    auto summary = [&](const float (&x)[8], uint32_t tile, bool store, bool to_memory) {
        float m = NEG;
#pragma unroll
        for (uint32_t e = 0; e < 8u; ++e) {
            m = fmaxf(m, x[e]);
        }
        // (the maximum over the 16 lanes of a tile: the rotated operand as the instruction's own)
        asm("s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_ror:1 row_mask:0xf bank_mask:0xf"
            : "+v"(m));
        const float top = m * c;
        float sum = 0.0f;
#pragma unroll
        for (uint32_t e = 0; e < 8u; ++e) {
            sum += __builtin_amdgcn_exp2f(__builtin_fmaf(x[e], c, -top));
        }
        sum += rotated16<0x128>(sum);
        sum += rotated16<0x124>(sum);
        sum += rotated16<0x122>(sum);
        sum += rotated16<0x121>(sum);
        // A NaN among the tile's values, a tile of nothing but -inf, a column at -inf where c2 is
        // 0: the sum comes out as a NaN, and the rare tile is summed again value by value.
        if (sum != sum) {
            sum = 0.0f;
#pragma unroll
            for (uint32_t e = 0; e < 8u; ++e) {
                sum += x[e] == x[e] && x[e] > NEG ? __builtin_amdgcn_exp2f(__builtin_fmaf(x[e], c, -top)) : 0.0f;
            }
            sum += rotated16<0x128>(sum);
            sum += rotated16<0x124>(sum);
            sum += rotated16<0x122>(sum);
            sum += rotated16<0x121>(sum);
        }
        if (store && sub == 0u) {
            // (a tile that holds +inf: inf - inf, as in the producer's epilogue)
            const float value = m > NEG ? (m < __builtin_huge_valf() ? sum : __builtin_nanf("")) : 0.0f;
            if (to_memory) {
                out_max[tile] = m;
                out_sum[tile] = value;
            } else {
                stash_max[tile - first_tile] = m;
                stash_sum[tile - first_tile] = value;
            }
        }
    };
    // (loads past the last whole tile ask for that tile again: every load is unconditional)
    auto fetch = [&](Got (&d)[LOADS], uint32_t b) {
#pragma unroll
        for (uint32_t u = 0; u < LOADS; ++u) {
            const uint32_t tile = b * PER_BLOCK + u * 16u + mine;
            const char* at = base + ((tile < full ? tile : full - 1u) * 128u + sub * 8u) * ELEM;
#pragma unroll
            for (uint32_t q = 0; q < PIECES; ++q) {
                d[u].p[q] = *reinterpret_cast<const piece_t*>(at + q * 16u);
            }
        }
    };
    auto fold = [&](const Got (&d)[LOADS], uint32_t b) {
#pragma unroll
        for (uint32_t u = 0; u < LOADS; ++u) {
            const uint32_t tile = b * PER_BLOCK + u * 16u + mine;
            float x[8];
            if constexpr (F32) {
#pragma unroll
                for (uint32_t e = 0; e < 4u; ++e) {
                    x[e] = d[u].p[0][e];
                    x[4u + e] = d[u].p[PIECES - 1u][e];
                }
            } else {
#pragma unroll
                for (uint32_t e = 0; e < 4u; ++e) {
                    x[2u * e] = __builtin_bit_cast(float, d[u].p[0][e] << 16);
                    x[2u * e + 1u] = __builtin_bit_cast(float, d[u].p[0][e] & 0xffff0000u);
                }
            }
            summary(x, tile, tile < full, false);
        }
    };
    if (b0 < b1) {
        // Three blocks a pass, every one of them asked for and reduced without a condition (a
        // load that one path leaves unread would make every pass wait for all loads); what is
        // left of the slice after whole passes sits in the first two places of the ring.
        Got ring0[LOADS], ring1[LOADS], ring2[LOADS];
        const uint32_t n = b1 - b0, whole = n / 3u * 3u, last = b1 - 1u;
        auto clamped = [&](uint32_t b) -> uint32_t { return b < last ? b : last; };
        fetch(ring0, b0);
        fetch(ring1, clamped(b0 + 1u));
        for (uint32_t i = b0; i < b0 + whole; i += 3u) {
            fetch(ring2, clamped(i + 2u));
            fold(ring0, i);
            fetch(ring0, clamped(i + 3u));
            fold(ring1, i + 1u);
            fetch(ring1, clamped(i + 4u));
            fold(ring2, i + 2u);
        }
        if (n - whole >= 1u) {
            fold(ring0, b0 + whole);
        }
        if (n - whole == 2u) {
            fold(ring1, b0 + whole + 1u);
        }
    }
    __syncthreads();
    const uint32_t held = (b1 * PER_BLOCK < full ? b1 * PER_BLOCK : full);
    for (uint32_t t = first_tile + threadIdx.x; t < held; t += 256u) {
        out_max[t] = stash_max[t - first_tile];
        out_sum[t] = stash_sum[t - first_tile];
    }
    if (blockIdx.y == gridDim.y - 1u && full < tiles_per_row && threadIdx.x < 64u) {
        float x[8];
#pragma unroll
        for (uint32_t e = 0; e < 8u; ++e) {
            const uint32_t col = full * 128u + sub * 8u + e;
            x[e] = NEG;
            if (mine == 0u && col < vocab) {
                if constexpr (F32) {
                    x[e] = reinterpret_cast<const float*>(base)[col];
                } else {
                    x[e] = __builtin_bit_cast(float, (uint32_t) reinterpret_cast<const uint16_t*>(base)[col] << 16);
                }
            }
        }
        summary(x, full, mine == 0u, true);
    }
}

// Codes to bf16 weights: w = q * scale + bias as one fused f32 operation, rounded to bf16 (nearest
// even) - the values the tiles of lm_head.hip form on their way into LDS.  A thread turns eight
// codes (4 or 8 bytes, side by side with its neighbours') into 16 bytes, side by side too; a
// group holds 8 weights or more, so the eight share a scale and a bias.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
template <int WBITS>
__global__ void __launch_bounds__(256)
k_head_weights_of_codes(const uint32_t* __restrict__ codes, uint64_t codes_stride,
                        const uint16_t* __restrict__ scales, const uint16_t* __restrict__ biases,
                        uint32_t group_shift, uint32_t d, uint32_t vocab, uint16_t* __restrict__ out) {
    constexpr int AHEAD = 4;
    constexpr uint32_t WORDS = WBITS / 4;   // words of eight codes
    const uint32_t eights = d / 8u;
    const uint64_t n = (uint64_t)vocab * eights, step = (uint64_t)gridDim.x * 256u;
    for (uint64_t i0 = (uint64_t)blockIdx.x * 256u + threadIdx.x; i0 < n; i0 += step * AHEAD) {
        uint32_t w[AHEAD][2], sb[AHEAD];
        uint64_t to[AHEAD];
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            const uint64_t i = i0 + step * (uint64_t)u < n ? i0 + step * (uint64_t)u : n - 1u;
            const uint32_t row = (uint32_t)(i / eights), eight = (uint32_t)(i % eights);
            const uint32_t* at = codes + (uint64_t)row * codes_stride + eight * WORDS;
            w[u][0] = at[0];
            w[u][1] = WORDS == 2u ? at[WORDS - 1u] : 0u;
            const uint64_t g = (uint64_t)row * (d >> group_shift) + ((eight * 8u) >> group_shift);
            sb[u] = (uint32_t)scales[g] | ((uint32_t)biases[g] << 16);
            to[u] = (uint64_t)row * d + eight * 8u;
        }
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            const float sc = __builtin_bit_cast(float, sb[u] << 16), bi = __builtin_bit_cast(float, sb[u] & 0xffff0000u);
            uint32_t pairs[4];
#pragma unroll
            for (uint32_t p = 0; p < 4u; ++p) {
                f32x2 f;
#pragma unroll
                for (uint32_t e = 0; e < 2u; ++e) {
                    const uint32_t j = 2u * p + e;
                    const uint32_t q = WBITS == 8 ? ((w[u][j >> 2] >> (8u * (j & 3u))) & 0xffu) : ((w[u][0] >> (4u * j)) & 0xfu);
                    f[e] = __builtin_fmaf((float)q, sc, bi);
                }
                pairs[p] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
            }
            if (i0 + step * (uint64_t)u < n) {
                *reinterpret_cast<u32x4*>(out + to[u]) = u32x4{pairs[0], pairs[1], pairs[2], pairs[3]};
            }
        }
    }
}

// ---- the vendor's library, by name
struct Vendor {
    bool tried = false, usable = false;
    decltype(&hipblasLtCreate) create = nullptr;
    decltype(&hipblasLtMatrixLayoutCreate) layout_create = nullptr;
    decltype(&hipblasLtMatrixLayoutDestroy) layout_destroy = nullptr;
    decltype(&hipblasLtMatmulDescCreate) desc_create = nullptr;
    decltype(&hipblasLtMatmulDescDestroy) desc_destroy = nullptr;
    decltype(&hipblasLtMatmulDescSetAttribute) desc_set = nullptr;
    decltype(&hipblasLtMatmulPreferenceCreate) pref_create = nullptr;
    decltype(&hipblasLtMatmulPreferenceDestroy) pref_destroy = nullptr;
    decltype(&hipblasLtMatmulPreferenceSetAttribute) pref_set = nullptr;
    decltype(&hipblasLtMatmulAlgoGetHeuristic) heuristic = nullptr;
    decltype(&hipblasLtMatmul) matmul = nullptr;
};

template <class F>
bool bind(void* so, const char* name, F* to) {
    *to = reinterpret_cast<F>(dlsym(so, name));
    return *to != nullptr;
}

const Vendor& vendor() {
    static Vendor v;
    if (v.tried) {
        return v;
    }
    v.tried = true;
    void* so = dlopen("libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
    if (so == nullptr) {
        so = dlopen("/opt/rocm/lib/libhipblaslt.so.1", RTLD_NOW | RTLD_LOCAL);
    }
    if (so == nullptr) {
        return v;
    }
    v.usable = bind(so, "hipblasLtCreate", &v.create) && bind(so, "hipblasLtMatrixLayoutCreate", &v.layout_create) &&
               bind(so, "hipblasLtMatrixLayoutDestroy", &v.layout_destroy) &&
               bind(so, "hipblasLtMatmulDescCreate", &v.desc_create) &&
               bind(so, "hipblasLtMatmulDescDestroy", &v.desc_destroy) &&
               bind(so, "hipblasLtMatmulDescSetAttribute", &v.desc_set) &&
               bind(so, "hipblasLtMatmulPreferenceCreate", &v.pref_create) &&
               bind(so, "hipblasLtMatmulPreferenceDestroy", &v.pref_destroy) &&
               bind(so, "hipblasLtMatmulPreferenceSetAttribute", &v.pref_set) &&
               bind(so, "hipblasLtMatmulAlgoGetHeuristic", &v.heuristic) && bind(so, "hipblasLtMatmul", &v.matmul);
    return v;
}

constexpr size_t WORKSPACE_BYTES = 64u << 20;

// One shape's descriptors and the algorithm the library's heuristic names for it.
struct Plan {
    uint64_t rows, d, vocab, hidden_stride, weight_stride, logits_stride;
    bool out_f32, ok;
    hipblasLtMatmulDesc_t desc;
    hipblasLtMatrixLayout_t weights, hidden, logits;
    hipblasLtMatmulAlgo_t algo;
};

// What one stream of one device calls the library with: a handle, a workspace of its own (calls
// on one stream follow each other; two streams must not share scratch memory), its plans, and
// the bf16 weights its codes were last turned into.
struct Caller {
    hipblasLtHandle_t handle = nullptr;
    void* workspace = nullptr;
    std::vector<Plan> plans;
    void* weights = nullptr;
    size_t weights_bytes = 0;
};

std::mutex g_mu;
std::map<std::pair<int, hipStream_t>, Caller> g_callers;

// logits^T [vocab x rows, column-major, ld logits_stride] = weight [d x vocab, ld weight_stride]^T
// x hidden [d x rows, ld hidden_stride]
Plan make_plan(const Vendor& v, Caller& c, uint64_t rows, uint64_t d, uint64_t vocab, uint64_t hidden_stride,
               uint64_t weight_stride, uint64_t logits_stride, bool out_f32) {
    Plan p = {};
    p.rows = rows, p.d = d, p.vocab = vocab, p.hidden_stride = hidden_stride, p.weight_stride = weight_stride;
    p.logits_stride = logits_stride, p.out_f32 = out_f32, p.ok = false;
    const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
    hipblasLtMatmulPreference_t pref = nullptr;
    const uint64_t room = WORKSPACE_BYTES;
    hipblasLtMatmulHeuristicResult_t found[1];
    int n_found = 0;
    if (v.desc_create(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS &&
        v.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed)) == HIPBLAS_STATUS_SUCCESS &&
        v.desc_set(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)) == HIPBLAS_STATUS_SUCCESS &&
        v.layout_create(&p.weights, HIP_R_16BF, d, vocab, (int64_t)weight_stride) == HIPBLAS_STATUS_SUCCESS &&
        v.layout_create(&p.hidden, HIP_R_16BF, d, rows, (int64_t)hidden_stride) == HIPBLAS_STATUS_SUCCESS &&
        v.layout_create(&p.logits, out_f32 ? HIP_R_32F : HIP_R_16BF, vocab, rows, (int64_t)logits_stride) ==
            HIPBLAS_STATUS_SUCCESS &&
        v.pref_create(&pref) == HIPBLAS_STATUS_SUCCESS &&
        v.pref_set(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &room, sizeof(room)) == HIPBLAS_STATUS_SUCCESS &&
        v.heuristic(c.handle, p.desc, p.weights, p.hidden, p.logits, p.logits, pref, 1, found, &n_found) ==
            HIPBLAS_STATUS_SUCCESS &&
        n_found >= 1 && found[0].state == HIPBLAS_STATUS_SUCCESS && found[0].workspaceSize <= WORKSPACE_BYTES) {
        p.algo = found[0].algo;
        p.ok = true;
    }
    if (pref != nullptr) {
        v.pref_destroy(pref);
    }
    return p;
}

Caller* caller_of(const Vendor& v, hipStream_t stream) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) {
        return nullptr;
    }
    Caller& c = g_callers[std::make_pair(device, stream)];
    if (c.handle == nullptr) {
        if (v.create(&c.handle) != HIPBLAS_STATUS_SUCCESS) {
            c.handle = nullptr;
            return nullptr;
        }
    }
    if (c.workspace == nullptr && hipMalloc(&c.workspace, WORKSPACE_BYTES) != hipSuccess) {
        c.workspace = nullptr;
        (void)hipGetLastError();
        return nullptr;
    }
    return &c;
}

}  // namespace

bool head_library_present() {
    std::lock_guard<std::mutex> hold(g_mu);
    return vendor().usable;
}

hipError_t launch_head_library(hipStream_t stream, const void* hidden, uint64_t hidden_stride, const void* weight,
                               uint64_t weight_stride, uint32_t rows, uint32_t d, uint32_t vocab, void* logits,
                               uint64_t logits_stride, bool out_f32, const HeadWeights& wq) {
    std::lock_guard<std::mutex> hold(g_mu);
    const Vendor& v = vendor();
    if (!v.usable) {
        return hipErrorNotSupported;
    }
    Caller* c = caller_of(v, stream);
    if (c == nullptr) {
        return hipErrorNotSupported;
    }
    if (wq.bits != 0u) {
        if ((wq.bits != 4u && wq.bits != 8u) || d % 8u != 0u || wq.group_shift < 3u) {
            return hipErrorNotSupported;
        }
        const size_t bytes = (size_t)vocab * d * 2u;
        if (c->weights_bytes < bytes) {
            if (c->weights != nullptr) {
                (void)hipStreamSynchronize(stream);
                (void)hipFree(c->weights);
                c->weights = nullptr, c->weights_bytes = 0;
            }
            if (hipMalloc(&c->weights, bytes) != hipSuccess) {
                c->weights = nullptr;
                (void)hipGetLastError();
                return hipErrorNotSupported;
            }
            c->weights_bytes = bytes;
        }
        const uint64_t blocks = ((uint64_t)vocab * (d / 8u) + 1023u) / 1024u;
        const uint32_t grid = (uint32_t)(blocks < 65536u ? blocks : 65536u);
        if (wq.bits == 4u) {
            hipLaunchKernelGGL(k_head_weights_of_codes<4>, dim3(grid), dim3(256), 0, stream,
                               static_cast<const uint32_t*>(weight), weight_stride,
                               static_cast<const uint16_t*>(wq.scales), static_cast<const uint16_t*>(wq.biases),
                               wq.group_shift, d, vocab, static_cast<uint16_t*>(c->weights));
        } else {
            hipLaunchKernelGGL(k_head_weights_of_codes<8>, dim3(grid), dim3(256), 0, stream,
                               static_cast<const uint32_t*>(weight), weight_stride,
                               static_cast<const uint16_t*>(wq.scales), static_cast<const uint16_t*>(wq.biases),
                               wq.group_shift, d, vocab, static_cast<uint16_t*>(c->weights));
        }
        if (hipError_t e = hipGetLastError(); e != hipSuccess) {
            return e;
        }
        weight = c->weights;
        weight_stride = d;
    }
    const Plan* plan = nullptr;
    for (const Plan& p : c->plans) {
        if (p.rows == rows && p.d == d && p.vocab == vocab && p.hidden_stride == hidden_stride &&
            p.weight_stride == weight_stride && p.logits_stride == logits_stride && p.out_f32 == out_f32) {
            plan = &p;
            break;
        }
    }
    if (plan == nullptr) {
        if (c->plans.size() >= 64u) {
            return hipErrorNotSupported;   // (a caller that never repeats a shape keeps to its own kernel)
        }
        c->plans.push_back(make_plan(v, *c, rows, d, vocab, hidden_stride, weight_stride, logits_stride, out_f32));
        plan = &c->plans.back();
    }
    if (!plan->ok) {
        return hipErrorNotSupported;
    }
    const float one = 1.0f, zero = 0.0f;
    const hipblasStatus_t st = v.matmul(c->handle, plan->desc, &one, weight, plan->weights, hidden, plan->hidden, &zero,
                                        logits, plan->logits, logits, plan->logits, &plan->algo, c->workspace,
                                        WORKSPACE_BYTES, stream);
    return st == HIPBLAS_STATUS_SUCCESS ? hipSuccess : hipErrorUnknown;
}

hipError_t launch_head_summaries(hipStream_t stream, const void* logits, uint64_t logits_stride, uint32_t rows,
                                 uint32_t vocab, const float* c2_of_row, float* tile_max, float* tile_sum,
                                 bool f32) {
    const uint32_t tiles = (vocab + LILY_TILE_COLS - 1u) / LILY_TILE_COLS;
    if (tiles > HEAD_LIBRARY_MAX_TILES) {
        return hipErrorInvalidValue;
    }
    // about a thousand workgroups: a row is cut into slices of whole blocks where the rows are few
    const uint32_t per_block = f32 ? 32u : 64u, blocks = (vocab / 128u + per_block - 1u) / per_block;
    const uint32_t want = (1024u + rows - 1u) / rows;
    const uint32_t per_slice = blocks == 0u ? 1u : (blocks + want - 1u) / want;
    const uint32_t slices = blocks == 0u ? 1u : (blocks + per_slice - 1u) / per_slice;
    const dim3 grid(rows, slices);
    if (f32) {
        hipLaunchKernelGGL(k_head_summaries<true>, grid, dim3(256), 0, stream, logits, logits_stride, vocab, c2_of_row,
                           tile_max, tile_sum, tiles, per_slice);
    } else {
        hipLaunchKernelGGL(k_head_summaries<false>, grid, dim3(256), 0, stream, logits, logits_stride, vocab,
                           c2_of_row, tile_max, tile_sum, tiles, per_slice);
    }
    return hipGetLastError();
}

}  // namespace lily
