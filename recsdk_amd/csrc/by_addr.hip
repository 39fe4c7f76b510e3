// By-address row lookup / update and the fused LazyAdam / Sgd row updates.
// All four are pure row streaming: one thread per 16-byte (or narrower) chunk of a row, consecutive threads on
// consecutive chunks of the same row so that every row is read and written with full cache lines.
// Compiled with -ffp-contract=off.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.h"

namespace recsdk {

typedef uint32_t Chunk16 __attribute__((ext_vector_type(4)));
typedef uint32_t Chunk8 __attribute__((ext_vector_type(2)));
typedef float RowVec __attribute__((ext_vector_type(4)));

template <int CH>
struct ChunkT;
template <>
struct ChunkT<16> {
    using type = Chunk16;
};
template <>
struct ChunkT<8> {
    using type = Chunk8;
};
template <>
struct ChunkT<4> {
    using type = uint32_t;
};
template <>
struct ChunkT<2> {
    using type = uint16_t;
};

// y[i, :] = *(row*)address[i]; address 0 -> zeros.  CH = bytes per thread.
// The block first copies the addresses of the rows it covers into LDS (one thread per row), so that the copy loop
// issues row loads and stores only; with every lane loading its row's address itself a third of the memory
// instructions were address loads.
template <int CH>
__global__ __launch_bounds__(kBlock) void k_lookup_by_addr(const int64_t* __restrict__ address, int64_t n,
                                                           int rowBytes, int chunksPerRow, char* __restrict__ y)
{
    using C = typename ChunkT<CH>::type;
    constexpr int kChunks = kBlock * kItems;
    __shared__ int64_t sAddr[kChunks + 2];
    const int64_t total = n * chunksPerRow;
    const int64_t g0 = (int64_t)blockIdx.x * kChunks;
    const int64_t i0 = g0 / chunksPerRow;
    const uint32_t r0 = (uint32_t)(g0 - i0 * chunksPerRow);
    const int rowsHere = (int)((r0 + (uint32_t)kChunks + (uint32_t)chunksPerRow - 1) / (uint32_t)chunksPerRow);
    for (int j = threadIdx.x; j < rowsHere; j += kBlock) {
        sAddr[j] = (i0 + j < n) ? address[i0 + j] : 0;
    }
    __syncthreads();
    C vals[kItems];
    int64_t dst[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        int64_t g = g0 + k * kBlock + threadIdx.x;
        dst[k] = -1;
        if (g < total) {
            const uint32_t q = r0 + (uint32_t)(k * kBlock + threadIdx.x);
            const uint32_t qi = q / (uint32_t)chunksPerRow;
            int64_t i = i0 + qi;
            int c = (int)(q - qi * (uint32_t)chunksPerRow);
            int64_t a = sAddr[qi];
            dst[k] = i * rowBytes + (int64_t)c * CH;
            if (a != 0) {
                const char* src = reinterpret_cast<const char*>(a) + (int64_t)c * CH;
                if ((reinterpret_cast<uintptr_t>(src) & (CH - 1)) == 0) {
                    vals[k] = *reinterpret_cast<const C*>(src);
                } else {
                    // address not aligned to the chunk: assemble from 16-bit pieces
                    uint16_t* pieces = reinterpret_cast<uint16_t*>(&vals[k]);
#pragma unroll
                    for (int b = 0; b < CH / 2; ++b) {
                        pieces[b] = reinterpret_cast<const uint16_t*>(src)[b];
                    }
                }
            } else {
                vals[k] = C{};
            }
        }
    }
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (dst[k] >= 0) {
            // the output is written once and read by a later kernel: streamed past the caches
            __builtin_nontemporal_store(vals[k], reinterpret_cast<C*>(y + dst[k]));
        }
    }
}

__device__ __forceinline__ void atomic_add_elem(float* p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomic_add_elem(int32_t* p, int32_t v) { atomicAdd(p, v); }

__device__ __forceinline__ float half_to_float(__half h) { return __half2float(h); }
__device__ __forceinline__ float half_to_float(__hip_bfloat16 h) { return __bfloat162float(h); }
__device__ __forceinline__ void float_to_half(float f, __half* h) { *h = __float2half(f); }
__device__ __forceinline__ void float_to_half(float f, __hip_bfloat16* h) { *h = __float2bfloat16(f); }

// 16-bit float atomic add through a CAS on the containing 32-bit word.
template <typename H>
__device__ __forceinline__ void atomic_add_half(H* p, H v)
{
    uintptr_t a = reinterpret_cast<uintptr_t>(p);
    uint32_t* word = reinterpret_cast<uint32_t*>(a & ~uintptr_t(3));
    const bool hi = (a & 2) != 0;
    uint32_t old = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    while (true) {
        uint16_t bits = hi ? (uint16_t)(old >> 16) : (uint16_t)(old & 0xffffu);
        H cur;
        __builtin_memcpy(&cur, &bits, 2);
        H sum;
        float_to_half(half_to_float(cur) + half_to_float(v), &sum);
        uint16_t nb;
        __builtin_memcpy(&nb, &sum, 2);
        uint32_t repl = hi ? ((old & 0x0000ffffu) | ((uint32_t)nb << 16)) : ((old & 0xffff0000u) | nb);
        uint32_t prev = atomicCAS(word, old, repl);
        if (prev == old) {
            break;
        }
        old = prev;
    }
}
__device__ __forceinline__ void atomic_add_elem(__half* p, __half v) { atomic_add_half<__half>(p, v); }
__device__ __forceinline__ void atomic_add_elem(__hip_bfloat16* p, __hip_bfloat16 v)
{
    atomic_add_half<__hip_bfloat16>(p, v);
}

// *(row*)address[i] (+)= emb[i, :].  One thread per element group of EPT elements.
template <typename T, int EPT>
__global__ __launch_bounds__(kBlock) void k_update_by_addr(const int64_t* __restrict__ address, int64_t n, int dim,
                                                           int groupsPerRow, const T* __restrict__ emb,
                                                           int updateType)
{
    const int64_t total = n * groupsPerRow;
    const int64_t g0 = (int64_t)blockIdx.x * (kBlock * kItems);
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        int64_t g = g0 + k * kBlock + threadIdx.x;
        if (g >= total) {
            continue;
        }
        int64_t i = g / groupsPerRow;
        int c = (int)(g - i * groupsPerRow);
        int64_t a = address[i];
        if (a == 0) {
            continue;
        }
        T* dst = reinterpret_cast<T*>(a) + c * EPT;
        const T* src = emb + i * dim + c * EPT;
        if (sizeof(T) * EPT == 16 && updateType == 1 && (c + 1) * EPT <= dim &&
            ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15) == 0) {
            // overwrite of a whole aligned 16-byte piece: one load, one store
            *reinterpret_cast<Chunk16*>(dst) = __builtin_nontemporal_load(reinterpret_cast<const Chunk16*>(src));
            continue;
        }
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            if (c * EPT + e < dim) {
                if (updateType == 0) {
                    atomic_add_elem(dst + e, src[e]);
                } else {
                    dst[e] = src[e];
                }
            }
        }
    }
}

// LazyAdam: rows indices[i] >= 0 of m, v, var updated in place (lazy_adam.cpp:168-185).
template <int VEC>
__global__ __launch_bounds__(kBlock) void k_lazy_adam(const float* __restrict__ grad,
                                                      const int32_t* __restrict__ indices, int64_t n, int dim,
                                                      int chunksPerRow, float* __restrict__ m, float* __restrict__ v,
                                                      float* __restrict__ var, float lr, float beta1, float beta2,
                                                      float eps)
{
    const int64_t total = n * chunksPerRow;
    const int64_t g0 = (int64_t)blockIdx.x * (kBlock * kItems);
    const float omb1 = 1.0f - beta1;
    const float omb2 = 1.0f - beta2;
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        int64_t g = g0 + k * kBlock + threadIdx.x;
        if (g >= total) {
            continue;
        }
        int64_t i = g / chunksPerRow;
        int c = (int)(g - i * chunksPerRow);
        int64_t idx = indices[i];
        if (idx < 0) {
            continue;
        }
        const int64_t e0 = idx * dim + (int64_t)c * VEC;
        const float* gp = grad + i * dim + (int64_t)c * VEC;
        float gv[VEC], mv[VEC], vv[VEC], wv[VEC];
        if (VEC == 4) {
            // every row is read and written once per call: streamed past the caches
            *reinterpret_cast<RowVec*>(gv) = __builtin_nontemporal_load(reinterpret_cast<const RowVec*>(gp));
            *reinterpret_cast<RowVec*>(mv) = __builtin_nontemporal_load(reinterpret_cast<const RowVec*>(m + e0));
            *reinterpret_cast<RowVec*>(vv) = __builtin_nontemporal_load(reinterpret_cast<const RowVec*>(v + e0));
            *reinterpret_cast<RowVec*>(wv) = __builtin_nontemporal_load(reinterpret_cast<const RowVec*>(var + e0));
        } else {
            gv[0] = gp[0];
            mv[0] = m[e0];
            vv[0] = v[e0];
            wv[0] = var[e0];
        }
#pragma unroll
        for (int x = 0; x < VEC; ++x) {
            float mn = mv[x] * beta1 + gv[x] * omb1;
            float vn = vv[x] * beta2 + (gv[x] * gv[x]) * omb2;
            float den = sqrtf(fabsf(vn)) + eps;
            float upd = (mn * -lr) / den;
            mv[x] = mn;
            vv[x] = vn;
            wv[x] = upd + wv[x];
        }
        if (VEC == 4) {
            __builtin_nontemporal_store(*reinterpret_cast<RowVec*>(mv), reinterpret_cast<RowVec*>(m + e0));
            __builtin_nontemporal_store(*reinterpret_cast<RowVec*>(vv), reinterpret_cast<RowVec*>(v + e0));
            __builtin_nontemporal_store(*reinterpret_cast<RowVec*>(wv), reinterpret_cast<RowVec*>(var + e0));
        } else {
            m[e0] = mv[0];
            v[e0] = vv[0];
            var[e0] = wv[0];
        }
    }
}

// Sgd: var[idx] += -lr * (g + wd * var[idx]) with an atomic add (sgd_kernel.h:83-95,169-184).
__global__ __launch_bounds__(kBlock) void k_sgd(const float* __restrict__ grad, const int32_t* __restrict__ indices,
                                                int64_t n, int dim, float* __restrict__ var, float neLr,
                                                float weightDecay)
{
    const int64_t total = n * dim;
    const int64_t g0 = (int64_t)blockIdx.x * (kBlock * kItems);
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        int64_t g = g0 + k * kBlock + threadIdx.x;
        if (g >= total) {
            continue;
        }
        int64_t i = g / dim;
        int c = (int)(g - i * dim);
        int64_t idx = indices[i];
        if (idx < 0) {
            continue;
        }
        float t = grad[g];
        float* dst = var + idx * dim + c;
        if (weightDecay != 0.0f) {
            t = t + weightDecay * (*dst);
        }
        unsafeAtomicAdd(dst, neLr * t);
    }
}

}  // namespace recsdk

using namespace recsdk;

static int elem_bytes(int dtype)
{
    switch (dtype) {
        case RECSDK_DT_F32:
        case RECSDK_DT_I32:
            return 4;
        case RECSDK_DT_F16:
        case RECSDK_DT_BF16:
            return 2;
        default:
            return 0;
    }
}

extern "C" int recsdk_lookup_by_addr(const int64_t* d_address, int64_t n, int32_t dim, int32_t dtype, void* d_y,
                                     void* stream)
{
    const int eb = elem_bytes(dtype);
    RECSDK_REQUIRE(eb != 0, RECSDK_EINVAL, "recsdk_lookup_by_addr: unknown dtype");
    RECSDK_REQUIRE(n >= 0 && dim > 0, RECSDK_EINVAL, "recsdk_lookup_by_addr: n must be >= 0 and dim > 0");
    if (n == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_address != nullptr && d_y != nullptr, RECSDK_ENULL, "recsdk_lookup_by_addr: NULL argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int rowBytes = dim * eb;
    const uintptr_t ya = reinterpret_cast<uintptr_t>(d_y);
    char* y = static_cast<char*>(d_y);
    auto launch = [&](auto chTag) -> int {
        constexpr int CH = decltype(chTag)::value;
        const int cpr = rowBytes / CH;
        const unsigned grid = (unsigned)cdiv(n * cpr, kBlock * kItems);
        RECSDK_LAUNCH(k_lookup_by_addr<CH>, dim3(grid), dim3(kBlock), s, d_address, n, rowBytes, cpr, y);
        return RECSDK_OK;
    };
    if (rowBytes % 16 == 0 && ya % 16 == 0) {
        return launch(std::integral_constant<int, 16>{});
    } else if (rowBytes % 8 == 0 && ya % 8 == 0) {
        return launch(std::integral_constant<int, 8>{});
    } else if (rowBytes % 4 == 0 && ya % 4 == 0) {
        return launch(std::integral_constant<int, 4>{});
    }
    return launch(std::integral_constant<int, 2>{});
}

extern "C" int recsdk_update_by_addr(const int64_t* d_address, int64_t n, int32_t dim, int32_t dtype,
                                     const void* d_embedding, int32_t update_type, void* stream)
{
    RECSDK_REQUIRE(elem_bytes(dtype) != 0, RECSDK_EINVAL, "recsdk_update_by_addr: unknown dtype");
    RECSDK_REQUIRE(n >= 0 && dim > 0, RECSDK_EINVAL, "recsdk_update_by_addr: n must be >= 0 and dim > 0");
    RECSDK_REQUIRE(update_type == 0 || update_type == 1, RECSDK_EINVAL, "recsdk_update_by_addr: update_type must be 0 or 1");
    if (n == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_address != nullptr && d_embedding != nullptr, RECSDK_ENULL, "recsdk_update_by_addr: NULL argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    constexpr int EPT = 4;
    const int gpr = (dim + EPT - 1) / EPT;
    const unsigned grid = (unsigned)cdiv(n * gpr, kBlock * kItems);
    // Atomic adds of 32-bit elements go one element per lane: the 64 atomics of a wave instruction then fall into 256
    // contiguous bytes (two lines) instead of one per 16 bytes over 1 KiB, which the L2 atomic units take 3.5 x faster.
    const unsigned grid1 = (unsigned)cdiv(n * (int64_t)dim, kBlock * kItems);
    switch (dtype) {
        case RECSDK_DT_F32:
            if (update_type == 0) {
                RECSDK_LAUNCH((k_update_by_addr<float, 1>), dim3(grid1), dim3(kBlock), s, d_address, n, dim, dim,
                              static_cast<const float*>(d_embedding), update_type);
            } else {
                RECSDK_LAUNCH((k_update_by_addr<float, EPT>), dim3(grid), dim3(kBlock), s, d_address, n, dim, gpr,
                              static_cast<const float*>(d_embedding), update_type);
            }
            break;
        case RECSDK_DT_I32:
            if (update_type == 0) {
                RECSDK_LAUNCH((k_update_by_addr<int32_t, 1>), dim3(grid1), dim3(kBlock), s, d_address, n, dim, dim,
                              static_cast<const int32_t*>(d_embedding), update_type);
            } else {
                RECSDK_LAUNCH((k_update_by_addr<int32_t, EPT>), dim3(grid), dim3(kBlock), s, d_address, n, dim, gpr,
                              static_cast<const int32_t*>(d_embedding), update_type);
            }
            break;
        case RECSDK_DT_F16:
            RECSDK_LAUNCH((k_update_by_addr<__half, EPT>), dim3(grid), dim3(kBlock), s, d_address, n, dim, gpr,
                               static_cast<const __half*>(d_embedding), update_type);
            break;
        default:
            RECSDK_LAUNCH((k_update_by_addr<__hip_bfloat16, EPT>), dim3(grid), dim3(kBlock), s, d_address, n,
                               dim, gpr, static_cast<const __hip_bfloat16*>(d_embedding), update_type);
            break;
    }
    RECSDK_LAUNCH_CHECK();
    return RECSDK_OK;
}

extern "C" int recsdk_lazy_adam(const float* d_grad, const int32_t* d_indices, int64_t n, int32_t dim, float* d_m,
                                float* d_v, float* d_var, float lr, float beta1, float beta2, float epsilon,
                                void* stream)
{
    RECSDK_REQUIRE(n >= 0 && dim > 0, RECSDK_EINVAL, "recsdk_lazy_adam: n must be >= 0 and dim > 0");
    if (n == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_grad && d_indices && d_m && d_v && d_var, RECSDK_ENULL, "recsdk_lazy_adam: NULL argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) % 16) == 0; };
    if (dim % 4 == 0 && al16(d_grad) && al16(d_m) && al16(d_v) && al16(d_var)) {
        const int cpr = dim / 4;
        const unsigned grid = (unsigned)cdiv(n * cpr, kBlock * kItems);
        RECSDK_LAUNCH(k_lazy_adam<4>, dim3(grid), dim3(kBlock), s, d_grad, d_indices, n, dim, cpr, d_m, d_v,
                           d_var, lr, beta1, beta2, epsilon);
    } else {
        const unsigned grid = (unsigned)cdiv(n * dim, kBlock * kItems);
        RECSDK_LAUNCH(k_lazy_adam<1>, dim3(grid), dim3(kBlock), s, d_grad, d_indices, n, dim, dim, d_m, d_v,
                           d_var, lr, beta1, beta2, epsilon);
    }
    RECSDK_LAUNCH_CHECK();
    return RECSDK_OK;
}

extern "C" int recsdk_sgd(const float* d_grad, const int32_t* d_indices, int64_t n, int32_t dim, float* d_var,
                          float lr, float weight_decay, void* stream)
{
    RECSDK_REQUIRE(n >= 0 && dim > 0, RECSDK_EINVAL, "recsdk_sgd: n must be >= 0 and dim > 0");
    if (n == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_grad && d_indices && d_var, RECSDK_ENULL, "recsdk_sgd: NULL argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned grid = (unsigned)cdiv(n * dim, kBlock * kItems);
    RECSDK_LAUNCH(k_sgd, dim3(grid), dim3(kBlock), s, d_grad, d_indices, n, dim, d_var, -lr, weight_decay);
    RECSDK_LAUNCH_CHECK();
    return RECSDK_OK;
}
