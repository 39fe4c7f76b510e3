// Row gather by (distinct key -> slot) and the fused "segment-reduce gradients + sparse optimizer" update.
//
// Gradient sums are formed in ascending lookup order, exactly as a sequential scatter-add would, so the
// result does not depend on scheduling:
//   - keys seen up to kListMax times: one wave per key sorts the key's (unordered) position list in
//     registers and adds the rows in order, up to 8 row loads in flight;
//   - keys seen more often: one block per (key, 32-column slice) streams the rows of the ordered position
//     list through a double-buffered LDS tile; one thread per column adds them in order.
// This file is compiled with -ffp-contract=off: the update formulas round like their scalar definition.
#include <algorithm>
#include <vector>

#include "common.h"
#include "dedup.h"

namespace recsdk {

struct RowsDesc {
    float* w;
    float* s1;
    float* s2;
    int64_t stride;
};

struct OptParams {
    int optim;
    float lr;
    float beta1;
    float beta2;
    float eps;
    float weightDecay;
};

template <int VEC>
struct VecT;
template <>
struct VecT<1> {
    using type = float;
};
template <>
struct VecT<2> {
    using type = float2;
};
template <>
struct VecT<4> {
    using type = float4;
};

template <int VEC>
__device__ __forceinline__ void vec_load(float (&dst)[VEC], const float* p)
{
    using V = typename VecT<VEC>::type;
    V v = *reinterpret_cast<const V*>(p);
    const float* f = reinterpret_cast<const float*>(&v);
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        dst[k] = f[k];
    }
}

template <int VEC>
__device__ __forceinline__ void vec_store(float* p, const float (&src)[VEC])
{
    using V = typename VecT<VEC>::type;
    V v;
    float* f = reinterpret_cast<float*>(&v);
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        f[k] = src[k];
    }
    *reinterpret_cast<V*>(p) = v;
}

// One element of the fused row update.  g is the summed gradient.
__device__ __forceinline__ void opt_update(const OptParams& p, float g, float& w, float& s1, float& s2)
{
    if (p.optim == RECSDK_OPT_ADAM) {
        // lazy_adam.cpp:168-185
        float mn = s1 * p.beta1 + g * (1.0f - p.beta1);
        float vn = s2 * p.beta2 + (g * g) * (1.0f - p.beta2);
        float den = sqrtf(fabsf(vn)) + p.eps;
        float upd = (mn * -p.lr) / den;
        s1 = mn;
        s2 = vn;
        w = upd + w;
    } else if (p.optim == RECSDK_OPT_ADAGRAD) {
        // adagrad_by_addr.py:101-125
        float st = s1 + g * g;
        float den = sqrtf(st + p.eps);
        float nd = (-p.lr * g) / den;
        s1 = st;
        w = w + nd;
    } else {
        // gradient_descent_by_addr.py:86-109
        float t = g;
        if (p.weightDecay != 0.0f) {
            t = t + p.weightDecay * w;
        }
        w = w + (-(t * p.lr));
    }
}

// ---- gather -------------------------------------------------------------------------------------
// One thread per VEC-wide chunk of an output row; consecutive threads cover consecutive chunks of a row.
template <int VEC>
__global__ __launch_bounds__(kBlock) void k_gather_unique(const RowsDesc* __restrict__ rows,
                                                          const int64_t* __restrict__ off, int T,
                                                          const int32_t* __restrict__ grank,
                                                          const int64_t* __restrict__ slots, float* __restrict__ out,
                                                          int dim, int chunksPerRow)
{
    __shared__ int sT0;
    const int64_t n = off[T];
    const int64_t totalChunks = n * chunksPerRow;
    const int64_t g0 = (int64_t)blockIdx.x * (kBlock * kItems);
    if (g0 >= totalChunks) {
        return;
    }
    if (threadIdx.x == 0) {
        sT0 = find_segment(off, T, g0 / chunksPerRow);
    }
    __syncthreads();
    int t = sT0;
    float vals[kItems][VEC];
    int64_t dstIdx[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        int64_t g = g0 + k * kBlock + threadIdx.x;
        dstIdx[k] = -1;
        if (g < totalChunks) {
            int64_t i = g / chunksPerRow;
            int c = (int)(g - i * chunksPerRow);
            t = advance_segment(off, t, i);
            int32_t R = grank[i];
            int64_t slot = (R >= 0) ? slots[R] : -1;
            dstIdx[k] = i * dim + (int64_t)c * VEC;
            if (slot >= 0) {
                const RowsDesc rd = rows[t];
                vec_load<VEC>(vals[k], rd.w + slot * rd.stride + (int64_t)c * VEC);
            } else {
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    vals[k][v] = 0.0f;
                }
            }
        }
    }
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (dstIdx[k] >= 0) {
            vec_store<VEC>(out + dstIdx[k], vals[k]);
        }
    }
}

// ---- short segments: one wave per distinct key ---------------------------------------------------
template <int VEC, int NJ>
__global__ __launch_bounds__(kBlock) void k_apply_short(const RowsDesc* __restrict__ rows,
                                                        const int64_t* __restrict__ uoff, int T,
                                                        const int64_t* __restrict__ total,
                                                        const uint32_t* __restrict__ ucount,
                                                        const uint32_t* __restrict__ useg,
                                                        const int32_t* __restrict__ posList,
                                                        const int64_t* __restrict__ slots,
                                                        const float* __restrict__ grad, int dim, OptParams prm)
{
    const int64_t U = total[0];
    const int64_t R = (int64_t)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);
    if (R >= U) {
        return;
    }
    const uint32_t c = ucount[R];
    if (c > (uint32_t)kListMax) {
        return;
    }
    const int64_t slot = slots[R];
    if (slot < 0) {
        return;
    }
    const int lane = lane_id();
    int32_t p = (lane < (int)c) ? posList[useg[R] + lane] : 0x7fffffff;
    if (c > 1) {
        // rank of every position among the key's positions, then permute into ascending order
        int rank = 0;
        for (uint32_t j = 0; j < c; ++j) {
            int32_t pj = __builtin_amdgcn_readlane(p, __builtin_amdgcn_readfirstlane(j));
            rank += (pj < p) ? 1 : 0;
        }
        if (lane >= (int)c) {
            rank = lane;
        }
        p = __builtin_amdgcn_ds_permute(rank << 2, p);
    }
    float acc[NJ][VEC];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            acc[j][v] = 0.0f;
        }
    }
    constexpr int kDepth = (NJ == 1) ? 8 : 4;
    for (uint32_t r = 0; r < c; r += kDepth) {
        float buf[kDepth][NJ][VEC];
#pragma unroll
        for (int k = 0; k < kDepth; ++k) {
            if (r + k < c) {
                int32_t pos = __builtin_amdgcn_readlane(p, __builtin_amdgcn_readfirstlane(r + k));
                const float* src = grad + (int64_t)pos * dim;
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    int e = (j * kWave + lane) * VEC;
                    if (e < dim) {
                        vec_load<VEC>(buf[k][j], src + e);
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < kDepth; ++k) {
            if (r + k < c) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    int e = (j * kWave + lane) * VEC;
                    if (e < dim) {
#pragma unroll
                        for (int v = 0; v < VEC; ++v) {
                            acc[j][v] += buf[k][j][v];
                        }
                    }
                }
            }
        }
    }
    const int t = find_segment(uoff, T, R);
    const RowsDesc rd = rows[t];
    const int64_t rowOff = slot * rd.stride;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        int e = (j * kWave + lane) * VEC;
        if (e < dim) {
            float w[VEC];
            float s1[VEC];
            float s2[VEC];
            vec_load<VEC>(w, rd.w + rowOff + e);
            if (prm.optim != RECSDK_OPT_SGD) {
                vec_load<VEC>(s1, rd.s1 + rowOff + e);
            }
            if (prm.optim == RECSDK_OPT_ADAM) {
                vec_load<VEC>(s2, rd.s2 + rowOff + e);
            }
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                opt_update(prm, acc[j][v], w[v], s1[v], s2[v]);
            }
            vec_store<VEC>(rd.w + rowOff + e, w);
            if (prm.optim != RECSDK_OPT_SGD) {
                vec_store<VEC>(rd.s1 + rowOff + e, s1);
            }
            if (prm.optim == RECSDK_OPT_ADAM) {
                vec_store<VEC>(rd.s2 + rowOff + e, s2);
            }
        }
    }
}

// ---- long segments: one block per (key, 32-column slice) -----------------------------------------
constexpr int kSlice = 32;       // columns per slice (128 bytes)
constexpr int kLongRows = 256;   // rows per LDS tile

__global__ __launch_bounds__(kBlock) void k_apply_long(const RowsDesc* __restrict__ rows,
                                                       const int64_t* __restrict__ uoff, int T,
                                                       const int32_t* __restrict__ longList,
                                                       const uint32_t* __restrict__ nLongPtr,
                                                       const uint32_t* __restrict__ ucount,
                                                       const uint32_t* __restrict__ useg,
                                                       const int32_t* __restrict__ posList,
                                                       const int64_t* __restrict__ slots,
                                                       const float* __restrict__ grad, int dim, int slices,
                                                       OptParams prm)
{
    __shared__ float tile[2][kLongRows][kSlice];
    const uint32_t nLong = nLongPtr[0];
    const int64_t items = (int64_t)nLong * slices;
    const int col4 = threadIdx.x & 7;   // float4 column inside the slice
    const int row0 = threadIdx.x >> 3;  // 0..31
    for (int64_t item = blockIdx.x; item < items; item += gridDim.x) {
        const int32_t R = longList[item / slices];
        const int slice = (int)(item % slices);
        const int64_t slot = slots[R];
        if (slot < 0) {
            continue;
        }
        const uint32_t c = ucount[R];
        const int32_t* list = posList + useg[R];
        const int colBase = slice * kSlice;
        const bool colOk = (colBase + col4 * 4) < dim;
        const uint32_t nb = (c + kLongRows - 1) / kLongRows;
        float4 regs[kLongRows / 32];
        auto issue = [&](uint32_t b) {
#pragma unroll
            for (int j = 0; j < kLongRows / 32; ++j) {
                uint32_t r = b * kLongRows + row0 + 32 * j;
                regs[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (r < c && colOk) {
                    int32_t pos = list[r];
                    regs[j] = *reinterpret_cast<const float4*>(grad + (int64_t)pos * dim + colBase + col4 * 4);
                }
            }
        };
        auto stash = [&](int bufIdx) {
#pragma unroll
            for (int j = 0; j < kLongRows / 32; ++j) {
                *reinterpret_cast<float4*>(&tile[bufIdx][row0 + 32 * j][col4 * 4]) = regs[j];
            }
        };
        float acc = 0.0f;
        issue(0);
        stash(0);
        __syncthreads();
        for (uint32_t b = 0; b < nb; ++b) {
            const int cur = b & 1;
            if (b + 1 < nb) {
                issue(b + 1);
            }
            if (threadIdx.x < kSlice) {
                uint32_t rowsHere = min((uint32_t)kLongRows, c - b * kLongRows);
                for (uint32_t r = 0; r < rowsHere; ++r) {
                    acc += tile[cur][r][threadIdx.x];
                }
            }
            if (b + 1 < nb) {
                stash(cur ^ 1);
            }
            __syncthreads();
        }
        if (threadIdx.x < kSlice && colBase + (int)threadIdx.x < dim) {
            const int t = find_segment(uoff, T, (int64_t)R);
            const RowsDesc rd = rows[t];
            const int64_t e = slot * rd.stride + colBase + threadIdx.x;
            float w = rd.w[e];
            float s1 = 0.0f;
            float s2 = 0.0f;
            if (prm.optim != RECSDK_OPT_SGD) {
                s1 = rd.s1[e];
            }
            if (prm.optim == RECSDK_OPT_ADAM) {
                s2 = rd.s2[e];
            }
            opt_update(prm, acc, w, s1, s2);
            rd.w[e] = w;
            if (prm.optim != RECSDK_OPT_SGD) {
                rd.s1[e] = s1;
            }
            if (prm.optim == RECSDK_OPT_ADAM) {
                rd.s2[e] = s2;
            }
        }
        __syncthreads();
    }
}

}  // namespace recsdk

using namespace recsdk;

struct recsdk_rows {
    int32_t T = 0;
    int32_t dim = 0;
    RowsDesc* descs = nullptr;  // device
    std::vector<RowsDesc> host;
};

extern "C" int recsdk_rows_create(int32_t T, int32_t dim, float* const* h_w, float* const* h_s1, float* const* h_s2,
                                  const int64_t* h_stride, recsdk_rows_t** out)
{
    RECSDK_REQUIRE(out != nullptr && h_w != nullptr && h_stride != nullptr, RECSDK_ENULL,
                   "recsdk_rows_create: NULL argument");
    RECSDK_REQUIRE(T > 0 && dim > 0, RECSDK_EINVAL, "recsdk_rows_create: T and dim must be positive");
    auto* r = new recsdk_rows();
    r->T = T;
    r->dim = dim;
    r->host.resize(T);
    for (int t = 0; t < T; ++t) {
        r->host[t].w = h_w[t];
        r->host[t].s1 = h_s1 ? h_s1[t] : nullptr;
        r->host[t].s2 = h_s2 ? h_s2[t] : nullptr;
        r->host[t].stride = h_stride[t];
    }
    if (hipMalloc(reinterpret_cast<void**>(&r->descs), sizeof(RowsDesc) * T) != hipSuccess ||
        hipMemcpy(r->descs, r->host.data(), sizeof(RowsDesc) * T, hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        if (r->descs) {
            (void)hipFree(r->descs);
        }
        delete r;
        set_error("recsdk_rows_create: hipMalloc/hipMemcpy failed");
        return RECSDK_ENOMEM;
    }
    *out = r;
    return RECSDK_OK;
}

extern "C" int recsdk_rows_destroy(recsdk_rows_t* rows)
{
    if (rows == nullptr) {
        return RECSDK_OK;
    }
    (void)hipFree(rows->descs);
    delete rows;
    return RECSDK_OK;
}

static bool rows_aligned(const recsdk_rows* rows, int vec, bool needS1, bool needS2)
{
    for (const RowsDesc& d : rows->host) {
        if ((reinterpret_cast<uintptr_t>(d.w) % (4 * vec)) != 0 || (d.stride % vec) != 0) {
            return false;
        }
        if (needS1 && (d.s1 == nullptr || (reinterpret_cast<uintptr_t>(d.s1) % (4 * vec)) != 0)) {
            return false;
        }
        if (needS2 && (d.s2 == nullptr || (reinterpret_cast<uintptr_t>(d.s2) % (4 * vec)) != 0)) {
            return false;
        }
    }
    return true;
}

extern "C" int recsdk_gather_unique(recsdk_rows_t* rows, recsdk_unique_t* u, const int64_t* d_slots, float* d_out,
                                    void* stream)
{
    RECSDK_REQUIRE(rows != nullptr && u != nullptr && d_slots != nullptr && d_out != nullptr, RECSDK_ENULL,
                   "recsdk_gather_unique: NULL argument");
    const UniqueView* v = recsdk_unique_view(u);
    RECSDK_REQUIRE(v->T == rows->T, RECSDK_EINVAL, "recsdk_gather_unique: table count of rows and unique differ");
    if (v->n == 0) {
        return RECSDK_OK;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int dim = rows->dim;
    const bool out16 = (reinterpret_cast<uintptr_t>(d_out) % 16) == 0;
    if (dim % 4 == 0 && out16 && rows_aligned(rows, 4, false, false)) {
        const int cpr = dim / 4;
        const unsigned grid = (unsigned)cdiv(v->n * cpr, kBlock * kItems);
        RECSDK_LAUNCH(k_gather_unique<4>, dim3(grid), dim3(kBlock), s, rows->descs, v->off, v->T, v->grank,
                           d_slots, d_out, dim, cpr);
    } else {
        const unsigned grid = (unsigned)cdiv(v->n * dim, kBlock * kItems);
        RECSDK_LAUNCH(k_gather_unique<1>, dim3(grid), dim3(kBlock), s, rows->descs, v->off, v->T, v->grank,
                           d_slots, d_out, dim, dim);
    }
    RECSDK_LAUNCH_CHECK();
    return RECSDK_OK;
}

template <int VEC, int NJ>
static int launch_short(const recsdk_rows* rows, const UniqueView* v, const int64_t* d_slots, const float* d_grad,
                         const OptParams& prm, hipStream_t s)
{
    const unsigned grid = (unsigned)cdiv(v->n, kBlock / kWave);
    RECSDK_LAUNCH((k_apply_short<VEC, NJ>), dim3(grid), dim3(kBlock), s, rows->descs, v->uoff, v->T, v->total,
                       v->ucount, v->useg, v->posList, d_slots, d_grad, rows->dim, prm);
    return RECSDK_OK;
}

extern "C" int recsdk_sparse_apply(recsdk_rows_t* rows, recsdk_unique_t* u, const int64_t* d_slots,
                                   const float* d_grad, int32_t optim, float lr, float beta1, float beta2, float eps,
                                   float weight_decay, void* stream)
{
    RECSDK_REQUIRE(rows != nullptr && u != nullptr && d_slots != nullptr && d_grad != nullptr, RECSDK_ENULL,
                   "recsdk_sparse_apply: NULL argument");
    RECSDK_REQUIRE(optim == RECSDK_OPT_SGD || optim == RECSDK_OPT_ADAGRAD || optim == RECSDK_OPT_ADAM, RECSDK_EINVAL,
                   "recsdk_sparse_apply: unknown optimizer");
    const UniqueView* v = recsdk_unique_view(u);
    RECSDK_REQUIRE(v->T == rows->T, RECSDK_EINVAL, "recsdk_sparse_apply: table count of rows and unique differ");
    RECSDK_REQUIRE(v->hasLists, RECSDK_EINVAL,
                   "recsdk_sparse_apply: the unique run carried input counts, no position lists were built");
    const int dim = rows->dim;
    RECSDK_REQUIRE(dim % 4 == 0 && dim <= 1024, RECSDK_EINVAL,
                   "recsdk_sparse_apply: dim must be a multiple of 4 and at most 1024");
    RECSDK_REQUIRE((reinterpret_cast<uintptr_t>(d_grad) % 16) == 0, RECSDK_EINVAL,
                   "recsdk_sparse_apply: d_grad must be 16-byte aligned");
    RECSDK_REQUIRE(rows_aligned(rows, 4, optim != RECSDK_OPT_SGD, optim == RECSDK_OPT_ADAM), RECSDK_EINVAL,
                   "recsdk_sparse_apply: row pointers must be 16-byte aligned, strides multiples of 4, and the "
                   "optimizer's state pointers present");
    if (v->n == 0) {
        return RECSDK_OK;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    OptParams prm{optim, lr, beta1, beta2, eps, weight_decay};
    // long segments first: they are the longest-running blocks
    if (v->n > kListMax) {
        const int slices = (dim + kSlice - 1) / kSlice;
        const unsigned grid = (unsigned)std::min<int64_t>((v->n / kListMax + 1) * slices, 8192);
        RECSDK_LAUNCH(k_apply_long, dim3(grid), dim3(kBlock), s, rows->descs, v->uoff, v->T, v->longList,
                           v->nLong, v->ucount, v->useg, v->posList, d_slots, d_grad, dim, slices, prm);
        RECSDK_LAUNCH_CHECK();
    }
    if (dim >= 256) {
        if (dim <= 256) {
            return launch_short<4, 1>(rows, v, d_slots, d_grad, prm, s);
        } else if (dim <= 512) {
            return launch_short<4, 2>(rows, v, d_slots, d_grad, prm, s);
        } else {
            return launch_short<4, 4>(rows, v, d_slots, d_grad, prm, s);
        }
    } else if (dim >= 128) {
        if (dim == 128) {
            return launch_short<2, 1>(rows, v, d_slots, d_grad, prm, s);
        } else {
            return launch_short<2, 2>(rows, v, d_slots, d_grad, prm, s);
        }
    } else if (dim > 64) {
        return launch_short<1, 2>(rows, v, d_slots, d_grad, prm, s);
    } else {
        return launch_short<1, 1>(rows, v, d_slots, d_grad, prm, s);
    }
    RECSDK_LAUNCH_CHECK();
    return RECSDK_OK;
}
