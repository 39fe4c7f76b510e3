// Row gather by (distinct key -> slot) and the fused "segment-reduce gradients + sparse optimizer" update.
//
// Gradient sums are formed in ascending lookup order, exactly as a sequential scatter-add would, so the
// result does not depend on scheduling:
//   - keys seen up to kListMax times: a group of lanes per key walks the key's ascending position list and adds
//     the rows in order, several row loads in flight;
//   - keys seen more often: one wave per (key, 32-column slice) streams the rows of the list through a
//     wave-private LDS tile, 64 rows per batch; one lane per column adds them in order.
// This file is compiled with -ffp-contract=off: the update formulas round like their scalar definition.
#include <stdlib.h>

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
// The descriptors of the tables a block touches are staged in LDS, row/chunk indices use 32-bit arithmetic
// relative to the block's first chunk, and the per-lookup rows leave through streaming stores.
constexpr int kDescCache = 32;

template <int VEC>
__global__ __launch_bounds__(kBlock) void k_gather_unique(const RowsDesc* __restrict__ rows,
                                                          const int64_t* __restrict__ off, int T,
                                                          const int32_t* __restrict__ grank,
                                                          const int64_t* __restrict__ slots, float* __restrict__ out,
                                                          int dim, int chunksPerRow)
{
    __shared__ int sT0;
    __shared__ const float* sW[kDescCache];
    __shared__ int64_t sStride[kDescCache];
    const int64_t n = off[T];
    const int64_t totalChunks = n * chunksPerRow;
    const int64_t g0 = (int64_t)blockIdx.x * (kBlock * kItems);
    if (g0 >= totalChunks) {
        return;
    }
    const int64_t i0 = g0 / chunksPerRow;
    const uint32_t r0 = (uint32_t)(g0 - i0 * chunksPerRow);
    if (threadIdx.x == 0) {
        sT0 = find_segment(off, T, i0);
    }
    __syncthreads();
    const int tBase = sT0;
    if (threadIdx.x < kDescCache && tBase + (int)threadIdx.x < T) {
        sW[threadIdx.x] = rows[tBase + threadIdx.x].w;
        sStride[threadIdx.x] = rows[tBase + threadIdx.x].stride;
    }
    __syncthreads();
    int t = tBase;
    float vals[kItems][VEC];
    int64_t dstIdx[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        const uint32_t q = r0 + (uint32_t)(k * kBlock + threadIdx.x);
        const uint32_t qi = q / (uint32_t)chunksPerRow;
        const int64_t i = i0 + qi;
        const int c = (int)(q - qi * (uint32_t)chunksPerRow);
        dstIdx[k] = -1;
        if (i < n) {
            t = advance_segment(off, t, i);
            int32_t R = grank[i];
            int64_t slot = (R >= 0) ? slots[R] : -1;
            dstIdx[k] = i * dim + (int64_t)c * VEC;
            if (slot >= 0) {
                const float* w;
                int64_t stride;
                if (t - tBase < kDescCache) {
                    w = sW[t - tBase];
                    stride = sStride[t - tBase];
                } else {
                    w = rows[t].w;
                    stride = rows[t].stride;
                }
                vec_load<VEC>(vals[k], w + slot * stride + (int64_t)c * VEC);
            } else {
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    vals[k][v] = 0.0f;
                }
            }
        }
    }
    // the per-lookup rows are written once and not read again by this library: streaming stores
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
        if (dstIdx[k] >= 0) {
            typedef float NtVec __attribute__((ext_vector_type(VEC)));
            NtVec v;
#pragma unroll
            for (int x = 0; x < VEC; ++x) {
                v[x] = vals[k][x];
            }
            __builtin_nontemporal_store(v, reinterpret_cast<NtVec*>(out + dstIdx[k]));
        }
    }
}

// ---- keys seen up to kListMax times: a group of G lanes per distinct key ------------------------------
// G = lanes per key (a power of two, 4 floats per lane and pass), NJ = passes over the row.  The key's position
// list is already in ascending order.  The row state (w, s1, s2) is requested before the gradient rows so that
// its latency overlaps theirs.
template <int G, int NJ>
__global__ __launch_bounds__(kBlock) void k_apply_short(const RowsDesc* __restrict__ rows,
                                                        const int64_t* __restrict__ uoff, int T,
                                                        const int64_t* __restrict__ total,
                                                        const uint32_t* __restrict__ ucount,
                                                        const uint32_t* __restrict__ useg,
                                                        const int32_t* __restrict__ posList,
                                                        const int64_t* __restrict__ slots,
                                                        const float* __restrict__ grad, int dim, OptParams prm)
{
    constexpr int kKeysPerBlock = kBlock / G;
    const int64_t U = total[0];
    const int64_t R = (int64_t)blockIdx.x * kKeysPerBlock + threadIdx.x / G;
    const int gl = threadIdx.x % G;
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
    const int32_t* list = posList + useg[R];
    const int t = find_segment(uoff, T, R);
    const RowsDesc rd = rows[t];
    const int64_t rowOff = slot * rd.stride;
    float w[NJ][4];
    float s1[NJ][4];
    float s2[NJ][4];
    float acc[NJ][4];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int e = (j * G + gl) * 4;
        if (e < dim) {
            vec_load<4>(w[j], rd.w + rowOff + e);
            if (prm.optim != RECSDK_OPT_SGD) {
                vec_load<4>(s1[j], rd.s1 + rowOff + e);
            }
            if (prm.optim == RECSDK_OPT_ADAM) {
                vec_load<4>(s2[j], rd.s2 + rowOff + e);
            }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            acc[j][v] = 0.0f;
        }
    }
    constexpr int kDepth = (NJ == 1) ? 4 : 2;
    for (uint32_t r = 0; r < c; r += kDepth) {
        float buf[kDepth][NJ][4];
#pragma unroll
        for (int k = 0; k < kDepth; ++k) {
            if (r + k < c) {
                const float* src = grad + (int64_t)list[r + k] * dim;
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const int e = (j * G + gl) * 4;
                    if (e < dim) {
                        vec_load<4>(buf[k][j], src + e);
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < kDepth; ++k) {
            if (r + k < c) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    if ((j * G + gl) * 4 < dim) {
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            acc[j][v] += buf[k][j][v];
                        }
                    }
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int e = (j * G + gl) * 4;
        if (e < dim) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                opt_update(prm, acc[j][v], w[j][v], s1[j][v], s2[j][v]);
            }
            vec_store<4>(rd.w + rowOff + e, w[j]);
            if (prm.optim != RECSDK_OPT_SGD) {
                vec_store<4>(rd.s1 + rowOff + e, s1[j]);
            }
            if (prm.optim == RECSDK_OPT_ADAM) {
                vec_store<4>(rd.s2 + rowOff + e, s2[j]);
            }
        }
    }
}

// ---- keys seen more than kListMax times: one wave per (key, column slice) ------------------------------
// A slice is SLICE columns wide (SLICE/4 lanes x 16 bytes per row), so one load instruction fetches 256/SLICE rows
// and a batch of 8 instructions 2048/SLICE rows; kPipe batches are in flight per wave, their list positions one
// round further ahead.  A batch goes through a wave-private 8 KiB LDS tile so that one lane per column can add its
// values in list order.  Narrow slices put more rows of one key in flight (more waves per key, more rows per
// instruction), which is what bounds the keys seen thousands of times: their sum is one long dependent chain and
// the memory system shares its bandwidth evenly among the waves that have loads in flight.
constexpr int kPipe = 4;          // batches of rows in flight per wave
constexpr int kSub = 8;           // load instructions per batch
constexpr int kHugeCount = 1024;  // keys seen more often take the narrow slices

__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int SLICE>
struct LongGeom {
    static constexpr int kLpr = SLICE / 4;         // lanes per row
    static constexpr int kRpi = kWave / kLpr;      // rows per load instruction
    static constexpr int kBatch = kRpi * kSub;     // rows per batch
};

// One batch of the pipeline: the list positions of a batch and, later, its rows.
template <int SLICE>
struct LongStage {
    using G = LongGeom<SLICE>;
    int32_t pos[kSub];
    float4 row[kSub];

    __device__ __forceinline__ void load_pos(const int32_t* __restrict__ list, uint32_t c, uint32_t b, int sub)
    {
#pragma unroll
        for (int j = 0; j < kSub; ++j) {
            const uint32_t r = b * G::kBatch + j * G::kRpi + sub;
            pos[j] = list[r < c ? r : c - 1];
        }
    }

    __device__ __forceinline__ void issue_rows(const float* __restrict__ gcol, int dim)
    {
#pragma unroll
        for (int j = 0; j < kSub; ++j) {
            row[j] = *reinterpret_cast<const float4*>(gcol + (int64_t)pos[j] * dim);
        }
    }
};

// Consume batch b from stage st: rows -> LDS tile (rows past the end of the list as zeros), refill the stage with
// batch b + kPipe (and the positions of batch b + 2*kPipe), then add the tile's rows in order.  The body has no
// data-dependent branches: adding the zero rows leaves the sum unchanged, lanes beyond the slice compute a value
// nobody reads.
template <int SLICE>
__device__ __forceinline__ void long_step(LongStage<SLICE>& st, float (*tile)[SLICE], float& acc,
                                          const int32_t* __restrict__ list, const float* __restrict__ gcol, int dim,
                                          uint32_t c, uint32_t b, int lane, int sub, int col4)
{
    using G = LongGeom<SLICE>;
#pragma unroll
    for (int j = 0; j < kSub; ++j) {
        const bool live = b * G::kBatch + j * G::kRpi + sub < c;
        float4 v = st.row[j];
        v.x = live ? v.x : 0.0f;
        v.y = live ? v.y : 0.0f;
        v.z = live ? v.z : 0.0f;
        v.w = live ? v.w : 0.0f;
        *reinterpret_cast<float4*>(&tile[j * G::kRpi + sub][col4 * 4]) = v;
    }
    wave_lds_fence();
    __builtin_amdgcn_sched_barrier(0);
    st.issue_rows(gcol, dim);
    st.load_pos(list, c, b + 2 * kPipe, sub);
    __builtin_amdgcn_sched_barrier(0);
    const int col = lane & (SLICE - 1);
#pragma unroll 16
    for (int r = 0; r < G::kBatch; ++r) {
        acc += tile[r][col];
    }
    wave_lds_fence();
    __builtin_amdgcn_sched_barrier(0);
}

// HUGE = true: keys seen more than kHugeCount times; false: the other keys of the long list.
template <int SLICE, bool HUGE>
__global__ __launch_bounds__(kBlock, 2) void k_apply_long(const RowsDesc* __restrict__ rows,
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
    using G = LongGeom<SLICE>;
    __shared__ float tileAll[kBlock / kWave][G::kBatch][SLICE];
    float(*tile)[SLICE] = tileAll[threadIdx.x >> 6];
    const uint32_t nLong = nLongPtr[0];
    const int64_t items = (int64_t)nLong * slices;
    const int lane = lane_id();
    const int col4 = lane % G::kLpr;  // float4 column inside the slice
    const int sub = lane / G::kLpr;   // row inside the group of rows one instruction fetches
    const int64_t wavesTotal = (int64_t)gridDim.x * (kBlock / kWave);
    for (int64_t item = (int64_t)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6); item < items; item += wavesTotal) {
        const int32_t R = longList[item / slices];
        const int slice = (int)(item % slices);
        const uint32_t c = ucount[R];
        if ((c > (uint32_t)kHugeCount) != HUGE) {
            continue;
        }
        const int64_t slot = slots[R];
        if (slot < 0) {
            continue;
        }
        const int32_t* list = posList + useg[R];
        const int colBase = slice * SLICE;
        const bool colOk = (colBase + col4 * 4) < dim;
        const uint32_t nb = (c + G::kBatch - 1) / G::kBatch;
        // Loads are unconditional (indices clamped to the last list entry, columns to the row) so that the
        // compiler keeps them in straight-line code with exact wait counts; surplus rows are never added.
        const float* gcol = grad + (colOk ? colBase + col4 * 4 : 0);
        LongStage<SLICE> st0, st1, st2, st3;
        static_assert(kPipe == 4, "the stages below are written out for four batches in flight");
        // memory returns in issue order: the scheduling barriers keep the loads in the order the steps consume them
        st0.load_pos(list, c, 0, sub);
        st1.load_pos(list, c, 1, sub);
        st2.load_pos(list, c, 2, sub);
        st3.load_pos(list, c, 3, sub);
        __builtin_amdgcn_sched_barrier(0);
        st0.issue_rows(gcol, dim);
        st0.load_pos(list, c, 4, sub);
        __builtin_amdgcn_sched_barrier(0);
        st1.issue_rows(gcol, dim);
        st1.load_pos(list, c, 5, sub);
        __builtin_amdgcn_sched_barrier(0);
        st2.issue_rows(gcol, dim);
        st2.load_pos(list, c, 6, sub);
        __builtin_amdgcn_sched_barrier(0);
        st3.issue_rows(gcol, dim);
        st3.load_pos(list, c, 7, sub);
        __builtin_amdgcn_sched_barrier(0);
        float acc = 0.0f;
        for (uint32_t b0 = 0; b0 < nb; b0 += kPipe) {
            long_step<SLICE>(st0, tile, acc, list, gcol, dim, c, b0 + 0, lane, sub, col4);
            long_step<SLICE>(st1, tile, acc, list, gcol, dim, c, b0 + 1, lane, sub, col4);
            long_step<SLICE>(st2, tile, acc, list, gcol, dim, c, b0 + 2, lane, sub, col4);
            long_step<SLICE>(st3, tile, acc, list, gcol, dim, c, b0 + 3, lane, sub, col4);
        }
        if (lane < SLICE && colBase + lane < dim) {
            const int t = find_segment(uoff, T, (int64_t)R);
            const RowsDesc rd = rows[t];
            const int64_t e = slot * rd.stride + colBase + lane;
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
    }
}

}  // namespace recsdk

using namespace recsdk;

struct recsdk_rows {
    int32_t T = 0;
    int32_t dim = 0;
    RowsDesc* descs = nullptr;  // device
    std::vector<RowsDesc> host;
    // the two update kernels touch disjoint rows; the long-list one runs on a side stream next to the other
    hipStream_t side = nullptr;
    hipEvent_t evFork = nullptr;
    hipEvent_t evJoin = nullptr;
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
    if (hipStreamCreateWithFlags(&r->side, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&r->evFork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&r->evJoin, hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError();
        set_error("recsdk_rows_create: could not create the side stream");
        recsdk_rows_destroy(r);
        return RECSDK_EHIP;
    }
    *out = r;
    return RECSDK_OK;
}

extern "C" int recsdk_rows_destroy(recsdk_rows_t* rows)
{
    if (rows == nullptr) {
        return RECSDK_OK;
    }
    if (rows->evFork) {
        (void)hipEventDestroy(rows->evFork);
    }
    if (rows->evJoin) {
        (void)hipEventDestroy(rows->evJoin);
    }
    if (rows->side) {
        (void)hipStreamDestroy(rows->side);
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

template <int G, int NJ>
static int launch_short(const recsdk_rows* rows, const UniqueView* v, const int64_t* d_slots, const float* d_grad,
                        const OptParams& prm, hipStream_t s)
{
    const unsigned grid = (unsigned)cdiv(v->n, kBlock / G);
    RECSDK_LAUNCH((k_apply_short<G, NJ>), dim3(grid), dim3(kBlock), s, rows->descs, v->uoff, v->T, v->total,
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
    // keys with long position lists go to the side stream: fork after everything queued on `s` so far
    const bool haveLong = v->n > kListMax;
    // RECSDK_NO_SIDE_STREAM=1 keeps every kernel on the caller's stream (for per-kernel measurements)
    static const bool serial = (getenv("RECSDK_NO_SIDE_STREAM") != nullptr);
    if (haveLong) {
        hipStream_t side = serial ? s : rows->side;
        if (!serial) {
            RECSDK_HIP_TRY(hipEventRecord(rows->evFork, s));
            RECSDK_HIP_TRY(hipStreamWaitEvent(side, rows->evFork, 0));
        }
        const int kWavesPerBlock = kBlock / kWave;
        if (v->n > kHugeCount) {
            // the longest chains first, in narrow slices
            const int slices = (dim + 7) / 8;
            const unsigned grid = (unsigned)std::min<int64_t>(cdiv((v->n / kHugeCount + 1) * slices, kWavesPerBlock), 4096);
            RECSDK_LAUNCH((k_apply_long<8, true>), dim3(grid), dim3(kBlock), side, rows->descs, v->uoff, v->T, v->longList,
                          v->nLong, v->ucount, v->useg, v->posList, d_slots, d_grad, dim, slices, prm);
        }
        const int slices = (dim + 31) / 32;
        const unsigned grid = (unsigned)std::min<int64_t>(cdiv((v->n / kListMax + 1) * slices, kWavesPerBlock), 4096);
        RECSDK_LAUNCH((k_apply_long<32, false>), dim3(grid), dim3(kBlock), side, rows->descs, v->uoff, v->T, v->longList,
                      v->nLong, v->ucount, v->useg, v->posList, d_slots, d_grad, dim, slices, prm);
        if (!serial) {
            RECSDK_HIP_TRY(hipEventRecord(rows->evJoin, side));
        }
    }
    const int chunks = dim / 4;
    int rc;
    if (chunks <= 4) {
        rc = launch_short<4, 1>(rows, v, d_slots, d_grad, prm, s);
    } else if (chunks <= 8) {
        rc = launch_short<8, 1>(rows, v, d_slots, d_grad, prm, s);
    } else if (chunks <= 16) {
        rc = launch_short<16, 1>(rows, v, d_slots, d_grad, prm, s);
    } else if (chunks <= 32) {
        rc = launch_short<32, 1>(rows, v, d_slots, d_grad, prm, s);
    } else if (chunks <= 64) {
        rc = launch_short<64, 1>(rows, v, d_slots, d_grad, prm, s);
    } else if (chunks <= 128) {
        rc = launch_short<64, 2>(rows, v, d_slots, d_grad, prm, s);
    } else {
        rc = launch_short<64, 4>(rows, v, d_slots, d_grad, prm, s);
    }
    if (haveLong && !serial) {
        RECSDK_HIP_TRY(hipStreamWaitEvent(s, rows->evJoin, 0));
    }
    return rc;
}
