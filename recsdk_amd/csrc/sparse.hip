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

#include "apply.h"
#include "common.h"
#include "dedup.h"


namespace recsdk {

// Rows of the update kernels are touched once per step: gradient rows are read once, a key's weights and optimizer
// state are read and written once.  Non-temporal loads and stores keep them from displacing what the neighbouring
// kernels reuse in L2 (hot rows of the gather, hash tables) and leave no dirty lines behind for the next kernel to
// write back (short-list update 364 -> 345-356 us, gather 265 -> 254 us, step 1.147 -> 1.121 ms).
template <int VEC>
__device__ __forceinline__ void vec_load(float (&dst)[VEC], const float* p)
{
    typedef float NtV __attribute__((ext_vector_type(VEC)));
    const NtV v = __builtin_nontemporal_load(reinterpret_cast<const NtV*>(p));
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        dst[k] = v[k];
    }
}

// ordinary (cached) load, for rows that several list entries share
__device__ __forceinline__ void vec_load4_cached(float (&dst)[4], const float* p)
{
    const float4 v = *reinterpret_cast<const float4*>(p);
    dst[0] = v.x;
    dst[1] = v.y;
    dst[2] = v.z;
    dst[3] = v.w;
}

template <int VEC>
__device__ __forceinline__ void vec_store(float* p, const float (&src)[VEC])
{
    typedef float NtV __attribute__((ext_vector_type(VEC)));
    NtV v;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        v[k] = src[k];
    }
    __builtin_nontemporal_store(v, reinterpret_cast<NtV*>(p));
}

// bf16 <-> fp32 (round to nearest even on store)
__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((u >> 16) | 0x40);
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// four consecutive weights starting at element e of a table stored as WT (float or uint16_t = bf16)
template <typename WT>
__device__ __forceinline__ void w_load4(float (&dst)[4], const void* base, int64_t e);
template <>
__device__ __forceinline__ void w_load4<float>(float (&dst)[4], const void* base, int64_t e)
{
    vec_load<4>(dst, static_cast<const float*>(base) + e);
}
template <>
__device__ __forceinline__ void w_load4<uint16_t>(float (&dst)[4], const void* base, int64_t e)
{
    uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + e);
    dst[0] = bf16_to_f32((uint16_t)(raw.x & 0xffffu));
    dst[1] = bf16_to_f32((uint16_t)(raw.x >> 16));
    dst[2] = bf16_to_f32((uint16_t)(raw.y & 0xffffu));
    dst[3] = bf16_to_f32((uint16_t)(raw.y >> 16));
}
template <typename WT>
__device__ __forceinline__ void w_store4(void* base, int64_t e, const float (&src)[4]);
template <>
__device__ __forceinline__ void w_store4<float>(void* base, int64_t e, const float (&src)[4])
{
    vec_store<4>(static_cast<float*>(base) + e, src);
}
template <>
__device__ __forceinline__ void w_store4<uint16_t>(void* base, int64_t e, const float (&src)[4])
{
    uint2 raw;
    raw.x = (uint32_t)f32_to_bf16(src[0]) | ((uint32_t)f32_to_bf16(src[1]) << 16);
    raw.y = (uint32_t)f32_to_bf16(src[2]) | ((uint32_t)f32_to_bf16(src[3]) << 16);
    *reinterpret_cast<uint2*>(static_cast<uint16_t*>(base) + e) = raw;
}
template <typename WT>
__device__ __forceinline__ float w_load1(const void* base, int64_t e);
template <>
__device__ __forceinline__ float w_load1<float>(const void* base, int64_t e)
{
    return static_cast<const float*>(base)[e];
}
template <>
__device__ __forceinline__ float w_load1<uint16_t>(const void* base, int64_t e)
{
    return bf16_to_f32(static_cast<const uint16_t*>(base)[e]);
}
template <typename WT>
__device__ __forceinline__ void w_store1(void* base, int64_t e, float v);
template <>
__device__ __forceinline__ void w_store1<float>(void* base, int64_t e, float v)
{
    static_cast<float*>(base)[e] = v;
}
template <>
__device__ __forceinline__ void w_store1<uint16_t>(void* base, int64_t e, float v)
{
    static_cast<uint16_t*>(base)[e] = f32_to_bf16(v);
}

// The rate of this launch: the caller's value, or what its device word holds now.
__device__ __forceinline__ void opt_resolve_rate(OptParams& p)
{
    if (p.lrDev != nullptr) {
        p.lr = *p.lrDev;
    }
}

// One element of the fused row update.  g is the summed gradient.
__device__ __forceinline__ void opt_update(const OptParams& p, float g, float& w, float& s1, float& s2)
{
    switch (p.optim) {
        case kOptAdam: {
            // lazy_adam.cpp:168-185
            float mn = s1 * p.beta1 + g * (1.0f - p.beta1);
            float vn = s2 * p.beta2 + (g * g) * (1.0f - p.beta2);
            float den = sqrtf(fabsf(vn)) + p.eps;
            float upd = (mn * -p.lr) / den;
            s1 = mn;
            s2 = vn;
            w = upd + w;
            break;
        }
        case kOptAdagrad: {
            // adagrad_by_addr.py:101-125
            float st = s1 + g * g;
            float den = sqrtf(st + p.eps);
            float nd = (-p.lr * g) / den;
            s1 = st;
            w = w + nd;
            break;
        }
        case kOptSgd: {
            // gradient_descent_by_addr.py:86-109
            float t = g;
            if (p.weightDecay != 0.0f) {
                t = t + p.weightDecay * w;
            }
            w = w + (-(t * p.lr));
            break;
        }
        case kOptTbeAdam: {
            // backward_codegen_adam_unweighted_exact_kernel.h:128-166
            float m1 = s1 * p.beta1 + g * (1.0f - p.beta1);
            float m2 = s2 * p.beta2 + (g * g) * (1.0f - p.beta2);
            float delta = (m1 / (sqrtf(m2) + p.eps)) * p.stepSize;
            s1 = m1;
            s2 = m2;
            w = w + delta;
            break;
        }
        case kOptTbeAdagrad: {
            // backward_codegen_adagrad_unweighted_exact_kernel.h:108-139
            float m1 = s1 + g * g;
            float delta = -((p.lr / (sqrtf(m1) + p.eps)) * g);
            s1 = m1;
            w = w + delta;
            break;
        }
        case kOptStoreSum: {
            w = g;
            break;
        }
        default: {
            // backward_codegen_sgd_unweighted_exact_kernel.h: w += -lr * G
            w = w + g * p.stepSize;
            break;
        }
    }
}

__device__ __forceinline__ bool dev_uses_s1(int optim)
{
    return optim != kOptSgd && optim != kOptTbeSgd && optim != kOptStoreSum;
}
__device__ __forceinline__ bool dev_uses_s2(int optim) { return optim == kOptAdam || optim == kOptTbeAdam; }

// ---- forward gather in two steps: one row address per distinct key, then a pure row copy per lookup ---------
// rowPtr[R] = address of the row of the R-th distinct key (NULL when the key has no slot).  Resolving the table
// and the slot once per distinct key keeps the per-lookup kernel free of table searches and block-wide set-up.
__global__ __launch_bounds__(kBlock) void k_row_ptrs(const RowsDesc* __restrict__ rows,
                                                     const int64_t* __restrict__ uoff, int T,
                                                     const int64_t* __restrict__ total,
                                                     const int64_t* __restrict__ slots,
                                                     const float** __restrict__ rowPtr)
{
    const int64_t R = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (R >= total[0]) {
        return;
    }
    const int64_t slot = slots[R];
    const float* p = nullptr;
    if (slot >= 0) {
        const int t = find_segment(uoff, T, R);
        p = static_cast<const float*>(rows[t].w) + slot * rows[t].stride;
    }
    rowPtr[R] = p;
}

// out[i, :] = row of lookup i's key (zeros without a row); VEC floats per thread and item, kGatherItems items per
// thread, streaming stores.  A block first resolves the row addresses of the lookups it covers (one thread per
// lookup: inverse index -> row address) into LDS; the copy loop then issues nothing but row loads and stores.  With
// every lane chasing the two index loads itself the memory pipeline spent a third of its instruction slots on
// them (4.0 TB/s, now 4.65); a plain random-row copy reaches 5.5-5.9 TB/s on the same device.
// DIRECT (at most kGatherTables tables): the block keeps the tables' bases, strides and first ranks in LDS and turns
// a lookup's rank into its row address itself (rank -> slot, two dependent loads as with the address array), so no
// kernel has to write one address per distinct key first.
constexpr int kGatherTables = 64;
template <int VEC, int kGatherItems, bool NT, bool DIRECT>
__global__ __launch_bounds__(kBlock) void k_gather_rows(const float* const* __restrict__ rowPtr,
                                                        const RowsDesc* __restrict__ rows,
                                                        const int64_t* __restrict__ uoff, int T,
                                                        const int64_t* __restrict__ slots,
                                                        const int32_t* __restrict__ grank, float* __restrict__ out,
                                                        int64_t n, int dim, int chunksPerRow)
{
    typedef float NtVec __attribute__((ext_vector_type(VEC)));
    constexpr int kChunks = kBlock * kGatherItems;
    __shared__ const float* sPtr[kChunks + 2];  // at most one lookup per chunk, plus the two partial rows
    __shared__ const float* sBase[DIRECT ? kGatherTables : 1];
    __shared__ int64_t sStride[DIRECT ? kGatherTables : 1];
    __shared__ int32_t sFirst[DIRECT ? kGatherTables + 1 : 1];  // ranks fit 31 bits
    const int64_t totalChunks = n * chunksPerRow;
    const int64_t g0 = (int64_t)blockIdx.x * kChunks;
    const int64_t i0 = g0 / chunksPerRow;
    const uint32_t r0 = (uint32_t)(g0 - i0 * chunksPerRow);
    const int rowsHere = (int)((r0 + (uint32_t)kChunks + (uint32_t)chunksPerRow - 1) / (uint32_t)chunksPerRow);
    if (DIRECT) {
        // the threads past the lookups stage the tables while the first ones fetch their ranks
        int32_t R = -1;
        int64_t slot = -1;
        if ((int)threadIdx.x < rowsHere && i0 + threadIdx.x < n) {
            R = grank[i0 + threadIdx.x];
            if (R >= 0) {
                slot = slots[R];
            }
        }
        const int tt = (int)threadIdx.x - (kBlock - kGatherTables - 1);
        if (tt >= 0 && tt <= T) {
            sFirst[tt] = (int32_t)uoff[tt];
            if (tt < T) {
                sBase[tt] = static_cast<const float*>(rows[tt].w);
                sStride[tt] = rows[tt].stride;
            }
        }
        __syncthreads();
        for (int j = threadIdx.x; j < rowsHere; j += kBlock) {
            if (j >= kBlock) {   // more lookups than threads (rows of fewer than kGatherItems pieces)
                R = -1;
                slot = -1;
                if (i0 + j < n) {
                    R = grank[i0 + j];
                    if (R >= 0) {
                        slot = slots[R];
                    }
                }
            }
            const float* p = nullptr;
            if (slot >= 0) {
                int lo = 0;
                int hi = T;   // sFirst[lo] <= R < sFirst[hi]
                while (hi - lo > 1) {
                    const int mid = (lo + hi) >> 1;
                    if (sFirst[mid] <= R) {
                        lo = mid;
                    } else {
                        hi = mid;
                    }
                }
                p = sBase[lo] + slot * sStride[lo];
            }
            sPtr[j] = p;
        }
    } else {
        for (int j = threadIdx.x; j < rowsHere; j += kBlock) {
            const int64_t i = i0 + j;
            const float* p = nullptr;
            if (i < n) {
                const int32_t R = grank[i];
                if (R >= 0) {
                    p = rowPtr[R];
                }
            }
            sPtr[j] = p;
        }
    }
    __syncthreads();
    NtVec vals[kGatherItems];
    int64_t dst[kGatherItems];
#pragma unroll
    for (int k = 0; k < kGatherItems; ++k) {
        const uint32_t q = r0 + (uint32_t)(k * kBlock + threadIdx.x);
        const uint32_t qi = q / (uint32_t)chunksPerRow;
        const int c = (int)(q - qi * (uint32_t)chunksPerRow);
        NtVec v;
#pragma unroll
        for (int x = 0; x < VEC; ++x) {
            v[x] = 0.0f;
        }
        dst[k] = -1;
        if (g0 + k * kBlock + threadIdx.x < totalChunks) {
            dst[k] = (i0 + qi) * dim + (int64_t)c * VEC;
            const float* p = sPtr[qi];
            if (p != nullptr) {
                v = *reinterpret_cast<const NtVec*>(p + c * VEC);
            }
        }
        vals[k] = v;
    }
#pragma unroll
    for (int k = 0; k < kGatherItems; ++k) {
        if (dst[k] >= 0) {
            if (NT) {
                __builtin_nontemporal_store(vals[k], reinterpret_cast<NtVec*>(out + dst[k]));
            } else {
                *reinterpret_cast<NtVec*>(out + dst[k]) = vals[k];
            }
        }
    }
}

// ---- small batches: one launch each -------------------------------------------------------------------------
// Forward gather of a small batch: every thread resolves the row of its lookup itself (rank -> table -> slot); the
// few kilobytes of index data sit in L1 / L2 after the first touch.
__global__ __launch_bounds__(kBlock) void k_gather_small(const RowsDesc* __restrict__ rows,
                                                         const int64_t* __restrict__ uoff, int T,
                                                         const int64_t* __restrict__ slots,
                                                         const int32_t* __restrict__ grank, float* __restrict__ out,
                                                         int64_t n, int dim)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;  // one float per thread: any dim, any alignment
    if (e >= n * dim) {
        return;
    }
    const int64_t i = e / dim;
    const int c = (int)(e - i * dim);
    const int32_t R = grank[i];
    float v = 0.0f;
    if (R >= 0) {
        const int64_t slot = slots[R];
        if (slot >= 0) {
            const int t = find_segment(uoff, T, (int64_t)R);
            v = static_cast<const float*>(rows[t].w)[slot * rows[t].stride + c];
        }
    }
    out[e] = v;
}

// Gradient reduce + optimizer of a small batch without position lists: G lanes per distinct key, 64 / G keys per
// wave, four waves per block.  The block first filters the inverse index: each wave reads a quarter of it, 512
// positions in flight at a time, and lists the positions that belong to one of the block's keys, in ascending order.
// Every wave then takes the positions of its own keys from the four lists in turn into a short per-key queue in
// LDS.  A full queue (and, at the end, what is left) is drained: its gradient rows are loaded four at a time and
// added in queue order, which is ascending position order, as the list-based kernels add them.  With n positions and
// U keys this reads U / (256 / G) * n index words instead of building lists with five more launches: at most a few
// thousand keys only.  (With every wave walking the whole index by itself, 64 rounds of a load, a ballot and a
// branch, the walk was two thirds of the kernel.)
constexpr int kSmallQueue = 16;

template <int G, int NJ, typename WT>
__global__ __launch_bounds__(kBlock) void k_apply_small(const RowsDesc* __restrict__ rows,
                                                        const int64_t* __restrict__ uoff, int T,
                                                        const int64_t* __restrict__ total,
                                                        const int32_t* __restrict__ grank, int64_t n,
                                                        const int64_t* __restrict__ slots, GradSrc gs, OptParams prm)
{
    opt_resolve_rate(prm);
    constexpr int kKeysPerWave = kWave / G;
    constexpr int kWaves = kBlock / kWave;
    __shared__ uint16_t sQueue[kWaves][kKeysPerWave][kSmallQueue];
    // positions that hold one of the block's keys, and which of its keys: wave q lists those of its part of the
    // inverse index, in ascending order
    constexpr int kPart = kSmallKeys / kWaves;
    constexpr int kBlockKeys = kWaves * kKeysPerWave;
    static_assert(kBlockKeys <= 256, "a key of the block is named by one byte");
    __shared__ uint16_t sHitPos[kWaves][kPart];
    __shared__ uint8_t sHitKey[kWaves][kPart];
    __shared__ int sHits[kWaves];
    const int64_t U = total[0];
    const int64_t Rb = (int64_t)blockIdx.x * kBlockKeys;
    if (Rb >= U) {
        return;
    }
    const int wave = threadIdx.x >> 6;
    const int lane = lane_id();
    const int myKey = lane / G;  // key of this lane inside its wave
    const int gl = lane % G;
    const int64_t R0 = ((int64_t)blockIdx.x * kWaves + wave) * kKeysPerWave;
    const int64_t R = R0 + myKey;
    const bool live = R < U;
    const int64_t slot = live ? slots[R] : -1;
    const bool useS1 = dev_uses_s1(prm.optim);
    const bool useS2 = dev_uses_s2(prm.optim);
    RowsDesc rd = rows[0];
    if (live && slot >= 0) {
        rd = rows[find_segment(uoff, T, R)];
    }
    const int dim = rd.dim;
    const int64_t rowOff = slot * rd.stride;
    const bool work = live && slot >= 0;
    float w[NJ][4];
    float s1[NJ][4];
    float s2[NJ][4];
    float acc[NJ][4];
    // A key seen more than kTwoLevelMin times is summed chunk by chunk (kChunkRows rows in order, then the chunk sums
    // in order).  How often a key is seen is known only at the end of the walk, so both sums are kept.
    float chk[NJ][4];
    float tot[NJ][4];
    int inChunk = 0;
    int seen = 0;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            chk[j][v] = 0.0f;
            tot[j][v] = 0.0f;
        }
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int e = (j * G + gl) * 4;
        if (work && e < dim) {
            w_load4<WT>(w[j], rd.w, rowOff + e);
            if (useS1) {
                vec_load<4>(s1[j], rd.s1 + rowOff + e);
            }
            if (useS2) {
                vec_load<4>(s2[j], rd.s2 + rowOff + e);
            }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            acc[j][v] = 0.0f;
        }
    }
    // the row loads above are in flight while the block filters the inverse index
    {
        // kAhead rounds of 64 positions are in flight together; what lies behind position n is masked
        constexpr int kAhead = 8;
        static_assert(kPart % (kAhead * kWave) == 0, "whole groups of rounds per part");
        const int last = (int)(n < (int64_t)(wave + 1) * kPart ? n : (int64_t)(wave + 1) * kPart);
        int found = 0;
        for (int c00 = wave * kPart; c00 < last; c00 += kAhead * kWave) {
            int32_t ahead[kAhead];
#pragma unroll
            for (int a = 0; a < kAhead; ++a) {
                const int p = c00 + a * kWave + lane;
                ahead[a] = grank[p < last ? p : last - 1];
            }
#pragma unroll
            for (int a = 0; a < kAhead; ++a) {
                const int p = c00 + a * kWave + lane;
                const uint32_t d = (uint32_t)(ahead[a] - (int)Rb);  // ranks of a small batch are below kSmallKeys
                const bool hit = p < last && ahead[a] >= 0 && d < (uint32_t)kBlockKeys;
                const unsigned long long mask = __ballot(hit);
                if (mask != 0) {
                    if (hit) {
                        const int at = found + __popcll(mask & ((1ull << lane) - 1ull));
                        sHitPos[wave][at] = (uint16_t)p;
                        sHitKey[wave][at] = (uint8_t)d;
                    }
                    found += __popcll(mask);
                }
            }
        }
        if (lane == 0) {
            sHits[wave] = found;
        }
    }
    __syncthreads();
    if (R0 >= U) {
        return;
    }
    const float* gbase = gs.base + rd.gradCol;
    uint16_t* queue = sQueue[wave][myKey];
    int queued = 0;  // the same in all lanes of a key
    // adds the queue's gradient rows in order, four loads in flight
    auto drain = [&]() {
        // the queue was written by the key's first lane: order those LDS writes before the reads of all its lanes
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        for (int q0 = 0; q0 < queued; q0 += 4) {
            float buf[4][NJ][4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (q0 + q < queued) {
                    const float* src = gbase + (int64_t)queue[q0 + q] * gs.stride;
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        const int e = (j * G + gl) * 4;
                        if (e < dim) {
                            vec_load<4>(buf[q][j], src + e);
                        }
                    }
                }
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (q0 + q < queued) {
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        if ((j * G + gl) * 4 < dim) {
#pragma unroll
                            for (int v = 0; v < 4; ++v) {
                                acc[j][v] += buf[q][j][v];
                                chk[j][v] += buf[q][j][v];
                            }
                        }
                    }
                    if (++inChunk == kChunkRows) {
#pragma unroll
                        for (int j = 0; j < NJ; ++j) {
#pragma unroll
                            for (int v = 0; v < 4; ++v) {
                                tot[j][v] += chk[j][v];
                                chk[j][v] = 0.0f;
                            }
                        }
                        inChunk = 0;
                    }
                }
            }
        }
        seen += queued;
        queued = 0;
    };
    // the wave's keys take their positions from the four lists in turn: ascending positions
    const int myFirst = wave * kKeysPerWave;  // the wave's first key inside the block
    for (int q = 0; q < kWaves; ++q) {
        const int cnt = sHits[q];
        for (int e0 = 0; e0 < cnt; e0 += kWave) {
            const int e = e0 + lane;
            const uint32_t d = e < cnt ? (uint32_t)((int)sHitKey[q][e] - myFirst) : 0xffffffffu;
            const int pos = e < cnt ? (int)sHitPos[q][e] : 0;
            unsigned long long hits = __ballot(d < (uint32_t)kKeysPerWave);
            while (hits != 0) {
                const int b = __ffsll((long long)hits) - 1;  // from a ballot: the same in every lane
                hits &= hits - 1;
                const int k = __builtin_amdgcn_readlane((int)d, b);
                const int at = __builtin_amdgcn_readlane(pos, b);
                if (k == myKey) {
                    if (queued == kSmallQueue) {
                        if (work) {
                            drain();
                        } else {
                            queued = 0;
                        }
                    }
                    if (gl == 0) {
                        queue[queued] = (uint16_t)at;
                    }
                    queued += 1;
                }
            }
        }
    }
    if (!work) {
        return;
    }
    drain();
    if (seen > kTwoLevelMin) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                acc[j][v] = inChunk > 0 ? tot[j][v] + chk[j][v] : tot[j][v];
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
            w_store4<WT>(rd.w, rowOff + e, w[j]);
            if (useS1) {
                vec_store<4>(rd.s1 + rowOff + e, s1[j]);
            }
            if (useS2) {
                vec_store<4>(rd.s2 + rowOff + e, s2[j]);
            }
        }
    }
}

// ---- keys seen up to kListMax times: a group of G lanes per distinct key ------------------------------
// G = lanes per key (a power of two, 4 elements per lane and pass), NJ = passes over the row.  The key's position
// list is already in ascending order.  WT = float or uint16_t (bf16 weights); SHARED = a gradient row is added to
// several keys (pooled layout: once per index of the bag), so it is loaded through the caches; a by-key gradient
// row is read once and streamed past them.  A list entry is the index of the
// gradient row to add (the lookup position; for the pooled layout the caller has rewritten it to the bag's sample and
// the table's columns start at the row descriptor's gradCol).
// One thread per key first resolves the key's metadata (count, slot, list start, table, row descriptor) into LDS,
// so that the memory pipeline of the other lanes carries row traffic only: with every lane fetching the metadata
// itself two thirds of the memory instructions of a wave were such fetches.  The group then loads its whole
// position list with one or two instructions and hands the positions round by lane shuffles.
struct __attribute__((aligned(16))) KeyMeta {
    const void* w;
    float* s1;
    float* s2;
    const float* gbase;   // gradient base including the table's column offset
    int64_t rowOff;       // slot * stride
    const int32_t* list;  // the key's position list
    uint32_t count;       // 0: nothing to do for this key
    int32_t dim;
};

template <int G, int NJ, typename WT, bool SHARED>
__global__ __launch_bounds__(kBlock) void k_apply_short(const RowsDesc* __restrict__ rows,
                                                        const int64_t* __restrict__ uoff, int T,
                                                        const int64_t* __restrict__ total,
                                                        const uint32_t* __restrict__ ucount,
                                                        const uint32_t* __restrict__ useg,
                                                        const int32_t* __restrict__ posList,
                                                        const int64_t* __restrict__ slots, GradSrc gs, OptParams prm)
{
    opt_resolve_rate(prm);
    constexpr int kKeysPerBlock = kBlock / G;
    __shared__ KeyMeta sMeta[kKeysPerBlock];
    const int64_t U = total[0];
    const int64_t R0 = (int64_t)blockIdx.x * kKeysPerBlock;
    if (R0 >= U) {
        return;
    }
    if (threadIdx.x < kKeysPerBlock) {
        const int64_t R = R0 + threadIdx.x;
        KeyMeta m;
        m.count = 0;
        m.w = nullptr;
        m.s1 = nullptr;
        m.s2 = nullptr;
        m.gbase = nullptr;
        m.rowOff = 0;
        m.list = nullptr;
        m.dim = 0;
        if (R < U) {
            const uint32_t c = ucount[R];
            const int64_t slot = slots[R];
            if (c <= (uint32_t)kListMax && slot >= 0) {
                const int t = find_segment(uoff, T, R);
                const RowsDesc rd = rows[t];
                m.count = c;
                m.w = rd.w;
                m.s1 = rd.s1;
                m.s2 = rd.s2;
                m.gbase = gs.base + rd.gradCol;
                m.rowOff = slot * rd.stride;
                m.list = posList + useg[R];
                m.dim = rd.dim;
            }
        }
        sMeta[threadIdx.x] = m;
    }
    __syncthreads();
    const KeyMeta m = sMeta[threadIdx.x / G];
    const int gl = threadIdx.x % G;
    const uint32_t c = m.count;
    if (c == 0) {
        return;
    }
    const int dim = m.dim;
    const int64_t rowOff = m.rowOff;
    const bool useS1 = dev_uses_s1(prm.optim);
    const bool useS2 = dev_uses_s2(prm.optim);
    // the whole list: lane gl holds positions gl, gl + G, ...
    constexpr int kListRegs = (kListMax + G - 1) / G;
    int32_t myPos[kListRegs];
#pragma unroll
    for (int q = 0; q < kListRegs; ++q) {
        const uint32_t r = (uint32_t)(q * G + gl);
        myPos[q] = (r < c) ? m.list[r] : 0;
    }
    float w[NJ][4];
    float s1[NJ][4];
    float s2[NJ][4];
    float acc[NJ][4];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int e = (j * G + gl) * 4;
        if (e < dim) {
            w_load4<WT>(w[j], m.w, rowOff + e);
            if (useS1) {
                vec_load<4>(s1[j], m.s1 + rowOff + e);
            }
            if (useS2) {
                vec_load<4>(s2[j], m.s2 + rowOff + e);
            }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            acc[j][v] = 0.0f;
        }
    }
    constexpr int kDepth = (NJ == 1) ? 4 : 2;  // two passes with four rows in flight: 327 -> 404 us (fewer waves resident)
    const int groupBase = (int)(threadIdx.x & (kWave - 1)) - gl;  // first lane of this key's group inside the wave
    for (uint32_t r = 0; r < c; r += kDepth) {
        float buf[kDepth][NJ][4];
#pragma unroll
        for (int k = 0; k < kDepth; ++k) {
            // position r + k sits in register (r + k) / G of lane (r + k) % G of the group
            const uint32_t rr = r + k;
            int32_t pos = 0;
#pragma unroll
            for (int q = 0; q < kListRegs; ++q) {
                const int32_t cand = __shfl(myPos[q], groupBase + (int)(rr % G), kWave);
                if ((int)(rr / G) == q) {
                    pos = cand;
                }
            }
            if (rr < c) {
                const float* src = m.gbase + (int64_t)pos * gs.stride;
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const int e = (j * G + gl) * 4;
                    if (e < dim) {
                        if (SHARED) {
                            vec_load4_cached(buf[k][j], src + e);
                        } else {
                            vec_load<4>(buf[k][j], src + e);
                        }
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
            w_store4<WT>(const_cast<void*>(m.w), rowOff + e, w[j]);
            if (useS1) {
                vec_store<4>(m.s1 + rowOff + e, s1[j]);
            }
            if (useS2) {
                vec_store<4>(m.s2 + rowOff + e, s2[j]);
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
constexpr int64_t kSplitLongMin = 500000;  // runs of at least this many keys launch the long-list kernel in two parts
constexpr int kPipe = 4;          // batches of rows in flight per wave
constexpr int kSub = 8;           // load instructions per batch

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

// One batch of the pipeline: the list positions of a batch and, later, its rows.  The positions are fetched with
// one load per 64 rows (lane l holds the position of row q*64 + l of the batch) and handed to the lanes that load a
// row by a lane shuffle: a load per row and lane would spend as many memory instructions on positions as on rows.
template <int SLICE>
struct LongStage {
    using G = LongGeom<SLICE>;
    static constexpr int kRaw = G::kBatch / kWave;
    static_assert(G::kBatch % kWave == 0 && kWave % G::kRpi == 0, "a batch is a whole number of 64-row groups");
    int32_t raw[kRaw];
    float4 row[kSub];

    __device__ __forceinline__ void load_pos(const int32_t* __restrict__ list, uint32_t c, uint32_t b, int lane)
    {
#pragma unroll
        for (int q = 0; q < kRaw; ++q) {
            const uint32_t r = b * G::kBatch + q * kWave + lane;
            raw[q] = list[r < c ? r : c - 1];
        }
    }

    // the gradient row of list entry p starts at gcol + p * stride
    __device__ __forceinline__ void issue_rows(const float* __restrict__ gcol, const GradSrc& gs, int sub)
    {
#pragma unroll
        for (int j = 0; j < kSub; ++j) {
            // row j * kRpi + sub of the batch: register (j * kRpi) / 64 of lane (j * kRpi) % 64 + sub
            const int32_t pos = __shfl(raw[(j * G::kRpi) / kWave], (j * G::kRpi) % kWave + sub, kWave);
            row[j] = *reinterpret_cast<const float4*>(gcol + (int64_t)pos * gs.stride);
        }
    }
};

// Consume batch b from stage st: rows -> LDS tile (rows past the end of the list as zeros), refill the stage with
// batch b + kPipe (and the positions of batch b + 2*kPipe), then add the tile's rows in order.  The body has no
// data-dependent branches: adding the zero rows leaves the sum unchanged, lanes beyond the slice compute a value
// nobody reads.
// The tile is column-major (tile[column][row], kTilePitch floats per column) so that the lane that owns a column
// fetches four consecutive rows with one 16-byte LDS read; the reads of the next 16 rows are issued before the 16
// dependent adds of the current ones, so the chain of adds never waits for LDS.
template <int SLICE>
struct LongTile {
    static constexpr int kPitch = LongGeom<SLICE>::kBatch + 4;  // +4: the column groups of one store land on different banks
    static constexpr int kFloats = SLICE * kPitch;
};

__device__ __forceinline__ void add4(float& acc, const float4& q)
{
    acc += q.x;
    acc += q.y;
    acc += q.z;
    acc += q.w;
}

// rows of a stage -> the wave's column-major tile (rows past the end of the list as zeros)
template <int SLICE>
__device__ __forceinline__ void tile_write(const LongStage<SLICE>& st, float* tile, uint32_t c, uint32_t b, int sub,
                                           int col4)
{
    using G = LongGeom<SLICE>;
    constexpr int kPitch = LongTile<SLICE>::kPitch;
#pragma unroll
    for (int j = 0; j < kSub; ++j) {
        const bool live = b * G::kBatch + j * G::kRpi + sub < c;
        const float4 v = st.row[j];
        float* dst = tile + (col4 * 4) * kPitch + j * G::kRpi + sub;
        dst[0] = live ? v.x : 0.0f;
        dst[kPitch] = live ? v.y : 0.0f;
        dst[2 * kPitch] = live ? v.z : 0.0f;
        dst[3 * kPitch] = live ? v.w : 0.0f;
    }
}

// acc += the tile's rows of this lane's column, in row order; the LDS reads run 16 rows ahead of the adds
template <int SLICE>
__device__ __forceinline__ void tile_add(const float* tile, float& acc, int lane)
{
    using G = LongGeom<SLICE>;
    constexpr int kPitch = LongTile<SLICE>::kPitch;
    const float4* colRows = reinterpret_cast<const float4*>(tile + (lane & (SLICE - 1)) * kPitch);
    static_assert(G::kBatch % 32 == 0, "the add loop takes 32 rows per round");
    float4 qa[4];
    float4 qb[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        qa[k] = colRows[k];
    }
#pragma unroll
    for (int g = 0; g < G::kBatch / 32; ++g) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            qb[k] = colRows[g * 8 + 4 + k];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            add4(acc, qa[k]);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (g + 1 < G::kBatch / 32) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                qa[k] = colRows[(g + 1) * 8 + k];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            add4(acc, qb[k]);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <int SLICE>
__device__ __forceinline__ void long_step(LongStage<SLICE>& st, float* tile, float& acc,
                                          const int32_t* __restrict__ list, const float* __restrict__ gcol,
                                          const GradSrc& gs, uint32_t c, uint32_t b, int lane, int sub, int col4)
{
    tile_write<SLICE>(st, tile, c, b, sub, col4);
    wave_lds_fence();
    __builtin_amdgcn_sched_barrier(0);
    st.issue_rows(gcol, gs, sub);
    st.load_pos(list, c, b + 2 * kPipe, lane);
    __builtin_amdgcn_sched_barrier(0);
    tile_add<SLICE>(tile, acc, lane);
    wave_lds_fence();
    __builtin_amdgcn_sched_barrier(0);
}

// The same without a refill, for lists that fit the stages already in flight.
template <int SLICE>
__device__ __forceinline__ void last_step(const LongStage<SLICE>& st, float* tile, float& acc, uint32_t c, uint32_t b,
                                          int lane, int sub, int col4)
{
    tile_write<SLICE>(st, tile, c, b, sub, col4);
    wave_lds_fence();
    tile_add<SLICE>(tile, acc, lane);
    wave_lds_fence();
}

// Per long key: everything a (key, column slice) item needs, resolved once so that an item starts with one
// record instead of a chain of eight dependent loads (most long keys are short enough that this chain was longer
// than their reduce).
__global__ __launch_bounds__(kBlock) void k_long_meta(const RowsDesc* __restrict__ rows,
                                                      const int64_t* __restrict__ uoff, int T,
                                                      const uint32_t* __restrict__ nLongPtr,
                                                      const int32_t* __restrict__ longList,
                                                      const uint32_t* __restrict__ longSeg,
                                                      const int32_t* __restrict__ longPos,
                                                      const uint32_t* __restrict__ ucount,
                                                      const int64_t* __restrict__ slots, GradSrc gs,
                                                      KeyMeta* __restrict__ meta, KeyMeta* __restrict__ chunkMeta,
                                                      float* __restrict__ chunkSums, int32_t* __restrict__ chunkList,
                                                      uint32_t* nChunks, int64_t chunkCap, int chunkPitch)
{
    const uint32_t lid = blockIdx.x * kBlock + threadIdx.x;
    const bool mine = lid < nLongPtr[0];   // no early return: the lanes of a wave write chunk records together below
    KeyMeta m;
    m.count = 0;
    m.w = nullptr;
    m.s1 = nullptr;
    m.s2 = nullptr;
    m.gbase = nullptr;
    m.rowOff = 0;
    m.list = nullptr;
    m.dim = 0;
    uint32_t nch = 0;   // > 0: this lane's key is summed chunk by chunk, its chunks are c0 .. c0 + nch - 1
    uint32_t c0 = 0;
    if (mine) {
        const int32_t R = longList[lid];
        const int64_t slot = slots[R];
        if (slot >= 0) {
            const int t = find_segment(uoff, T, (int64_t)R);
            const RowsDesc rd = rows[t];
            m.count = ucount[R];
            m.w = rd.w;
            m.s1 = rd.s1;
            m.s2 = rd.s2;
            m.gbase = gs.base + rd.gradCol;
            m.rowOff = slot * rd.stride;
            m.list = longPos + longSeg[lid];
            m.dim = rd.dim;
            if (m.count > (uint32_t)kTwoLevelMin && chunkMeta != nullptr) {
                // Two-level sum: every chunk of kChunkRows list entries becomes a work item of its own whose "row"
                // is a row of chunkSums (summed in list order and stored, not applied); the key itself then adds
                // its chunks' sums in chunk order and applies the optimizer once.
                nch = (m.count + kChunkRows - 1) / kChunkRows;
                c0 = atomicAdd(nChunks, nch);
                if ((int64_t)c0 + nch > chunkCap) {
                    nch = 0;   // no room (cannot happen with the workspace sized for the handle): one chain
                }
            }
        }
    }
    // The chunk records of a key are written by its whole wave (a key seen 150 000 times has 586 of them; one
    // thread writing them one after the other took as long as the reduce itself).
    unsigned long long todo = __ballot(nch != 0);
    const int lane = lane_id();
    while (todo != 0) {
        const int src = __ffsll((long long)todo) - 1;
        todo &= todo - 1;
        const uint32_t kNch = (uint32_t)__shfl((int)nch, src, kWave);
        const uint32_t kC0 = (uint32_t)__shfl((int)c0, src, kWave);
        const uint32_t kCount = (uint32_t)__shfl((int)m.count, src, kWave);
        const int kDim = __shfl(m.dim, src, kWave);
        const unsigned long long gb = (unsigned long long)reinterpret_cast<uintptr_t>(m.gbase);
        const unsigned long long ls = (unsigned long long)reinterpret_cast<uintptr_t>(m.list);
        const unsigned long long kGbase = ((unsigned long long)(uint32_t)__shfl((int)(gb >> 32), src, kWave) << 32) |
                                          (uint32_t)__shfl((int)gb, src, kWave);
        const unsigned long long kList = ((unsigned long long)(uint32_t)__shfl((int)(ls >> 32), src, kWave) << 32) |
                                         (uint32_t)__shfl((int)ls, src, kWave);
        for (uint32_t j = (uint32_t)lane; j < kNch; j += kWave) {
            KeyMeta cm;
            cm.w = chunkSums + (int64_t)(kC0 + j) * chunkPitch;
            cm.s1 = nullptr;
            cm.s2 = nullptr;
            cm.gbase = reinterpret_cast<const float*>(static_cast<uintptr_t>(kGbase));
            cm.rowOff = 0;
            cm.list = reinterpret_cast<const int32_t*>(static_cast<uintptr_t>(kList)) + (int64_t)j * kChunkRows;
            cm.count = (j + 1 < kNch) ? (uint32_t)kChunkRows : kCount - j * (uint32_t)kChunkRows;
            cm.dim = kDim;
            chunkMeta[kC0 + j] = cm;
            chunkList[kC0 + j] = (int32_t)((int64_t)(kC0 + j) * chunkPitch / gs.stride);
        }
    }
    if (!mine) {
        return;
    }
    if (nch != 0) {
        m.gbase = chunkSums;
        m.list = chunkList + c0;
        m.count = nch;
    }
    meta[lid] = m;
}

// One (long key, column slice) item: the wave walks the key's ascending position list with kPipe batches in flight.
template <int SLICE, typename WT>
__device__ __forceinline__ void long_item(const KeyMeta& m, int slice, const GradSrc& gs, const OptParams& prm,
                                          float* tile, int lane)
{
    using G = LongGeom<SLICE>;
    const int col4 = lane % G::kLpr;  // float4 column inside the slice
    const int sub = lane / G::kLpr;   // row inside the group of rows one instruction fetches
    const uint32_t c = m.count;
    const int dim = m.dim;
    const int colBase = slice * SLICE;
    if (c == 0 || colBase >= dim) {
        return;
    }
    const int32_t* list = m.list;
    const bool colOk = (colBase + col4 * 4) < dim;
    const uint32_t nb = (c + G::kBatch - 1) / G::kBatch;
    // Loads are unconditional (indices clamped to the last list entry, columns to the row) so that the
    // compiler keeps them in straight-line code with exact wait counts; surplus rows are never added.
    const float* gcol = m.gbase + (colOk ? colBase + col4 * 4 : 0);
    LongStage<SLICE> st0, st1, st2, st3;
    static_assert(kPipe == 4, "the stages below are written out for four batches in flight");
    float acc = 0.0f;
    if (nb <= (uint32_t)kPipe) {
        // the whole list fits the stages: fetch exactly its batches, then consume them (most long keys are here,
        // and a full pipeline round with its refills would cost them more than their own rows)
        st0.load_pos(list, c, 0, lane);
        if (nb > 1) {
            st1.load_pos(list, c, 1, lane);
        }
        if (nb > 2) {
            st2.load_pos(list, c, 2, lane);
        }
        if (nb > 3) {
            st3.load_pos(list, c, 3, lane);
        }
        st0.issue_rows(gcol, gs, sub);
        if (nb > 1) {
            st1.issue_rows(gcol, gs, sub);
        }
        if (nb > 2) {
            st2.issue_rows(gcol, gs, sub);
        }
        if (nb > 3) {
            st3.issue_rows(gcol, gs, sub);
        }
        last_step<SLICE>(st0, tile, acc, c, 0, lane, sub, col4);
        if (nb > 1) {
            last_step<SLICE>(st1, tile, acc, c, 1, lane, sub, col4);
        }
        if (nb > 2) {
            last_step<SLICE>(st2, tile, acc, c, 2, lane, sub, col4);
        }
        if (nb > 3) {
            last_step<SLICE>(st3, tile, acc, c, 3, lane, sub, col4);
        }
    } else {
        // memory returns in issue order: the scheduling barriers keep the loads in the order the steps consume them
        st0.load_pos(list, c, 0, lane);
        st1.load_pos(list, c, 1, lane);
        st2.load_pos(list, c, 2, lane);
        st3.load_pos(list, c, 3, lane);
        __builtin_amdgcn_sched_barrier(0);
        st0.issue_rows(gcol, gs, sub);
        st0.load_pos(list, c, 4, lane);
        __builtin_amdgcn_sched_barrier(0);
        st1.issue_rows(gcol, gs, sub);
        st1.load_pos(list, c, 5, lane);
        __builtin_amdgcn_sched_barrier(0);
        st2.issue_rows(gcol, gs, sub);
        st2.load_pos(list, c, 6, lane);
        __builtin_amdgcn_sched_barrier(0);
        st3.issue_rows(gcol, gs, sub);
        st3.load_pos(list, c, 7, lane);
        __builtin_amdgcn_sched_barrier(0);
        for (uint32_t b0 = 0; b0 < nb; b0 += kPipe) {
            long_step<SLICE>(st0, tile, acc, list, gcol, gs, c, b0 + 0, lane, sub, col4);
            long_step<SLICE>(st1, tile, acc, list, gcol, gs, c, b0 + 1, lane, sub, col4);
            long_step<SLICE>(st2, tile, acc, list, gcol, gs, c, b0 + 2, lane, sub, col4);
            long_step<SLICE>(st3, tile, acc, list, gcol, gs, c, b0 + 3, lane, sub, col4);
        }
    }
    if (lane < SLICE && colBase + lane < dim) {
        const int64_t e = m.rowOff + colBase + lane;
        float w = w_load1<WT>(m.w, e);
        float s1 = 0.0f;
        float s2 = 0.0f;
        if (dev_uses_s1(prm.optim)) {
            s1 = m.s1[e];
        }
        if (dev_uses_s2(prm.optim)) {
            s2 = m.s2[e];
        }
        opt_update(prm, acc, w, s1, s2);
        w_store1<WT>(const_cast<void*>(m.w), e, w);
        if (dev_uses_s1(prm.optim)) {
            m.s1[e] = s1;
        }
        if (dev_uses_s2(prm.optim)) {
            m.s2[e] = s2;
        }
    }
}

// One launch covers every long key, longest lists first: (key, 8-column slice) items for the keys seen more than
// kVeryHugeMin times (the longest dependent chains: narrow slices put the most rows of one key in flight),
// (key, 16-column slice) items for those seen more than kHugeMin times, then the (key, 32-column slice) items of the
// other long keys, which fill the machine while the longest chains finish.  Narrow slices cost adds: only SLICE of
// the 64 lanes own a column, so they are kept for the keys whose chain would otherwise set the kernel's duration.
template <typename WT>
__global__ __launch_bounds__(kBlock, 2) void k_apply_long(const KeyMeta* __restrict__ meta,
                                                          const int32_t* __restrict__ hugeIds,
                                                          const uint32_t* __restrict__ nHugePtr,
                                                          const uint32_t* __restrict__ nVeryHugePtr,
                                                          const int32_t* __restrict__ longIds,
                                                          const uint32_t* __restrict__ nRestPtr, GradSrc gs,
                                                          int slices8, int slices16, int slices32, OptParams prm,
                                                          uint32_t* consumed)
{
    opt_resolve_rate(prm);
    // the chunk counter of the pass before this one has been read by then: the next reduce starts from zero
    if (consumed != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
        *consumed = 0;
    }
    constexpr int kTileFloats = LongTile<8>::kFloats > LongTile<32>::kFloats
                                    ? (LongTile<8>::kFloats > LongTile<16>::kFloats ? LongTile<8>::kFloats
                                                                                  : LongTile<16>::kFloats)
                                    : (LongTile<32>::kFloats > LongTile<16>::kFloats ? LongTile<32>::kFloats
                                                                                   : LongTile<16>::kFloats);
    __shared__ __attribute__((aligned(16))) float tileAll[kBlock / kWave][kTileFloats];
    float* tile = tileAll[threadIdx.x >> 6];
    const int64_t nVery = nVeryHugePtr[0];
    const int64_t items8 = nVery * slices8;
    const int64_t items16 = ((int64_t)nHugePtr[0] - nVery) * slices16;
    const int64_t items = items8 + items16 + (int64_t)nRestPtr[0] * slices32;
    const int lane = lane_id();
    const int64_t wavesTotal = (int64_t)gridDim.x * (kBlock / kWave);
    for (int64_t item = (int64_t)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6); item < items; item += wavesTotal) {
        // the item, hence the key, is the same for the whole wave
        if (item < items8) {
            const int32_t lid = __builtin_amdgcn_readfirstlane(hugeIds[item / slices8]);
            const KeyMeta m = meta[lid];
            long_item<8, WT>(m, (int)(item % slices8), gs, prm, tile, lane);
        } else if (item < items8 + items16) {
            const int64_t j = item - items8;
            const int32_t lid = __builtin_amdgcn_readfirstlane(hugeIds[nVery + j / slices16]);
            const KeyMeta m = meta[lid];
            long_item<16, WT>(m, (int)(j % slices16), gs, prm, tile, lane);
        } else {
            const int64_t j = item - items8 - items16;
            const int32_t lid = __builtin_amdgcn_readfirstlane(longIds[j / slices32]);
            const KeyMeta m = meta[lid];
            long_item<32, WT>(m, (int)(j % slices32), gs, prm, tile, lane);
        }
    }
}

// ---- launch --------------------------------------------------------------------------------------------
template <int G, int NJ, typename WT, bool SHARED>
static int launch_short(const ApplyCtx& c)
{
    const UniqueView* v = c.v;
    const unsigned grid = (unsigned)cdiv(v->n, kBlock / G);
    hipStream_t s = c.stream;
    RECSDK_LAUNCH((k_apply_short<G, NJ, WT, SHARED>), dim3(grid), dim3(kBlock), s, c.d_rows, v->uoff, v->T, v->total,
                  v->ucount, v->useg, v->posList, c.d_slots, c.g, c.prm);
    return RECSDK_OK;
}

template <int G, int NJ, typename WT>
static int launch_small(const ApplyCtx& c)
{
    const UniqueView* v = c.v;
    const unsigned grid = (unsigned)cdiv(v->n, (kBlock / kWave) * (kWave / G));
    hipStream_t s = c.stream;
    RECSDK_LAUNCH_AS("k_apply_small", (k_apply_small<G, NJ, WT>), dim3(grid), dim3(kBlock), s, c.d_rows, v->uoff, v->T,
                     v->total, v->grank, v->n, c.d_slots, c.g, c.prm);
    return RECSDK_OK;
}

template <typename WT>
static int apply_launch_t(const ApplyCtx& c)
{
    const UniqueView* v = c.v;
    const int dim = c.maxDim;
    hipStream_t s = c.stream;
    if (v->scanReduce) {
        // a small run: no position lists, one launch
        const int ch = (dim + 3) / 4;
        if (ch <= 4) {
            return launch_small<4, 1, WT>(c);
        } else if (ch <= 8) {
            return launch_small<8, 1, WT>(c);
        } else if (ch <= 16) {
            return launch_small<16, 1, WT>(c);
        } else if (ch <= 32) {
            return launch_small<32, 1, WT>(c);
        } else if (ch <= 64) {
            return launch_small<64, 1, WT>(c);
        } else if (ch <= 128) {
            return launch_small<64, 2, WT>(c);
        } else if (ch <= 256) {
            return launch_small<64, 4, WT>(c);
        }
        return launch_small<64, 8, WT>(c);
    }
    if (v->listsReady != nullptr) {
        RECSDK_HIP_TRY(hipStreamWaitEvent(s, v->listsReady, 0));
    }
    // Keys seen more than kTwoLevelMin times: chunk sums first (a pass of the long-list kernel over the chunks, which
    // stores the sums), then the keys add their chunk sums like any other list.  The chunk pass is a few hundred
    // waves walking chains of dependent adds and moves little data, so it runs on a side stream next to the
    // short-list kernel, which is bound by memory traffic; the long-list kernel follows when both are done.  (Running
    // ALL long-list work beside the short-list kernel measured no gain: both are bound by memory traffic.  With the
    // chunk pass beside it the step of 26 x 65536 keys went from 1.014 to 0.964 ms.)
    const bool haveLong = v->n > kListMax;
    const bool twoLevel = haveLong && v->n > kTwoLevelMin && c.uq != nullptr;
    const bool fork = twoLevel && c.side != nullptr;
    const int kWavesPerBlock = kBlock / kWave;
    const int slices8 = (dim + 7) / 8;
    const int slices16 = (dim + 15) / 16;
    const int slices32 = (dim + 31) / 32;
    KeyMeta* meta = static_cast<KeyMeta*>(v->longMeta);
    // part 0: every long key; 1: only those of at most kHugeMin positions, which need no chunk sums; 2: only the others
    auto long_lists = [&](int part) -> int {
        const int64_t itemsMax = (part != 1 ? (v->n / kHugeMin + 1) * slices8 : 0) +
                                 (part != 2 ? (v->n / kListMax + 1) * slices32 : 0);
        const unsigned grid = (unsigned)std::min<int64_t>(cdiv(itemsMax, kWavesPerBlock), 4096);
        RECSDK_LAUNCH((k_apply_long<WT>), dim3(grid), dim3(kBlock), s, meta, v->hugeIds, part != 1 ? v->nHuge : v->zero,
                      part != 1 ? v->nVeryHuge : v->zero, v->longIds, part != 2 ? v->nLongRest : v->zero, c.g, slices8,
                      slices16, slices32, c.prm, (twoLevel && part != 1) ? v->nChunks : (uint32_t*)nullptr);
        return RECSDK_OK;
    };
    // With many keys the long-list kernel goes in two: the keys that need no chunk sums right behind the short-list
    // kernel, the others when the chunk pass has ended.  That pass runs beside the short-list kernel and ends some
    // 25 us after it (26 x 65536 keys), which the whole long-list kernel used to wait for.  With few keys one more
    // launch costs more than the wait.
    static_assert(kTwoLevelMin == kHugeMin, "the keys summed through chunks are the ones listed in hugeIds");
    const bool split = fork && c.evMeta != nullptr && v->n >= kSplitLongMin;
    if (haveLong) {
        hipStream_t side = fork ? c.side : s;
        if (twoLevel) {
            const int rc = recsdk_unique_chunk_buffers(c.uq, dim);
            if (rc != RECSDK_OK) {
                return rc;
            }
        }
        if (fork) {
            RECSDK_HIP_TRY(hipEventRecord(c.evFork, s));
            RECSDK_HIP_TRY(hipStreamWaitEvent(side, c.evFork, 0));
        }
        if (v->classesReady != nullptr) {
            // every long-list launch below is ordered after this stream's k_long_meta
            RECSDK_HIP_TRY(hipStreamWaitEvent(side, v->classesReady, 0));
        }
        RECSDK_LAUNCH(k_long_meta, dim3((unsigned)cdiv(v->n / kListMax + 1, kBlock)), dim3(kBlock), side, c.d_rows,
                      v->uoff, v->T, v->nLong, v->longList, v->longSeg, v->longPos, v->ucount, c.d_slots, c.g, meta,
                      twoLevel ? static_cast<KeyMeta*>(v->chunkMeta) : (KeyMeta*)nullptr, v->chunkSums, v->chunkList,
                      v->nChunks, v->chunkCap, (int)v->chunkPitch);
        if (split) {
            RECSDK_HIP_TRY(hipEventRecord(c.evMeta, side));
        }
        if (twoLevel) {
            OptParams store = c.prm;
            store.optim = kOptStoreSum;
            const unsigned cgrid = (unsigned)std::min<int64_t>(cdiv(v->chunkCap * slices32, kWavesPerBlock), 4096);
            RECSDK_LAUNCH_AS("k_apply_long_chunks", (k_apply_long<float>), dim3(cgrid), dim3(kBlock), side,
                             static_cast<const KeyMeta*>(v->chunkMeta), v->hugeIds, v->zero, v->zero, v->chunkIds,
                             v->nChunks, c.g, slices8, slices16, slices32, store, (uint32_t*)nullptr);
        }
        if (fork) {
            RECSDK_HIP_TRY(hipEventRecord(c.evJoin, side));
        } else {
            const int rc = long_lists(0);
            if (rc != RECSDK_OK) {
                return rc;
            }
        }
    }
    const int chunks = (dim + 3) / 4;
    int rc;
    // From 36 columns on a key gets half the lanes its row would fill and takes the row in two passes: twice the keys
    // per wave with the same bytes in flight per key (26 x 65536 keys of 128 columns: 335 -> 327 us; a quarter of the
    // lanes and four passes: 357 us, the registers cost more residency than the keys bring).
    if (chunks > 8 && chunks <= 16) {
        rc = c.gradShared ? launch_short<8, 2, WT, true>(c) : launch_short<8, 2, WT, false>(c);
    } else if (chunks > 16 && chunks <= 32) {
        rc = c.gradShared ? launch_short<16, 2, WT, true>(c) : launch_short<16, 2, WT, false>(c);
    } else if (chunks > 32 && chunks <= 64) {
        rc = c.gradShared ? launch_short<32, 2, WT, true>(c) : launch_short<32, 2, WT, false>(c);
    } else if (chunks <= 4) {
        rc = c.gradShared ? launch_short<4, 1, WT, true>(c) : launch_short<4, 1, WT, false>(c);
    } else if (chunks <= 8) {
        rc = c.gradShared ? launch_short<8, 1, WT, true>(c) : launch_short<8, 1, WT, false>(c);
    } else if (chunks <= 16) {
        rc = c.gradShared ? launch_short<16, 1, WT, true>(c) : launch_short<16, 1, WT, false>(c);
    } else if (chunks <= 32) {
        rc = c.gradShared ? launch_short<32, 1, WT, true>(c) : launch_short<32, 1, WT, false>(c);
    } else if (chunks <= 64) {
        rc = c.gradShared ? launch_short<64, 1, WT, true>(c) : launch_short<64, 1, WT, false>(c);
    } else if (chunks <= 128) {
        rc = c.gradShared ? launch_short<64, 2, WT, true>(c) : launch_short<64, 2, WT, false>(c);
    } else if (chunks <= 256) {
        rc = c.gradShared ? launch_short<64, 4, WT, true>(c) : launch_short<64, 4, WT, false>(c);
    } else {
        rc = c.gradShared ? launch_short<64, 8, WT, true>(c) : launch_short<64, 8, WT, false>(c);
    }
    if (fork && rc == RECSDK_OK) {
        if (split) {
            RECSDK_HIP_TRY(hipStreamWaitEvent(s, c.evMeta, 0));
            rc = long_lists(1);
            if (rc != RECSDK_OK) {
                return rc;
            }
        }
        RECSDK_HIP_TRY(hipStreamWaitEvent(s, c.evJoin, 0));
        rc = long_lists(split ? 2 : 0);
    }
    return rc;
}

int apply_launch(const ApplyCtx& c)
{
    if (c.v->n == 0) {
        return RECSDK_OK;
    }
    return c.wBf16 ? apply_launch_t<uint16_t>(c) : apply_launch_t<float>(c);
}

}  // namespace recsdk

using namespace recsdk;

struct recsdk_rows {
    int32_t T = 0;
    int32_t dim = 0;
    RowsDesc* descs = nullptr;  // device
    std::vector<RowsDesc> host;
    // the update kernels for long and short position lists touch disjoint rows; the former run on a side stream
    hipStream_t side = nullptr;
    hipEvent_t evFork = nullptr;
    hipEvent_t evJoin = nullptr;
    hipEvent_t evMeta = nullptr;
    // one row address per distinct key of the unique run being gathered (grown on demand)
    const float** rowPtr = nullptr;
    int64_t rowPtrCap = 0;
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
        r->host[t].dim = dim;
        r->host[t].gradCol = 0;
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
        hipEventCreateWithFlags(&r->evJoin, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&r->evMeta, hipEventDisableTiming) != hipSuccess) {
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
    if (rows->evMeta) {
        (void)hipEventDestroy(rows->evMeta);
    }
    if (rows->side) {
        (void)hipStreamDestroy(rows->side);
    }
    (void)hipFree(rows->descs);
    if (rows->rowPtr != nullptr) {
        (void)hipFree(rows->rowPtr);
    }
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
    if (v->n <= small_batch_keys()) {
        RECSDK_LAUNCH(k_gather_small, dim3((unsigned)cdiv(v->n * dim, kBlock)), dim3(kBlock), s, rows->descs, v->uoff,
                      v->T, d_slots, v->grank, d_out, v->n, dim);
        return RECSDK_OK;
    }
    const bool out16 = (reinterpret_cast<uintptr_t>(d_out) % 16) == 0;
    const bool vec4 = dim % 4 == 0 && out16 && rows_aligned(rows, 4, false, false);
    if (v->T <= kGatherTables) {
        if (vec4) {
            const int cpr = dim / 4;
            const unsigned grid = (unsigned)cdiv(v->n * cpr, kBlock * 4);
            RECSDK_LAUNCH((k_gather_rows<4, 4, true, true>), dim3(grid), dim3(kBlock), s, (const float* const*)nullptr,
                          rows->descs, v->uoff, v->T, d_slots, v->grank, d_out, v->n, dim, cpr);
        } else {
            const unsigned grid = (unsigned)cdiv(v->n * dim, kBlock * 4);
            RECSDK_LAUNCH((k_gather_rows<1, 4, true, true>), dim3(grid), dim3(kBlock), s, (const float* const*)nullptr,
                          rows->descs, v->uoff, v->T, d_slots, v->grank, d_out, v->n, dim, dim);
        }
        return RECSDK_OK;
    }
    if (rows->rowPtrCap < v->n) {
        // hipFree waits for the device, so no kernel still reads the old buffer
        if (rows->rowPtr != nullptr) {
            RECSDK_HIP_TRY(hipFree(rows->rowPtr));
            rows->rowPtr = nullptr;
            rows->rowPtrCap = 0;
        }
        const int64_t cap = std::max<int64_t>(v->n, 1024);
        RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&rows->rowPtr), sizeof(float*) * cap));
        rows->rowPtrCap = cap;
    }
    RECSDK_LAUNCH(k_row_ptrs, dim3((unsigned)cdiv(v->n, kBlock)), dim3(kBlock), s, rows->descs, v->uoff, v->T, v->total,
                  d_slots, rows->rowPtr);
    if (vec4) {
        const int cpr = dim / 4;
        const unsigned grid = (unsigned)cdiv(v->n * cpr, kBlock * 4);
        RECSDK_LAUNCH((k_gather_rows<4, 4, true, false>), dim3(grid), dim3(kBlock), s, rows->rowPtr, rows->descs,
                      v->uoff, v->T, d_slots, v->grank, d_out, v->n, dim, cpr);
    } else {
        const unsigned grid = (unsigned)cdiv(v->n * dim, kBlock * 4);
        RECSDK_LAUNCH((k_gather_rows<1, 4, true, false>), dim3(grid), dim3(kBlock), s, rows->rowPtr, rows->descs,
                      v->uoff, v->T, d_slots, v->grank, d_out, v->n, dim, dim);
    }
    return RECSDK_OK;
}

static int sparse_apply_impl(recsdk_rows_t* rows, recsdk_unique_t* u, const int64_t* d_slots, const float* d_grad,
                             int32_t optim, float lr, const float* d_lr, float beta1, float beta2, float eps,
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
    RECSDK_REQUIRE(dim % 4 == 0 && dim <= 2048, RECSDK_EINVAL,
                   "recsdk_sparse_apply: dim must be a multiple of 4 and at most 2048");
    RECSDK_REQUIRE((reinterpret_cast<uintptr_t>(d_grad) % 16) == 0, RECSDK_EINVAL,
                   "recsdk_sparse_apply: d_grad must be 16-byte aligned");
    RECSDK_REQUIRE(rows_aligned(rows, 4, optim != RECSDK_OPT_SGD, optim == RECSDK_OPT_ADAM), RECSDK_EINVAL,
                   "recsdk_sparse_apply: row pointers must be 16-byte aligned, strides multiples of 4, and the "
                   "optimizer's state pointers present");
    ApplyCtx c;
    c.d_rows = rows->descs;
    c.T = rows->T;
    c.maxDim = dim;
    c.uq = u;
    c.wBf16 = false;
    c.v = v;
    c.d_slots = d_slots;
    c.g = GradSrc{d_grad, dim};
    c.prm = OptParams{optim, lr, beta1, beta2, eps, weight_decay, 0.0f, d_lr};
    c.stream = static_cast<hipStream_t>(stream);
    c.side = rows->side;
    c.evFork = rows->evFork;
    c.evJoin = rows->evJoin;
    c.evMeta = rows->evMeta;
    return apply_launch(c);
}

extern "C" int recsdk_sparse_apply(recsdk_rows_t* rows, recsdk_unique_t* u, const int64_t* d_slots,
                                   const float* d_grad, int32_t optim, float lr, float beta1, float beta2, float eps,
                                   float weight_decay, void* stream)
{
    return sparse_apply_impl(rows, u, d_slots, d_grad, optim, lr, nullptr, beta1, beta2, eps, weight_decay, stream);
}

extern "C" int recsdk_sparse_apply_lr_dev(recsdk_rows_t* rows, recsdk_unique_t* u, const int64_t* d_slots,
                                          const float* d_grad, int32_t optim, const float* d_lr, float beta1,
                                          float beta2, float eps, float weight_decay, void* stream)
{
    RECSDK_REQUIRE(d_lr != nullptr, RECSDK_ENULL, "recsdk_sparse_apply_lr_dev: d_lr is NULL");
    return sparse_apply_impl(rows, u, d_slots, d_grad, optim, 0.0f, d_lr, beta1, beta2, eps, weight_decay, stream);
}
