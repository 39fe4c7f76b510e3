// Split-embedding (fbgemm-style, table-batched) pooled lookup forward and the exact backward with fused optimizer.
//
// forward : one group of lanes per bag (t, b) adds the bag's rows in index order, 4 row loads in flight, and
//           writes out[b, D_offsets[t] : D_offsets[t+1]]; bf16 tables are widened to fp32 before adding.
// backward: the touched rows are found with the same dedup as the key path (keys = row indices, one segment per
//           table), which also yields every row's ascending list of positions; each position maps to its bag's
//           sample b, so the gradient row of position k is grad_output[b, D-slice of t] (times 1/len for mean).
//           The shared row-update kernels then add those rows in list order and apply the optimizer once per row.
// Compiled with -ffp-contract=off.
#include <algorithm>
#include <cstdlib>

#include "apply.h"
#include "common.h"
#include "dedup.h"

namespace recsdk {

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

template <typename WT>
__device__ __forceinline__ void tbe_load4(float (&dst)[4], const void* base, int64_t e);
template <>
__device__ __forceinline__ void tbe_load4<float>(float (&dst)[4], const void* base, int64_t e)
{
    float4 v = *reinterpret_cast<const float4*>(static_cast<const float*>(base) + e);
    dst[0] = v.x;
    dst[1] = v.y;
    dst[2] = v.z;
    dst[3] = v.w;
}
template <>
__device__ __forceinline__ void tbe_load4<uint16_t>(float (&dst)[4], const void* base, int64_t e)
{
    uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + e);
    dst[0] = bf16_bits_to_f32((uint16_t)(raw.x & 0xffffu));
    dst[1] = bf16_bits_to_f32((uint16_t)(raw.x >> 16));
    dst[2] = bf16_bits_to_f32((uint16_t)(raw.y & 0xffffu));
    dst[3] = bf16_bits_to_f32((uint16_t)(raw.y >> 16));
}

// E columns of a row: E = 4 as above; E = 8 (bf16 rows only) is one 16-byte load of eight values where the row has
// them, four values and four zeros at the end of a row whose width is a multiple of 4 but not of 8.
template <typename WT, int E>
__device__ __forceinline__ void tbe_load_cols(float (&dst)[E], const void* base, int64_t e, int left)
{
    if constexpr (E == 4) {
        tbe_load4<WT>(dst, base, e);
    } else {
        static_assert(E == 8 && sizeof(WT) == 2, "eight columns per lane are for 2-byte rows");
        if (left >= 8) {
            const uint4 raw = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(base) + e);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                dst[2 * k] = bf16_bits_to_f32((uint16_t)(w[k] & 0xffffu));
                dst[2 * k + 1] = bf16_bits_to_f32((uint16_t)(w[k] >> 16));
            }
        } else {
            float lo[4];
            tbe_load4<WT>(lo, base, e);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                dst[k] = lo[k];
                dst[4 + k] = 0.0f;
            }
        }
    }
}

// E columns of a row as they come from memory (16 bytes, 8 for four bf16 values): rows waiting in registers for their
// turn in the sum take a quarter of the space of their float values.
template <typename WT, int E>
struct RawCols {
    uint32_t w[(E * (int)sizeof(WT)) / 4];

    __device__ __forceinline__ void load(const void* base, int64_t e, int left)
    {
        if constexpr (sizeof(WT) == 4) {
            const uint4 v = *reinterpret_cast<const uint4*>(static_cast<const float*>(base) + e);
            w[0] = v.x;
            w[1] = v.y;
            w[2] = v.z;
            w[3] = v.w;
        } else if constexpr (E == 4) {
            const uint2 v = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + e);
            w[0] = v.x;
            w[1] = v.y;
        } else {
            if (left >= 8) {
                const uint4 v = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(base) + e);
                w[0] = v.x;
                w[1] = v.y;
                w[2] = v.z;
                w[3] = v.w;
            } else {   // the last four columns of a row whose width is no multiple of 8: four values and four zeros
                const uint2 v = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + e);
                w[0] = v.x;
                w[1] = v.y;
                w[2] = 0u;
                w[3] = 0u;
            }
        }
    }
    __device__ __forceinline__ float value(int k) const
    {
        if constexpr (sizeof(WT) == 4) {
            return __uint_as_float(w[k]);
        } else {
            return bf16_bits_to_f32((uint16_t)((k & 1) ? (w[k >> 1] >> 16) : (w[k >> 1] & 0xffffu)));
        }
    }
};

// ---- forward, sum / mean --------------------------------------------------------------------------------
// A group of G lanes per bag, 4 columns per lane and pass.  One thread per bag first resolves the bag's metadata
// (table, column range, index range, weight base) into LDS, and a group fetches G indices with one load and hands
// them round by lane shuffles, so that the memory pipeline carries row loads rather than one index load per row
// and lane.
struct BagMeta {
    int64_t s;       // first index of the bag
    int64_t e;       // one past its last index
    int64_t base;    // first element of the table in the weight buffer
    int64_t outOff;  // b * totalD + d0
    int32_t D;       // 0: nothing to do
    int32_t pad;
};

// A block takes kFwdRounds bags per group and hands them out longest first (odd rounds backwards): the groups of a
// wave then work on bags of nearly the same length.  With bags of 1..50 indices taken in input order a wave waited
// for the longest of its four bags: 523 us for 10.9 M indices of 128-byte rows, 385 us now; bags of one length 338 us.
// Four or eight bags per group sort better but leave fewer, longer blocks: 384 and 425 us.
constexpr int kFwdRounds = 2;

// E = columns per lane and pass: 4, or 8 for bf16 rows (half as many lanes per bag and as many 16-byte loads as an
// fp32 row of the same width takes: 10.9 M indices of 128-byte bf16 rows 386 -> 373 us; what bounds the kernel is
// the rate of random 128-byte lines from beyond the L2, not the loads' width).
template <int G, int NJ, typename WT, int E>
__global__ __launch_bounds__(kBlock) void k_tbe_forward(const void* __restrict__ weights, int64_t numel,
                                                        const int64_t* __restrict__ wOff,
                                                        const int32_t* __restrict__ dOff,
                                                        const int64_t* __restrict__ indices,
                                                        const int64_t* __restrict__ offsets, int T, int64_t B,
                                                        int mean, float* __restrict__ out, int64_t totalD)
{
    constexpr int kGroups = kBlock / G;
    constexpr int kBagsPerBlock = kGroups * kFwdRounds;  // <= kBlock because G >= 4
    __shared__ BagMeta sMeta[kBagsPerBlock];
    __shared__ int32_t sLen[kBagsPerBlock];
    __shared__ int16_t sOrder[kBagsPerBlock];
    const int64_t bag0 = (int64_t)blockIdx.x * kBagsPerBlock;
    if (threadIdx.x < kBagsPerBlock) {
        const int64_t bag = bag0 + threadIdx.x;
        BagMeta m;
        m.D = 0;
        m.s = 0;
        m.e = 0;
        m.base = 0;
        m.outOff = 0;
        m.pad = 0;
        if (bag < (int64_t)T * B) {
            const int t = (int)(bag / B);
            const int64_t b = bag - (int64_t)t * B;
            const int d0 = dOff[t];
            m.D = dOff[t + 1] - d0;
            m.s = offsets[bag];
            m.e = offsets[bag + 1];
            m.base = wOff[t];
            m.outOff = b * totalD + d0;
        }
        sMeta[threadIdx.x] = m;
        const int64_t len = m.e - m.s;
        sLen[threadIdx.x] = (m.D == 0 || len < 0) ? -1 : (int32_t)(len > 0x7fffffff ? 0x7fffffff : len);
    }
    __syncthreads();
    if (threadIdx.x < kBagsPerBlock) {
        // place among the block's bags, longest first (ties in input order)
        const int32_t mine = sLen[threadIdx.x];
        int rank = 0;
        for (int k = 0; k < kBagsPerBlock; ++k) {
            const int32_t other = sLen[k];
            rank += (other > mine || (other == mine && k < (int)threadIdx.x)) ? 1 : 0;
        }
        sOrder[rank] = (int16_t)threadIdx.x;
    }
    __syncthreads();
    const int gl = threadIdx.x % G;
    const int groupBase = (int)(threadIdx.x & (kWave - 1)) - gl;  // first lane of this group inside the wave
    for (int round = 0; round < kFwdRounds; ++round) {
        // odd rounds run through the groups backwards, so that no wave gets the longest bags of every round
        const int g = (int)(threadIdx.x / G);
        const BagMeta m = sMeta[sOrder[round * kGroups + ((round & 1) ? kGroups - 1 - g : g)]];
        const int D = m.D;
        if (D == 0) {
            continue;
        }
        const int64_t s = m.s;
        const int64_t e = m.e;
        const int64_t base = m.base;
        float scale = 1.0f;
        if (mean && e > s) {
            scale = 1.0f / (float)(e - s);
        }
        float acc[NJ][E];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
#pragma unroll
            for (int v = 0; v < E; ++v) {
                acc[j][v] = 0.0f;
            }
        }
        if constexpr (NJ == 1) {
            // A row fits the group.  What bounds this path is the chain index -> row -> add of one bag: every round
            // fetches up to kIdxRegs * G indices at once, then the rows in batches of kBatch loads that are all in flight
            // together, the next batch issued before the current one is added (10.9 M indices of 128-byte rows in bags
            // of 1..50: 375 us with four rows in flight and one index load per G rows).
            constexpr int kBatch = G < 8 ? G : 8;
            constexpr int kBatchesPerReg = G / kBatch;
            constexpr int kIdxRegs = (G >= 32) ? 1 : (G >= 16 ? 2 : 4);
            constexpr int kBatches = kIdxRegs * kBatchesPerReg;
            const int c = gl * E;
            const bool colOk = c < D;
            for (int64_t k0 = s; k0 < e; k0 += (int64_t)G * kIdxRegs) {
                long long myRow[kIdxRegs];
#pragma unroll
                for (int r = 0; r < kIdxRegs; ++r) {
                    const int64_t at = k0 + (int64_t)r * G + gl;
                    myRow[r] = at < e ? indices[at] : -1;
                }
                const int cnt = (int)((e - k0) < (int64_t)(G * kIdxRegs) ? (e - k0) : (int64_t)(G * kIdxRegs));
                RawCols<WT, E> buf[2][kBatch];
                bool ok[2][kBatch];
                auto issue = [&](int b) {
#pragma unroll
                    for (int q = 0; q < kBatch; ++q) {
                        const int qq = b * kBatch + q;                       // index of the round
                        const long long row = __shfl(myRow[(b / kBatchesPerReg) < kIdxRegs ? b / kBatchesPerReg : 0],
                                                     groupBase + (qq % G), kWave);
                        const int64_t at = base + row * D;
                        ok[b & 1][q] = qq < cnt && row >= 0 && at + D <= numel && colOk;
                        if (ok[b & 1][q]) {
                            buf[b & 1][q].load(weights, at + c, D - c);
                        }
                    }
                };
                issue(0);
#pragma unroll
                for (int b = 0; b < kBatches; ++b) {
                    if (b + 1 < kBatches && (b + 1) * kBatch < cnt) {
                        issue(b + 1);
                    }
                    if (b * kBatch < cnt) {
#pragma unroll
                        for (int q = 0; q < kBatch; ++q) {
                            if (ok[b & 1][q]) {
#pragma unroll
                                for (int v = 0; v < E; ++v) {
                                    float x = buf[b & 1][q].value(v);
                                    if (mean) {
                                        x = x * scale;
                                    }
                                    acc[0][v] += x;
                                }
                            }
                        }
                    }
                }
            }
        } else {
        constexpr int kDepth = 2;
        for (int64_t k0 = s; k0 < e; k0 += G) {
            // G indices of the bag with one load; lane gl holds index k0 + gl
            const long long myRow = (k0 + gl < e) ? indices[k0 + gl] : -1;
            const int cnt = (int)((e - k0) < (int64_t)G ? (e - k0) : (int64_t)G);
            for (int q0 = 0; q0 < cnt; q0 += kDepth) {
                float buf[kDepth][NJ][E];
                bool ok[kDepth];
#pragma unroll
                for (int q = 0; q < kDepth; ++q) {
                    const int qq = q0 + q;
                    const long long row = __shfl(myRow, groupBase + (qq < G ? qq : 0), kWave);
                    const int64_t at = base + row * D;
                    // rows outside the weight buffer contribute nothing
                    ok[q] = qq < cnt && row >= 0 && at + D <= numel;
                    if (ok[q]) {
#pragma unroll
                        for (int j = 0; j < NJ; ++j) {
                            const int c = (j * G + gl) * E;
                            if (c < D) {
                                tbe_load_cols<WT, E>(buf[q][j], weights, at + c, D - c);
                            }
                        }
                    }
                }
#pragma unroll
                for (int q = 0; q < kDepth; ++q) {
                    if (ok[q]) {
#pragma unroll
                        for (int j = 0; j < NJ; ++j) {
                            if ((j * G + gl) * E < D) {
#pragma unroll
                                for (int v = 0; v < E; ++v) {
                                    float x = buf[q][j][v];
                                    if (mean) {
                                        x = x * scale;
                                    }
                                    acc[j][v] += x;
                                }
                            }
                        }
                    }
                }
            }
        }
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int c = (j * G + gl) * E;
            if (c < D) {
                *reinterpret_cast<float4*>(out + m.outOff + c) =
                    make_float4(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
                if constexpr (E == 8) {
                    if (c + 4 < D) {
                        *reinterpret_cast<float4*>(out + m.outOff + c + 4) =
                            make_float4(acc[j][4], acc[j][5], acc[j][6], acc[j][7]);
                    }
                }
            }
        }
    }
}

// ---- forward, no pooling: out[k, :] = row of indices[k] ----------------------------------------------------
template <typename WT>
__global__ __launch_bounds__(kBlock) void k_tbe_forward_nobag(const void* __restrict__ weights, int64_t numel,
                                                              const int64_t* __restrict__ wOff,
                                                              const int64_t* __restrict__ indices,
                                                              const int64_t* __restrict__ offsets, int T, int64_t B,
                                                              float* __restrict__ out, int D, int chunksPerRow)
{
    const int64_t nnz = offsets[(int64_t)T * B];
    const int64_t total = nnz * chunksPerRow;
#pragma unroll
    for (int q = 0; q < kItems; ++q) {
        const int64_t g = (int64_t)blockIdx.x * (kBlock * kItems) + q * kBlock + threadIdx.x;
        if (g >= total) {
            continue;
        }
        const int64_t k = g / chunksPerRow;
        const int c = (int)(g - k * chunksPerRow) * 4;
        // table of position k: largest t with offsets[t*B] <= k
        int lo = 0;
        int hi = T - 1;
        while (lo < hi) {
            int mid = (lo + hi + 1) >> 1;
            if (offsets[(int64_t)mid * B] <= k) {
                lo = mid;
            } else {
                hi = mid - 1;
            }
        }
        const int64_t row = indices[k];
        const int64_t at = wOff[lo] + row * D;
        float v[4] = {0.f, 0.f, 0.f, 0.f};
        if (row >= 0 && at + D <= numel) {
            tbe_load4<WT>(v, weights, at + c);
        }
        *reinterpret_cast<float4*>(out + k * D + c) = make_float4(v[0], v[1], v[2], v[3]);
    }
}

// ---- backward helpers ------------------------------------------------------------------------------------
// Segment boundaries in `indices` and the row descriptors of the update kernels.  Features that read one table carry
// the same hash_size_cumsum entry (and are adjacent); their positions form ONE segment, owned by the last feature of
// the group, and the features before it get empty segments: the rows of a table are then grouped across its features.
__global__ __launch_bounds__(kBlock) void k_tbe_prepare(void* weights, int wBf16, float* m1, float* m2,
                                                        const int64_t* __restrict__ wOff,
                                                        const int32_t* __restrict__ dOff,
                                                        const int64_t* __restrict__ offsets,
                                                        const int64_t* __restrict__ cumsum, int T, int64_t B,
                                                        int64_t* tb, RowsDesc* descs)
{
    for (int t = threadIdx.x; t <= T; t += kBlock) {
        int f = t;
        if (t < T) {
            while (f > 0 && cumsum[f - 1] == cumsum[t]) {
                --f;
            }
        }
        tb[t] = offsets[(int64_t)f * B];
        if (t < T) {
            RowsDesc d;
            const int64_t o = wOff[t];
            d.w = wBf16 ? static_cast<void*>(static_cast<uint16_t*>(weights) + o)
                        : static_cast<void*>(static_cast<float*>(weights) + o);
            d.s1 = m1 ? m1 + o : nullptr;
            d.s2 = m2 ? m2 + o : nullptr;
            d.dim = dOff[t + 1] - dOff[t];
            d.stride = d.dim;
            d.gradCol = 0;  // the list entries carry the whole offset of the gradient row, see k_tbe_bagmap
            descs[t] = d;
        }
    }
}

// One wave per bag: where the gradient row of each of the bag's positions starts, in units of 4 floats:
// grad_output[b, D_offsets[t]] for the pooled modes, grad_output[k, 0] for position k without pooling.  The update
// kernels read list entry * 4 floats past the gradient base, so one list may mix positions of several features.
__global__ __launch_bounds__(kBlock) void k_tbe_bagmap(const int64_t* __restrict__ offsets,
                                                       const int32_t* __restrict__ dOff, int T, int64_t B,
                                                       int64_t totalD, int nobag, int32_t* __restrict__ rowOf,
                                                       const int64_t* __restrict__ rows,
                                                       const int64_t* __restrict__ rowBase, uint32_t sentinel,
                                                       uint32_t* __restrict__ sortKey, uint32_t* __restrict__ sortVal)
{
    // sixteen lanes per bag: bags of a few dozen positions leave most of a whole wave idle
    constexpr int kBagLanes = 16;
    const int64_t bag = (int64_t)blockIdx.x * (kBlock / kBagLanes) + (threadIdx.x / kBagLanes);
    if (bag >= (int64_t)T * B) {
        return;
    }
    const int sub = threadIdx.x % kBagLanes;
    const int64_t s = offsets[bag];
    const int64_t e = offsets[bag + 1];
    const int t = (int)(bag / B);
    const int64_t b = bag - (int64_t)t * B;
    const int64_t D4 = (dOff[t + 1] - dOff[t]) / 4;
    const int32_t pooled = (int32_t)((b * totalD + dOff[t]) / 4);
    if (sortKey != nullptr) {
        // the grouping sort's input written here, where the table of a position is known from its bag: key = the row
        // in one numbering over all tables (the sentinel for a row outside its table), value = the gradient row
        // features that share a table have equal bases: the table ends where the next larger base begins
        const int64_t base = rowBase[t];
        int tl = t;
        while (tl + 1 < T && rowBase[tl + 1] == base) {
            ++tl;
        }
        const int64_t size = rowBase[tl + 1] - base;
        for (int64_t k = s + sub; k < e; k += kBagLanes) {
            const int64_t row = rows[k];
            sortKey[k] = (row >= 0 && row < size) ? (uint32_t)(base + row) : sentinel;
            sortVal[k] = (uint32_t)(nobag ? (int32_t)(k * D4) : pooled);
        }
        return;
    }
    for (int64_t k = s + sub; k < e; k += kBagLanes) {
        rowOf[k] = nobag ? (int32_t)(k * D4) : pooled;
    }
}

// Mean pooling: every position of bag (t, b) contributes grad[b, columns of t] / len(bag).  The quotient is the same
// for all positions of the bag, so it is formed once per bag and column here and the update kernels add plain rows.
__global__ __launch_bounds__(kBlock) void k_tbe_scale_grad(const float* __restrict__ grad,
                                                           const int64_t* __restrict__ offsets,
                                                           const int32_t* __restrict__ dOff, int T, int64_t B,
                                                           int64_t totalD, float* __restrict__ scaled)
{
    const int64_t total4 = B * (totalD / 4);
    for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total4; e += (int64_t)gridDim.x * kBlock) {
        const int64_t b = e / (totalD / 4);
        const int32_t col = (int32_t)(e - b * (totalD / 4)) * 4;
        // table of the column (table widths are multiples of 4, so the four columns share it)
        int lo = 0;
        int hi = T - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (dOff[mid] <= col) {
                lo = mid;
            } else {
                hi = mid - 1;
            }
        }
        const int64_t bag = (int64_t)lo * B + b;
        const int64_t len = offsets[bag + 1] - offsets[bag];
        const float sc = len > 0 ? 1.0f / (float)len : 1.0f;
        float4 g = *reinterpret_cast<const float4*>(grad + b * totalD + col);
        g.x = g.x * sc;
        g.y = g.y * sc;
        g.z = g.z * sc;
        g.w = g.w * sc;
        *reinterpret_cast<float4*>(scaled + b * totalD + col) = g;
    }
}

// Position lists -> gradient-row lists, in place: entry p becomes the start of p's gradient row.  Without this the
// update kernels would chase rowOf[p] in front of every gradient row, which serialises their loads.  total[2] = end
// of the last list.
__global__ __launch_bounds__(kBlock) void k_tbe_translate(const int64_t* __restrict__ total,
                                                          const int32_t* __restrict__ rowOf,
                                                          int32_t* __restrict__ posList)
{
    const int64_t m = total[2];
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < m; i += (int64_t)gridDim.x * kBlock) {
        posList[i] = rowOf[posList[i]];
    }
}

// slot of each touched row = its index, or -1 when it lies outside its table
__global__ __launch_bounds__(kBlock) void k_tbe_slots(const int64_t* __restrict__ uniq,
                                                      const int64_t* __restrict__ uoff, int T,
                                                      const int64_t* __restrict__ total,
                                                      const int64_t* __restrict__ hashSizeCumsum,
                                                      int64_t* __restrict__ slots)
{
    const int64_t R = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (R >= total[0]) {
        return;
    }
    const int t = find_segment(uoff, T, R);
    const int64_t rows = hashSizeCumsum[t + 1] - hashSizeCumsum[t];
    const int64_t row = uniq[R];
    slots[R] = (row >= 0 && row < rows) ? row : -1;
}

// Unique variant: distinct key R of the grouping is a place j in the caller's unique_ids (the sort key was
// unique_offsets[t] + unique_inverse[k]); its table row is unique_ids[j], or -1 when that lies outside the table.
__global__ __launch_bounds__(kBlock) void k_tbe_unique_rows(const int64_t* __restrict__ uniq,
                                                            const int64_t* __restrict__ total,
                                                            const int64_t* __restrict__ uniqueIds,
                                                            const int64_t* __restrict__ uniqueOffsets, int T,
                                                            const int64_t* __restrict__ hashSizeCumsum,
                                                            int64_t* __restrict__ slots)
{
    const int64_t R = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (R >= total[0]) {
        return;
    }
    const int64_t j = uniq[R];
    const int t = find_segment(uniqueOffsets, T, j);
    const int64_t rows = hashSizeCumsum[t + 1] - hashSizeCumsum[t];
    const int64_t row = uniqueIds[j];
    slots[R] = (row >= 0 && row < rows) ? row : -1;
}

}  // namespace recsdk

using namespace recsdk;

template <typename WT>
static int tbe_forward_t(const void* w, int64_t numel, const int64_t* wOff, const int32_t* dOff, int64_t totalD,
                         int32_t maxD, const int64_t* indices, const int64_t* offsets, int32_t T, int64_t B,
                         int64_t nnz, int32_t mode, float* out, hipStream_t s)
{
    if (mode == RECSDK_POOL_NONE) {
        if (nnz == 0) {
            return RECSDK_OK;
        }
        const int D = (int)(totalD / T);
        const int cpr = D / 4;
        const unsigned grid = (unsigned)cdiv(nnz * cpr, kBlock * kItems);
        RECSDK_LAUNCH(k_tbe_forward_nobag<WT>, dim3(grid), dim3(kBlock), s, w, numel, wOff, indices, offsets, T, B, out,
                      D, cpr);
        return RECSDK_OK;
    }
    const int mean = (mode == RECSDK_POOL_MEAN) ? 1 : 0;
    const int64_t bags = (int64_t)T * B;
    // bf16 rows: eight columns per lane (one 16-byte load), fp32 rows: four
    constexpr int kCols = sizeof(WT) == 2 ? 8 : 4;
    const int chunks = (maxD + kCols - 1) / kCols;
#define TBE_FWD(G, NJ)                                                                                               \
    do {                                                                                                             \
        const unsigned grid = (unsigned)cdiv(bags, (kBlock / G) * kFwdRounds);                                       \
        RECSDK_LAUNCH((k_tbe_forward<G, NJ, WT, kCols>), dim3(grid), dim3(kBlock), s, w, numel, wOff, dOff, indices, \
                      offsets, T, B, mean, out, totalD);                                                             \
    } while (0)
    if (chunks <= 4) {
        TBE_FWD(4, 1);
    } else if (chunks <= 8) {
        TBE_FWD(8, 1);
    } else if (chunks <= 16) {
        TBE_FWD(16, 1);
    } else if (chunks <= 32) {
        TBE_FWD(32, 1);
    } else if (chunks <= 64) {
        TBE_FWD(64, 1);
    } else if (chunks <= 128) {
        TBE_FWD(64, 2);
    } else if (chunks <= 256) {
        TBE_FWD(64, 4);
    } else {
        TBE_FWD(64, 8);
    }
#undef TBE_FWD
    return RECSDK_OK;
}

extern "C" int recsdk_tbe_forward(const void* d_dev_weights, int32_t weights_dtype, int64_t weights_numel,
                                  const int64_t* d_weights_offsets, const int32_t* d_D_offsets, int64_t total_D,
                                  int32_t max_D, const int64_t* d_indices, const int64_t* d_offsets, int32_t T,
                                  int64_t B, int64_t nnz, int32_t pooling_mode, float* d_out, void* stream)
{
    RECSDK_REQUIRE(weights_dtype == RECSDK_DT_F32 || weights_dtype == RECSDK_DT_BF16, RECSDK_EINVAL,
                   "recsdk_tbe_forward: weights must be fp32 or bf16");
    RECSDK_REQUIRE(T > 0 && B >= 0 && nnz >= 0 && total_D > 0 && max_D > 0, RECSDK_EINVAL,
                   "recsdk_tbe_forward: bad sizes");
    RECSDK_REQUIRE(max_D % 4 == 0 && total_D % 4 == 0 && max_D <= 2048, RECSDK_EINVAL,
                   "recsdk_tbe_forward: embedding dims must be multiples of 4 (the reference requires 8) and <= 2048");
    RECSDK_REQUIRE(pooling_mode >= RECSDK_POOL_SUM && pooling_mode <= RECSDK_POOL_NONE, RECSDK_EINVAL,
                   "recsdk_tbe_forward: bad pooling mode");
    RECSDK_REQUIRE(pooling_mode != RECSDK_POOL_NONE || total_D % T == 0, RECSDK_EINVAL,
                   "recsdk_tbe_forward: pooling NONE needs the same dim for every table");
    if (B == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_dev_weights && d_weights_offsets && d_D_offsets && d_offsets && d_out && (nnz == 0 || d_indices),
                   RECSDK_ENULL, "recsdk_tbe_forward: NULL argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (weights_dtype == RECSDK_DT_BF16) {
        return tbe_forward_t<uint16_t>(d_dev_weights, weights_numel, d_weights_offsets, d_D_offsets, total_D, max_D,
                                       d_indices, d_offsets, T, B, nnz, pooling_mode, d_out, s);
    }
    return tbe_forward_t<float>(d_dev_weights, weights_numel, d_weights_offsets, d_D_offsets, total_D, max_D, d_indices,
                                d_offsets, T, B, nnz, pooling_mode, d_out, s);
}

struct recsdk_tbe {
    int32_t maxTables = 0;
    int64_t maxNnz = 0;
    recsdk_unique_t* uq = nullptr;
    int64_t* tb = nullptr;       // [T+1] table boundaries in indices
    RowsDesc* descs = nullptr;   // [T]
    int32_t* rowOf = nullptr;    // [nnz] sample of each position
    float* scaled = nullptr;     // mean pooling: the gradient divided by the bag lengths, [B, total_D] (grown on demand)
    int64_t scaledCap = 0;
    int64_t* slots = nullptr;    // [nnz] row index of each touched row (or -1)
    int64_t totalRows = -1;      // rows of all tables, read from hash_size_cumsum on the first backward call
    const int64_t* sizesFrom = nullptr;
    int32_t sizesT = 0;
    hipStream_t side = nullptr;
    hipEvent_t evFork = nullptr;
    hipEvent_t evJoin = nullptr;
    hipEvent_t evMeta = nullptr;
};

extern "C" int recsdk_tbe_destroy(recsdk_tbe_t* h)
{
    if (h == nullptr) {
        return RECSDK_OK;
    }
    recsdk_unique_destroy(h->uq);
    void* ptrs[] = {h->tb, h->descs, h->rowOf, h->scaled, h->slots};
    for (void* p : ptrs) {
        if (p) {
            (void)hipFree(p);
        }
    }
    if (h->evFork) {
        (void)hipEventDestroy(h->evFork);
    }
    if (h->evJoin) {
        (void)hipEventDestroy(h->evJoin);
    }
    if (h->evMeta) {
        (void)hipEventDestroy(h->evMeta);
    }
    if (h->side) {
        (void)hipStreamDestroy(h->side);
    }
    delete h;
    return RECSDK_OK;
}

extern "C" int recsdk_tbe_create(int32_t max_tables, int64_t max_nnz, recsdk_tbe_t** out)
{
    RECSDK_REQUIRE(out != nullptr, RECSDK_ENULL, "recsdk_tbe_create: out is NULL");
    RECSDK_REQUIRE(max_tables > 0 && max_nnz > 0, RECSDK_EINVAL, "recsdk_tbe_create: sizes must be positive");
    auto* h = new recsdk_tbe();
    h->maxTables = max_tables;
    h->maxNnz = max_nnz;
    int rc = recsdk_unique_create(max_nnz, max_tables, &h->uq);
    if (rc != RECSDK_OK) {
        delete h;
        return rc;
    }
    bool ok = true;
    auto alloc = [&](auto** p, size_t bytes) {
        if (ok && hipMalloc(reinterpret_cast<void**>(p), bytes) != hipSuccess) {
            ok = false;
        }
    };
    alloc(&h->tb, sizeof(int64_t) * (max_tables + 1));
    alloc(&h->descs, sizeof(RowsDesc) * max_tables);
    alloc(&h->rowOf, sizeof(int32_t) * max_nnz);
    alloc(&h->slots, sizeof(int64_t) * max_nnz);
    if (ok && (hipStreamCreateWithFlags(&h->side, hipStreamNonBlocking) != hipSuccess ||
               hipEventCreateWithFlags(&h->evFork, hipEventDisableTiming) != hipSuccess ||
               hipEventCreateWithFlags(&h->evJoin, hipEventDisableTiming) != hipSuccess ||
               hipEventCreateWithFlags(&h->evMeta, hipEventDisableTiming) != hipSuccess)) {
        ok = false;
    }
    if (!ok) {
        (void)hipGetLastError();
        recsdk_tbe_destroy(h);
        set_error("recsdk_tbe_create: allocation failed");
        return RECSDK_ENOMEM;
    }
    *out = h;
    return RECSDK_OK;
}

// The unique arrays are all NULL (plain form) or all given (the caller's distinct rows and inverse index).
static int tbe_backward_impl(recsdk_tbe_t* h, int32_t optim, const float* d_grad_output, void* d_dev_weights,
                             int32_t weights_dtype, const int64_t* d_weights_offsets, const int32_t* d_D_offsets,
                             int64_t total_D, int32_t max_D, const int64_t* d_hash_size_cumsum, const int64_t* d_indices,
                             const int64_t* d_offsets, int32_t T, int64_t B, int64_t nnz, int32_t pooling_mode,
                             const int64_t* d_unique_ids, const int64_t* d_unique_offsets,
                             const int64_t* d_unique_inverse, int64_t num_unique, float* d_momentum1,
                             float* d_momentum2, float lr, float eps, float beta1, float beta2, int64_t iter,
                             void* stream)
{
    const bool unique = d_unique_ids != nullptr;
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "recsdk_tbe_backward: NULL handle");
    RECSDK_REQUIRE(optim == RECSDK_OPT_SGD || optim == RECSDK_OPT_ADAGRAD || optim == RECSDK_OPT_ADAM, RECSDK_EINVAL,
                   "recsdk_tbe_backward: unknown optimizer");
    RECSDK_REQUIRE(weights_dtype == RECSDK_DT_F32 || weights_dtype == RECSDK_DT_BF16, RECSDK_EINVAL,
                   "recsdk_tbe_backward: weights must be fp32 or bf16");
    RECSDK_REQUIRE(T > 0 && T <= h->maxTables && nnz >= 0 && nnz <= h->maxNnz, RECSDK_ECAPACITY,
                   "recsdk_tbe_backward: T or nnz exceeds what the handle was created for");
    RECSDK_REQUIRE(pooling_mode >= RECSDK_POOL_SUM && pooling_mode <= RECSDK_POOL_NONE, RECSDK_EINVAL,
                   "recsdk_tbe_backward: bad pooling mode");
    RECSDK_REQUIRE(max_D > 0 && max_D % 4 == 0 && max_D <= 2048 && total_D % 4 == 0, RECSDK_EINVAL,
                   "recsdk_tbe_backward: embedding dims must be multiples of 4 and <= 2048");
    const bool nobag = pooling_mode == RECSDK_POOL_NONE;
    RECSDK_REQUIRE(!nobag || total_D == (int64_t)max_D * T, RECSDK_EINVAL,
                   "recsdk_tbe_backward: pooling NONE needs the same dim for every table");
    // the lists name a gradient row by its start in units of 4 floats, as a 32-bit number
    RECSDK_REQUIRE((nobag ? nnz * max_D : B * total_D) / 4 < (int64_t)0x7fffffff, RECSDK_EINVAL,
                   "recsdk_tbe_backward: grad_output holds 2^33 elements or more");
    // op_host/backward_codegen_adagrad_unweighted_exact.cpp:91-96 rejects beta == 1
    RECSDK_REQUIRE(optim != RECSDK_OPT_ADAM || (beta1 != 1.0f && beta2 != 1.0f), RECSDK_EINVAL,
                   "recsdk_tbe_backward: beta1 and beta2 can not be 1.0");
    if (nnz == 0 || B == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_grad_output && d_dev_weights && d_weights_offsets && d_D_offsets && d_hash_size_cumsum &&
                       d_offsets && (unique || d_indices),
                   RECSDK_ENULL, "recsdk_tbe_backward: NULL argument");
    RECSDK_REQUIRE(!unique || (d_unique_offsets != nullptr && d_unique_inverse != nullptr), RECSDK_ENULL,
                   "recsdk_tbe_backward_unique: unique_offsets or unique_inverse is NULL");
    RECSDK_REQUIRE(!unique || (num_unique > 0 && num_unique < (int64_t)0xFFFFFFFFLL), RECSDK_EINVAL,
                   "recsdk_tbe_backward_unique: num_unique must be in (0, 2^32)");
    RECSDK_REQUIRE(optim == RECSDK_OPT_SGD || d_momentum1 != nullptr, RECSDK_ENULL,
                   "recsdk_tbe_backward: momentum1 is NULL");
    RECSDK_REQUIRE(optim != RECSDK_OPT_ADAM || d_momentum2 != nullptr, RECSDK_ENULL,
                   "recsdk_tbe_backward: momentum2 is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int mean = (pooling_mode == RECSDK_POOL_MEAN) ? 1 : 0;
    const int wBf16 = (weights_dtype == RECSDK_DT_BF16) ? 1 : 0;
    // features of one table are told by equal table starts: hash_size_cumsum, or unique_offsets in the unique form
    // (training/.../test_split_embedding_codegen_lookup_function.py:268-287 builds them with that property)
    RECSDK_LAUNCH(k_tbe_prepare, dim3(1), dim3(kBlock), s, d_dev_weights, wBf16, d_momentum1, d_momentum2,
                  d_weights_offsets, d_D_offsets, d_offsets, d_hash_size_cumsum, T, B, h->tb, h->descs);
    const float* grad = d_grad_output;
    if (mean) {
        const int64_t need = B * total_D;
        if (h->scaledCap < need) {
            if (h->scaled != nullptr) {
                RECSDK_HIP_TRY(hipFree(h->scaled));  // waits for the device: no kernel still reads it
                h->scaled = nullptr;
                h->scaledCap = 0;
            }
            RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&h->scaled), sizeof(float) * need));
            h->scaledCap = need;
        }
        const unsigned grid = (unsigned)std::min<int64_t>(cdiv(need / 4, kBlock), 256 * 32);
        RECSDK_LAUNCH(k_tbe_scale_grad, dim3(grid), dim3(kBlock), s, d_grad_output, d_offsets, d_D_offsets, T, B,
                      total_D, h->scaled);
        grad = h->scaled;
    }
    // The number of rows of all tables decides how the touched rows are grouped; it is read once per handle (the
    // tables of a module do not change size) because the bit count of the sort is a host-side argument.
    if (!unique && (h->totalRows < 0 || h->sizesFrom != d_hash_size_cumsum || h->sizesT != T)) {
        int64_t total = 0;
        RECSDK_HIP_TRY(hipMemcpyAsync(&total, d_hash_size_cumsum + T, sizeof(int64_t), hipMemcpyDeviceToHost, s));
        RECSDK_HIP_TRY(hipStreamSynchronize(s));
        h->totalRows = total;
        h->sizesFrom = d_hash_size_cumsum;
        h->sizesT = T;
    }
    const UniqueView* v = recsdk_unique_view(h->uq);
    int rc;
    // RECSDK_TBE_HASHED=1 forces the hashed path (the tests run both)
    const char* forceHashed = getenv("RECSDK_TBE_HASHED");
    const bool hashed = forceHashed != nullptr && forceHashed[0] == '1';
    // one wave per bag: the gradient row of every position and, for the grouping sort, its key (the bag's table
    // gives the row base, so no kernel has to search the table of every position again)
    const unsigned bagGrid = (unsigned)cdiv((int64_t)T * B, kBlock / 16);   // sixteen lanes per bag
    uint32_t* sortKey = nullptr;
    uint32_t* sortVal = nullptr;
    rc = recsdk_unique_group_input(h->uq, &sortKey, &sortVal);
    if (rc != RECSDK_OK) {
        return rc;
    }
    if (unique) {
        // the caller's inverse index names the group of every position: stable sort of (unique_offsets[t] +
        // unique_inverse[k], gradient row of k) over log2(num_unique) bits instead of log2(rows of all tables);
        // distinct key R of the grouping is then a place in unique_ids
        RECSDK_LAUNCH(k_tbe_bagmap, dim3(bagGrid), dim3(kBlock), s, d_offsets, d_D_offsets, T, B, total_D, nobag ? 1 : 0,
                      h->rowOf, d_unique_inverse, d_unique_offsets, (uint32_t)num_unique, sortKey, sortVal);
        rc = recsdk_unique_run_grouped(h->uq, d_unique_inverse, h->tb, d_unique_offsets, T, nnz, num_unique, nullptr,
                                       h->slots, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
        RECSDK_LAUNCH(k_tbe_unique_rows, dim3((unsigned)cdiv(nnz, kBlock)), dim3(kBlock), s, v->uniq, v->total,
                      d_unique_ids, d_unique_offsets, T, d_hash_size_cumsum, h->slots);
    } else if (!hashed && h->totalRows > 0 && h->totalRows < (int64_t)0xFFFFFFFFLL) {
        // stable sort of (table base + row, gradient row of the position): the lists come out as gradient rows
        RECSDK_LAUNCH(k_tbe_bagmap, dim3(bagGrid), dim3(kBlock), s, d_offsets, d_D_offsets, T, B, total_D, nobag ? 1 : 0,
                      h->rowOf, d_indices, d_hash_size_cumsum, (uint32_t)h->totalRows, sortKey, sortVal);
        rc = recsdk_unique_run_grouped(h->uq, d_indices, h->tb, d_hash_size_cumsum, T, nnz, h->totalRows, nullptr,
                                       h->slots, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
    } else {
        // 2^32 rows or more: hashed dedup, then the position lists are rewritten to gradient rows
        RECSDK_LAUNCH(k_tbe_bagmap, dim3(bagGrid), dim3(kBlock), s, d_offsets, d_D_offsets, T, B, total_D, nobag ? 1 : 0,
                      h->rowOf, (const int64_t*)nullptr, (const int64_t*)nullptr, 0u, (uint32_t*)nullptr,
                      (uint32_t*)nullptr);
        rc = recsdk_unique_run_lists(h->uq, d_indices, nullptr, h->tb, T, nnz, 0, 0, false, stream);
        if (rc != RECSDK_OK) {
            return rc;
        }
        {
            const unsigned grid = (unsigned)cdiv(nnz, kBlock);
            RECSDK_LAUNCH(k_tbe_slots, dim3(grid), dim3(kBlock), s, v->uniq, v->uoff, T, v->total, d_hash_size_cumsum,
                          h->slots);
        }
        if (v->listsReady != nullptr) {
            RECSDK_HIP_TRY(hipStreamWaitEvent(s, v->listsReady, 0));
        }
        {
            const unsigned grid = (unsigned)std::min<int64_t>(cdiv(nnz, kBlock), 256 * 32);
            RECSDK_LAUNCH(k_tbe_translate, dim3(grid), dim3(kBlock), s, v->total, h->rowOf, v->posList);
        }
    }
    ApplyCtx c;
    c.d_rows = h->descs;
    c.T = T;
    c.maxDim = max_D;
    c.wBf16 = wBf16 != 0;
    c.gradShared = true;
    c.v = v;
    c.uq = h->uq;
    c.d_slots = h->slots;
    c.g = GradSrc{grad, 4};  // list entries count in units of 4 floats
    OptParams prm{};
    prm.lr = lr;
    prm.eps = eps;
    prm.beta1 = beta1;
    prm.beta2 = beta2;
    if (optim == RECSDK_OPT_ADAM) {
        // op_host/backward_codegen_adagrad_unweighted_exact.cpp:98-108: pow in double, narrowed to float
        float b1c = static_cast<float>(1 - pow(static_cast<double>(beta1), static_cast<double>(iter)));
        float b2c = static_cast<float>(1 - pow(static_cast<double>(beta2), static_cast<double>(iter)));
        float beta2sqrt = sqrtf(b2c) / b1c;
        prm.optim = kOptTbeAdam;
        prm.stepSize = -lr * beta2sqrt;
    } else if (optim == RECSDK_OPT_ADAGRAD) {
        prm.optim = kOptTbeAdagrad;
    } else {
        prm.optim = kOptTbeSgd;
        prm.stepSize = -lr;
    }
    c.prm = prm;
    c.stream = s;
    c.side = h->side;
    c.evFork = h->evFork;
    c.evJoin = h->evJoin;
    c.evMeta = h->evMeta;
    return apply_launch(c);
}

extern "C" int recsdk_tbe_backward(recsdk_tbe_t* h, int32_t optim, const float* d_grad_output, void* d_dev_weights,
                                   int32_t weights_dtype, const int64_t* d_weights_offsets, const int32_t* d_D_offsets,
                                   int64_t total_D, int32_t max_D, const int64_t* d_hash_size_cumsum,
                                   const int64_t* d_indices, const int64_t* d_offsets, int32_t T, int64_t B,
                                   int64_t nnz, int32_t pooling_mode, float* d_momentum1, float* d_momentum2, float lr,
                                   float eps, float beta1, float beta2, int64_t iter, void* stream)
{
    RECSDK_REQUIRE(nnz == 0 || B == 0 || d_indices != nullptr, RECSDK_ENULL, "recsdk_tbe_backward: d_indices is NULL");
    return tbe_backward_impl(h, optim, d_grad_output, d_dev_weights, weights_dtype, d_weights_offsets, d_D_offsets,
                             total_D, max_D, d_hash_size_cumsum, d_indices, d_offsets, T, B, nnz, pooling_mode, nullptr,
                             nullptr, nullptr, 0, d_momentum1, d_momentum2, lr, eps, beta1, beta2, iter, stream);
}

extern "C" int recsdk_tbe_backward_unique(recsdk_tbe_t* h, int32_t optim, const float* d_grad_output,
                                          void* d_dev_weights, int32_t weights_dtype, const int64_t* d_weights_offsets,
                                          const int32_t* d_D_offsets, int64_t total_D, int32_t max_D,
                                          const int64_t* d_hash_size_cumsum, const int64_t* d_offsets, int32_t T,
                                          int64_t B, int64_t nnz, int32_t pooling_mode, const int64_t* d_unique_ids,
                                          const int64_t* d_unique_offsets, const int64_t* d_unique_inverse,
                                          int64_t num_unique, float* d_momentum1, float* d_momentum2, float lr,
                                          float eps, float beta1, float beta2, int64_t iter, void* stream)
{
    RECSDK_REQUIRE(nnz == 0 || B == 0 || d_unique_ids != nullptr, RECSDK_ENULL,
                   "recsdk_tbe_backward_unique: d_unique_ids is NULL");
    if (nnz == 0 || B == 0) {
        return RECSDK_OK;
    }
    return tbe_backward_impl(h, optim, d_grad_output, d_dev_weights, weights_dtype, d_weights_offsets, d_D_offsets,
                             total_D, max_D, d_hash_size_cumsum, nullptr, d_offsets, T, B, nnz, pooling_mode,
                             d_unique_ids, d_unique_offsets, d_unique_inverse, num_unique, d_momentum1, d_momentum2, lr,
                             eps, beta1, beta2, iter, stream);
}
