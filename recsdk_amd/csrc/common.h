// Shared host/device helpers of the HIP library (gfx950, wave64).
#ifndef RECSDK_CSRC_COMMON_H
#define RECSDK_CSRC_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/recsdk_hip.h"

namespace recsdk {

constexpr int kWave = 64;
constexpr int kBlock = 256;                 // threads per block used by the streaming kernels
constexpr int kItems = 4;                   // items per thread in scan tiles
constexpr int kTile = kBlock * kItems;      // 1024 items per scan tile
constexpr long long kEmptyKey = -1;         // INVALID_KEY_VALUE doubles as the empty marker of hash slots
constexpr long long kTombKey = (long long)0x8000000000000000ULL;  // erased slot of the persistent tables
constexpr int kListMax = 64;                // segments up to this length are reduced by one wave
constexpr int kHugeMin = 1024;              // keys seen more often than this take 16-column slices
constexpr int kVeryHugeMin = 4096;          // ... and more often than this 8-column slices (longest chains)
constexpr int kTwoLevelMin = 1024;          // keys seen more often than this are summed chunk by chunk: chunks of
constexpr int kChunkRows = 256;             // kChunkRows rows in order, then the chunk sums in order
constexpr int kSmallKeys = 4096;            // batches up to this size (and kSmallTables tables) take the one-launch
constexpr int kSmallTables = 64;            // paths: such a batch is bound by its launches, not by its traffic
constexpr int kSmallBlock = 1024;           // threads of the one block that runs such a path

void set_error(const char* fmt, ...);

// Largest batch (keys per call) that takes the one-launch paths; recsdk_set_small_batch_keys changes it.
int64_t small_batch_keys();

#define RECSDK_HIP_TRY(expr)                                                                   \
    do {                                                                                       \
        hipError_t _e = (expr);                                                                \
        if (_e != hipSuccess) {                                                                \
            ::recsdk::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
            return RECSDK_EHIP;                                                                \
        }                                                                                      \
    } while (0)

#define RECSDK_REQUIRE(cond, code, msg)          \
    do {                                         \
        if (!(cond)) {                           \
            ::recsdk::set_error("%s", msg);      \
            return code;                         \
        }                                        \
    } while (0)

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Optional per-kernel timing with HIP events (off by default; see recsdk_profile_* in the header).
// A KernelScope brackets one kernel launch with a start/stop event pair on the launch stream when the
// kernel's name is selected.
bool profile_begin(const char* name, hipStream_t stream, int* slot);
void profile_end(int slot, hipStream_t stream);

struct KernelScope {
    int slot = -1;
    hipStream_t stream;
    KernelScope(const char* name, hipStream_t s) : stream(s) { profile_begin(name, s, &slot); }
    ~KernelScope()
    {
        if (slot >= 0) {
            profile_end(slot, stream);
        }
    }
};

// Checks the launch of the kernel just enqueued.
#define RECSDK_LAUNCH_CHECK() RECSDK_HIP_TRY(hipGetLastError())

// Launch `kernel` on `stream` (timed when profiling selects its name) and check the launch.
#define RECSDK_LAUNCH(kernel, grid, block, stream, ...)                               \
    do {                                                                              \
        {                                                                             \
            ::recsdk::KernelScope _scope(#kernel, stream);                            \
            hipLaunchKernelGGL(kernel, grid, block, 0, stream, __VA_ARGS__);          \
        }                                                                             \
        RECSDK_LAUNCH_CHECK();                                                        \
    } while (0)

// The same with an explicit name for the per-kernel timing (two launch sites of one template that should be told apart).
#define RECSDK_LAUNCH_AS(name, kernel, grid, block, stream, ...)                      \
    do {                                                                              \
        {                                                                             \
            ::recsdk::KernelScope _scope(name, stream);                               \
            hipLaunchKernelGGL(kernel, grid, block, 0, stream, __VA_ARGS__);          \
        }                                                                             \
        RECSDK_LAUNCH_CHECK();                                                        \
    } while (0)

#ifdef __HIPCC__

__device__ __forceinline__ uint64_t hash64(uint64_t x)
{
    x ^= x >> 33;
    x *= 0xff51afd7ed558ccdULL;
    x ^= x >> 33;
    x *= 0xc4ceb9fe1a85ec53ULL;
    x ^= x >> 33;
    return x;
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Largest t in [0, T) with off[t] <= i (off non-decreasing, off[0] <= i < off[T]).
__device__ __forceinline__ int find_segment(const int64_t* __restrict__ off, int T, int64_t i)
{
    int lo = 0;
    int hi = T - 1;
    while (lo < hi) {
        int mid = (lo + hi + 1) >> 1;
        if (off[mid] <= i) {
            lo = mid;
        } else {
            hi = mid - 1;
        }
    }
    return lo;
}

// Advance a segment hint: t such that off[t] <= i < off[t+1], starting from a t with off[t] <= i.
__device__ __forceinline__ int advance_segment(const int64_t* __restrict__ off, int t, int64_t i)
{
    while (i >= off[t + 1]) {
        ++t;
    }
    return t;
}

// counters[idx] += number of lanes with pred, with one atomic per distinct idx among the calling lanes instead of
// one per lane (thousands of atomics on one address serialise in L2).  May be called in divergent code.
__device__ __forceinline__ void wave_count_add(unsigned long long* counters, int idx, bool pred)
{
    unsigned long long todo = __ballot(pred);
    while (todo != 0) {
        const int leader = __ffsll((long long)todo) - 1;
        const int lidx = __shfl(idx, leader, kWave);
        const unsigned long long same = __ballot(pred && idx == lidx);
        if (lane_id() == leader) {
            atomicAdd(counters + lidx, (unsigned long long)__popcll(same));
        }
        todo &= ~same;
    }
}

// Every calling lane with pred takes a distinct value of *counter (one atomic per wave; the values of a wave are
// consecutive, in lane order).  Lanes without pred get an unspecified value.  May be called in divergent code.
__device__ __forceinline__ unsigned long long wave_take(unsigned long long* counter, bool pred)
{
    const unsigned long long mask = __ballot(pred);
    if (mask == 0) {
        return 0;
    }
    const int leader = __ffsll((long long)mask) - 1;
    unsigned long long base = 0;
    if (lane_id() == leader) {
        base = atomicAdd(counter, (unsigned long long)__popcll(mask));
    }
    const uint32_t lo = __shfl((uint32_t)base, leader, kWave);
    const uint32_t hi = __shfl((uint32_t)(base >> 32), leader, kWave);
    const unsigned long long below = mask & ((1ull << lane_id()) - 1ull);
    return (((unsigned long long)hi << 32) | lo) + (unsigned long long)__popcll(below);
}

// Unordered append of sparse (64-bit, 32-bit) pairs found by a block's grid-stride loop: the pairs collect in LDS and
// go out with ONE global atomic per flush.  A compaction whose hits are rare (one in hundreds of slots) gains nothing
// from wave aggregation and one atomic per hit serialises on the counter's address (about 10 ns each).
// Use: every thread of the block calls push() once per loop round (pred = it has a pair), then maybe_flush(); after
// the loop flush().  The loop must have the same trip count for all threads of the block.
template <int CAP>
struct BlockAppend {
    unsigned long long a[CAP];
    uint32_t b[CAP];
    uint32_t count;
    unsigned long long base;

    __device__ __forceinline__ void init()
    {
        if (threadIdx.x == 0) {
            count = 0;
        }
        __syncthreads();
    }
    __device__ __forceinline__ void push(bool pred, unsigned long long va, uint32_t vb)
    {
        if (pred) {
            const uint32_t at = atomicAdd(&count, 1u);  // LDS atomic; never reaches CAP, see maybe_flush
            a[at] = va;
            b[at] = vb;
        }
    }
    __device__ __forceinline__ void flush(unsigned long long* counter, unsigned long long* outA, uint32_t* outB,
                                          int64_t cap)
    {
        __syncthreads();
        const uint32_t m = count;
        if (m != 0) {
            if (threadIdx.x == 0) {
                base = atomicAdd(counter, (unsigned long long)m);
            }
            __syncthreads();
            for (uint32_t j = threadIdx.x; j < m; j += blockDim.x) {
                if ((int64_t)(base + j) < cap) {
                    outA[base + j] = a[j];
                    if (outB != nullptr) {
                        outB[base + j] = b[j];
                    }
                }
            }
            __syncthreads();
            if (threadIdx.x == 0) {
                count = 0;
            }
        }
        __syncthreads();
    }
    // flush when another round of `perThread` pairs per thread might not fit
    __device__ __forceinline__ void maybe_flush(unsigned long long* counter, unsigned long long* outA, uint32_t* outB,
                                                int64_t cap, uint32_t perThread = 1)
    {
        __syncthreads();
        if (count + perThread * blockDim.x > (uint32_t)CAP) {  // uniform: every thread reads the same count after the barrier
            flush(counter, outA, outB, cap);
        }
    }
};

// Inclusive scan over the 64 lanes of a wave.
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v)
{
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        uint32_t o = __shfl_up(v, d, kWave);
        if (lane_id() >= d) {
            v += o;
        }
    }
    return v;
}

// Exclusive scan of one value per thread over a 256-thread block; *total gets the block sum.
// `smem` must hold 4 uint32 (one per wave) + 1.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* smem, uint32_t* total)
{
    uint32_t inc = wave_inclusive_scan(v);
    int w = threadIdx.x >> 6;
    if (lane_id() == kWave - 1) {
        smem[w] = inc;
    }
    __syncthreads();
    uint32_t base = 0;
    uint32_t sum = 0;
#pragma unroll
    for (int k = 0; k < kBlock / kWave; ++k) {
        uint32_t s = smem[k];
        if (k < w) {
            base += s;
        }
        sum += s;
    }
    __syncthreads();
    *total = sum;
    return base + inc - v;
}

// The same for a block of NT threads (a multiple of 64, at most 1024); `smem` must hold NT / 64 uint32.
template <int NT>
__device__ __forceinline__ uint32_t block_exclusive_scan_n(uint32_t v, uint32_t* smem, uint32_t* total)
{
    constexpr int kW = NT / kWave;
    uint32_t inc = wave_inclusive_scan(v);
    const int w = threadIdx.x >> 6;
    if (lane_id() == kWave - 1) {
        smem[w] = inc;
    }
    __syncthreads();
    uint32_t base = 0;
    uint32_t sum = 0;
#pragma unroll
    for (int k = 0; k < kW; ++k) {
        const uint32_t s = smem[k];
        if (k < w) {
            base += s;
        }
        sum += s;
    }
    __syncthreads();
    *total = sum;
    return base + inc - v;
}

// Rank at the first key of every segment (and the total, for segments that start at or past n): the exclusive scan
// of the tile sums at the segment's tile plus the flags set before the segment's first key inside that tile.
// `flags` holds one byte (0 or 1) per key, whole tiles of it, 16-byte aligned.  Called by a whole block of kBlock
// threads: one wave per segment, the flags of a tile in one 16-byte load per lane, eight segments in flight per wave
// (a serial walk over the tile's bytes made this the slowest part of the single-block scan kernels).
template <typename OUT>
__device__ __forceinline__ void segment_start_ranks(const uint8_t* __restrict__ flags,
                                                    const uint32_t* __restrict__ tileBase,
                                                    const int64_t* __restrict__ off, int T, int64_t n, uint32_t total,
                                                    OUT* __restrict__ out)
{
    static_assert(kTile == kWave * 16, "one 16-byte load per lane covers a tile");
    constexpr int kWaves = kBlock / kWave;
    constexpr int kFlight = 8;
    const int lane = lane_id();
    for (int t0 = threadIdx.x >> 6; t0 <= T; t0 += kWaves * kFlight) {
        uint32_t part[kFlight];
        uint32_t base[kFlight];
#pragma unroll
        for (int q = 0; q < kFlight; ++q) {
            const int t = t0 + q * kWaves;
            part[q] = 0;
            base[q] = total;
            if (t <= T) {
                const int64_t o = off[t];
                if (o < n) {
                    const int64_t tile = o / kTile;
                    base[q] = tileBase[tile];
                    const int64_t first = tile * kTile + lane * 16;
                    if (first < o) {
                        const uint4 v = *reinterpret_cast<const uint4*>(flags + first);
                        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
                        const int valid = (int)(o - first < 16 ? o - first : 16);
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            const int nb = valid - 4 * k;
                            const uint32_t mask = nb >= 4 ? 0x01010101u : (nb <= 0 ? 0u : (0x01010101u >> (8 * (4 - nb))));
                            part[q] += (uint32_t)__popc(w[k] & mask);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int q = 0; q < kFlight; ++q) {
            uint32_t p = part[q];
#pragma unroll
            for (int d = kWave / 2; d > 0; d >>= 1) {
                p += __shfl_down(p, d, kWave);
            }
            const int t = t0 + q * kWaves;
            if (lane == 0 && t <= T) {
                out[t] = (OUT)(base[q] + p);
            }
        }
    }
}

#endif  // __HIPCC__

}  // namespace recsdk

#endif
