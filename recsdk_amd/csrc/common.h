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

void set_error(const char* fmt, ...);

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

#endif  // __HIPCC__

}  // namespace recsdk

#endif
