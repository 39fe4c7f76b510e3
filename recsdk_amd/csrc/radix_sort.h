// Stable least-significant-digit radix sort of (key, 32-bit value) pairs for gfx950, written for this library's
// index work: positions by the rank of their key, gradient rows by table row, cache slots by their stamps.
//
// One counting kernel reads the keys once and counts the digits of every pass (a second, tiny one adds the blocks'
// counts up); each pass is then ONE kernel
// ("one sweep"): a block takes the next tile of the input in order, ranks its keys inside the tile with wave-wide
// digit matching (64-lane ballots, one LDS add per distinct digit and wave), publishes the tile's digit counts,
// obtains the counts of all earlier tiles by looking back over their published words (decoupled look-back: a tile
// never waits for more than its predecessors' counting, not for their scatter), and writes keys and values to their
// final places of the pass through LDS, so that equal digits leave the block as runs.
//
// Nothing here calls hipMemsetAsync, and no state survives a call: the look-back words and the tile tickets of all
// passes are cleared by the counting kernel, so a captured stream holds kernel nodes only and the workspace needs no
// initialisation.  There is no fence either: blocks of one kernel talk through relaxed device-wide atomics whose
// words carry the data themselves (a release fence writes the L2 back and costs tens of microseconds here).
// Calls that share a workspace must not overlap on the device.
#ifndef RECSDK_CSRC_RADIX_SORT_H
#define RECSDK_CSRC_RADIX_SORT_H

#include <algorithm>
#include <type_traits>

#include "common.h"

namespace recsdk {
namespace rsort {

constexpr int kMaxPasses = 8;         // 64-bit keys in digits of 8 bits
constexpr int kMaxRadix = 1024;       // digits of at most 10 bits
constexpr uint32_t kFlagAggregate = 1u << 30;   // the word holds this tile's count
constexpr uint32_t kFlagInclusive = 2u << 30;   // the word holds the count of this tile and all before it
constexpr uint32_t kFlagMask = 3u << 30;
constexpr uint32_t kValueMask = ~kFlagMask;
constexpr int kLookBack = 8;         // predecessors polled per round of a tile's look-back
constexpr int kHistThreads = 1024;
constexpr int kHistItems = 8;         // keys per thread and round of the histogram kernel's loop
constexpr int kHistMaxBlocks = 512;   // blocks of the histogram kernel at most (two per compute unit)
constexpr int kHistPartialWords = 3072;   // digits times passes at most: 3 x 1024 (32-bit keys), 8 x 256 (64-bit keys)
constexpr int kTicketWords = kMaxPasses;

// Device memory of one sorter; nothing in it has to be initialised.
struct Workspace {
    uint32_t* totals = nullptr;    // [kMaxPasses][kMaxRadix] keys per digit, per pass
    uint32_t* ticket = nullptr;    // [kMaxPasses] next tile of every pass
    uint32_t* partial = nullptr;   // [kHistMaxBlocks][kHistPartialWords] digit counts of every block of the counting kernel
    uint32_t* status = nullptr;    // look-back words: per pass, tile and digit
    int64_t statusWords = 0;
    void* tmpKeys = nullptr;       // intermediate results of passes that do not write the caller's output
    uint32_t* tmpVals = nullptr;
    int64_t maxN = 0;
    int keyBytes = 4;
};

// Digit width that needs the fewest passes for `bits` key bits (the narrowest on a tie: smaller tables in LDS).
inline int digit_bits_for(int bits)
{
    int best = 8;
    for (int digit = 9; digit <= 10; ++digit) {
        if ((bits + digit - 1) / digit < (bits + best - 1) / best) {
            best = digit;
        }
    }
    return best;
}

// Tile shapes.  Small sorts are bound by the chain launch -> ticket -> load -> rank -> look-back of a single tile
// (small tiles, many blocks), big ones by the work per pair (big tiles: fewer tickets and look-back words, longer runs
// of equal digits in the stores; at 16 pairs per thread half as many waves meet at every barrier).  Measured on
// 32-bit pairs: 131072 pairs over 17 bits 33 / 28 / 31 us with tiles of 2048 / 4096 / 8192 pairs, 1.7 M pairs over
// 19 bits 156 / 83 / 60 us (66 us as 512 threads x 16), 10.9 M pairs over 26 bits 264 us as 1024 x 8, 221 us as 512 x 16.
enum TileShape { kShapeSmall = 0, kShapeMedium = 1, kShapeBig = 2, kShapeHuge = 3 };
constexpr int kTilePairs[4] = {256 * 8, 512 * 8, 1024 * 8, 512 * 16};
constexpr int64_t kMediumTileMin = 100000;
constexpr int64_t kBigTileMin = int64_t(1) << 20;
constexpr int64_t kHugeTileMin = int64_t(1) << 22;
// tuning knobs for experiments (a forced tile shape + 1, the counting kernel's grid); the defaults are what ships
inline int& forced_shape() { static int v = 0; return v; }
inline int& hist_max_blocks() { static int v = kHistMaxBlocks; return v; }
inline int tile_shape_for(int64_t n)
{
    if (forced_shape() >= 1 && forced_shape() <= 4) {
        return forced_shape() - 1;
    }
    return n >= kHugeTileMin ? kShapeHuge : (n >= kBigTileMin ? kShapeBig : (n >= kMediumTileMin ? kShapeMedium : kShapeSmall));
}

// Look-back words a sort of up to maxN pairs can need at most: the tiles of the shape each size takes, and 3 passes
// of 1024 digits (32-bit keys) or 8 passes of 256 digits (64-bit keys) per tile.
inline int64_t status_words_for(int64_t maxN)
{
    const int64_t small = cdiv(std::min<int64_t>(maxN, kMediumTileMin), kTilePairs[kShapeSmall]);
    const int64_t medium = maxN >= kMediumTileMin ? cdiv(std::min<int64_t>(maxN, kBigTileMin), kTilePairs[kShapeMedium]) : 0;
    const int64_t big = maxN >= kBigTileMin ? cdiv(maxN, kTilePairs[kShapeBig]) : 0;   // the huge tile has as many pairs
    return std::max<int64_t>(small, std::max<int64_t>(medium, big)) * 3072 + 4;
}

// Blocks of the histogram kernel: one per kHistThreads * kHistItems keys, at most kHistMaxBlocks.
inline int hist_blocks_for(int64_t n)
{
    return (int)std::max<int64_t>(1, std::min<int64_t>(cdiv(n, (int64_t)kHistThreads * kHistItems), hist_max_blocks()));
}

// Bytes of one allocation that workspace_carve() cuts into the arrays above.
inline size_t workspace_bytes(int64_t maxN, int keyBytes)
{
    auto up = [](size_t x) { return (x + 255) / 256 * 256; };
    const size_t fixed = up(sizeof(uint32_t) * kMaxPasses * kMaxRadix) + up(sizeof(uint32_t) * kTicketWords) +
                         up(sizeof(uint32_t) * (size_t)kHistMaxBlocks * kHistPartialWords);
    return fixed + up(sizeof(uint32_t) * (size_t)status_words_for(maxN)) + up((size_t)keyBytes * (size_t)maxN) +
           up(sizeof(uint32_t) * (size_t)maxN);
}

// Cuts `mem` (workspace_bytes(maxN, keyBytes) bytes, 256-byte aligned) into a workspace.
inline Workspace workspace_carve(void* mem, int64_t maxN, int keyBytes)
{
    auto up = [](size_t x) { return (x + 255) / 256 * 256; };
    Workspace w;
    char* p = static_cast<char*>(mem);
    w.totals = reinterpret_cast<uint32_t*>(p);
    p += up(sizeof(uint32_t) * kMaxPasses * kMaxRadix);
    w.ticket = reinterpret_cast<uint32_t*>(p);
    p += up(sizeof(uint32_t) * kTicketWords);
    w.partial = reinterpret_cast<uint32_t*>(p);
    p += up(sizeof(uint32_t) * (size_t)kHistMaxBlocks * kHistPartialWords);
    w.status = reinterpret_cast<uint32_t*>(p);
    w.statusWords = status_words_for(maxN);
    p += up(sizeof(uint32_t) * (size_t)w.statusWords);
    w.tmpKeys = p;
    p += up((size_t)keyBytes * (size_t)maxN);
    w.tmpVals = reinterpret_cast<uint32_t*>(p);
    w.maxN = maxN;
    w.keyBytes = keyBytes;
    return w;
}

#ifdef __HIPCC__

// The sorted order is ascending in ordered(key): the key itself, or its complement for a descending sort.
template <typename KeyT, bool DESC>
__device__ __forceinline__ KeyT ordered(KeyT k)
{
    return DESC ? (KeyT)~k : k;
}

// Lanes of the wave whose digit equals this lane's; all 64 lanes must call it.  Per bit one ballot; a lane collects
// the lanes that differ from it in some bit (ballot XOR its own bit spread over a word), two bits per OR.
template <int DIGIT>
__device__ __forceinline__ unsigned long long match_digit(uint32_t d)
{
    uint32_t diffLo = 0;
    uint32_t diffHi = 0;
#pragma unroll
    for (int b = 0; b < DIGIT; ++b) {
        const int mine = __builtin_amdgcn_sbfe((int)d, b, 1);                     // all ones when this lane's bit is set
        const unsigned long long set = __builtin_amdgcn_ballot_w64(mine < 0);    // lanes whose bit is set
        diffLo |= (uint32_t)set ^ (uint32_t)mine;
        diffHi |= (uint32_t)(set >> 32) ^ (uint32_t)mine;
    }
    return ~(((unsigned long long)diffHi << 32) | diffLo);
}

// counters[d] += 1 for every lane with `valid`; all 64 lanes must call it.  A wave whose lanes all hold the same digit
// (the high digits of keys that arrive grouped, such as table base + row) adds once: LDS atomics of one instruction on
// one address are served one after the other, and 64 of them cost as much as a hundred conflict-free instructions.
__device__ __forceinline__ void wave_count_digit(uint32_t* counters, uint32_t d, bool valid)
{
    const unsigned long long live = __builtin_amdgcn_ballot_w64(valid);
    if (live == 0) {
        return;
    }
    const int first = __ffsll((long long)live) - 1;
    const uint32_t d0 = (uint32_t)__shfl((int)d, first, kWave);
    const unsigned long long same = __builtin_amdgcn_ballot_w64(valid && d == d0);
    if (same == live) {
        if (lane_id() == first) {
            atomicAdd(&counters[d0], (uint32_t)__popcll(live));
        }
    } else if (valid) {
        atomicAdd(&counters[d], 1u);
    }
}

// Counts the digits of all passes over a slice of the keys per block (plain stores of the block's counts: no atomics,
// no fences, the kernel boundary publishes them) and clears the look-back words and tickets of the passes.
template <typename KeyT, int DIGIT, bool DESC>
__global__ __launch_bounds__(kHistThreads) void k_rsort_count(const KeyT* __restrict__ keys, int64_t n, int passes,
                                                             uint32_t* __restrict__ partial,
                                                             uint32_t* __restrict__ ticket,
                                                             uint32_t* __restrict__ status, int64_t statusWords)
{
    constexpr int RADIX = 1 << DIGIT;
    constexpr int PMAX = ((int)sizeof(KeyT) * 8 + DIGIT - 1) / DIGIT;
    // Several copies of the counters, lane l of a wave counts in copy l % COPIES: keys with a heavy head (a few rows
    // that hold a tenth of the lookups each, high digits that barely vary) put dozens of lanes of one instruction on one
    // counter, and LDS atomics on one address are served one after the other.
    constexpr int COPIES = PMAX * RADIX * 8 <= 16384 ? 8 : (PMAX * RADIX * 4 <= 16384 ? 4 : 2);
    __shared__ uint32_t sH[COPIES * PMAX * RADIX];
    const int bins = passes * RADIX;
    for (int i = threadIdx.x; i < COPIES * PMAX * RADIX; i += kHistThreads) {
        sH[i] = 0;
    }
    if (blockIdx.x == 0 && threadIdx.x < kMaxPasses) {
        ticket[threadIdx.x] = 0;
    }
    __syncthreads();
    uint32_t* mineH = sH + (threadIdx.x & (COPIES - 1)) * (PMAX * RADIX);
    const int64_t chunk = (int64_t)kHistThreads * kHistItems;
    for (int64_t first = (int64_t)blockIdx.x * chunk; first < n; first += (int64_t)gridDim.x * chunk) {
        KeyT k[kHistItems];
#pragma unroll
        for (int j = 0; j < kHistItems; ++j) {
            const int64_t i = first + (int64_t)j * kHistThreads + threadIdx.x;
            k[j] = i < n ? ordered<KeyT, DESC>(keys[i]) : (KeyT)0;
        }
#pragma unroll
        for (int j = 0; j < kHistItems; ++j) {
            const int64_t i = first + (int64_t)j * kHistThreads + threadIdx.x;
            if (i < n) {
                for (int p = 0; p < passes; ++p) {
                    atomicAdd(&mineH[p * RADIX + (int)((k[j] >> (p * DIGIT)) & (KeyT)(RADIX - 1))], 1u);
                }
            }
        }
    }
    // the look-back words of all passes, 16 bytes per store
    {
        uint4* s4 = reinterpret_cast<uint4*>(status);
        const int64_t quads = statusWords / 4;   // statusWords is a multiple of 4
        for (int64_t i = (int64_t)blockIdx.x * kHistThreads + threadIdx.x; i < quads; i += (int64_t)gridDim.x * kHistThreads) {
            s4[i] = make_uint4(0u, 0u, 0u, 0u);
        }
    }
    __syncthreads();
    uint32_t* mine = partial + (size_t)blockIdx.x * kHistPartialWords;
    for (int i = threadIdx.x; i < bins; i += kHistThreads) {
        uint32_t c = 0;
#pragma unroll
        for (int q = 0; q < COPIES; ++q) {
            c += sH[q * (PMAX * RADIX) + i];
        }
        mine[i] = c;
    }
}

// Adds the blocks' counts up: block (pass, group of 64 digits), lane = digit, every wave a share of the counting
// blocks.  totals[pass][digit] is what the pass kernels scan.
template <int SLICES>
__global__ __launch_bounds__(SLICES * kWave) void k_rsort_totals(const uint32_t* __restrict__ partial, int blocks, int radix,
                                                       uint32_t* __restrict__ totals)
{
    __shared__ uint32_t sPart[SLICES][kWave];
    const int groupsPerPass = radix / kWave;
    const int pass = blockIdx.x / groupsPerPass;
    const int d = (blockIdx.x % groupsPerPass) * kWave + (threadIdx.x & (kWave - 1));
    const int slice = threadIdx.x >> 6;
    uint32_t sum = 0;
    for (int b0 = slice; b0 < blocks; b0 += SLICES * 8) {
        uint32_t v[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const int b = b0 + q * SLICES;
            v[q] = b < blocks ? partial[(size_t)b * kHistPartialWords + pass * radix + d] : 0u;
        }
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            sum += v[q];
        }
    }
    sPart[slice][threadIdx.x & (kWave - 1)] = sum;
    __syncthreads();
    if (slice == 0) {
        uint32_t t = 0;
#pragma unroll
        for (int q = 0; q < SLICES; ++q) {
            t += sPart[q][threadIdx.x];
        }
        totals[pass * kMaxRadix + d] = t;
    }
}

// Resident waves per SIMD the pass kernel is compiled for (its register budget): two blocks of 1024 threads or of
// 512 threads with 16 pairs each, three of 512 threads with 8 pairs each.
template <int THREADS, int ITEMS, int KEY_BYTES>
constexpr int pass_waves_per_simd()
{
    // 64-bit keys: the exchange buffers of the two biggest shapes leave room for one block per compute unit
    return KEY_BYTES == 8 ? (THREADS * ITEMS == 8192 ? THREADS / 256 : 4)
                          : (THREADS == 1024 ? 8 : (THREADS == 512 && ITEMS == 8 ? 6 : 4));
}

// One pass over one digit.  Tiles are taken in input order through a ticket, so a tile's predecessors are always
// running or done when it looks back.  A tile counts its digits and publishes the counts BEFORE it ranks its keys, so
// that the tiles behind it find them while they rank their own.
template <typename KeyT, int THREADS, int ITEMS, int DIGIT, bool DESC>
__global__ __launch_bounds__(THREADS, (pass_waves_per_simd<THREADS, ITEMS, (int)sizeof(KeyT)>())) void k_rsort_pass(
    const KeyT* __restrict__ keysIn, KeyT* __restrict__ keysOut, const uint32_t* __restrict__ valsIn,
    uint32_t* __restrict__ valsOut, int64_t n, int shift, const uint32_t* __restrict__ totals, uint32_t* status,
    uint32_t* ticket)
{
    constexpr int RADIX = 1 << DIGIT;
    constexpr int NW = THREADS / kWave;
    constexpr int TILE = THREADS * ITEMS;
    constexpr int DPT = (RADIX + THREADS - 1) / THREADS;   // digits per thread in the per-digit steps
    constexpr size_t kHistBytes = sizeof(uint32_t) * NW * RADIX;
    constexpr size_t kXchgBytes = (sizeof(KeyT) + sizeof(uint32_t)) * TILE;
    constexpr size_t kUnionBytes = kHistBytes > kXchgBytes ? kHistBytes : kXchgBytes;
    // per-wave digit counters first, the exchange buffers of keys and values once the counters are dead
    __shared__ __align__(16) unsigned char sUnion[kUnionBytes];
    __shared__ uint32_t sDigitStart[RADIX];   // first index of every digit in the tile's sorted order
    __shared__ uint32_t sGlobalOff[RADIX];    // output index of the tile's sorted index 0 of every digit, minus its start
    __shared__ uint32_t sScan[NW];
    __shared__ uint32_t sTile;
    uint32_t* sHist = reinterpret_cast<uint32_t*>(sUnion);
    KeyT* sKeys = reinterpret_cast<KeyT*>(sUnion);
    uint32_t* sVals = reinterpret_cast<uint32_t*>(sUnion + sizeof(KeyT) * TILE);

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & (kWave - 1);
    if (tid == 0) {
        sTile = atomicAdd(ticket, 1u);
    }
    for (int i = tid; i < NW * RADIX; i += THREADS) {
        sHist[i] = 0;
    }
    __syncthreads();
    const uint32_t tile = sTile;
    const int64_t tileBase = (int64_t)tile * TILE;
    const int64_t left = n - tileBase;
    const int valid = (int)(left < TILE ? left : TILE);

    // keys of this thread: item i of lane l of wave w is element w * 64 * ITEMS + i * 64 + l of the tile
    KeyT key[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const int at = wave * kWave * ITEMS + i * kWave + lane;
        // slots past the end count as the largest key: they sort behind everything and are never written
        key[i] = at < valid ? ordered<KeyT, DESC>(keysIn[tileBase + at]) : (KeyT)~(KeyT)0;
    }
    // first output index of every digit: exclusive scan of the digits' totals (every block does its own)
    {
        uint32_t tot[DPT];
        uint32_t tsum = 0;
#pragma unroll
        for (int j = 0; j < DPT; ++j) {
            const int d = tid * DPT + j;
            tot[j] = d < RADIX ? totals[d] : 0u;
            tsum += tot[j];
        }
        uint32_t all;
        uint32_t e = block_exclusive_scan_n<THREADS>(tsum, sScan, &all);
#pragma unroll
        for (int j = 0; j < DPT; ++j) {
            const int d = tid * DPT + j;
            if (d < RADIX) {
                sGlobalOff[d] = e;
            }
            e += tot[j];
        }
    }
    // digit counts of every wave
    uint32_t* myHist = sHist + wave * RADIX;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        wave_count_digit(myHist, (uint32_t)((key[i] >> shift) & (KeyT)(RADIX - 1)), true);
    }
    __syncthreads();
    // per digit: counts of the waves -> starts of the waves inside the digit, count of the tile, published at once
    uint32_t cnt[DPT];
    uint32_t sum = 0;
#pragma unroll
    for (int j = 0; j < DPT; ++j) {
        const int d = tid * DPT + j;
        uint32_t running = 0;
        if (d < RADIX) {
            constexpr int kBatch = NW < 8 ? NW : 8;   // counters read together
#pragma unroll
            for (int w0 = 0; w0 < NW; w0 += kBatch) {
                uint32_t c[kBatch];
#pragma unroll
                for (int w = 0; w < kBatch; ++w) {
                    c[w] = sHist[(w0 + w) * RADIX + d];
                }
#pragma unroll
                for (int w = 0; w < kBatch; ++w) {
                    sHist[(w0 + w) * RADIX + d] = running;
                    running += c[w];
                }
            }
            __hip_atomic_store(&status[(int64_t)tile * RADIX + d], (tile == 0 ? kFlagInclusive : kFlagAggregate) | running,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        cnt[j] = running;
        sum += running;
    }
    uint32_t total;
    uint32_t excl = block_exclusive_scan_n<THREADS>(sum, sScan, &total);
    {
        uint32_t e = excl;
#pragma unroll
        for (int j = 0; j < DPT; ++j) {
            const int d = tid * DPT + j;
            if (d < RADIX) {
                sDigitStart[d] = e;
            }
            e += cnt[j];
        }
    }
    __syncthreads();
    // Place of every pair in the tile's sorted order: start of its digit + the keys of the digit in the waves before
    // its own + those before it in its own wave.  Lanes of a wave with equal digits find each other by ballots; the
    // lowest of them moves the wave's counter of the digit on by their number.
    uint32_t pos[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const uint32_t d = (uint32_t)((key[i] >> shift) & (KeyT)(RADIX - 1));
        const unsigned long long same = match_digit<DIGIT>(d);
        const int leader = __ffsll((long long)same) - 1;
        uint32_t before = 0;
        if (lane == leader) {
            before = atomicAdd(&myHist[d], (uint32_t)__popcll(same));
        }
        before = __shfl(before, leader, kWave);
        pos[i] = sDigitStart[d] + before + (uint32_t)__popcll(same & ((1ull << lane) - 1ull));
    }
    // the values travel late: their loads are in flight while the tile looks back
    uint32_t val[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const int at = wave * kWave * ITEMS + i * kWave + lane;
        val[i] = at < valid ? valsIn[tileBase + at] : 0u;
    }
    // Counts of the tiles before this one, per digit.  kLookBack predecessors are polled per round with all loads in
    // flight together: every poll is a trip to the memory side, and a chain of single polls would cost one trip per
    // tile walked (the blocks that start together walk about sqrt(2 * resident tiles / kLookBack) rounds).
#pragma unroll
    for (int j = 0; j < DPT; ++j) {
        const int d = tid * DPT + j;
        if (d < RADIX) {
            uint32_t prefix = 0;
            if (tile != 0) {
                int64_t t = (int64_t)tile - 1;
                bool done = false;
                while (!done) {
                    uint32_t st[kLookBack];
#pragma unroll
                    for (int k = 0; k < kLookBack; ++k) {
                        st[k] = t - k >= 0 ? __hip_atomic_load(&status[(t - k) * RADIX + d], __ATOMIC_RELAXED,
                                                               __HIP_MEMORY_SCOPE_AGENT)
                                           : kFlagInclusive;   // before the first tile: nothing, and the walk ends
                    }
                    bool open = true;
                    int used = 0;
#pragma unroll
                    for (int k = 0; k < kLookBack; ++k) {
                        if (open && !done) {
                            if ((st[k] & kFlagMask) == 0) {
                                open = false;   // not published yet: poll again from this tile
                            } else {
                                prefix += st[k] & kValueMask;
                                ++used;
                                done = (st[k] & kFlagInclusive) != 0;
                            }
                        }
                    }
                    t -= used;
                }
                __hip_atomic_store(&status[(int64_t)tile * RADIX + d], kFlagInclusive | (prefix + cnt[j]), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            }
            sGlobalOff[d] += prefix - excl;   // each digit's word is read and written by this thread alone
        }
        excl += cnt[j];
    }
    __syncthreads();   // the counters are dead: their memory becomes the exchange buffers
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        sKeys[pos[i]] = key[i];
        sVals[pos[i]] = val[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const int p = i * THREADS + tid;
        if (p < valid) {
            const KeyT k = sKeys[p];
            const uint32_t d = (uint32_t)((k >> shift) & (KeyT)(RADIX - 1));
            const uint32_t dst = sGlobalOff[d] + (uint32_t)p;
            keysOut[dst] = ordered<KeyT, DESC>(k);
            valsOut[dst] = sVals[p];
        }
    }
}

template <typename KeyT, int DIGIT, bool DESC>
static int sort_pairs_digit(const Workspace& w, const char* name, const KeyT* keysIn, KeyT* keysOut,
                            const uint32_t* valsIn, uint32_t* valsOut, int64_t n, int bits, hipStream_t s)
{
    constexpr int RADIX = 1 << DIGIT;
    const int passes = (bits + DIGIT - 1) / DIGIT;
    const int shape = tile_shape_for(n);
    const int64_t tiles = cdiv(n, kTilePairs[shape]);
    const int64_t words = (tiles * RADIX * passes + 3) / 4 * 4;
    if (words > w.statusWords || n > w.maxN || passes > kMaxPasses || passes * RADIX > kHistPartialWords ||
        (int)sizeof(KeyT) > w.keyBytes) {
        set_error("radix sort: %lld pairs over %d bits exceed the workspace", (long long)n, bits);
        return RECSDK_ECAPACITY;
    }
    KernelScope scope(name, s);
    {
        const int grid = hist_blocks_for(n);
        hipLaunchKernelGGL((k_rsort_count<KeyT, DIGIT, DESC>), dim3((unsigned)grid), dim3(kHistThreads), 0, s, keysIn, n,
                           passes, w.partial, w.ticket, w.status, words);
        RECSDK_LAUNCH_CHECK();
        hipLaunchKernelGGL(k_rsort_totals<16>, dim3((unsigned)(passes * RADIX / kWave)), dim3(16 * kWave), 0, s, w.partial, grid,
                           RADIX, w.totals);
        RECSDK_LAUNCH_CHECK();
    }
    const KeyT* srcK = keysIn;
    const uint32_t* srcV = valsIn;
    for (int p = 0; p < passes; ++p) {
        const bool toOut = ((passes - 1 - p) % 2) == 0;
        KeyT* dstK = toOut ? keysOut : static_cast<KeyT*>(w.tmpKeys);
        uint32_t* dstV = toOut ? valsOut : w.tmpVals;
        uint32_t* status = w.status + (int64_t)p * tiles * RADIX;
#define RECSDK_RSORT_PASS(THREADS, ITEMS)                                                                           \
    hipLaunchKernelGGL((k_rsort_pass<KeyT, THREADS, ITEMS, DIGIT, DESC>), dim3((unsigned)tiles),                       \
                       dim3(THREADS), 0, s, srcK, dstK, srcV, dstV, n, p * DIGIT, w.totals + p * kMaxRadix, status, \
                       w.ticket + p)
        switch (shape) {
        case kShapeHuge:
            RECSDK_RSORT_PASS(512, 16);
            break;
        case kShapeBig:
            RECSDK_RSORT_PASS(1024, 8);
            break;
        case kShapeMedium:
            RECSDK_RSORT_PASS(512, 8);
            break;
        default:
            RECSDK_RSORT_PASS(256, 8);
            break;
        }
#undef RECSDK_RSORT_PASS
        RECSDK_LAUNCH_CHECK();
        srcK = dstK;
        srcV = dstV;
    }
    return RECSDK_OK;
}

// Stable sort of n pairs by the low `bits` bits of their keys (the keys hold nothing above them), ascending, or
// descending with DESC.  keysIn / valsIn are left as they are; keysOut / valsOut must not overlap them.  `name` is
// the label of the whole sort in the library's per-kernel timing.
template <typename KeyT, bool DESC = false>
static int sort_pairs(const Workspace& w, const char* name, const KeyT* keysIn, KeyT* keysOut, const uint32_t* valsIn,
                      uint32_t* valsOut, int64_t n, int bits, hipStream_t s)
{
    static_assert(std::is_same<KeyT, uint32_t>::value || std::is_same<KeyT, uint64_t>::value, "32- or 64-bit keys");
    if (n <= 0) {
        return RECSDK_OK;
    }
    bits = std::max(1, std::min(bits, (int)sizeof(KeyT) * 8));
    if constexpr (sizeof(KeyT) == 8) {
        // digits of 10 bits where they save a pass and the counting kernel's per-block counts still fit (3 passes)
        if (bits <= 30 && digit_bits_for(bits) == 10) {
            return sort_pairs_digit<KeyT, 10, DESC>(w, name, keysIn, keysOut, valsIn, valsOut, n, bits, s);
        }
        return sort_pairs_digit<KeyT, 8, DESC>(w, name, keysIn, keysOut, valsIn, valsOut, n, bits, s);
    } else {
        switch (digit_bits_for(bits)) {
        case 9:
            return sort_pairs_digit<KeyT, 9, DESC>(w, name, keysIn, keysOut, valsIn, valsOut, n, bits, s);
        case 10:
            return sort_pairs_digit<KeyT, 10, DESC>(w, name, keysIn, keysOut, valsIn, valsOut, n, bits, s);
        default:
            return sort_pairs_digit<KeyT, 8, DESC>(w, name, keysIn, keysOut, valsIn, valsOut, n, bits, s);
        }
    }
}

#endif  // __HIPCC__

}  // namespace rsort
}  // namespace recsdk

#endif
