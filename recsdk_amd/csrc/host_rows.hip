// Host-DRAM row store behind the HBM cache, its row initializers, and the device kernels that move rows between
// the two.
//
// Reference: EmbLocalTable (AccCTR embedding_cache/embedding_local_table/emb_local_table.cpp:106-335) keeps one
// malloc'd row of extEmbeddingSize floats per key behind a hash map; new rows come from a pool that background
// threads pre-fill by running every initializer over the row (address_mapper.h:72-231); initializers are
// constant / random normal / truncated normal over a column range of the row, one std::default_random_engine per
// initializer object seeded once (initializer/*/*.cpp).
// Here the rows live in ONE pinned, device-mapped arena (row index instead of address) so that swap-in and
// swap-out are device kernels that read / write host memory over the host link, with no staging copy and no host
// memcpy threads.  The key -> row map lives on the DEVICE (one static key -> slot table: rows are handed out in
// array order, freed rows are reused last-freed-first), so a swap of keys the cache planner produced on the device
// needs no host work at all; the calls that take host keys upload them, resolve them on the device and download
// the rows.  The j-th row ever created receives the j-th row of the initializer stream (what a single refill thread
// of the reference's pool produces): the host generates that stream ahead into a pinned ring and the swap-in kernel
// copies row j of it.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <random>
#include <thread>
#include <unordered_set>
#include <vector>

#include "common.h"
#include "dedup.h"
#include "fileio.h"
#include "tables.h"

namespace recsdk {

// limits the reference clamps to (embedding_cache/common.h:55-62)
constexpr float kMeanMax = 1e9f, kMeanMin = -1e9f, kStdMax = 100.0f, kStdMin = 0.0f;
constexpr float kConstMax = 1e9f, kConstMin = -1e9f, kInitKMax = 10000.0f, kInitKMin = -10000.0f;

inline float clampf(float v, float lo, float hi) { return v > hi ? hi : (v < lo ? lo : v); }

// The value stream of std::normal_distribution<float>(mean, stddev) over std::default_random_engine(seed), which is what
// the reference's initializers draw from (initializer/random_normal_initializer/random_normal_initializer.cpp:24-79),
// produced many values at a time on several host threads.  libstdc++'s engine is minstd_rand0 (x <- 16807 x mod
// 2^31 - 1), its generate_canonical<float, 24> takes one draw, (x - 1) / 2^31 (1 is replaced by the float below it), and
// its normal distribution is Marsaglia's polar method in float: attempts of two draws each until x^2 + y^2 lies in
// (0, 1], then y * mult and, on the next call, the saved x * mult.  Every attempt takes exactly two draws, so attempt a
// starts at draw 2a whatever the attempts before it decided, and the engine jumps ahead by modular exponentiation: a
// stretch of attempts is cut into pieces that threads evaluate on their own, and the accepted values are strung together
// in attempt order.  The stream is the sequential one bit for bit (same float operations, same libm).
class NormalStream {
public:
    NormalStream() = default;
    NormalStream(uint32_t seed, float mean, float stddev) : mean_(mean), stddev_(stddev)
    {
        state_ = seed % kModulus;
        if (state_ == 0) {
            state_ = 1;
        }
    }
    // the next value of the stream
    float Next()
    {
        if (head_ == buf_.size()) {
            Produce(4096);
        }
        return buf_[head_++];
    }
    // make sure `n` more values can be taken without generating one by one
    void Reserve(size_t n)
    {
        const size_t have = buf_.size() - head_;
        if (have < n) {
            Produce(n - have);
        }
    }

private:
    static constexpr uint64_t kModulus = 2147483647u;
    static constexpr uint64_t kMultiplier = 16807u;
    static constexpr size_t kPieceAttempts = 1 << 16;   // attempts per piece of work of a thread
    static constexpr int kMaxThreads = 16;

    static uint64_t PowMod(uint64_t base, uint64_t e)
    {
        uint64_t r = 1;
        base %= kModulus;
        while (e != 0) {
            if (e & 1) {
                r = r * base % kModulus;
            }
            base = base * base % kModulus;
            e >>= 1;
        }
        return r;
    }
    static float Canonical(uint64_t x)
    {
        const float r = static_cast<float>(static_cast<uint32_t>(x) - 1u) / 2147483648.0f;
        return r >= 1.0f ? std::nextafterf(1.0f, 0.0f) : r;
    }
    // attempts [first, first + count) of the stream that starts at engine state `start`: the accepted values, in order,
    // to out[0 ..]; returns their number (at most 2 * count)
    size_t Piece(uint64_t start, uint64_t first, uint64_t count, float* out) const
    {
        uint64_t x = start * PowMod(kMultiplier, 2 * first) % kModulus;
        size_t m = 0;
        for (uint64_t a = 0; a < count; ++a) {
            x = x * kMultiplier % kModulus;
            const float u = 2.0f * Canonical(x) - 1.0f;
            x = x * kMultiplier % kModulus;
            const float v = 2.0f * Canonical(x) - 1.0f;
            const float r2 = u * u + v * v;
            if (r2 > 1.0f || r2 == 0.0f) {
                continue;
            }
            const float mult = std::sqrt(-2.0f * std::log(r2) / r2);
            out[m++] = v * mult * stddev_ + mean_;
            out[m++] = u * mult * stddev_ + mean_;
        }
        return m;
    }
    void Produce(size_t need)
    {
        // an attempt is accepted with probability pi / 4 and yields two values
        const uint64_t attempts = static_cast<uint64_t>(static_cast<double>(need) / 1.5) + 64;
        const uint64_t pieces = (attempts + kPieceAttempts - 1) / kPieceAttempts;
        // every piece writes where its attempts would land if all were accepted; the buffers keep their size from call
        // to call (fresh pages per call cost more than the arithmetic)
        if (scratch_.size() < 2 * attempts) {
            scratch_.resize(2 * attempts);
        }
        pieceCount_.assign(pieces, 0);
        const unsigned hw = std::thread::hardware_concurrency();
        const int threads = static_cast<int>(std::min<uint64_t>(pieces, std::min<unsigned>(hw == 0 ? 1 : hw, kMaxThreads)));
        auto work = [&](int t) {
            for (uint64_t p = t; p < pieces; p += threads) {
                const uint64_t first = p * kPieceAttempts;
                pieceCount_[p] = Piece(state_, first, std::min<uint64_t>(kPieceAttempts, attempts - first),
                                       scratch_.data() + 2 * first);
            }
        };
        if (threads <= 1) {
            work(0);
        } else {
            std::vector<std::thread> pool;
            for (int t = 1; t < threads; ++t) {
                pool.emplace_back(work, t);
            }
            work(0);
            for (std::thread& th : pool) {
                th.join();
            }
        }
        // drop what has been consumed, append the pieces in attempt order, move the engine past the attempts
        const size_t left = buf_.size() - head_;
        if (head_ != 0) {
            std::memmove(buf_.data(), buf_.data() + head_, sizeof(float) * left);
        }
        head_ = 0;
        size_t total = left;
        for (uint64_t p = 0; p < pieces; ++p) {
            total += pieceCount_[p];
        }
        buf_.resize(total);
        size_t at = left;
        for (uint64_t p = 0; p < pieces; ++p) {
            std::memcpy(buf_.data() + at, scratch_.data() + 2 * p * kPieceAttempts, sizeof(float) * pieceCount_[p]);
            at += pieceCount_[p];
        }
        state_ = state_ * PowMod(kMultiplier, 2 * attempts) % kModulus;
    }

    uint64_t state_ = 1;     // engine state before the first attempt not yet evaluated
    float mean_ = 0.0f;
    float stddev_ = 1.0f;
    std::vector<float> buf_;   // values produced and not yet taken
    size_t head_ = 0;
    std::vector<float> scratch_;        // where the pieces of a refill write
    std::vector<size_t> pieceCount_;    // accepted values per piece
};

// One initializer over columns [start, start+len) of a row.
struct RowInit {
    int32_t kind;
    uint32_t start;
    uint32_t len;
    float value;  // constant: initK * value
    float initK;
    float minBound, maxBound;
    NormalStream stream;

    explicit RowInit(const recsdk_initializer_desc_t& d) : kind(d.kind), start(d.start), len(d.len)
    {
        initK = clampf(d.init_k, kInitKMin, kInitKMax);
        minBound = 0.0f;
        maxBound = 0.0f;
        if (kind == RECSDK_INIT_CONSTANT) {
            value = initK * clampf(d.value_or_mean, kConstMin, kConstMax);
        } else {
            const float mean = clampf(d.value_or_mean, kMeanMin, kMeanMax);
            const float stddev = clampf(d.stddev, kStdMin, kStdMax);
            stream = NormalStream(d.seed, mean, stddev);
            // truncated_normal_initializer.cpp:69-70, boundNum = 2 (include/embedding_cache.h:133)
            minBound = initK * (mean - 2.0f * stddev);
            maxBound = initK * (mean + 2.0f * stddev);
            value = 0.0f;
        }
    }

    // `rows` rows are about to be generated: have their values produced in one go (a truncated normal rejects about
    // one value in twenty; what is missing is produced as the rows ask for it)
    void Reserve(int64_t rows)
    {
        if (kind != RECSDK_INIT_CONSTANT && rows > 0) {
            const double perRow = kind == RECSDK_INIT_TRUNCATED_NORMAL ? len * 1.06 : len;
            stream.Reserve(static_cast<size_t>(perRow * static_cast<double>(rows)));
        }
    }

    void Generate(float* row)
    {
        float* p = row + start;
        if (kind == RECSDK_INIT_CONSTANT) {
            std::fill_n(p, len, value);
        } else if (kind == RECSDK_INIT_RANDOM_NORMAL) {
            for (uint32_t j = 0; j < len; ++j) {
                p[j] = initK * stream.Next();
            }
        } else {
            for (uint32_t j = 0; j < len; ++j) {
                float t = initK * stream.Next();
                while (t < minBound || t > maxBound) {
                    t = initK * stream.Next();
                }
                p[j] = t;
            }
        }
    }
};

// device row <-> host row, one 16-byte chunk per thread; hostRow / devSlot index the two row arrays.
// Swap-in: a key whose row was created by this call (rank >= 0) takes row (created + rank) of the initializer
// stream, which also becomes the content of its host row.  `prefilledFrom` (may be NULL): host rows from
// prefilledFrom[0] on already hold that content, so the write over the host link is left out for them.
__global__ __launch_bounds__(kBlock) void k_rows_host_to_dev(float* __restrict__ arena, int64_t hostStride,
                                                             const int64_t* __restrict__ hostRow,
                                                             const int64_t* __restrict__ rank,
                                                             const float* __restrict__ pool, int64_t poolCap,
                                                             const int64_t* __restrict__ created,
                                                             const int64_t* __restrict__ prefilledFrom,
                                                             float* __restrict__ cache, int64_t cacheStride,
                                                             const int64_t* __restrict__ devSlot, int64_t n,
                                                             int32_t chunksPerRow)
{
    const int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t i = q / chunksPerRow;
    const int c = (int)(q - i * chunksPerRow);
    if (i >= n) {
        return;
    }
    const int64_t row = hostRow[i];
    if (row < 0) {
        return;  // the store is full (reported by the next synchronising call)
    }
    const int64_t r = rank[i];
    float4 v;
    if (r >= 0) {
        v = *reinterpret_cast<const float4*>(pool + ((created[0] + r) % poolCap) * hostStride + c * 4);
        if (prefilledFrom == nullptr || row < prefilledFrom[0]) {
            *reinterpret_cast<float4*>(arena + row * hostStride + c * 4) = v;
        }
    } else {
        v = *reinterpret_cast<const float4*>(arena + row * hostStride + c * 4);
    }
    *reinterpret_cast<float4*>(cache + devSlot[i] * cacheStride + c * 4) = v;
}

__global__ __launch_bounds__(kBlock) void k_rows_dev_to_host(float* __restrict__ arena, int64_t hostStride,
                                                             const int64_t* __restrict__ hostRow,
                                                             const float* __restrict__ cache, int64_t cacheStride,
                                                             const int64_t* __restrict__ devSlot, int64_t n,
                                                             int32_t chunksPerRow)
{
    const int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t i = q / chunksPerRow;
    const int c = (int)(q - i * chunksPerRow);
    if (i >= n || hostRow[i] < 0) {
        return;
    }
    const float4 v = *reinterpret_cast<const float4*>(cache + devSlot[i] * cacheStride + c * 4);
    *reinterpret_cast<float4*>(arena + hostRow[i] * hostStride + c * 4) = v;
}

// victims' cache rows -> a dense HBM buffer, so that their slots may be overwritten while the copy to the host runs
__global__ __launch_bounds__(kBlock) void k_rows_stage(float* __restrict__ stage, int64_t stageStride,
                                                       const float* __restrict__ cache, int64_t cacheStride,
                                                       const int64_t* __restrict__ devSlot, int64_t n,
                                                       int32_t chunksPerRow)
{
    const int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t i = q / chunksPerRow;
    const int c = (int)(q - i * chunksPerRow);
    if (i >= n) {
        return;
    }
    *reinterpret_cast<float4*>(stage + i * stageStride + c * 4) =
        *reinterpret_cast<const float4*>(cache + devSlot[i] * cacheStride + c * 4);
}

// Both directions of the host link in one launch: even blocks move rows out (staged row i -> host row outRow[i]),
// odd blocks bring rows in (as k_rows_host_to_dev), so that reads and writes over the link are in flight together.
// The grid is small and every block walks its direction's 16-byte chunks with a stride: a few hundred KB in flight
// per direction saturate the link, and a kernel of tens of thousands of blocks, all waiting for the link, would keep
// the kernels of other streams (the dedup of a later batch, the update of an earlier one) off the CUs for as long as
// it runs.  The two sets of host rows are disjoint (different keys), and the staged rows are not in the cache any
// more.  Even and odd on purpose: consecutive blocks go to consecutive XCDs, so each direction has four XCDs to
// itself; with the first half of the grid going out and the second coming in, both on all eight, the host-backed-cache
// configuration's step takes 3.63 instead of 3.15 ms.
constexpr unsigned kLinkBlocks = 64;   // per direction
constexpr int kLinkDepth = 8;          // 16-byte chunks per thread and round

// UN chunks per thread and round, their loads in flight together (the rows that come in are read over the host link
// with microseconds of latency).  What fills the link is the number of waves that read over it: with 8 or 16 loads
// per thread alike, 16 / 32 / 64 blocks of 256 threads per direction move 18 / 25 / 35 GB/s each way in the
// host-backed-cache configuration, and 256 blocks of 64 threads as much as 64 of 256.  More waves than that gain
// nothing on the link and take from the kernels of the other two stages, which already run several times slower
// while rows cross the link (one chunk per thread and 128 blocks per direction: 3.37 ms per step of that
// configuration; 8 chunks and 64 blocks: 3.13-3.17 ms).
template <int UN>
__global__ __launch_bounds__(kBlock) void k_rows_both_ways(float* __restrict__ arena, int64_t hostStride,
                                                                const int64_t* __restrict__ outRow,
                                                                const float* __restrict__ stage, int64_t nOut,
                                                                const int64_t* __restrict__ inRow,
                                                                const int64_t* __restrict__ rank,
                                                                const float* __restrict__ pool, int64_t poolCap,
                                                                const int64_t* __restrict__ created,
                                                                const int64_t* __restrict__ prefilledFrom,
                                                                float* __restrict__ cache, int64_t cacheStride,
                                                                const int64_t* __restrict__ devSlot, int64_t nIn,
                                                                int32_t chunksPerRow)
{
    const bool out = (blockIdx.x & 1) == 0;
    const int64_t stride = (int64_t)(gridDim.x >> 1) * blockDim.x;
    const int64_t chunks = (out ? nOut : nIn) * chunksPerRow;
    const int64_t made = created[0];
    const int64_t frontier = prefilledFrom != nullptr ? prefilledFrom[0] : INT64_MAX;
    for (int64_t q0 = (int64_t)(blockIdx.x >> 1) * blockDim.x + threadIdx.x; q0 < chunks; q0 += stride * UN) {
        float4 v[UN];
        int64_t dst[UN];     // element offset of the destination chunk, -1: none
        int64_t dst2[UN];    // "in" only: a second destination in the host arena (a new row taken from the pool)
        const float* src[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int64_t q = q0 + u * stride;
            dst[u] = -1;
            dst2[u] = -1;
            src[u] = nullptr;
            if (q < chunks) {
                const int64_t i = q / chunksPerRow;
                const int c = (int)(q - i * chunksPerRow);
                if (out) {
                    const int64_t row = outRow[i];
                    if (row >= 0) {
                        src[u] = stage + i * hostStride + c * 4;
                        dst[u] = row * hostStride + c * 4;
                    }
                } else {
                    const int64_t row = inRow[i];
                    if (row >= 0) {
                        const int64_t r = rank[i];
                        if (r >= 0) {
                            src[u] = pool + ((made + r) % poolCap) * hostStride + c * 4;
                            if (row < frontier || prefilledFrom == nullptr) {
                                dst2[u] = row * hostStride + c * 4;
                            }
                        } else {
                            src[u] = arena + row * hostStride + c * 4;
                        }
                        dst[u] = devSlot[i] * cacheStride + c * 4;
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            if (src[u] != nullptr) {
                v[u] = *reinterpret_cast<const float4*>(src[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            if (dst[u] >= 0) {
                if (out) {
                    *reinterpret_cast<float4*>(arena + dst[u]) = v[u];
                } else {
                    if (dst2[u] >= 0) {
                        *reinterpret_cast<float4*>(arena + dst2[u]) = v[u];
                    }
                    *reinterpret_cast<float4*>(cache + dst[u]) = v[u];
                }
            }
        }
    }
}

// every host row := the one row of a constant initializer stream (16-byte chunks, grid-stride)
__global__ __launch_bounds__(kBlock) void k_rows_prefill(float* __restrict__ arena, int64_t chunks,
                                                         const float* __restrict__ row, int32_t chunksPerRow)
{
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x; q < chunks; q += stride) {
        const int c = (int)(q % chunksPerRow);
        *reinterpret_cast<float4*>(arena + q * 4) = *reinterpret_cast<const float4*>(row + c * 4);
    }
}

__global__ __launch_bounds__(kBlock) void k_rows_fill(int64_t* __restrict__ p, int64_t n, int64_t value)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) {
        p[i] = value;
    }
}

__global__ void k_rows_set_offsets(int64_t* off, int64_t n)
{
    off[0] = 0;
    off[1] = n;
}

// created[1] += number of keys this call created; k_rows_commit then moves it into created[0]
__global__ __launch_bounds__(kBlock) void k_rows_count_created(const int64_t* __restrict__ rank, int64_t n,
                                                               unsigned long long* created)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    wave_count_add(created, 1, i < n && rank[i] >= 0);
}

__global__ void k_rows_commit(int64_t* created)
{
    created[0] += created[1];
    created[1] = 0;
}

}  // namespace recsdk

using namespace recsdk;

struct recsdk_initializer {
    std::vector<RowInit> inits;
};

static int check_descs(const recsdk_initializer_desc_t* descs, int32_t n, int32_t extDim, const char* who)
{
    RECSDK_REQUIRE(n >= 0 && (n == 0 || descs != nullptr), RECSDK_ENULL, "initializer descriptors missing");
    for (int32_t k = 0; k < n; ++k) {
        RECSDK_REQUIRE(descs[k].kind >= RECSDK_INIT_CONSTANT && descs[k].kind <= RECSDK_INIT_TRUNCATED_NORMAL,
                       RECSDK_EINVAL, "Invalid Initializer Type.");
        RECSDK_REQUIRE(extDim <= 0 || (uint64_t)descs[k].start + descs[k].len <= (uint64_t)extDim, RECSDK_EINVAL,
                       "an initializer's start + len is larger than the row");
    }
    (void)who;
    return RECSDK_OK;
}

extern "C" int recsdk_initializer_create(const recsdk_initializer_desc_t* descs, int32_t n_descs,
                                         recsdk_initializer_t** out)
{
    RECSDK_REQUIRE(out != nullptr, RECSDK_ENULL, "recsdk_initializer_create: out is NULL");
    int rc = check_descs(descs, n_descs, 0, "recsdk_initializer_create");
    if (rc != RECSDK_OK) {
        return rc;
    }
    auto* h = new recsdk_initializer();
    for (int32_t k = 0; k < n_descs; ++k) {
        h->inits.emplace_back(descs[k]);
    }
    *out = h;
    return RECSDK_OK;
}

extern "C" int recsdk_initializer_destroy(recsdk_initializer_t* h)
{
    delete h;
    return RECSDK_OK;
}

extern "C" int recsdk_initializer_generate(recsdk_initializer_t* h, float* h_rows, int64_t rows, int32_t ext_dim)
{
    RECSDK_REQUIRE(h != nullptr && (rows == 0 || h_rows != nullptr), RECSDK_ENULL,
                   "recsdk_initializer_generate: NULL argument");
    for (const RowInit& ri : h->inits) {
        RECSDK_REQUIRE((uint64_t)ri.start + ri.len <= (uint64_t)ext_dim, RECSDK_EINVAL,
                       "recsdk_initializer_generate: an initializer's start + len is larger than ext_dim");
    }
    for (RowInit& ri : h->inits) {
        ri.Reserve(rows);
    }
    for (int64_t r = 0; r < rows; ++r) {
        for (RowInit& ri : h->inits) {
            ri.Generate(h_rows + r * ext_dim);
        }
    }
    return RECSDK_OK;
}

// ---- host row store ----------------------------------------------------------------------------------------
struct recsdk_hostrows {
    int64_t vocab = 0;
    int32_t ext = 0;
    float* arena = nullptr;      // pinned host memory, vocab * ext floats
    float* arenaDev = nullptr;   // the same memory as the device sees it
    std::vector<RowInit> inits;
    bool allConst = true;        // every initializer is a constant: the stream repeats one row
    recsdk_tables_t* dmap = nullptr;  // key -> row on the device (one static table of `vocab` rows)
    recsdk_unique_t* uq = nullptr;    // dedup of the calls that take host keys
    int64_t maxCall = 0;              // keys per device call; longer calls go in pieces
    // device scratch, maxCall entries each
    int64_t* dKeys = nullptr;
    int64_t* dRows = nullptr;    // row per distinct key / per key of a device call
    int64_t* dRank = nullptr;    // creation rank per distinct key, -1 = existed
    int64_t* dRowsOcc = nullptr; // row per occurrence
    int64_t* dOff = nullptr;     // [2]
    int64_t* dCreated = nullptr; // [0] rows ever created = position in the initializer stream, [1] of the call in flight
    // pinned staging, maxCall entries each
    int64_t* hKeys = nullptr;
    int64_t* hRows = nullptr;
    int64_t* hRowsU = nullptr;
    int64_t* hRank = nullptr;
    // initializer stream: ring of poolCap rows, row j of the stream at j % poolCap, rows below `generated` exist
    float* pool = nullptr;
    float* poolDev = nullptr;
    float* poolHbm = nullptr;    // constant initializers: device copy of the one stream row
    bool prefilled = false;      // constant initializers: every host row not handed out yet holds that row
    float* stage = nullptr;      // HBM copy of the rows a combined swap sends out, stageRows rows of ext floats
    int64_t stageRows = 0;
    hipEvent_t linkStart = nullptr;  // caller's event, recorded by a combined swap right before its link kernel
    int64_t poolCap = 0;
    int64_t generated = 0;

    void Generate(int64_t upTo)
    {
        for (RowInit& ri : inits) {
            ri.Reserve(upTo - generated);
        }
        for (; generated < upTo; ++generated) {
            float* row = pool + (generated % poolCap) * ext;
            for (RowInit& ri : inits) {
                ri.Generate(row);  // columns no initializer covers stay 0
            }
        }
    }
    const float* StreamRow(int64_t j)
    {
        if (allConst) {
            return pool;
        }
        Generate(j + 1);
        return pool + (j % poolCap) * ext;
    }
};

static void hostrows_free_pool(recsdk_hostrows* h)
{
    if (h->pool != nullptr) {
        (void)hipHostFree(h->pool);
        h->pool = nullptr;
        h->poolDev = nullptr;
        h->poolCap = 0;
    }
}

// ring of `cap` stream rows; rows [from, generated) of the old ring are kept
static int hostrows_alloc_pool(recsdk_hostrows* h, int64_t cap, int64_t from)
{
    float* fresh = nullptr;
    float* freshDev = nullptr;
    const size_t bytes = sizeof(float) * (size_t)cap * (size_t)h->ext;
    if (hipHostMalloc(reinterpret_cast<void**>(&fresh), bytes, hipHostMallocMapped) != hipSuccess ||
        hipHostGetDevicePointer(reinterpret_cast<void**>(&freshDev), fresh, 0) != hipSuccess) {
        (void)hipGetLastError();
        if (fresh != nullptr) {
            (void)hipHostFree(fresh);
        }
        set_error("host row store: pinned allocation of the initializer ring failed");
        return RECSDK_ENOMEM;
    }
    std::memset(fresh, 0, bytes);
    for (int64_t j = from; j < h->generated && h->pool != nullptr; ++j) {
        std::memcpy(fresh + (j % cap) * h->ext, h->pool + (j % h->poolCap) * h->ext, sizeof(float) * h->ext);
    }
    hostrows_free_pool(h);
    h->pool = fresh;
    h->poolDev = freshDev;
    h->poolCap = cap;
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_destroy(recsdk_hostrows_t* h)
{
    if (h == nullptr) {
        return RECSDK_OK;
    }
    (void)hipDeviceSynchronize();  // kernels of the handle may still read the pinned buffers
    recsdk_tables_destroy(h->dmap);
    recsdk_unique_destroy(h->uq);
    void* dev[] = {h->dKeys, h->dRows, h->dRank, h->dRowsOcc, h->dOff, h->dCreated, h->poolHbm, h->stage};
    for (void* p : dev) {
        if (p != nullptr) {
            (void)hipFree(p);
        }
    }
    void* pinned[] = {h->hKeys, h->hRows, h->hRowsU, h->hRank, h->arena};
    for (void* p : pinned) {
        if (p != nullptr) {
            (void)hipHostFree(p);
        }
    }
    hostrows_free_pool(h);
    delete h;
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_create(int64_t vocab_size, int32_t ext_dim, const recsdk_initializer_desc_t* descs,
                                      int32_t n_descs, recsdk_hostrows_t** out)
{
    RECSDK_REQUIRE(out != nullptr, RECSDK_ENULL, "recsdk_hostrows_create: out is NULL");
    RECSDK_REQUIRE(vocab_size > 0 && ext_dim > 0 && ext_dim % 4 == 0, RECSDK_EINVAL,
                   "recsdk_hostrows_create: vocab_size must be positive and ext_dim a positive multiple of 4");
    int rc = check_descs(descs, n_descs, ext_dim, "recsdk_hostrows_create");
    if (rc != RECSDK_OK) {
        return rc;
    }
    auto* h = new recsdk_hostrows();
    h->vocab = vocab_size;
    h->ext = ext_dim;
    for (int32_t k = 0; k < n_descs; ++k) {
        h->inits.emplace_back(descs[k]);
        if (descs[k].kind != RECSDK_INIT_CONSTANT) {
            h->allConst = false;
        }
    }
    h->maxCall = std::min<int64_t>(std::max<int64_t>(vocab_size, 1024), int64_t(1) << 20);
    const size_t bytes = sizeof(float) * (size_t)vocab_size * (size_t)ext_dim;
    bool ok = hipHostMalloc(reinterpret_cast<void**>(&h->arena), bytes, hipHostMallocMapped) == hipSuccess &&
              hipHostGetDevicePointer(reinterpret_cast<void**>(&h->arenaDev), h->arena, 0) == hipSuccess;
    auto dalloc = [&](int64_t** p, int64_t count) {
        ok = ok && hipMalloc(reinterpret_cast<void**>(p), sizeof(int64_t) * count) == hipSuccess;
    };
    auto palloc = [&](int64_t** p, int64_t count) {
        ok = ok && hipHostMalloc(reinterpret_cast<void**>(p), sizeof(int64_t) * count, hipHostMallocDefault) == hipSuccess;
    };
    dalloc(&h->dKeys, h->maxCall);
    dalloc(&h->dRows, h->maxCall);
    dalloc(&h->dRank, h->maxCall);
    dalloc(&h->dRowsOcc, h->maxCall);
    dalloc(&h->dOff, 2);
    dalloc(&h->dCreated, 2);
    palloc(&h->hKeys, h->maxCall);
    palloc(&h->hRows, h->maxCall);
    palloc(&h->hRowsU, h->maxCall);
    palloc(&h->hRank, h->maxCall);
    ok = ok && hipMemset(h->dCreated, 0, sizeof(int64_t) * 2) == hipSuccess;
    if (ok) {
        const int64_t vocabArr[1] = {vocab_size};
        ok = recsdk_tables_create(1, vocabArr, nullptr, nullptr, nullptr, h->maxCall, &h->dmap) == RECSDK_OK &&
             recsdk_unique_create(h->maxCall, 1, &h->uq) == RECSDK_OK &&
             recsdk_unique_set_lists(h->uq, 0) == RECSDK_OK;
    }
    // constant initializers: the stream is one row repeated; otherwise a ring that grows with the calls
    ok = ok && hostrows_alloc_pool(h, h->allConst ? 1 : 4096, 0) == RECSDK_OK;
    if (!ok) {
        (void)hipGetLastError();
        recsdk_hostrows_destroy(h);
        set_error("recsdk_hostrows_create: allocation failed");
        return RECSDK_ENOMEM;
    }
    if (h->allConst) {
        // the one row every new key starts from is read from HBM, not over the host link
        h->Generate(1);
        if (hipMalloc(reinterpret_cast<void**>(&h->poolHbm), sizeof(float) * ext_dim) != hipSuccess ||
            hipMemcpy(h->poolHbm, h->pool, sizeof(float) * ext_dim, hipMemcpyHostToDevice) != hipSuccess) {
            (void)hipGetLastError();
            recsdk_hostrows_destroy(h);
            set_error("recsdk_hostrows_create: allocation failed");
            return RECSDK_ENOMEM;
        }
        h->poolDev = h->poolHbm;
        // Every host row starts as that row, written once here over the host link.  A key that takes a row nobody has
        // used before then finds its initial values in place, and its swap-in writes the cache row only; rows that
        // come back from the freed list are written as before.
        const int64_t chunks = vocab_size * (int64_t)(ext_dim / 4);
        hipLaunchKernelGGL(k_rows_prefill, dim3((unsigned)std::min<int64_t>(cdiv(chunks, kBlock), 256 * 8)), dim3(kBlock), 0,
                           nullptr, h->arenaDev, chunks, h->poolHbm, ext_dim / 4);
        if (hipGetLastError() != hipSuccess || hipStreamSynchronize(nullptr) != hipSuccess) {
            (void)hipGetLastError();
            recsdk_hostrows_destroy(h);
            set_error("recsdk_hostrows_create: filling the host rows failed");
            return RECSDK_EHIP;
        }
        h->prefilled = true;
    }
    *out = h;
    return RECSDK_OK;
}

// parallel row copies over `threads` host threads (contiguous index ranges, like the reference's split)
template <typename F>
static void for_rows(int64_t n, int32_t threads, F&& body)
{
    if (threads <= 1 || n < 4096) {
        for (int64_t i = 0; i < n; ++i) {
            body(i);
        }
        return;
    }
    std::vector<std::thread> pool;
    const int64_t per = (n + threads - 1) / threads;
    for (int32_t t = 0; t < threads; ++t) {
        const int64_t b = std::min<int64_t>(n, per * t);
        const int64_t e = std::min<int64_t>(n, b + per);
        pool.emplace_back([=, &body]() {
            for (int64_t i = b; i < e; ++i) {
                body(i);
            }
        });
    }
    for (auto& t : pool) {
        t.join();
    }
}

// Rows of host keys, found or (create) created in array order; synchronous, on the null stream.  rows[i] = row of
// keys[i] or -1.  Created rows receive their initial values.  Key -1 is reserved and has no row.
static int resolve_rows(recsdk_hostrows* h, const int64_t* keys, int64_t n, bool create, int64_t* rows,
                        const char* who)
{
    hipStream_t s = nullptr;
    if (create) {
        for (int64_t i = 0; i < n; ++i) {
            if (keys[i] == -1) {
                set_error("%s: key -1 is reserved and has no row", who);
                return RECSDK_EINVAL;
            }
        }
    }
    for (int64_t b = 0; b < n; b += h->maxCall) {
        const int64_t m = std::min<int64_t>(h->maxCall, n - b);
        std::memcpy(h->hKeys, keys + b, sizeof(int64_t) * m);
        RECSDK_HIP_TRY(hipMemcpyAsync(h->dKeys, h->hKeys, sizeof(int64_t) * m, hipMemcpyHostToDevice, s));
        RECSDK_LAUNCH(k_rows_set_offsets, dim3(1), dim3(1), s, h->dOff, m);
        int rc = recsdk_unique_run(h->uq, h->dKeys, nullptr, h->dOff, 1, m, 0, 0, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
        const UniqueView* v = recsdk_unique_view(h->uq);
        int64_t U = 0;
        rc = recsdk_unique_total(h->uq, s, &U);
        if (rc != RECSDK_OK) {
            return rc;
        }
        RECSDK_HIP_TRY(hipMemcpyAsync(h->dRows, v->uniq, sizeof(int64_t) * U, hipMemcpyDeviceToDevice, s));
        RECSDK_LAUNCH(k_rows_fill, dim3((unsigned)cdiv(std::max<int64_t>(U, 1), kBlock)), dim3(kBlock), s, h->dRank, U,
                      (int64_t)-1);
        rc = recsdk_tables_key2offset_ranked(h->dmap, h->dRows, v->uoff, 1, m,
                                             create ? RECSDK_CHANNEL_TRAIN : RECSDK_CHANNEL_EVAL, h->dRank, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
        rc = recsdk_unique_expand(h->uq, h->dRows, -1, h->dRowsOcc, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
        int64_t created = 0;
        RECSDK_HIP_TRY(hipMemcpyAsync(h->hRows, h->dRowsOcc, sizeof(int64_t) * m, hipMemcpyDeviceToHost, s));
        RECSDK_HIP_TRY(hipMemcpyAsync(h->hRowsU, h->dRows, sizeof(int64_t) * U, hipMemcpyDeviceToHost, s));
        RECSDK_HIP_TRY(hipMemcpyAsync(h->hRank, h->dRank, sizeof(int64_t) * U, hipMemcpyDeviceToHost, s));
        RECSDK_HIP_TRY(hipMemcpyAsync(&created, h->dCreated, sizeof(int64_t), hipMemcpyDeviceToHost, s));
        RECSDK_HIP_TRY(hipStreamSynchronize(s));
        std::memcpy(rows + b, h->hRows, sizeof(int64_t) * m);
        if (create) {
            // distinct keys are in first-occurrence order, so creation ranks ascend with R
            int64_t fresh = 0;
            for (int64_t R = 0; R < U; ++R) {
                if (h->hRank[R] < 0) {
                    continue;
                }
                if (h->hRowsU[R] < 0) {
                    set_error("%s: host vocabulary size is too small", who);
                    return RECSDK_ECAPACITY;
                }
                std::memcpy(h->arena + h->hRowsU[R] * h->ext, h->StreamRow(created + h->hRank[R]),
                            sizeof(float) * h->ext);
                fresh += 1;
            }
            if (fresh > 0) {
                created += fresh;
                RECSDK_HIP_TRY(hipMemcpy(h->dCreated, &created, sizeof(int64_t), hipMemcpyHostToDevice));
            }
        }
    }
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_find_rows(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, int32_t create,
                                         int64_t* h_rows)
{
    RECSDK_REQUIRE(h != nullptr && (n == 0 || (h_keys != nullptr && h_rows != nullptr)), RECSDK_ENULL,
                   "recsdk_hostrows_find_rows: NULL argument");
    return resolve_rows(h, h_keys, n, create != 0, h_rows, "recsdk_hostrows_find_rows");
}

extern "C" int recsdk_hostrows_gather(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, float* h_dst,
                                      int32_t threads)
{
    RECSDK_REQUIRE(h != nullptr && (n == 0 || (h_keys != nullptr && h_dst != nullptr)), RECSDK_ENULL,
                   "recsdk_hostrows_gather: NULL argument");
    std::vector<int64_t> rows(n);
    int rc = resolve_rows(h, h_keys, n, true, rows.data(), "recsdk_hostrows_gather");
    if (rc != RECSDK_OK) {
        return rc;
    }
    const size_t rb = sizeof(float) * h->ext;
    for_rows(n, threads, [&](int64_t i) { std::memcpy(h_dst + i * h->ext, h->arena + rows[i] * h->ext, rb); });
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_scatter(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, const float* h_src,
                                       int32_t threads)
{
    RECSDK_REQUIRE(h != nullptr && (n == 0 || (h_keys != nullptr && h_src != nullptr)), RECSDK_ENULL,
                   "recsdk_hostrows_scatter: NULL argument");
    std::vector<int64_t> rows(n);
    int rc = resolve_rows(h, h_keys, n, true, rows.data(), "recsdk_hostrows_scatter");
    if (rc != RECSDK_OK) {
        return rc;
    }
    const size_t rb = sizeof(float) * h->ext;
    // rows of one key written twice keep the later copy, as a sequential loop would
    for_rows(n, 1, [&](int64_t i) { std::memcpy(h->arena + rows[i] * h->ext, h_src + i * h->ext, rb); });
    (void)threads;
    return RECSDK_OK;
}

// erase host keys from the device map (rows go to the free stack in array order); synchronous
static int erase_keys(recsdk_hostrows* h, const int64_t* keys, int64_t n)
{
    hipStream_t s = nullptr;
    for (int64_t b = 0; b < n; b += h->maxCall) {
        const int64_t m = std::min<int64_t>(h->maxCall, n - b);
        std::memcpy(h->hKeys, keys + b, sizeof(int64_t) * m);
        RECSDK_HIP_TRY(hipMemcpyAsync(h->dKeys, h->hKeys, sizeof(int64_t) * m, hipMemcpyHostToDevice, s));
        RECSDK_LAUNCH(k_rows_set_offsets, dim3(1), dim3(1), s, h->dOff, m);
        int rc = recsdk_unique_run(h->uq, h->dKeys, nullptr, h->dOff, 1, m, 0, 0, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
        const UniqueView* v = recsdk_unique_view(h->uq);
        rc = recsdk_tables_evict(h->dmap, v->uniq, v->uoff, 1, m, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
        RECSDK_HIP_TRY(hipStreamSynchronize(s));
    }
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_gather_and_remove(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, float* h_dst)
{
    RECSDK_REQUIRE(h != nullptr && (n == 0 || (h_keys != nullptr && h_dst != nullptr)), RECSDK_ENULL,
                   "recsdk_hostrows_gather_and_remove: NULL argument");
    std::vector<int64_t> rows(n);
    int rc = resolve_rows(h, h_keys, n, false, rows.data(), "recsdk_hostrows_gather_and_remove");
    if (rc != RECSDK_OK) {
        return rc;
    }
    int64_t created = 0;
    RECSDK_HIP_TRY(hipMemcpy(&created, h->dCreated, sizeof(int64_t), hipMemcpyDeviceToHost));
    const int64_t before = created;
    const size_t rb = sizeof(float) * h->ext;
    std::unordered_set<int64_t> gone;
    for (int64_t i = 0; i < n; ++i) {
        if (rows[i] >= 0 && gone.insert(h_keys[i]).second) {
            std::memcpy(h_dst + i * h->ext, h->arena + rows[i] * h->ext, rb);
        } else {
            // a key that has no row (any more) gets the next row of the initializer stream and is not stored
            // (emb_local_table.cpp:247-253)
            std::memcpy(h_dst + i * h->ext, h->StreamRow(created), rb);
            created += 1;
        }
    }
    if (created != before) {
        RECSDK_HIP_TRY(hipMemcpy(h->dCreated, &created, sizeof(int64_t), hipMemcpyHostToDevice));
    }
    return erase_keys(h, h_keys, n);
}

extern "C" int recsdk_hostrows_remove(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n)
{
    RECSDK_REQUIRE(h != nullptr && (n == 0 || h_keys != nullptr), RECSDK_ENULL, "recsdk_hostrows_remove: NULL argument");
    return erase_keys(h, h_keys, n);
}

extern "C" int recsdk_hostrows_size(recsdk_hostrows_t* h, int64_t* h_live)
{
    RECSDK_REQUIRE(h != nullptr && h_live != nullptr, RECSDK_ENULL, "recsdk_hostrows_size: NULL argument");
    const int rc = recsdk_tables_stats(h->dmap, nullptr, nullptr, h_live, nullptr);
    if (rc == RECSDK_EOVERFLOW) {
        set_error("recsdk_hostrows_size: host vocabulary size is too small (a swap left keys without a row)");
        return RECSDK_ECAPACITY;
    }
    return rc;
}

extern "C" int recsdk_hostrows_arena(recsdk_hostrows_t* h, float** h_base)
{
    RECSDK_REQUIRE(h != nullptr && h_base != nullptr, RECSDK_ENULL, "recsdk_hostrows_arena: NULL argument");
    *h_base = h->arena;
    return RECSDK_OK;
}

// all (key, row) pairs in ascending key order
static int sorted_pairs(recsdk_hostrows* h, std::vector<int64_t>* keys, std::vector<int64_t>* rows)
{
    int64_t live = 0;
    int rc = recsdk_tables_stats(h->dmap, nullptr, nullptr, &live, nullptr);
    if (rc != RECSDK_OK && rc != RECSDK_EOVERFLOW) {
        return rc;
    }
    keys->assign((size_t)live, 0);
    rows->assign((size_t)live, 0);
    if (live == 0) {
        return RECSDK_OK;
    }
    int64_t* dk = nullptr;
    int64_t* dv = nullptr;
    auto body = [&]() -> int {
        RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&dk), sizeof(int64_t) * live));
        RECSDK_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&dv), sizeof(int64_t) * live));
        int64_t count = 0;
        const int r2 = recsdk_tables_export(h->dmap, 0, dk, dv, live, nullptr, &count);
        if (r2 != RECSDK_OK) {
            return r2;
        }
        std::vector<int64_t> k((size_t)count), v((size_t)count);
        RECSDK_HIP_TRY(hipMemcpy(k.data(), dk, sizeof(int64_t) * count, hipMemcpyDeviceToHost));
        RECSDK_HIP_TRY(hipMemcpy(v.data(), dv, sizeof(int64_t) * count, hipMemcpyDeviceToHost));
        std::vector<int64_t> order((size_t)count);
        for (int64_t i = 0; i < count; ++i) {
            order[(size_t)i] = i;
        }
        std::sort(order.begin(), order.end(), [&](int64_t a, int64_t b) { return k[(size_t)a] < k[(size_t)b]; });
        keys->resize((size_t)count);
        rows->resize((size_t)count);
        for (int64_t i = 0; i < count; ++i) {
            (*keys)[(size_t)i] = k[(size_t)order[(size_t)i]];
            (*rows)[(size_t)i] = v[(size_t)order[(size_t)i]];
        }
        return RECSDK_OK;
    };
    rc = body();
    if (dk != nullptr) {
        (void)hipFree(dk);
    }
    if (dv != nullptr) {
        (void)hipFree(dv);
    }
    return rc;
}

extern "C" int recsdk_hostrows_export(recsdk_hostrows_t* h, int64_t* h_keys, float* h_rows, int64_t cap,
                                      int64_t* h_count)
{
    RECSDK_REQUIRE(h != nullptr && h_count != nullptr, RECSDK_ENULL, "recsdk_hostrows_export: NULL argument");
    std::vector<int64_t> keys, rows;
    const int rc = sorted_pairs(h, &keys, &rows);
    if (rc != RECSDK_OK) {
        return rc;
    }
    *h_count = (int64_t)keys.size();
    if (h_keys == nullptr || h_rows == nullptr || cap < *h_count) {
        return RECSDK_OK;
    }
    for (size_t i = 0; i < keys.size(); ++i) {
        h_keys[i] = keys[i];
        std::memcpy(h_rows + i * h->ext, h->arena + rows[i] * h->ext, sizeof(float) * h->ext);
    }
    return RECSDK_OK;
}

// ---- serialized forms -----------------------------------------------------------------------------------

extern "C" int recsdk_hostrows_serialize(recsdk_hostrows_t* h, char* h_buf, int64_t cap, int64_t* h_bytes)
{
    RECSDK_REQUIRE(h != nullptr && h_bytes != nullptr, RECSDK_ENULL, "recsdk_hostrows_serialize: NULL argument");
    std::vector<int64_t> keys, rows;
    const int rc = sorted_pairs(h, &keys, &rows);
    if (rc != RECSDK_OK) {
        return rc;
    }
    const size_t rec = sizeof(uint64_t) + sizeof(float) * h->ext;
    *h_bytes = (int64_t)(rec * keys.size());
    if (h_buf == nullptr || cap < *h_bytes) {
        return RECSDK_OK;
    }
    char* p = h_buf;
    for (size_t i = 0; i < keys.size(); ++i) {
        const uint64_t k = (uint64_t)keys[i];
        std::memcpy(p, &k, sizeof(k));
        std::memcpy(p + sizeof(k), h->arena + rows[i] * h->ext, sizeof(float) * h->ext);
        p += rec;
    }
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_deserialize(recsdk_hostrows_t* h, const char* h_buf, int64_t bytes)
{
    RECSDK_REQUIRE(h != nullptr && (bytes == 0 || h_buf != nullptr), RECSDK_ENULL,
                   "recsdk_hostrows_deserialize: NULL argument");
    const int64_t rec = (int64_t)(sizeof(uint64_t) + sizeof(float) * h->ext);
    // records the buffer holds in full, and the one it may end in (its key is still taken, its floats as far as
    // they go, then the reference reports failure)
    const int64_t whole = bytes / rec;
    const int64_t tail = bytes - whole * rec;
    const bool cutKey = tail >= (int64_t)sizeof(uint64_t);
    std::vector<int64_t> keys((size_t)(whole + (cutKey ? 1 : 0)));
    for (size_t i = 0; i < keys.size(); ++i) {
        uint64_t k;
        std::memcpy(&k, h_buf + (int64_t)i * rec, sizeof(k));
        keys[i] = (int64_t)k;
    }
    std::vector<int64_t> rows(keys.size());
    const int rc = resolve_rows(h, keys.data(), (int64_t)keys.size(), true, rows.data(), "recsdk_hostrows_deserialize");
    if (rc != RECSDK_OK) {
        return rc;
    }
    for (int64_t i = 0; i < whole; ++i) {
        std::memcpy(h->arena + rows[(size_t)i] * h->ext, h_buf + i * rec + sizeof(uint64_t), sizeof(float) * h->ext);
    }
    if (tail != 0) {
        if (cutKey) {
            const int64_t have = (tail - (int64_t)sizeof(uint64_t)) / (int64_t)sizeof(float);
            std::memcpy(h->arena + rows[(size_t)whole] * h->ext, h_buf + whole * rec + sizeof(uint64_t),
                        sizeof(float) * have);
        }
        set_error("get data failed!");
        return RECSDK_EINVAL;
    }
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_save(recsdk_hostrows_t* h, const char* prefix, int32_t emb_dim, int32_t optim_num)
{
    RECSDK_REQUIRE(h != nullptr && prefix != nullptr, RECSDK_ENULL, "recsdk_hostrows_save: NULL argument");
    RECSDK_REQUIRE(emb_dim > 0 && optim_num >= 0 && optim_num <= 2 && (int64_t)emb_dim * (1 + optim_num) <= h->ext,
                   RECSDK_EINVAL, "recsdk_hostrows_save: emb_dim * (1 + optim_num) exceeds the row width");
    std::vector<int64_t> keys, rows;
    int rc = sorted_pairs(h, &keys, &rows);
    if (rc != RECSDK_OK) {
        return rc;
    }
    const int64_t count = (int64_t)keys.size();
    const std::string base(prefix);
    rc = write_file(base + "/key/slice.data", keys.data(), sizeof(int64_t) * keys.size());
    const int64_t keyAttr[2] = {(int64_t)sizeof(int64_t), count};
    if (rc == RECSDK_OK) {
        rc = write_file(base + "/key/slice.attribute", keyAttr, sizeof(keyAttr));
    }
    const int64_t rowAttr[3] = {(int64_t)sizeof(float), count, emb_dim};
    // embedding at float 0 of the row, momentum1 at embDim, momentum2 at optimNum * embDim
    const char* dirs[3] = {"/embedding", "/momentum1", "/momentum2"};
    const int64_t at[3] = {0, emb_dim, (int64_t)optim_num * emb_dim};
    std::vector<float> packed((size_t)count * emb_dim);
    for (int part = 0; part <= optim_num && rc == RECSDK_OK; ++part) {
        for (int64_t i = 0; i < count; ++i) {
            std::memcpy(packed.data() + i * emb_dim, h->arena + rows[(size_t)i] * h->ext + at[part],
                        sizeof(float) * emb_dim);
        }
        rc = write_file(base + dirs[part] + "/slice.data", packed.data(), sizeof(float) * packed.size());
        if (rc == RECSDK_OK) {
            rc = write_file(base + dirs[part] + "/slice.attribute", rowAttr, sizeof(rowAttr));
        }
    }
    return rc;
}

static int read_attribute(const std::string& path, int count, std::vector<int64_t>* out)
{
    std::vector<char> raw;
    const int rc = read_file(path, 1, &raw);
    if (rc != RECSDK_OK) {
        return rc;
    }
    if (raw.size() < sizeof(int64_t) * (size_t)count) {
        set_error("Read key attribute file error, expect read bytes:%zu, actual read bytes:%zu, file:%s",
                  sizeof(int64_t) * (size_t)count, raw.size(), path.c_str());
        return RECSDK_EIO;
    }
    out->resize((size_t)count);
    std::memcpy(out->data(), raw.data(), sizeof(int64_t) * (size_t)count);
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_load(recsdk_hostrows_t* h, const char* prefix, int32_t emb_dim, int32_t optim_num)
{
    RECSDK_REQUIRE(h != nullptr && prefix != nullptr, RECSDK_ENULL, "recsdk_hostrows_load: NULL argument");
    RECSDK_REQUIRE(emb_dim > 0 && optim_num >= 0 && optim_num <= 2 && (int64_t)emb_dim * (1 + optim_num) <= h->ext,
                   RECSDK_EINVAL, "recsdk_hostrows_load: emb_dim * (1 + optim_num) exceeds the row width");
    const std::string base(prefix);
    std::vector<int64_t> attr;
    int rc = read_attribute(base + "/key/slice.attribute", 2, &attr);
    if (rc != RECSDK_OK) {
        return rc;
    }
    if (attr[1] < 0 || attr[1] > 1000000000LL) {
        set_error("Read key attribute file error, keys count is invalid:%ld, file:%s.", (long)attr[1],
                  (base + "/key/slice.attribute").c_str());
        return RECSDK_EINVAL;
    }
    std::vector<char> rawKeys;
    rc = read_file(base + "/key/slice.data", 1, &rawKeys);
    if (rc != RECSDK_OK) {
        return rc;
    }
    if (rawKeys.size() % sizeof(int64_t) != 0 || (int64_t)(rawKeys.size() / sizeof(int64_t)) != attr[1]) {
        set_error("Key file bytes is not an integer multiple of type int64_t, key file:%s",
                  (base + "/key/slice.data").c_str());
        return RECSDK_EINVAL;
    }
    const int64_t count = attr[1];
    const int64_t* keys = reinterpret_cast<const int64_t*>(rawKeys.data());
    const char* dirs[3] = {"/embedding", "/momentum1", "/momentum2"};
    const int64_t at[3] = {0, emb_dim, (int64_t)optim_num * emb_dim};
    std::vector<std::vector<char>> parts((size_t)optim_num + 1);
    for (int part = 0; part <= optim_num; ++part) {
        const std::string dataFile = base + dirs[part] + "/slice.data";
        rc = read_attribute(base + dirs[part] + "/slice.attribute", 3, &attr);
        if (rc != RECSDK_OK) {
            return rc;
        }
        if (attr[2] != emb_dim) {
            set_error("Embedding or momentum dim error, load data dim from attribute:%ld, current table dim:%d, file:%s.",
                      (long)attr[2], emb_dim, (base + dirs[part] + "/slice.attribute").c_str());
            return RECSDK_EINVAL;
        }
        rc = read_file(dataFile, 1, &parts[part]);
        if (rc != RECSDK_OK) {
            return rc;
        }
        if ((int64_t)parts[part].size() != count * emb_dim * (int64_t)sizeof(float)) {
            set_error("Read data to file error, expect read bytes:%ld, actual read bytes:%zu, file:%s",
                      (long)(count * emb_dim * (int64_t)sizeof(float)), parts[part].size(), dataFile.c_str());
            return RECSDK_EIO;
        }
    }
    // InsertOrAssign: the row of each key becomes [embedding | momentum1 | momentum2]
    std::vector<int64_t> rows((size_t)count);
    rc = resolve_rows(h, keys, count, true, rows.data(), "recsdk_hostrows_load");
    if (rc != RECSDK_OK) {
        return rc;
    }
    for (int64_t i = 0; i < count; ++i) {
        const int64_t row = rows[(size_t)i];
        for (int part = 0; part <= optim_num; ++part) {
            std::memcpy(h->arena + row * h->ext + at[part], parts[part].data() + i * emb_dim * sizeof(float),
                        sizeof(float) * emb_dim);
        }
    }
    return RECSDK_OK;
}

// rows [created, created + m) of a non-constant initializer stream must be in the ring before a kernel reads them
static int hostrows_generate_ahead(recsdk_hostrows* h, int64_t m, hipStream_t s)
{
    int64_t created = 0;
    RECSDK_HIP_TRY(hipMemcpyAsync(&created, h->dCreated, sizeof(int64_t), hipMemcpyDeviceToHost, s));
    RECSDK_HIP_TRY(hipStreamSynchronize(s));
    if (h->poolCap < m) {
        int64_t cap = h->poolCap;
        while (cap < m) {
            cap <<= 1;
        }
        const int rc = hostrows_alloc_pool(h, cap, std::max<int64_t>(created, h->generated - h->poolCap));
        if (rc != RECSDK_OK) {
            return rc;
        }
    }
    h->Generate(created + m);
    return RECSDK_OK;
}

// ---- swaps ------------------------------------------------------------------------------------------------
// Rows of the (distinct) device keys are found or created on the device, then one kernel moves the rows.  Nothing
// here waits for the host unless the initializer stream has to be generated ahead (non-constant initializers).
static int swap_device(recsdk_hostrows* h, const int64_t* d_keys, int64_t n, const int64_t* d_slots, float* d_cache,
                       int64_t cache_stride, bool toHost, hipStream_t s)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "host row store handle is NULL");
    if (n <= 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_keys != nullptr && d_slots != nullptr && d_cache != nullptr, RECSDK_ENULL, "NULL argument");
    RECSDK_REQUIRE(cache_stride >= h->ext && cache_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(d_cache) % 16) == 0,
                   RECSDK_EINVAL, "cache rows must be 16-byte aligned, their stride a multiple of 4 and >= ext_dim");
    const int32_t cpr = h->ext / 4;
    for (int64_t b = 0; b < n; b += h->maxCall) {
        const int64_t m = std::min<int64_t>(h->maxCall, n - b);
        if (!h->allConst) {
            const int rc = hostrows_generate_ahead(h, m, s);
            if (rc != RECSDK_OK) {
                return rc;
            }
        }
        RECSDK_HIP_TRY(hipMemcpyAsync(h->dRows, d_keys + b, sizeof(int64_t) * m, hipMemcpyDeviceToDevice, s));
        RECSDK_LAUNCH(k_rows_fill, dim3((unsigned)cdiv(m, kBlock)), dim3(kBlock), s, h->dRank, m, (int64_t)-1);
        RECSDK_LAUNCH(k_rows_set_offsets, dim3(1), dim3(1), s, h->dOff, m);
        const int rc = recsdk_tables_key2offset_ranked(h->dmap, h->dRows, h->dOff, 1, m, RECSDK_CHANNEL_TRAIN, h->dRank, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
        const unsigned grid = (unsigned)cdiv(m * cpr, kBlock);
        if (toHost) {
            RECSDK_LAUNCH(k_rows_dev_to_host, dim3(grid), dim3(kBlock), s, h->arenaDev, (int64_t)h->ext, h->dRows, d_cache,
                          cache_stride, d_slots + b, m, cpr);
        } else {
            RECSDK_LAUNCH(k_rows_host_to_dev, dim3(grid), dim3(kBlock), s, h->arenaDev, (int64_t)h->ext, h->dRows,
                          h->dRank, h->poolDev, h->poolCap, h->dCreated,
                          h->prefilled ? recsdk_tables_frontier_snapshot(h->dmap) : nullptr, d_cache, cache_stride,
                          d_slots + b, m, cpr);
        }
        // a created row consumes its row of the initializer stream whether or not its values were used
        RECSDK_LAUNCH(k_rows_count_created, dim3((unsigned)cdiv(m, kBlock)), dim3(kBlock), s, h->dRank, m,
                      reinterpret_cast<unsigned long long*>(h->dCreated));
        RECSDK_LAUNCH(k_rows_commit, dim3(1), dim3(1), s, h->dCreated);
    }
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_swap_dev(recsdk_hostrows_t* h, const int64_t* d_out_keys, int64_t n_out,
                                        const int64_t* d_out_slots, const int64_t* d_in_keys, int64_t n_in,
                                        const int64_t* d_in_slots, float* d_cache, int64_t cache_stride, void* stream)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "host row store handle is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (n_out <= 0 || n_in <= 0 || n_out > h->maxCall || n_in > h->maxCall) {
        // one direction only, or lists longer than one device call: one after the other
        const int rc = swap_device(h, d_out_keys, n_out, d_out_slots, d_cache, cache_stride, true, s);
        return rc != RECSDK_OK ? rc : swap_device(h, d_in_keys, n_in, d_in_slots, d_cache, cache_stride, false, s);
    }
    RECSDK_REQUIRE(d_out_keys != nullptr && d_out_slots != nullptr && d_in_keys != nullptr && d_in_slots != nullptr &&
                       d_cache != nullptr, RECSDK_ENULL, "recsdk_hostrows_swap_dev: NULL argument");
    RECSDK_REQUIRE(cache_stride >= h->ext && cache_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(d_cache) % 16) == 0,
                   RECSDK_EINVAL, "cache rows must be 16-byte aligned, their stride a multiple of 4 and >= ext_dim");
    if (h->stageRows < n_out) {
        RECSDK_HIP_TRY(hipStreamSynchronize(s));
        if (h->stage != nullptr) {
            RECSDK_HIP_TRY(hipFree(h->stage));
            h->stage = nullptr;
            h->stageRows = 0;
        }
        const int64_t rows = std::min<int64_t>(h->maxCall, std::max<int64_t>(n_out + n_out / 4, 1024));
        if (hipMalloc(reinterpret_cast<void**>(&h->stage), sizeof(float) * (size_t)rows * (size_t)h->ext) != hipSuccess) {
            (void)hipGetLastError();
            set_error("recsdk_hostrows_swap_dev: no device memory for %lld staged rows", (long long)rows);
            return RECSDK_ENOMEM;
        }
        h->stageRows = rows;
    }
    const int32_t cpr = h->ext / 4;
    // rows of the keys that go out (a key never seen takes a row, and its row of the initializer stream, like
    // recsdk_hostrows_swap_out_dev), and their values out of the cache
    RECSDK_HIP_TRY(hipMemcpyAsync(h->dRowsOcc, d_out_keys, sizeof(int64_t) * n_out, hipMemcpyDeviceToDevice, s));
    RECSDK_LAUNCH(k_rows_fill, dim3((unsigned)cdiv(n_out, kBlock)), dim3(kBlock), s, h->dRank, n_out, (int64_t)-1);
    RECSDK_LAUNCH(k_rows_set_offsets, dim3(1), dim3(1), s, h->dOff, n_out);
    int rc = recsdk_tables_key2offset_ranked(h->dmap, h->dRowsOcc, h->dOff, 1, n_out, RECSDK_CHANNEL_TRAIN, h->dRank, s);
    if (rc != RECSDK_OK) {
        return rc;
    }
    RECSDK_LAUNCH(k_rows_count_created, dim3((unsigned)cdiv(n_out, kBlock)), dim3(kBlock), s, h->dRank, n_out,
                  reinterpret_cast<unsigned long long*>(h->dCreated));
    RECSDK_LAUNCH(k_rows_commit, dim3(1), dim3(1), s, h->dCreated);
    const unsigned outBlocks = (unsigned)cdiv(n_out * cpr, kBlock);
    RECSDK_LAUNCH(k_rows_stage, dim3(outBlocks), dim3(kBlock), s, h->stage, (int64_t)h->ext, d_cache, cache_stride,
                  d_out_slots, n_out, cpr);
    // rows of the keys that come in
    if (!h->allConst) {
        rc = hostrows_generate_ahead(h, n_in, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
    }
    RECSDK_HIP_TRY(hipMemcpyAsync(h->dRows, d_in_keys, sizeof(int64_t) * n_in, hipMemcpyDeviceToDevice, s));
    RECSDK_LAUNCH(k_rows_fill, dim3((unsigned)cdiv(n_in, kBlock)), dim3(kBlock), s, h->dRank, n_in, (int64_t)-1);
    RECSDK_LAUNCH(k_rows_set_offsets, dim3(1), dim3(1), s, h->dOff, n_in);
    rc = recsdk_tables_key2offset_ranked(h->dmap, h->dRows, h->dOff, 1, n_in, RECSDK_CHANNEL_TRAIN, h->dRank, s);
    if (rc != RECSDK_OK) {
        return rc;
    }
    const unsigned perWay =
        (unsigned)std::min<int64_t>(kLinkBlocks, cdiv(std::max(n_out, n_in) * cpr, (int64_t)kBlock * kLinkDepth));
    if (h->linkStart != nullptr) {
        RECSDK_HIP_TRY(hipEventRecord(h->linkStart, s));
    }
    RECSDK_LAUNCH_AS("k_rows_both_ways", (k_rows_both_ways<kLinkDepth>), dim3(2 * std::max(perWay, 1u)), dim3(kBlock), s,
                     h->arenaDev, (int64_t)h->ext, h->dRowsOcc, h->stage, n_out, h->dRows, h->dRank, h->poolDev,
                     h->poolCap, h->dCreated, h->prefilled ? recsdk_tables_frontier_snapshot(h->dmap) : nullptr, d_cache,
                     cache_stride, d_in_slots, n_in, cpr);
    RECSDK_LAUNCH(k_rows_count_created, dim3((unsigned)cdiv(n_in, kBlock)), dim3(kBlock), s, h->dRank, n_in,
                  reinterpret_cast<unsigned long long*>(h->dCreated));
    RECSDK_LAUNCH(k_rows_commit, dim3(1), dim3(1), s, h->dCreated);
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_on_link_start(recsdk_hostrows_t* h, void* event)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "recsdk_hostrows_on_link_start: NULL handle");
    h->linkStart = static_cast<hipEvent_t>(event);
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_swap_out_dev(recsdk_hostrows_t* h, const int64_t* d_keys, int64_t n,
                                            const int64_t* d_slots, const float* d_cache, int64_t cache_stride,
                                            void* stream)
{
    return swap_device(h, d_keys, n, d_slots, const_cast<float*>(d_cache), cache_stride, true,
                       static_cast<hipStream_t>(stream));
}

extern "C" int recsdk_hostrows_swap_in_dev(recsdk_hostrows_t* h, const int64_t* d_keys, int64_t n,
                                           const int64_t* d_slots, float* d_cache, int64_t cache_stride, void* stream)
{
    return swap_device(h, d_keys, n, d_slots, d_cache, cache_stride, false, static_cast<hipStream_t>(stream));
}

// host keys: uploaded piece by piece (the stream is drained first: the staging buffers are the handle's)
static int swap_host_keys(recsdk_hostrows* h, const int64_t* h_keys, int64_t n, const int64_t* d_slots, float* d_cache,
                          int64_t cache_stride, bool toHost, hipStream_t s)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "host row store handle is NULL");
    if (n <= 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(h_keys != nullptr, RECSDK_ENULL, "NULL argument");
    for (int64_t b = 0; b < n; b += h->maxCall) {
        const int64_t m = std::min<int64_t>(h->maxCall, n - b);
        RECSDK_HIP_TRY(hipStreamSynchronize(s));
        RECSDK_HIP_TRY(hipMemcpy(h->dKeys, h_keys + b, sizeof(int64_t) * m, hipMemcpyHostToDevice));
        const int rc = swap_device(h, h->dKeys, m, d_slots + b, d_cache, cache_stride, toHost, s);
        if (rc != RECSDK_OK) {
            return rc;
        }
    }
    return RECSDK_OK;
}

extern "C" int recsdk_hostrows_swap_out(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, const int64_t* d_slots,
                                        const float* d_cache, int64_t cache_stride, void* stream)
{
    return swap_host_keys(h, h_keys, n, d_slots, const_cast<float*>(d_cache), cache_stride, true,
                          static_cast<hipStream_t>(stream));
}

extern "C" int recsdk_hostrows_swap_in(recsdk_hostrows_t* h, const int64_t* h_keys, int64_t n, const int64_t* d_slots,
                                       float* d_cache, int64_t cache_stride, void* stream)
{
    return swap_host_keys(h, h_keys, n, d_slots, d_cache, cache_stride, false, static_cast<hipStream_t>(stream));
}
