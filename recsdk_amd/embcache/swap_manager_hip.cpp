// Embcache::SwapManager over the HIP library: a drop-in for the reference's
// training/torch_rec_v1/torchrec_embcache/src/torchrec_embcache/csrc/embedding_cache/swap_manager.cpp.
//
// It compiles against the reference's own header (embedding_cache/swap_manager.h:27-54, in place in the reference
// checkout) and defines the class's member functions, so that embcache_manager.cpp:89-282 links against it unchanged:
// ComputeSwapInfo keeps its host-vector signature (the keys go up to the device, the five lists come back), the plan
// itself is made by recsdk_swap_compute.  The class has no destructor to release a handle and EmbcacheManager keeps
// its SwapManagers by value in a std::vector (embcache_manager.h:209), which moves them as it grows: the device state
// therefore lives in a registry keyed by a number the constructor draws and stores in swapIdx_ (a member this
// implementation has no other use for; it travels with the object), and stays until
// recsdk_embcache_release_swap_managers() or the end of the process.  A copy of a SwapManager shares its state.
#include "embedding_cache/swap_manager.h"

#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>

#include <hip/hip_runtime_api.h>

#include "recsdk_hip.h"
#include "thread_stream.h"

namespace {

struct DeviceState {
    recsdk_swap_t* h = nullptr;
    int64_t maxKeys = 0;
    int64_t* keys = nullptr;      // [maxKeys] the batch
    int64_t* out[5] = {};         // [maxKeys] each: swap-out keys / offsets, swap-in keys / offsets, batch offsets
    bool keysStale = true;        // the host copy of the slots' keys (GetKey) is older than the device state
};

std::mutex g_lock;
std::unordered_map<int64_t, DeviceState> g_states;
int64_t g_nextToken = 1;

void Check(hipError_t e, const char* what)
{
    if (e != hipSuccess) {
        throw std::runtime_error(std::string("SwapManager (HIP): ") + what + ": " + hipGetErrorString(e));
    }
}

void Check(int rc, const char* what)
{
    if (rc != RECSDK_OK) {
        throw std::runtime_error(std::string("SwapManager (HIP): ") + what + ": " + recsdk_last_error());
    }
}

// Largest batch a SwapManager accepts (the planner's workspace is sized for it once): RECSDK_EMBCACHE_MAX_KEYS,
// default 2^20 keys per table and call.
int64_t MaxKeys()
{
    const char* env = std::getenv("RECSDK_EMBCACHE_MAX_KEYS");
    const long long v = env != nullptr ? std::atoll(env) : 0;
    return v > 0 ? v : (1LL << 20);
}

void Release(DeviceState& s)
{
    if (s.h != nullptr) {
        (void)recsdk_swap_destroy(s.h);
    }
    if (s.keys != nullptr) {
        (void)hipFree(s.keys);
    }
    for (auto& p : s.out) {
        if (p != nullptr) {
            (void)hipFree(p);
        }
    }
    s = DeviceState{};
}

// The device state of a SwapManager, created on first use.  It is built aside and entered into the registry only
// when every allocation has succeeded: a failure half way leaves no entry whose buffers are missing.
DeviceState& StateOf(int64_t token, int64_t cacheSize, int64_t memStart)
{
    std::lock_guard<std::mutex> lock(g_lock);
    auto it = g_states.find(token);
    if (it != g_states.end()) {
        return it->second;
    }
    DeviceState fresh;
    try {
        fresh.maxKeys = MaxKeys();
        Check(recsdk_swap_create(cacheSize, memStart, fresh.maxKeys, &fresh.h), "recsdk_swap_create");
        Check(hipMalloc(reinterpret_cast<void**>(&fresh.keys), sizeof(int64_t) * fresh.maxKeys), "hipMalloc");
        for (auto& p : fresh.out) {
            Check(hipMalloc(reinterpret_cast<void**>(&p), sizeof(int64_t) * fresh.maxKeys), "hipMalloc");
        }
    } catch (...) {
        (void)hipGetLastError();
        Release(fresh);
        throw;
    }
    return g_states.emplace(token, fresh).first->second;
}

using recsdk_embcache::CopyDown;
using recsdk_embcache::CopyUp;
using recsdk_embcache::ThreadStream;
constexpr const char* kWho = "SwapManager";

std::vector<int64_t> Download(const int64_t* d, int64_t n)
{
    std::vector<int64_t> v(static_cast<size_t>(n));
    CopyDown(v.data(), d, sizeof(int64_t) * static_cast<size_t>(n), kWho);
    return v;
}

}  // namespace

namespace Embcache {

SwapManager::SwapManager(int64_t cacheSize, int64_t memStartOffset) : cacheSize_(cacheSize)
{
    if (memStartOffset != 0) {
        memStartOffset_ = memStartOffset;
        occupiedNum_ = memStartOffset;
    }
    std::lock_guard<std::mutex> lock(g_lock);
    swapIdx_ = g_nextToken++;
}

ComputeSwapRet SwapManager::ComputeSwapInfo(const std::vector<int64_t>& keys)
{
    DeviceState& s = StateOf(swapIdx_, cacheSize_, memStartOffset_);
    const int64_t n = static_cast<int64_t>(keys.size());
    if (n > s.maxKeys) {
        throw std::runtime_error("SwapManager (HIP): batch of " + std::to_string(n) +
                                 " keys exceeds RECSDK_EMBCACHE_MAX_KEYS = " + std::to_string(s.maxKeys));
    }
    CopyUp(s.keys, keys.data(), sizeof(int64_t) * static_cast<size_t>(n), kWho);
    Check(recsdk_swap_compute(s.h, s.keys, n, s.out[0], s.out[1], s.out[2], s.out[3], s.out[4], ThreadStream()),
          "recsdk_swap_compute");
    int64_t swapouts = 0;
    int64_t swapins = 0;
    int64_t occupied = 0;
    const int rc = recsdk_swap_counts(s.h, ThreadStream(), &swapouts, &swapins, &occupied);
    if (rc == RECSDK_EOVERFLOW) {
        throw std::runtime_error("cacheSize_ too small");  // the reference's message (swap_manager.cpp:103-105)
    }
    Check(rc, "recsdk_swap_counts");
    occupiedNum_ = occupied;
    nowVersion_ += 1;
    s.keysStale = true;
    return std::make_tuple(Download(s.out[0], swapouts), Download(s.out[1], swapouts), Download(s.out[2], swapins),
                           Download(s.out[3], swapins), Download(s.out[4], n));
}

int64_t SwapManager::GetKey(int64_t off)
{
    if (off < 0 || off >= occupiedNum_) {
        throw std::out_of_range("off is out of bounds: " + std::to_string(off) +
                                ", occupiedNum: " + std::to_string(occupiedNum_));
    }
    DeviceState& s = StateOf(swapIdx_, cacheSize_, memStartOffset_);
    if (s.keysStale) {
        // embcache_manager.cpp:298-305 walks every occupied slot when it saves: fetch the slots' keys once per change
        int64_t* d = nullptr;
        Check(hipMalloc(reinterpret_cast<void**>(&d), sizeof(int64_t) * cacheSize_), "hipMalloc");
        Check(recsdk_swap_export(s.h, d, ThreadStream()), "recsdk_swap_export");
        std::vector<int64_t> host = Download(d, cacheSize_);
        Check(hipFree(d), "hipFree");
        cache_.resize(static_cast<size_t>(cacheSize_));
        for (int64_t i = 0; i < cacheSize_; ++i) {
            cache_[i].key = host[i];
        }
        s.keysStale = false;
    }
    return cache_[off].key;
}

void SwapManager::RemoveKeys(const std::vector<int64_t>& keys)
{
    DeviceState& s = StateOf(swapIdx_, cacheSize_, memStartOffset_);
    const int64_t total = static_cast<int64_t>(keys.size());
    for (int64_t first = 0; first < total; first += s.maxKeys) {
        const int64_t m = std::min(s.maxKeys, total - first);
        CopyUp(s.keys, keys.data() + first, sizeof(int64_t) * static_cast<size_t>(m), kWho);
        Check(recsdk_swap_remove(s.h, s.keys, m, ThreadStream()), "recsdk_swap_remove");
        Check(hipStreamSynchronize(ThreadStream()), "hipStreamSynchronize");   // s.keys is reused by the next piece
    }
    s.keysStale = true;
}

int64_t SwapManager::GetMemStartOffset() const
{
    return memStartOffset_;
}

}  // namespace Embcache

// Frees the device state of every SwapManager made so far (they must not be used afterwards).
extern "C" __attribute__((visibility("default"))) void recsdk_embcache_release_swap_managers()
{
    std::lock_guard<std::mutex> lock(g_lock);
    for (auto& kv : g_states) {
        Release(kv.second);
    }
    g_states.clear();
}
