// Library-level entry points: version and per-thread error text.
#include <stdarg.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"

namespace recsdk {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

}  // namespace recsdk

namespace recsdk {

// ---- optional per-kernel timing -------------------------------------------------------------------
struct ProfState {
    bool on = false;
    std::string prefix;                 // empty = every kernel
    std::vector<hipEvent_t> start;      // event pool, reused between sessions
    std::vector<hipEvent_t> stop;
    std::vector<int> nameOf;            // per used pair: index into names
    std::vector<std::string> names;
    int used = 0;
};
static ProfState g_prof;
static std::mutex g_profMutex;
constexpr int kMaxPairs = 1 << 16;

bool profile_begin(const char* name, hipStream_t stream, int* slot)
{
    *slot = -1;
    if (!g_prof.on) {
        return false;
    }
    std::lock_guard<std::mutex> lock(g_profMutex);
    // launch sites stringify their kernel expression: strip a leading parenthesis
    const char* n = (name[0] == '(') ? name + 1 : name;
    if (!g_prof.prefix.empty() && strncmp(n, g_prof.prefix.c_str(), g_prof.prefix.size()) != 0) {
        return false;
    }
    if (g_prof.used >= kMaxPairs) {
        return false;
    }
    if (g_prof.used >= (int)g_prof.start.size()) {
        hipEvent_t a;
        hipEvent_t b;
        if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) {
            return false;
        }
        g_prof.start.push_back(a);
        g_prof.stop.push_back(b);
    }
    std::string key(n);
    size_t cut = key.find_first_of("<)");
    if (cut != std::string::npos) {
        key.resize(cut);
    }
    int id = -1;
    for (size_t i = 0; i < g_prof.names.size(); ++i) {
        if (g_prof.names[i] == key) {
            id = (int)i;
        }
    }
    if (id < 0) {
        id = (int)g_prof.names.size();
        g_prof.names.push_back(key);
    }
    int s = g_prof.used++;
    g_prof.nameOf.resize(g_prof.used);
    g_prof.nameOf[s] = id;
    (void)hipEventRecord(g_prof.start[s], stream);
    *slot = s;
    return true;
}

void profile_end(int slot, hipStream_t stream) { (void)hipEventRecord(g_prof.stop[slot], stream); }

}  // namespace recsdk

namespace {
std::atomic<int64_t> g_smallBatchKeys{recsdk::kSmallKeys};
}  // namespace

namespace recsdk {
int64_t small_batch_keys() { return g_smallBatchKeys.load(std::memory_order_relaxed); }
}  // namespace recsdk

extern "C" int recsdk_set_small_batch_keys(int64_t max_keys)
{
    RECSDK_REQUIRE(max_keys >= 0 && max_keys <= recsdk::kSmallKeys, RECSDK_EINVAL,
                   "recsdk_set_small_batch_keys: the limit must be in [0, 4096]");
    g_smallBatchKeys.store(max_keys, std::memory_order_relaxed);
    return RECSDK_OK;
}

extern "C" int recsdk_version(void) { return 1; }

extern "C" int recsdk_profile_start(const char* kernel_prefix)
{
    std::lock_guard<std::mutex> lock(recsdk::g_profMutex);
    recsdk::g_prof.prefix = kernel_prefix ? kernel_prefix : "";
    recsdk::g_prof.used = 0;
    recsdk::g_prof.names.clear();
    recsdk::g_prof.nameOf.clear();
    recsdk::g_prof.on = true;
    return RECSDK_OK;
}

extern "C" int recsdk_profile_stop(void)
{
    std::lock_guard<std::mutex> lock(recsdk::g_profMutex);
    recsdk::g_prof.on = false;
    return (int)recsdk::g_prof.names.size();
}

extern "C" int recsdk_profile_get(int32_t index, char* name, int32_t name_cap, int64_t* launches, double* total_ms)
{
    using namespace recsdk;
    std::lock_guard<std::mutex> lock(g_profMutex);
    RECSDK_REQUIRE(index >= 0 && index < (int)g_prof.names.size(), RECSDK_EINVAL, "recsdk_profile_get: bad index");
    RECSDK_REQUIRE(name != nullptr && name_cap > 0 && launches != nullptr && total_ms != nullptr, RECSDK_ENULL,
                   "recsdk_profile_get: NULL argument");
    snprintf(name, (size_t)name_cap, "%s", g_prof.names[index].c_str());
    int64_t cnt = 0;
    double ms = 0.0;
    for (int s = 0; s < g_prof.used; ++s) {
        if (g_prof.nameOf[s] != index) {
            continue;
        }
        RECSDK_HIP_TRY(hipEventSynchronize(g_prof.stop[s]));
        float t = 0.0f;
        RECSDK_HIP_TRY(hipEventElapsedTime(&t, g_prof.start[s], g_prof.stop[s]));
        ms += t;
        cnt++;
    }
    *launches = cnt;
    *total_ms = ms;
    return RECSDK_OK;
}

namespace recsdk {

// A plain streaming copy (16 bytes per lane, two requests in flight per lane, loads and stores past the caches): the
// fastest of the shapes tried on MI355X (6.1 TB/s; four per lane 5.7, eight 4.3, hipMemcpy 4.8), i.e. what this
// device moves when nothing but the memory system is in the way.
typedef float CopyVec __attribute__((ext_vector_type(4)));
constexpr int kCopyItems = 2;

__global__ __launch_bounds__(kBlock) void k_calib_copy(const CopyVec* __restrict__ src, CopyVec* __restrict__ dst,
                                                       int64_t n)
{
    const int64_t first = (int64_t)blockIdx.x * kBlock * kCopyItems + threadIdx.x;
    CopyVec v[kCopyItems];
#pragma unroll
    for (int k = 0; k < kCopyItems; ++k) {
        const int64_t j = first + (int64_t)k * kBlock;
        if (j < n) {
            v[k] = __builtin_nontemporal_load(src + j);
        }
    }
#pragma unroll
    for (int k = 0; k < kCopyItems; ++k) {
        const int64_t j = first + (int64_t)k * kBlock;
        if (j < n) {
            __builtin_nontemporal_store(v[k], dst + j);
        }
    }
}

}  // namespace recsdk

extern "C" int recsdk_calib_copy(void* d_dst, const void* d_src, int64_t bytes, void* stream)
{
    using namespace recsdk;
    RECSDK_REQUIRE(bytes >= 0 && bytes % 16 == 0, RECSDK_EINVAL, "recsdk_calib_copy: bytes must be a multiple of 16");
    if (bytes == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_dst != nullptr && d_src != nullptr, RECSDK_ENULL, "recsdk_calib_copy: NULL argument");
    RECSDK_REQUIRE(reinterpret_cast<uintptr_t>(d_dst) % 16 == 0 && reinterpret_cast<uintptr_t>(d_src) % 16 == 0,
                   RECSDK_EINVAL, "recsdk_calib_copy: buffers must be 16-byte aligned");
    const int64_t n = bytes / 16;
    const int64_t grid = cdiv(n, (int64_t)kBlock * kCopyItems);
    RECSDK_REQUIRE(grid < (int64_t(1) << 31), RECSDK_EINVAL, "recsdk_calib_copy: too large for one launch");
    RECSDK_LAUNCH(k_calib_copy, dim3((unsigned)grid), dim3(kBlock), static_cast<hipStream_t>(stream),
                  static_cast<const CopyVec*>(d_src), static_cast<CopyVec*>(d_dst), n);
    return RECSDK_OK;
}

extern "C" int recsdk_graph_node_kinds(void* hip_graph, int32_t* h_kinds, int64_t cap, int64_t* h_count)
{
    using namespace recsdk;
    RECSDK_REQUIRE(hip_graph != nullptr && h_count != nullptr, RECSDK_ENULL, "recsdk_graph_node_kinds: NULL argument");
    RECSDK_REQUIRE(cap == 0 || h_kinds != nullptr, RECSDK_ENULL, "recsdk_graph_node_kinds: h_kinds is NULL");
    hipGraph_t graph = static_cast<hipGraph_t>(hip_graph);
    size_t n = 0;
    RECSDK_HIP_TRY(hipGraphGetNodes(graph, nullptr, &n));
    *h_count = (int64_t)n;
    if (n == 0 || cap <= 0) {
        return RECSDK_OK;
    }
    hipGraphNode_t* nodes = new hipGraphNode_t[n];
    size_t got = n;
    hipError_t e = hipGraphGetNodes(graph, nodes, &got);
    for (size_t i = 0; e == hipSuccess && i < got && (int64_t)i < cap; ++i) {
        hipGraphNodeType type;
        e = hipGraphNodeGetType(nodes[i], &type);
        h_kinds[i] = (int32_t)type;
    }
    delete[] nodes;
    RECSDK_HIP_TRY(e);
    return RECSDK_OK;
}

extern "C" const char* recsdk_last_error(void) { return recsdk::g_err; }
