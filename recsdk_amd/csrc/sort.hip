// C ABI of the library's radix sort (radix_sort.h): a sorter handle that owns the workspace, and one call that sorts
// (key, 32-bit value) pairs.  The library's own paths (position lists, row grouping, shard regrouping) include the
// header directly; this entry point lets callers and tests reach the same kernels.
#include <hip/hip_runtime.h>

#include "common.h"
#include "radix_sort.h"

using namespace recsdk;

struct recsdk_sorter {
    int64_t maxPairs = 0;
    int keyBytes = 4;
    void* mem = nullptr;
    rsort::Workspace ws;
};

extern "C" int recsdk_sorter_create(int64_t max_pairs, int32_t key_bytes, recsdk_sorter_t** out)
{
    RECSDK_REQUIRE(out != nullptr, RECSDK_ENULL, "recsdk_sorter_create: out is NULL");
    RECSDK_REQUIRE(max_pairs > 0 && max_pairs <= (int64_t(1) << 28), RECSDK_EINVAL,
                   "recsdk_sorter_create: max_pairs must be in (0, 2^28]");
    RECSDK_REQUIRE(key_bytes == 4 || key_bytes == 8, RECSDK_EINVAL, "recsdk_sorter_create: key_bytes must be 4 or 8");
    auto* h = new recsdk_sorter();
    h->maxPairs = max_pairs;
    h->keyBytes = key_bytes;
    if (hipMalloc(&h->mem, rsort::workspace_bytes(max_pairs, key_bytes)) != hipSuccess) {
        (void)hipGetLastError();
        delete h;
        set_error("recsdk_sorter_create: hipMalloc failed for %lld pairs", (long long)max_pairs);
        return RECSDK_ENOMEM;
    }
    h->ws = rsort::workspace_carve(h->mem, max_pairs, key_bytes);
    *out = h;
    return RECSDK_OK;
}

extern "C" int recsdk_sorter_destroy(recsdk_sorter_t* h)
{
    if (h == nullptr) {
        return RECSDK_OK;
    }
    if (h->mem != nullptr) {
        (void)hipFree(h->mem);
    }
    delete h;
    return RECSDK_OK;
}

extern "C" int recsdk_sort_pairs(recsdk_sorter_t* h, const void* d_keys_in, void* d_keys_out, const uint32_t* d_values_in,
                                 uint32_t* d_values_out, int64_t n, int32_t bits, int32_t descending, void* stream)
{
    RECSDK_REQUIRE(h != nullptr, RECSDK_ENULL, "recsdk_sort_pairs: NULL handle");
    RECSDK_REQUIRE(n >= 0 && n <= h->maxPairs, RECSDK_ECAPACITY, "recsdk_sort_pairs: n exceeds the sorter's max_pairs");
    RECSDK_REQUIRE(bits >= 1 && bits <= 8 * h->keyBytes, RECSDK_EINVAL, "recsdk_sort_pairs: bits out of range");
    if (n == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_keys_in != nullptr && d_keys_out != nullptr && d_values_in != nullptr && d_values_out != nullptr,
                   RECSDK_ENULL, "recsdk_sort_pairs: NULL argument");
    RECSDK_REQUIRE(d_keys_in != d_keys_out && d_values_in != d_values_out, RECSDK_EINVAL,
                   "recsdk_sort_pairs: the outputs must not be the inputs");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (h->keyBytes == 4) {
        const uint32_t* in = static_cast<const uint32_t*>(d_keys_in);
        uint32_t* out = static_cast<uint32_t*>(d_keys_out);
        return descending ? rsort::sort_pairs<uint32_t, true>(h->ws, "sort_pairs", in, out, d_values_in, d_values_out, n, bits, s)
                          : rsort::sort_pairs<uint32_t, false>(h->ws, "sort_pairs", in, out, d_values_in, d_values_out, n, bits, s);
    }
    const uint64_t* in = static_cast<const uint64_t*>(d_keys_in);
    uint64_t* out = static_cast<uint64_t*>(d_keys_out);
    return descending ? rsort::sort_pairs<uint64_t, true>(h->ws, "sort_pairs", in, out, d_values_in, d_values_out, n, bits, s)
                      : rsort::sort_pairs<uint64_t, false>(h->ws, "sort_pairs", in, out, d_values_in, d_values_out, n, bits, s);
}
