// Batch ingestion: the step right before the dedup.
//
// ReadEmbKeyV2::EnqueueBatchData / ParseTimestampAndCheck (training/tf_rec_v1/src/ops_tf/hybrid_dataset_ops.cpp:467-531):
// the input pipeline hands over ONE tensor per batch, [timestamp?][keys of table 0][keys of table 1]..., int32 or int64;
// table i takes splits[i] elements, tables the key process does not know are skipped.  Here the per-table batches of
// one step become one int64 key array + offsets[T_used+1] on the device, the layout every other entry point takes.
// KeyProcess::PushPaddingKeysTensors (key_process.cpp:1808-1827): mask 0 for values in a small set, 1 otherwise.
#include <algorithm>
#include <vector>

#include "common.h"

namespace recsdk {

constexpr int kIngestSegs = 64;   // contiguous source runs per launch (passed by value)
constexpr int kMaskVals = 64;     // padding values per launch

struct IngestSegs {
    int64_t src[kIngestSegs];      // first source element of the run
    int64_t dst[kIngestSegs + 1];  // first destination element; dst[count] = end
    int32_t count;
};

template <typename SrcT>
__global__ __launch_bounds__(kBlock) void k_ingest_copy(const SrcT* __restrict__ sample, int64_t* __restrict__ keys,
                                                        const IngestSegs segs)
{
    const int64_t first = segs.dst[0];
    const int64_t end = segs.dst[segs.count];
    for (int64_t i = first + (int64_t)blockIdx.x * kBlock + threadIdx.x; i < end; i += (int64_t)gridDim.x * kBlock) {
        int lo = 0;
        int hi = segs.count - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (segs.dst[mid] <= i) {
                lo = mid;
            } else {
                hi = mid - 1;
            }
        }
        keys[i] = (int64_t)sample[segs.src[lo] + (i - segs.dst[lo])];
    }
}

struct OffsetVals {
    int64_t v[kIngestSegs];
    int32_t count;
    int32_t first;
};

__global__ void k_ingest_offsets(int64_t* __restrict__ offsets, const OffsetVals o)
{
    if ((int)threadIdx.x < o.count) {
        offsets[o.first + threadIdx.x] = o.v[threadIdx.x];
    }
}

struct MaskVals {
    int64_t v[kMaskVals];
    int32_t count;
};

template <bool FIRST>
__global__ __launch_bounds__(kBlock) void k_padding_mask(const int64_t* __restrict__ values, int64_t n,
                                                         int32_t* __restrict__ mask, const MaskVals pad)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) {
        return;
    }
    const int64_t x = values[i];
    int32_t m = FIRST ? 1 : mask[i];
    for (int j = 0; j < pad.count; ++j) {
        if (pad.v[j] == x) {
            m = 0;
        }
    }
    mask[i] = m;
}

}  // namespace recsdk

using namespace recsdk;

extern "C" int recsdk_read_emb_key(const void* d_sample, int32_t sample_dtype, int64_t data_size,
                                   const int64_t* h_splits, const uint8_t* h_table_used, int32_t n_tables,
                                   int32_t is_timestamp, int64_t field_num, int64_t* d_keys, int64_t* d_offsets,
                                   int64_t* h_offsets, int64_t* h_timestamp, void* stream)
{
    RECSDK_REQUIRE(h_splits != nullptr && (d_sample != nullptr || data_size == 0), RECSDK_ENULL,
                   "recsdk_read_emb_key: NULL argument");
    RECSDK_REQUIRE(sample_dtype == RECSDK_DT_I32 || sample_dtype == RECSDK_DT_I64, RECSDK_EINVAL,
                   "recsdk_read_emb_key: the sample tensor must be int32 or int64");
    RECSDK_REQUIRE(n_tables >= 0 && data_size >= 0, RECSDK_EINVAL, "recsdk_read_emb_key: negative size");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t elem = sample_dtype == RECSDK_DT_I32 ? 4 : 8;
    int64_t offset = 0;
    if (is_timestamp) {
        // ParseTimestampAndCheck: exactly one element more than the feature fields; the first 8 bytes are a unix time > 0
        if (data_size - field_num != 1) {
            set_error("Timestamp field not found, dataSize:%ld, fieldNum:%ld.", (long)data_size, (long)field_num);
            return RECSDK_EINVAL;
        }
        RECSDK_REQUIRE((size_t)data_size * elem >= sizeof(int64_t), RECSDK_EINVAL,
                       "recsdk_read_emb_key: the sample tensor is shorter than a timestamp");
        int64_t ts = 0;
        RECSDK_HIP_TRY(hipMemcpyAsync(&ts, d_sample, sizeof(int64_t), hipMemcpyDeviceToHost, s));
        RECSDK_HIP_TRY(hipStreamSynchronize(s));
        if (ts <= 0) {
            set_error("Timestamp should greater than 0, get:%ld.", (long)ts);
            return RECSDK_EINVAL;
        }
        if (h_timestamp != nullptr) {
            *h_timestamp = ts;
        }
        offset = 1;  // one element, whatever its width
    } else if (h_timestamp != nullptr) {
        *h_timestamp = -1;
    }
    // source runs of the used tables (neighbours merge into one run)
    std::vector<int64_t> offs(1, 0);
    std::vector<int64_t> runSrc;
    std::vector<int64_t> runDst;
    int64_t total = 0;
    bool open = false;
    for (int i = 0; i < n_tables; ++i) {
        const int64_t len = h_splits[i];
        RECSDK_REQUIRE(len >= 0, RECSDK_EINVAL, "recsdk_read_emb_key: negative split");
        RECSDK_REQUIRE(offset + len <= data_size, RECSDK_EINVAL,
                       "recsdk_read_emb_key: the splits add up to more than the sample tensor holds");
        if (h_table_used != nullptr && !h_table_used[i]) {
            open = false;
        } else {
            if (!open && len > 0) {
                runSrc.push_back(offset);
                runDst.push_back(total);
                open = true;
            }
            total += len;
            offs.push_back(total);
        }
        offset += len;
    }
    RECSDK_REQUIRE(total == 0 || d_keys != nullptr, RECSDK_ENULL, "recsdk_read_emb_key: d_keys is NULL");
    if (h_offsets != nullptr) {
        for (size_t j = 0; j < offs.size(); ++j) {
            h_offsets[j] = offs[j];
        }
    }
    if (d_offsets != nullptr) {
        for (size_t b = 0; b < offs.size(); b += kIngestSegs) {
            OffsetVals o;
            o.first = (int32_t)b;
            o.count = (int32_t)std::min<size_t>(kIngestSegs, offs.size() - b);
            for (int j = 0; j < o.count; ++j) {
                o.v[j] = offs[b + j];
            }
            RECSDK_LAUNCH(k_ingest_offsets, dim3(1), dim3(kIngestSegs), s, d_offsets, o);
        }
    }
    runDst.push_back(total);
    const size_t runs = runSrc.size();
    for (size_t b = 0; b < runs; b += kIngestSegs) {
        IngestSegs g;
        g.count = (int32_t)std::min<size_t>(kIngestSegs, runs - b);
        for (int j = 0; j < g.count; ++j) {
            g.src[j] = runSrc[b + j];
            g.dst[j] = runDst[b + j];
        }
        g.dst[g.count] = runDst[b + g.count];
        const int64_t span = g.dst[g.count] - g.dst[0];
        const unsigned grid = (unsigned)std::min<int64_t>(std::max<int64_t>(cdiv(span, kBlock), 1), 1 << 16);
        if (sample_dtype == RECSDK_DT_I32) {
            RECSDK_LAUNCH(k_ingest_copy<int32_t>, dim3(grid), dim3(kBlock), s, static_cast<const int32_t*>(d_sample),
                          d_keys, g);
        } else {
            RECSDK_LAUNCH(k_ingest_copy<int64_t>, dim3(grid), dim3(kBlock), s, static_cast<const int64_t*>(d_sample),
                          d_keys, g);
        }
    }
    return RECSDK_OK;
}

extern "C" int recsdk_padding_keys_mask(const int64_t* d_values, int64_t n, const int64_t* h_padding, int32_t n_padding,
                                        int32_t* d_mask, void* stream)
{
    RECSDK_REQUIRE(n >= 0 && n_padding >= 0, RECSDK_EINVAL, "recsdk_padding_keys_mask: negative size");
    if (n == 0) {
        return RECSDK_OK;
    }
    RECSDK_REQUIRE(d_values != nullptr && d_mask != nullptr && (n_padding == 0 || h_padding != nullptr), RECSDK_ENULL,
                   "recsdk_padding_keys_mask: NULL argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned grid = (unsigned)cdiv(n, kBlock);
    int32_t b = 0;
    do {
        MaskVals p;
        p.count = std::min<int32_t>(kMaskVals, n_padding - b);
        for (int j = 0; j < p.count; ++j) {
            p.v[j] = h_padding[b + j];
        }
        if (b == 0) {
            RECSDK_LAUNCH(k_padding_mask<true>, dim3(grid), dim3(kBlock), s, d_values, n, d_mask, p);
        } else {
            RECSDK_LAUNCH(k_padding_mask<false>, dim3(grid), dim3(kBlock), s, d_values, n, d_mask, p);
        }
        b += kMaskVals;
    } while (b < n_padding);
    return RECSDK_OK;
}
