// Checkpoint files of the device-resident tables, in the reference's on-disk layout.
//
// EmbeddingStatic::SaveKey / LoadKey        training/tf_rec_v1/src/core/emb_table/embedding_static.cpp:137-239
// EmbeddingDynamic::SaveKey / SaveEmbData / SaveOptimData / LoadKey / LoadEmbAndOptim
//                                           training/tf_rec_v1/src/core/emb_table/embedding_dynamic.cpp:178-387
// LocalFileSystem::WriteEmbedding / ReadEmbedding
//                                           training/tf_rec_v1/src/core/file_system/local_file_system/local_file_system.cpp:165-224,317-381
// A key file is the raw int64 keys; a row file holds, for the i-th key of the key file, embSize floats.  The reference
// copies row by row between the device and the file; here a kernel packs (unpacks) a chunk of rows into (from) pinned
// host memory and the file is written (read) in chunks, two buffers in flight.
#include <algorithm>
#include <vector>

#include "common.h"
#include "fileio.h"

namespace recsdk {

constexpr int64_t kChunkBytes = int64_t(32) << 20;  // pinned staging per buffer

// rows at device addresses -> dense [m, dim] staging (pinned host memory seen from the device)
__global__ __launch_bounds__(kBlock) void k_ckpt_pack(const int64_t* __restrict__ addr, int64_t byteOffset, int64_t m,
                                                      int32_t dim, float* __restrict__ stage)
{
    const int64_t total = m * dim;
    for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total; e += (int64_t)gridDim.x * kBlock) {
        const int64_t i = e / dim;
        const int32_t c = (int32_t)(e - i * dim);
        const float* row = reinterpret_cast<const float*>(addr[i] + byteOffset);
        stage[e] = row[c];
    }
}

// dense [m, dim] staging -> rows first + (row0 + i) * ext floats
__global__ __launch_bounds__(kBlock) void k_ckpt_unpack(const float* __restrict__ stage, int64_t m, int32_t dim,
                                                        float* __restrict__ first, int64_t row0, int64_t ext)
{
    const int64_t total = m * dim;
    for (int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x; e < total; e += (int64_t)gridDim.x * kBlock) {
        const int64_t i = e / dim;
        const int32_t c = (int32_t)(e - i * dim);
        first[(row0 + i) * ext + c] = stage[e];
    }
}

struct Staging {
    float* host[2] = {nullptr, nullptr};
    float* dev[2] = {nullptr, nullptr};
    hipEvent_t done[2] = {nullptr, nullptr};
    ~Staging()
    {
        for (int k = 0; k < 2; ++k) {
            if (host[k] != nullptr) {
                (void)hipHostFree(host[k]);
            }
            if (done[k] != nullptr) {
                (void)hipEventDestroy(done[k]);
            }
        }
    }
    int Init(size_t bytes)
    {
        for (int k = 0; k < 2; ++k) {
            RECSDK_HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&host[k]), bytes, hipHostMallocMapped));
            RECSDK_HIP_TRY(hipHostGetDevicePointer(reinterpret_cast<void**>(&dev[k]), host[k], 0));
            RECSDK_HIP_TRY(hipEventCreateWithFlags(&done[k], hipEventDisableTiming));
        }
        return RECSDK_OK;
    }
};

}  // namespace recsdk

using namespace recsdk;

extern "C" int recsdk_ckpt_write_keys(const char* path, const int64_t* d_keys, int64_t n, void* stream)
{
    RECSDK_REQUIRE(path != nullptr && (n == 0 || d_keys != nullptr), RECSDK_ENULL, "recsdk_ckpt_write_keys: NULL argument");
    RECSDK_REQUIRE(n >= 0, RECSDK_EINVAL, "recsdk_ckpt_write_keys: negative size");
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::vector<int64_t> keys((size_t)n);
    if (n > 0) {
        RECSDK_HIP_TRY(hipMemcpyAsync(keys.data(), d_keys, sizeof(int64_t) * n, hipMemcpyDeviceToHost, s));
        RECSDK_HIP_TRY(hipStreamSynchronize(s));
    }
    return write_file(path, keys.data(), sizeof(int64_t) * (size_t)n);
}

extern "C" int recsdk_ckpt_read_keys(const char* path, int32_t rank_id, int32_t rank_size, int32_t is_dp,
                                     int64_t* h_keys, int64_t* h_load_offset, int64_t cap, int64_t* h_count)
{
    RECSDK_REQUIRE(path != nullptr && h_count != nullptr, RECSDK_ENULL, "recsdk_ckpt_read_keys: NULL argument");
    RECSDK_REQUIRE(rank_size > 0 && rank_id >= 0 && rank_id < rank_size, RECSDK_EINVAL,
                   "recsdk_ckpt_read_keys: bad rank id / rank size");
    std::vector<char> raw;
    const int rc = read_file(path, sizeof(int64_t), &raw);
    if (rc != RECSDK_OK) {
        return rc;
    }
    const int64_t* buf = reinterpret_cast<const int64_t*>(raw.data());
    const int64_t total = (int64_t)(raw.size() / sizeof(int64_t));
    int64_t m = 0;
    for (int64_t i = 0; i < total; ++i) {
        // model parallel: the rank keeps the keys with key % rankSize == rankId (C++ remainder, as the reference)
        if (!is_dp && buf[i] % rank_size != rank_id) {
            continue;
        }
        if (m < cap && h_keys != nullptr) {
            h_keys[m] = buf[i];
        }
        if (m < cap && h_load_offset != nullptr) {
            h_load_offset[m] = i;
        }
        ++m;
    }
    *h_count = m;
    if (m > cap) {
        set_error("recsdk_ckpt_read_keys: %ld keys for this rank, the buffers take %ld", (long)m, (long)cap);
        return RECSDK_ECAPACITY;
    }
    return RECSDK_OK;
}

extern "C" int recsdk_ckpt_write_rows(const char* path, const int64_t* d_addr, int64_t n, int32_t emb_size,
                                      int64_t byte_offset, void* stream)
{
    RECSDK_REQUIRE(path != nullptr && (n == 0 || d_addr != nullptr), RECSDK_ENULL, "recsdk_ckpt_write_rows: NULL argument");
    RECSDK_REQUIRE(n >= 0 && emb_size > 0 && byte_offset % 4 == 0, RECSDK_EINVAL,
                   "recsdk_ckpt_write_rows: sizes must be positive and the offset a multiple of 4");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!make_parent_dirs(path)) {
        set_error("Create directory for %s failed: %s", path, strerror(errno));
        return RECSDK_EIO;
    }
    const int fd = open(path, O_RDWR | O_CREAT | O_TRUNC, 0640);
    if (fd == -1) {
        set_error("Open file %s to write failed.", path);
        return RECSDK_EIO;
    }
    const int64_t rowBytes = (int64_t)emb_size * 4;
    const int64_t chunkRows = std::max<int64_t>(kChunkBytes / rowBytes, 1);
    Staging st;
    auto body = [&]() -> int {
        if (n == 0) {
            return RECSDK_OK;
        }
        int rc = st.Init((size_t)(std::min(chunkRows, n) * rowBytes));
        if (rc != RECSDK_OK) {
            return rc;
        }
        const int64_t chunks = cdiv(n, chunkRows);
        // chunk c is packed into buffer c % 2 while chunk c - 1 goes to the file
        for (int64_t c = 0; c <= chunks; ++c) {
            if (c < chunks) {
                const int64_t r0 = c * chunkRows;
                const int64_t m = std::min(chunkRows, n - r0);
                const unsigned grid = (unsigned)std::min<int64_t>(cdiv(m * emb_size, kBlock), 256 * 16);
                RECSDK_LAUNCH(k_ckpt_pack, dim3(grid), dim3(kBlock), s, d_addr + r0, byte_offset, m, emb_size,
                              st.dev[c & 1]);
                RECSDK_HIP_TRY(hipEventRecord(st.done[c & 1], s));
            }
            if (c > 0) {
                const int64_t p = c - 1;
                const int64_t r0 = p * chunkRows;
                const int64_t m = std::min(chunkRows, n - r0);
                RECSDK_HIP_TRY(hipEventSynchronize(st.done[p & 1]));
                if (!write_all(fd, st.host[p & 1], (size_t)(m * rowBytes))) {
                    set_error("Error writing to local file %s, please check the disk space or file permissions!", path);
                    return RECSDK_EIO;
                }
            }
        }
        return RECSDK_OK;
    };
    const int rc = body();
    (void)hipStreamSynchronize(s);  // no kernel may still write the staging buffers when they are freed
    close(fd);
    return rc;
}

extern "C" int recsdk_ckpt_read_rows(const char* path, const int64_t* h_load_offset, int64_t n, int32_t emb_size,
                                     float* d_first, int64_t ext_emb_size, void* stream)
{
    RECSDK_REQUIRE(path != nullptr && (n == 0 || d_first != nullptr), RECSDK_ENULL, "recsdk_ckpt_read_rows: NULL argument");
    RECSDK_REQUIRE(n >= 0 && emb_size > 0 && ext_emb_size >= emb_size, RECSDK_EINVAL,
                   "recsdk_ckpt_read_rows: bad sizes");
    if (n == 0) {
        return RECSDK_OK;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t size = file_size_of(path);
    const int fd = size < 0 ? -1 : open(path, O_RDONLY);
    if (fd == -1) {
        set_error("Failed to open read file: %s.", path);
        return RECSDK_EIO;
    }
    const int64_t rowBytes = (int64_t)emb_size * 4;
    const int64_t chunkRows = std::max<int64_t>(kChunkBytes / rowBytes, 1);
    Staging st;
    auto body = [&]() -> int {
        int rc = st.Init((size_t)(std::min(chunkRows, n) * rowBytes));
        if (rc != RECSDK_OK) {
            return rc;
        }
        bool used[2] = {false, false};
        for (int64_t c = 0; c * chunkRows < n; ++c) {
            const int k = (int)(c & 1);
            const int64_t r0 = c * chunkRows;
            const int64_t m = std::min(chunkRows, n - r0);
            if (used[k]) {
                RECSDK_HIP_TRY(hipEventSynchronize(st.done[k]));  // the kernel that read this buffer two chunks ago
            }
            // file rows loadOffset[r0 .. r0+m): neighbouring rows are read with one call
            int64_t i = 0;
            while (i < m) {
                const int64_t f0 = h_load_offset != nullptr ? h_load_offset[r0 + i] : r0 + i;
                int64_t j = i + 1;
                while (j < m && (h_load_offset != nullptr ? h_load_offset[r0 + j] : r0 + j) == f0 + (j - i)) {
                    ++j;
                }
                if (f0 < 0 || (f0 + (j - i)) * rowBytes > size) {
                    set_error("Failed to read file path: %s (row %ld is outside the file).", path, (long)f0);
                    return RECSDK_EIO;
                }
                if (!read_all_at(fd, reinterpret_cast<char*>(st.host[k]) + i * rowBytes, (size_t)((j - i) * rowBytes),
                                 f0 * rowBytes)) {
                    set_error("Failed to read file path: %s.", path);
                    return RECSDK_EIO;
                }
                i = j;
            }
            const unsigned grid = (unsigned)std::min<int64_t>(cdiv(m * emb_size, kBlock), 256 * 16);
            RECSDK_LAUNCH(k_ckpt_unpack, dim3(grid), dim3(kBlock), s, st.dev[k], m, emb_size, d_first, r0, ext_emb_size);
            RECSDK_HIP_TRY(hipEventRecord(st.done[k], s));
            used[k] = true;
        }
        return RECSDK_OK;
    };
    const int rc = body();
    (void)hipStreamSynchronize(s);
    close(fd);
    return rc;
}
