// hybrid::IdsMapper as a torch class for ROCm tensors, over librecsdk_hip.so.
//
// The reference registers the class in TORCH_LIBRARY(hybrid, m) (training/torch_rec_v1/hybrid_torchrec/src/
// bind_torch_lib.cpp:9-19) with a constructor (init_max_index, only_device_mem) and three methods, all working on
// host tensors with a host hash map (src/ids_process/ids_mapper.cpp:24-285):
//   ids2indices_unique(global_ids) -> (hash_indices, unique, unique_inverse)          :24-61
//   ids2indices_unique_out(global_ids, hash_indices, offset, unique, unique_ids, unique_inverse, unique_offset,
//                          table_id)                                                   :63-174
//   parallel_ids2indices_unique_out(mappers, global_ids, hash_indices, offsets, unique, unique_ids, unique_inverse,
//                                   unique_offset)   (static, one mapper per table)    :176-285
// Here the same names take int64 tensors on a ROCm device: an id gets the next dense index of its mapper the first
// time it is seen (first-occurrence order inside a call), `unique` / `unique_ids` list a table's distinct indices /
// ids in that order, `unique_inverse` maps every position to its place in that list.  `offset` and `unique_offset`
// may live on the host or on the device; they are small and are read / written through the host.
// only_device_mem == false tells the reference not to bound the indices by init_max_index (they address a cache
// there); this implementation then sizes its table for 8 x init_max_index ids.
#include <algorithm>
#include <vector>

#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/custom_class.h>
#include <torch/library.h>

#include "recsdk_hip.h"

namespace {

using at::Tensor;

void check(int rc, const char* what)
{
    TORCH_CHECK(rc == RECSDK_OK, what, " failed: ", recsdk_last_error());
}

class IdsMapper : public torch::CustomClassHolder {
public:
    IdsMapper(int64_t initMaxIndex, bool onlyDeviceMem) : initMaxIndex_(initMaxIndex), onlyDeviceMem_(onlyDeviceMem)
    {
        TORCH_CHECK(initMaxIndex > 0, "init_max_index must be positive");
    }

    ~IdsMapper() override
    {
        if (tables_ != nullptr) {
            recsdk_tables_destroy(tables_);
        }
        Release();
    }

    std::tuple<Tensor, Tensor, Tensor> UniqueAndLookup(const Tensor& globalIds)
    {
        CheckIds(globalIds);
        const int64_t n = globalIds.numel();
        const Tensor ids = globalIds.contiguous().view({-1});
        Tensor hashIndices = at::empty({n}, ids.options());
        if (n == 0) {
            return {hashIndices.view_as(globalIds), at::empty({0}, ids.options()), at::empty({0}, ids.options())};
        }
        const c10::DeviceGuard guard(ids.device());
        void* s = Stream(ids);
        Tensor uniqueIdx = at::empty({n}, ids.options());
        const int64_t distinct = Map(ids, hashIndices, uniqueIdx, nullptr, nullptr, s);
        // UniqueParallel (src/ids_process/unique.cpp:110-118): the distinct indices in ascending order + inverse
        Tensor sorted = at::empty({n}, ids.options());
        Tensor inverse = at::empty({n}, ids.options());
        const int64_t off[2] = {0, n};
        const Tensor dOff = at::tensor(at::ArrayRef<int64_t>(off, 2), ids.options());
        check(recsdk_unique_run(unique_, hashIndices.data_ptr<int64_t>(), nullptr, dOff.data_ptr<int64_t>(), 1, n, 0, 0, s),
              "recsdk_unique_run");
        check(recsdk_unique_sorted(regroup_, unique_, sorted.data_ptr<int64_t>(), inverse.data_ptr<int64_t>(), s),
              "recsdk_unique_sorted");
        return {hashIndices.view_as(globalIds), sorted.slice(0, 0, distinct), inverse};
    }

    void UniqueAndLookupOut(const Tensor& globalIds, const Tensor& hashIndices, const Tensor& offset, const Tensor& unique,
                            const Tensor& uniqueIds, const Tensor& uniqueInverse, const Tensor& uniqueOffset,
                            int64_t tableId)
    {
        CheckIds(globalIds);
        for (const Tensor* t : {&hashIndices, &unique, &uniqueIds, &uniqueInverse}) {
            TORCH_CHECK(t->scalar_type() == at::kLong && t->is_contiguous() && t->device() == globalIds.device(),
                        "the output tensors must be contiguous int64 tensors on the device of global_ids");
        }
        TORCH_CHECK(offset.numel() - 1 > tableId && tableId >= 0, "offset must be equal to table size + 1");
        TORCH_CHECK(uniqueOffset.scalar_type() == at::kLong && uniqueOffset.numel() > tableId + 1,
                    "unique_offset must be an int64 tensor of table size + 1 entries");
        const Tensor hostOffset = offset.to(at::kCPU, at::kLong).contiguous();
        Tensor hostUnique = uniqueOffset.to(at::kCPU).contiguous();
        const int64_t start = hostOffset.data_ptr<int64_t>()[tableId];
        const int64_t end = hostOffset.data_ptr<int64_t>()[tableId + 1];
        int64_t* uo = hostUnique.data_ptr<int64_t>();
        if (tableId == 0) {
            uo[0] = 0;
        }
        const int64_t base = uo[tableId];
        int64_t distinct = 0;
        if (end > start) {
            TORCH_CHECK(start >= 0 && end <= globalIds.numel() && end <= hashIndices.numel() && end <= uniqueInverse.numel(),
                        "offset reaches past the tensors");
            const c10::DeviceGuard guard(globalIds.device());
            const Tensor ids = globalIds.contiguous().view({-1}).slice(0, start, end);
            Tensor idx = hashIndices.view({-1}).slice(0, start, end);
            Tensor inv = uniqueInverse.view({-1}).slice(0, start, end);
            Tensor uniqueIdx = at::empty({end - start}, ids.options());
            Tensor distinctIds = at::empty({end - start}, ids.options());
            distinct = Map(ids, idx, uniqueIdx, &distinctIds, &inv, Stream(ids));
            TORCH_CHECK(base + distinct <= unique.numel() && base + distinct <= uniqueIds.numel(),
                        "unique / unique_ids are too small for the distinct ids of table ", tableId);
            unique.view({-1}).slice(0, base, base + distinct).copy_(uniqueIdx.slice(0, 0, distinct));
            uniqueIds.view({-1}).slice(0, base, base + distinct).copy_(distinctIds.slice(0, 0, distinct));
        }
        uo[tableId + 1] = base + distinct;
        uniqueOffset.copy_(hostUnique);
    }

    static void ParallelUniqueHashOut(const c10::List<c10::intrusive_ptr<IdsMapper>>& mappers, const Tensor& globalIds,
                                      const Tensor& hashIndices, const Tensor& offsets, const Tensor& unique,
                                      const Tensor& uniqueIds, const Tensor& uniqueInverse, const Tensor& uniqueOffset)
    {
        const int64_t tables = (int64_t)mappers.size();
        TORCH_CHECK(offsets.numel() == tables + 1, "offsets must hold one more entry than there are mappers");
        for (int64_t t = 0; t < tables; ++t) {
            c10::intrusive_ptr<IdsMapper> m = mappers.get(t);
            m->UniqueAndLookupOut(globalIds, hashIndices, offsets, unique, uniqueIds, uniqueInverse, uniqueOffset, t);
        }
    }

private:
    static void* Stream(const Tensor& t) { return c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

    static void CheckIds(const Tensor& globalIds)
    {
        TORCH_CHECK(globalIds.scalar_type() == at::kLong,
                    "globalIds must be int64_t tensor expected but got a tensor with dtype: ", globalIds.scalar_type());
        TORCH_CHECK(globalIds.is_cuda(), "globalIds must be on a ROCm device");
        if (globalIds.numel() > 0) {
            const int64_t smallest = globalIds.min().item<int64_t>();
            TORCH_CHECK(smallest >= 0, " Invalid key value: ", smallest);
        }
    }

    void Release()
    {
        if (unique_ != nullptr) {
            recsdk_unique_destroy(unique_);
            unique_ = nullptr;
        }
        if (regroup_ != nullptr) {
            recsdk_regroup_destroy(regroup_);
            regroup_ = nullptr;
        }
        cap_ = 0;
    }

    // workspaces for n ids per call; the id -> index table is created once and lives as long as the mapper
    void Reserve(int64_t n)
    {
        if (tables_ == nullptr) {
            const int64_t vocab = onlyDeviceMem_ ? initMaxIndex_ : 8 * initMaxIndex_;
            check(recsdk_tables_create(1, &vocab, nullptr, nullptr, nullptr, kChunk, &tables_), "recsdk_tables_create");
        }
        if (n > cap_) {
            Release();
            int64_t cap = 1024;
            while (cap < n) {
                cap *= 2;
            }
            check(recsdk_unique_create(cap, 1, &unique_), "recsdk_unique_create");
            check(recsdk_unique_set_lists(unique_, 0), "recsdk_unique_set_lists");
            check(recsdk_regroup_create(cap, &regroup_), "recsdk_regroup_create");
            cap_ = cap;
        }
    }

    // ids -> dense indices.  hashIndices[i] = index of ids[i]; uniqueIdx[0..U) = indices of the distinct ids in order of
    // first occurrence; optionally the distinct ids themselves and the inverse (position -> place among the distinct).
    int64_t Map(const Tensor& ids, Tensor& hashIndices, Tensor& uniqueIdx, Tensor* distinctIds, Tensor* inverse, void* s)
    {
        const int64_t n = ids.numel();
        Reserve(n);
        const int64_t off[2] = {0, n};
        const Tensor dOff = at::tensor(at::ArrayRef<int64_t>(off, 2), ids.options());
        check(recsdk_unique_run(unique_, ids.data_ptr<int64_t>(), nullptr, dOff.data_ptr<int64_t>(), 1, n, 0, 0, s),
              "recsdk_unique_run");
        Tensor inv32 = inverse != nullptr ? at::empty({n}, ids.options().dtype(at::kInt)) : Tensor();
        Tensor uOff = at::empty({2}, ids.options());
        check(recsdk_unique_fetch(unique_, uniqueIdx.data_ptr<int64_t>(), uOff.data_ptr<int64_t>(),
                                  inverse != nullptr ? inv32.data_ptr<int32_t>() : nullptr, nullptr, s),
              "recsdk_unique_fetch");
        int64_t distinct = 0;
        check(recsdk_unique_total(unique_, s, &distinct), "recsdk_unique_total");
        if (distinctIds != nullptr) {
            distinctIds->slice(0, 0, distinct).copy_(uniqueIdx.slice(0, 0, distinct));
        }
        // distinct ids -> indices, in place, kChunk ids per call (new ids take indices in array order)
        for (int64_t first = 0; first < distinct; first += kChunk) {
            const int64_t m = std::min<int64_t>(kChunk, distinct - first);
            const int64_t chunkOff[2] = {0, m};
            const Tensor dChunk = at::tensor(at::ArrayRef<int64_t>(chunkOff, 2), ids.options());
            check(recsdk_tables_key2offset(tables_, uniqueIdx.data_ptr<int64_t>() + first, dChunk.data_ptr<int64_t>(), 1, m,
                                           RECSDK_CHANNEL_TRAIN, s),
                  "recsdk_tables_key2offset");
        }
        const int rc = recsdk_tables_stats(tables_, s, nullptr, nullptr, nullptr);
        TORCH_CHECK(rc != RECSDK_EOVERFLOW, "Ids map reached maxIndex = ", initMaxIndex_,
                    " please reallocate a larger buffer.");
        check(rc, "recsdk_tables_stats");
        check(recsdk_unique_expand(unique_, uniqueIdx.data_ptr<int64_t>(), -1, hashIndices.data_ptr<int64_t>(), s),
              "recsdk_unique_expand");
        if (inverse != nullptr) {
            inverse->copy_(inv32);
        }
        return distinct;
    }

    static constexpr int64_t kChunk = 1 << 20;
    int64_t initMaxIndex_;
    bool onlyDeviceMem_;
    recsdk_tables_t* tables_ = nullptr;
    recsdk_unique_t* unique_ = nullptr;
    recsdk_regroup_t* regroup_ = nullptr;
    int64_t cap_ = 0;
};

}  // namespace

TORCH_LIBRARY(hybrid, m)
{
    m.class_<IdsMapper>("IdsMapper")
        .def(torch::init<int64_t, bool>())
        .def("ids2indices_unique", &IdsMapper::UniqueAndLookup)
        .def("ids2indices_unique_out", &IdsMapper::UniqueAndLookupOut)
        .def_static("parallel_ids2indices_unique_out", &IdsMapper::ParallelUniqueHashOut);
}
