// The reference's torch operator surface for the pooled lookup, registered for ROCm tensors over librecsdk_hip.so.
//
// The reference registers these schemas in TORCH_LIBRARY_FRAGMENT(fbgemm, ...) and implements them with Ascend
// aclnn calls (cust_op/framework/torch_plugin/torch_library/2.6.0/split_embedding_codegen_forward_unweighted/):
//   split_embedding_codegen_forward_unweighted_cuda                     split_embedding_codegen_forward_unweighted.cpp:75-100
//   split_embedding_backward_codegen_adagrad_unweighted_exact_cuda      backward_codegen_adagrad_unweighted_exact.cpp:333-372
//   split_embedding_backward_codegen_adam_unweighted_exact_cuda         backward_codegen_adam_unweighted_exact.cpp:467-512
//   split_embedding_backward_codegen_sgd_unweighted_exact_cuda          backward_codegen_sgd_unweighted_exact.cpp:387-422
//   split_embedding_codegen_lookup_{adagrad,adam,sgd}_function          the same files :282-331, :414-465, :334-385
// Here the same names and argument lists resolve, for tensors on a ROCm device, to recsdk_tbe_forward /
// recsdk_tbe_backward on the caller's current stream.  A model written against the reference's operators (or
// fbgemm_gpu's, whose names these are) runs unchanged after torch.ops.load_library(<this library>).
//
// hash_indices, when given, replaces indices in the forward and the backward (the reference's kernels read rows by it:
// split_embedding_codegen_forward_unweighted_kernel.h:103-107, backward_codegen_unweighted_exact_kernel.h:314,373-374);
// unique_ids / unique_offsets / unique_inverse, when given, select the unique variant of the backward
// (backward_codegen_unweighted_exact_kernel_unique.h), which groups the positions by the caller's inverse index.
// Arguments the reference accepts and ignores on its device (uvm / lxu cache tensors, placements, stochastic
// rounding, the vbe and gwd arguments, offset_per_key) are accepted and ignored here too.
#include <algorithm>
#include <map>
#include <mutex>
#include <string>
#include <tuple>

#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/autograd.h>
#include <torch/library.h>

#include "recsdk_hip.h"

namespace {

using at::Tensor;
using c10::optional;

void check(int rc, const char* what)
{
    TORCH_CHECK(rc == RECSDK_OK, what, " failed: ", recsdk_last_error());
}

void* current_stream(const Tensor& t)
{
    return c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

int32_t weights_dtype(const Tensor& w)
{
    TORCH_CHECK(w.scalar_type() == at::kFloat || w.scalar_type() == at::kBFloat16,
                "dev_weights must be float32 or bfloat16, got ", w.scalar_type());
    return w.scalar_type() == at::kFloat ? RECSDK_DT_F32 : RECSDK_DT_BF16;
}

// an optional tensor argument that the caller filled in
bool given(const Tensor& t)
{
    return t.defined() && t.numel() > 0;
}

// the index tensors in the layout the library takes (they already are in the usual case)
struct Layout {
    Tensor weightsOffsets, dOffsets, indices, offsets;
    int32_t T;
    int64_t B;
    int64_t nnz;
};

Layout make_layout(const Tensor& dev_weights, const Tensor& weights_offsets, const Tensor& D_offsets,
                   const Tensor& indices, const Tensor& offsets)
{
    TORCH_CHECK(dev_weights.is_cuda(), "dev_weights must be on a ROCm device");
    TORCH_CHECK(dev_weights.is_contiguous(), "dev_weights must be contiguous");
    for (const Tensor* t : {&weights_offsets, &D_offsets, &indices, &offsets}) {
        TORCH_CHECK(t->device() == dev_weights.device(), "all tensors must be on the device of dev_weights");
    }
    Layout l;
    l.weightsOffsets = weights_offsets.to(at::kLong).contiguous();
    l.dOffsets = D_offsets.to(at::kInt).contiguous();
    l.indices = indices.to(at::kLong).contiguous();
    l.offsets = offsets.to(at::kLong).contiguous();
    l.T = (int32_t)weights_offsets.numel();
    TORCH_CHECK(l.T > 0 && D_offsets.numel() == l.T + 1, "D_offsets must hold one more entry than weights_offsets");
    TORCH_CHECK(offsets.numel() >= 1 && (offsets.numel() - 1) % l.T == 0, "offsets must hold T * B + 1 entries");
    l.B = (offsets.numel() - 1) / l.T;
    l.nnz = indices.numel();
    return l;
}

Tensor forward_op(const Tensor& dev_weights, const Tensor& /*uvm_weights*/, const Tensor& /*lxu_cache_weights*/,
                  const Tensor& /*weights_placements*/, const Tensor& weights_offsets, const Tensor& D_offsets,
                  c10::SymInt total_D_, c10::SymInt max_D_, const Tensor& indices, const Tensor& offsets,
                  int64_t pooling_mode, const Tensor& /*lxu_cache_locations*/, const Tensor& /*uvm_cache_stats*/,
                  int64_t /*output_dtype*/, bool /*is_experimental*/, const Tensor& hash_indices,
                  const Tensor& /*offset_per_key*/)
{
    const int64_t total_D = total_D_.expect_int();
    const int64_t max_D = max_D_.expect_int();
    const Layout l = make_layout(dev_weights, weights_offsets, D_offsets, given(hash_indices) ? hash_indices : indices,
                                 offsets);
    const c10::DeviceGuard guard(dev_weights.device());
    Tensor out = pooling_mode == RECSDK_POOL_NONE
                     ? at::empty({l.nnz, total_D / l.T}, dev_weights.options().dtype(at::kFloat))
                     : at::empty({l.B, total_D}, dev_weights.options().dtype(at::kFloat));
    check(recsdk_tbe_forward(dev_weights.data_ptr(), weights_dtype(dev_weights), dev_weights.numel(),
                             l.weightsOffsets.data_ptr<int64_t>(), l.dOffsets.data_ptr<int32_t>(), total_D,
                             (int32_t)max_D, l.indices.data_ptr<int64_t>(), l.offsets.data_ptr<int64_t>(), l.T, l.B,
                             l.nnz, (int32_t)pooling_mode, out.data_ptr<float>(), current_stream(dev_weights)),
          "split_embedding_codegen_forward_unweighted_cuda");
    return out;
}

// One backward workspace per device.  The library reads the tables' sizes from hash_size_cumsum once per handle, so
// the workspace keeps the tensor it was created for alive (its memory cannot be handed to another tensor meanwhile)
// and is rebuilt when a call brings a different one.
struct Workspace {
    recsdk_tbe_t* h = nullptr;
    int32_t tables = 0;
    int64_t nnz = 0;
    Tensor cumsum;
};
std::mutex g_wsLock;
std::map<int, Workspace> g_ws;

recsdk_tbe_t* workspace(const Tensor& hash_size_cumsum, int32_t T, int64_t nnz)
{
    std::lock_guard<std::mutex> lock(g_wsLock);
    Workspace& w = g_ws[(int)hash_size_cumsum.device().index()];
    const bool sameTables = w.cumsum.defined() && w.cumsum.data_ptr() == hash_size_cumsum.data_ptr() && w.tables == T;
    if (w.h == nullptr || !sameTables || w.nnz < nnz) {
        if (w.h != nullptr) {
            recsdk_tbe_destroy(w.h);
            w.h = nullptr;
        }
        int64_t cap = std::max<int64_t>(w.nnz, 1024);
        while (cap < nnz) {
            cap *= 2;
        }
        check(recsdk_tbe_create(T, cap, &w.h), "recsdk_tbe_create");
        w.tables = T;
        w.nnz = cap;
        w.cumsum = hash_size_cumsum;
    }
    return w.h;
}

void backward_common(int32_t optim, const Tensor& grad_output, const Tensor& dev_weights, const Tensor& weights_offsets,
                     const Tensor& D_offsets, int64_t max_D, const Tensor& hash_size_cumsum, const Tensor& indices,
                     const Tensor& offsets, int64_t pooling_mode, const Tensor* momentum1, const Tensor* momentum2,
                     const Tensor& hash_indices, const Tensor& unique_ids, const Tensor& unique_offsets,
                     const Tensor& unique_inverse, double eps, double learning_rate, double beta1, double beta2,
                     int64_t iter, const char* name)
{
    const Layout l = make_layout(dev_weights, weights_offsets, D_offsets, given(hash_indices) ? hash_indices : indices,
                                 offsets);
    const c10::DeviceGuard guard(dev_weights.device());
    TORCH_CHECK(grad_output.device() == dev_weights.device(), name, ": grad_output is on another device");
    const Tensor grad = grad_output.to(at::kFloat).contiguous();
    const Tensor cumsum = hash_size_cumsum.scalar_type() == at::kLong && hash_size_cumsum.is_contiguous()
                              ? hash_size_cumsum
                              : hash_size_cumsum.to(at::kLong).contiguous();
    TORCH_CHECK(cumsum.device() == dev_weights.device() && cumsum.numel() >= l.T + 1, name,
                ": hash_size_cumsum must hold T + 1 entries on the device");
    float* m1 = nullptr;
    float* m2 = nullptr;
    for (auto pm : {std::make_pair(momentum1, &m1), std::make_pair(momentum2, &m2)}) {
        if (pm.first != nullptr) {
            TORCH_CHECK(pm.first->scalar_type() == at::kFloat && pm.first->is_contiguous() &&
                            pm.first->device() == dev_weights.device() && pm.first->numel() == dev_weights.numel(),
                        name, ": optimizer state must be a contiguous float32 tensor laid out like dev_weights");
            *pm.second = pm.first->data_ptr<float>();
        }
    }
    const int64_t total_D = grad.dim() == 2 ? (pooling_mode == RECSDK_POOL_NONE ? grad.size(1) * l.T : grad.size(1)) : 0;
    recsdk_tbe_t* h = workspace(cumsum, l.T, l.nnz);
    if (given(unique_ids)) {
        TORCH_CHECK(given(unique_inverse) && unique_offsets.defined() && unique_offsets.numel() == l.T + 1, name,
                    ": unique_ids needs unique_inverse and unique_offsets with one entry per feature plus one");
        TORCH_CHECK(unique_inverse.numel() == l.nnz, name, ": unique_inverse must hold one entry per index");
        for (const Tensor* t : {&unique_ids, &unique_offsets, &unique_inverse}) {
            TORCH_CHECK(t->device() == dev_weights.device(), name, ": the unique tensors must be on the device of dev_weights");
        }
        const Tensor ids = unique_ids.to(at::kLong).contiguous();
        const Tensor uoff = unique_offsets.to(at::kLong).contiguous();
        const Tensor inv = unique_inverse.to(at::kLong).contiguous();
        check(recsdk_tbe_backward_unique(h, optim, grad.data_ptr<float>(), dev_weights.data_ptr(),
                                         weights_dtype(dev_weights), l.weightsOffsets.data_ptr<int64_t>(),
                                         l.dOffsets.data_ptr<int32_t>(), total_D, (int32_t)max_D,
                                         cumsum.data_ptr<int64_t>(), l.offsets.data_ptr<int64_t>(), l.T, l.B, l.nnz,
                                         (int32_t)pooling_mode, ids.data_ptr<int64_t>(), uoff.data_ptr<int64_t>(),
                                         inv.data_ptr<int64_t>(), ids.numel(), m1, m2, (float)learning_rate, (float)eps,
                                         (float)beta1, (float)beta2, iter, current_stream(dev_weights)),
              name);
        return;
    }
    check(recsdk_tbe_backward(h, optim, grad.data_ptr<float>(), dev_weights.data_ptr(), weights_dtype(dev_weights),
                              l.weightsOffsets.data_ptr<int64_t>(), l.dOffsets.data_ptr<int32_t>(), total_D,
                              (int32_t)max_D, cumsum.data_ptr<int64_t>(), l.indices.data_ptr<int64_t>(),
                              l.offsets.data_ptr<int64_t>(), l.T, l.B, l.nnz, (int32_t)pooling_mode, m1, m2,
                              (float)learning_rate, (float)eps, (float)beta1, (float)beta2, iter,
                              current_stream(dev_weights)),
          name);
}

// the argument block every backward operator starts with
#define BACKWARD_HEAD                                                                                                \
    const Tensor &grad_output, const Tensor &dev_weights, const Tensor & /*uvm_weights*/,                            \
        const Tensor & /*lxu_cache_weights*/, const Tensor & /*weights_placements*/, const Tensor &weights_offsets,  \
        const Tensor &D_offsets, c10::SymInt max_D, const Tensor &hash_size_cumsum, int64_t /*total_hash_size_bits*/, \
        const Tensor &indices, const Tensor &offsets, int64_t pooling_mode, const Tensor & /*lxu_cache_locations*/,   \
        int64_t /*unused_*/, int64_t /*max_segment_length_per_warp*/, bool /*stochastic_rounding*/,                   \
        int64_t /*info_B_num_bits*/, int64_t /*info_B_mask_int64*/, bool /*use_uniq_cache_locations*/,                \
        bool /*use_homogeneous_placements*/
#define BACKWARD_TAIL                                                                                                \
    const Tensor &hash_indices, const Tensor &unique_ids, const Tensor &unique_offsets,                              \
        const Tensor &unique_inverse, const Tensor & /*offset_per_key*/

Tensor backward_adagrad_op(BACKWARD_HEAD, const Tensor& momentum1_dev, const Tensor& /*momentum1_uvm*/,
                           const Tensor& /*momentum1_placements*/, const Tensor& /*momentum1_offsets*/, BACKWARD_TAIL,
                           double eps, double learning_rate)
{
    backward_common(RECSDK_OPT_ADAGRAD, grad_output, dev_weights, weights_offsets, D_offsets, max_D.expect_int(),
                    hash_size_cumsum, indices, offsets, pooling_mode, &momentum1_dev, nullptr, hash_indices, unique_ids,
                    unique_offsets, unique_inverse, eps, learning_rate, 0, 0, 0,
                    "split_embedding_backward_codegen_adagrad_unweighted_exact_cuda");
    return Tensor();
}

Tensor backward_adam_op(BACKWARD_HEAD, const Tensor& momentum1_dev, const Tensor& /*momentum1_uvm*/,
                        const Tensor& /*momentum1_placements*/, const Tensor& /*momentum1_offsets*/,
                        const Tensor& momentum2_dev, const Tensor& /*momentum2_uvm*/,
                        const Tensor& /*momentum2_placements*/, const Tensor& /*momentum2_offsets*/, BACKWARD_TAIL,
                        double eps, double learning_rate, double beta1, double beta2, int64_t iter)
{
    backward_common(RECSDK_OPT_ADAM, grad_output, dev_weights, weights_offsets, D_offsets, max_D.expect_int(),
                    hash_size_cumsum, indices, offsets, pooling_mode, &momentum1_dev, &momentum2_dev, hash_indices, unique_ids,
                    unique_offsets, unique_inverse, eps, learning_rate, beta1, beta2, iter,
                    "split_embedding_backward_codegen_adam_unweighted_exact_cuda");
    return Tensor();
}

Tensor backward_sgd_op(BACKWARD_HEAD, BACKWARD_TAIL, double learning_rate)
{
    backward_common(RECSDK_OPT_SGD, grad_output, dev_weights, weights_offsets, D_offsets, max_D.expect_int(),
                    hash_size_cumsum, indices, offsets, pooling_mode, nullptr, nullptr, hash_indices, unique_ids, unique_offsets,
                    unique_inverse, 0, learning_rate, 0, 0, 0,
                    "split_embedding_backward_codegen_sgd_unweighted_exact_cuda");
    return Tensor();
}

// ---- the lookup functions: forward now, fused backward + optimizer when the gradient of the output arrives ----
struct LookupArgs {
    int32_t optim = RECSDK_OPT_SGD;
    int64_t maxD = 0;
    int64_t poolingMode = 0;
    double eps = 0, lr = 0, beta1 = 0, beta2 = 0;
    int64_t iter = 0;
};

class LookupFunction : public torch::autograd::Function<LookupFunction> {
public:
    static Tensor forward(torch::autograd::AutogradContext* ctx, const Tensor& /*placeholder*/, const Tensor& dev_weights,
                          const Tensor& weights_offsets, const Tensor& D_offsets, int64_t total_D,
                          const Tensor& hash_size_cumsum, const Tensor& indices, const Tensor& offsets,
                          const Tensor& momentum1, const Tensor& momentum2, const Tensor& hash_indices,
                          const Tensor& unique_ids, const Tensor& unique_offsets, const Tensor& unique_inverse,
                          LookupArgs args)
    {
        ctx->save_for_backward({dev_weights, weights_offsets, D_offsets, hash_size_cumsum, indices, offsets, momentum1,
                                momentum2, hash_indices, unique_ids, unique_offsets, unique_inverse});
        ctx->saved_data["optim"] = (int64_t)args.optim;
        ctx->saved_data["max_D"] = args.maxD;
        ctx->saved_data["pooling_mode"] = args.poolingMode;
        ctx->saved_data["eps"] = args.eps;
        ctx->saved_data["lr"] = args.lr;
        ctx->saved_data["beta1"] = args.beta1;
        ctx->saved_data["beta2"] = args.beta2;
        ctx->saved_data["iter"] = args.iter;
        const Tensor none;
        return forward_op(dev_weights, none, none, none, weights_offsets, D_offsets, total_D, args.maxD, indices, offsets,
                          args.poolingMode, none, none, 0, false, hash_indices, none);
    }

    static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                   torch::autograd::variable_list grad_outputs)
    {
        const auto saved = ctx->get_saved_variables();
        const Tensor& dev_weights = saved[0];
        const Tensor& momentum1 = saved[6];
        const Tensor& momentum2 = saved[7];
        const int32_t optim = (int32_t)ctx->saved_data["optim"].toInt();
        backward_common(optim, grad_outputs[0], dev_weights, saved[1], saved[2], ctx->saved_data["max_D"].toInt(), saved[3],
                        saved[4], saved[5], ctx->saved_data["pooling_mode"].toInt(),
                        optim != RECSDK_OPT_SGD ? &momentum1 : nullptr, optim == RECSDK_OPT_ADAM ? &momentum2 : nullptr,
                        saved[8], saved[9], saved[10], saved[11], ctx->saved_data["eps"].toDouble(), ctx->saved_data["lr"].toDouble(),
                        ctx->saved_data["beta1"].toDouble(), ctx->saved_data["beta2"].toDouble(),
                        ctx->saved_data["iter"].toInt(), "split_embedding_codegen_lookup_function (backward)");
        // the weights are updated in place; no input receives a gradient tensor
        return torch::autograd::variable_list(15);
    }
};

#define LOOKUP_HEAD                                                                                                  \
    const Tensor &placeholder_autograd_tensor, const Tensor &dev_weights, const Tensor & /*uvm_weights*/,            \
        const Tensor & /*lxu_cache_weights*/, const Tensor & /*weights_placements*/, const Tensor &weights_offsets,  \
        const Tensor &D_offsets, c10::SymInt total_D, c10::SymInt max_D, const Tensor &hash_size_cumsum,             \
        int64_t /*total_hash_size_bits*/, const Tensor &indices, const Tensor &offsets, int64_t pooling_mode,        \
        const optional<Tensor> & /*indice_weights*/, const optional<Tensor> & /*feature_requires_grad*/,             \
        const Tensor & /*lxu_cache_locations*/, bool /*gradient_clipping*/, double /*max_gradient*/,                 \
        bool /*stochastic_rounding*/
#define LOOKUP_UNIQUE                                                                                                \
    const optional<Tensor> &hash_indices, const optional<Tensor> &unique_ids,                                        \
        const optional<Tensor> &unique_offsets, const optional<Tensor> &unique_inverse
#define LOOKUP_UNIQUE_ARGS hash_indices, unique_ids, unique_offsets, unique_inverse
#define LOOKUP_VBE                                                                                                   \
    int64_t /*output_dtype*/, const optional<Tensor> & /*B_offsets*/,                                                \
        const optional<Tensor> & /*vbe_output_offsets_feature_rank*/,                                                \
        const optional<Tensor> & /*vbe_B_offsets_rank_per_feature*/, c10::SymInt /*max_B*/,                          \
        c10::SymInt /*max_B_feature_rank*/, c10::SymInt /*vbe_output_size*/, bool /*is_experimental*/,               \
        bool /*use_uniq_cache_locations_bwd*/, bool /*use_homogeneous_placements*/,                                  \
        const optional<Tensor> & /*uvm_cache_stats*/, const optional<Tensor> & /*prev_iter_dev*/

Tensor lookup(int32_t optim, const Tensor& placeholder, const Tensor& dev_weights, const Tensor& weights_offsets,
              const Tensor& D_offsets, const c10::SymInt& total_D, const c10::SymInt& max_D, const Tensor& hash_size_cumsum,
              const Tensor& indices, const Tensor& offsets, int64_t pooling_mode, const Tensor& m1, const Tensor& m2,
              const optional<Tensor>& hash_indices, const optional<Tensor>& unique_ids,
              const optional<Tensor>& unique_offsets, const optional<Tensor>& unique_inverse, double eps, double lr,
              double beta1, double beta2, int64_t iter)
{
    LookupArgs a;
    a.optim = optim;
    a.maxD = max_D.expect_int();
    a.poolingMode = pooling_mode;
    a.eps = eps;
    a.lr = lr;
    a.beta1 = beta1;
    a.beta2 = beta2;
    a.iter = iter;
    // an optimizer without that state passes an empty tensor (autograd functions take defined tensors only)
    const Tensor absent = at::empty({0}, dev_weights.options().dtype(at::kFloat));
    const Tensor noIndex = at::empty({0}, dev_weights.options().dtype(at::kLong));
    auto index = [&](const optional<Tensor>& t) { return t.has_value() && t->defined() ? *t : noIndex; };
    return LookupFunction::apply(placeholder, dev_weights, weights_offsets, D_offsets, total_D.expect_int(),
                                 hash_size_cumsum, indices, offsets, m1.defined() ? m1 : absent,
                                 m2.defined() ? m2 : absent, index(hash_indices), index(unique_ids),
                                 index(unique_offsets), index(unique_inverse), a);
}

Tensor lookup_adagrad(LOOKUP_HEAD, const Tensor& momentum1_dev, const Tensor& /*momentum1_uvm*/,
                      const Tensor& /*momentum1_placements*/, const Tensor& /*momentum1_offsets*/, LOOKUP_UNIQUE, double eps,
                      double learning_rate, LOOKUP_VBE, int64_t /*iter*/, bool /*apply_global_weight_decay*/,
                      double /*gwd_lower_bound*/)
{
    return lookup(RECSDK_OPT_ADAGRAD, placeholder_autograd_tensor, dev_weights, weights_offsets, D_offsets, total_D, max_D,
                  hash_size_cumsum, indices, offsets, pooling_mode, momentum1_dev, Tensor(), LOOKUP_UNIQUE_ARGS, eps,
                  learning_rate, 0, 0, 0);
}

Tensor lookup_adam(LOOKUP_HEAD, const Tensor& momentum1_dev, const Tensor& /*momentum1_uvm*/,
                   const Tensor& /*momentum1_placements*/, const Tensor& /*momentum1_offsets*/, const Tensor& momentum2_dev,
                   const Tensor& /*momentum2_uvm*/, const Tensor& /*momentum2_placements*/,
                   const Tensor& /*momentum2_offsets*/, LOOKUP_UNIQUE, double eps, double learning_rate, double beta1,
                   double beta2, double /*weight_decay*/, int64_t iter, LOOKUP_VBE, bool /*apply_global_weight_decay*/,
                   double /*gwd_lower_bound*/)
{
    return lookup(RECSDK_OPT_ADAM, placeholder_autograd_tensor, dev_weights, weights_offsets, D_offsets, total_D, max_D,
                  hash_size_cumsum, indices, offsets, pooling_mode, momentum1_dev, momentum2_dev, LOOKUP_UNIQUE_ARGS, eps,
                  learning_rate, beta1, beta2, iter);
}

Tensor lookup_sgd(LOOKUP_HEAD, LOOKUP_UNIQUE, double learning_rate, LOOKUP_VBE, int64_t /*iter*/,
                  bool /*apply_global_weight_decay*/, double /*gwd_lower_bound*/)
{
    return lookup(RECSDK_OPT_SGD, placeholder_autograd_tensor, dev_weights, weights_offsets, D_offsets, total_D, max_D,
                  hash_size_cumsum, indices, offsets, pooling_mode, Tensor(), Tensor(), LOOKUP_UNIQUE_ARGS, 0, learning_rate, 0,
                  0, 0);
}

// ---- schemas: the reference's, argument for argument ----------------------------------------------------------------
const std::string kTables =
    "Tensor(a!) dev_weights, Tensor(b!) uvm_weights, Tensor lxu_cache_weights, Tensor weights_placements, "
    "Tensor weights_offsets, Tensor D_offsets, ";
const std::string kBackwardHead =
    "Tensor grad_output, " + kTables +
    "SymInt max_D, Tensor hash_size_cumsum, int total_hash_size_bits, Tensor indices, Tensor offsets, int pooling_mode, "
    "Tensor lxu_cache_locations, int unused_, int max_segment_length_per_warp, bool stochastic_rounding, "
    "int info_B_num_bits, int info_B_mask_int64, bool use_uniq_cache_locations, bool use_homogeneous_placements, ";
const std::string kBackwardTail =
    "Tensor hash_indices = None, Tensor unique_ids = None, Tensor unique_offsets = None, Tensor unique_inverse = None, "
    "Tensor offset_per_key = None, ";
const std::string kMomentum1 =
    "Tensor momentum1_dev, Tensor momentum1_uvm, Tensor momentum1_placements, Tensor momentum1_offsets, ";
const std::string kMomentum2 =
    "Tensor momentum2_dev, Tensor momentum2_uvm, Tensor momentum2_placements, Tensor momentum2_offsets, ";
const std::string kLookupHead =
    "Tensor placeholder_autograd_tensor, " + kTables +
    "SymInt total_D, SymInt max_D, Tensor hash_size_cumsum, int total_hash_size_bits, Tensor indices, Tensor offsets, "
    "int pooling_mode, Tensor? indice_weights, Tensor? feature_requires_grad, Tensor lxu_cache_locations, "
    "bool gradient_clipping, float max_gradient, bool stochastic_rounding, ";
const std::string kLookupUnique =
    "Tensor? hash_indices = None, Tensor? unique_ids = None, Tensor? unique_offsets = None, "
    "Tensor? unique_inverse = None, ";
const std::string kLookupVbe =
    "int output_dtype=0, Tensor? B_offsets=None, Tensor? vbe_output_offsets_feature_rank=None, "
    "Tensor? vbe_B_offsets_rank_per_feature=None, SymInt max_B=-1, SymInt max_B_feature_rank=-1, "
    "SymInt vbe_output_size=-1, bool is_experimental=False, bool use_uniq_cache_locations_bwd=False, "
    "bool use_homogeneous_placements=False, Tensor? uvm_cache_stats=None, Tensor? prev_iter_dev=None, ";
const std::string kGwd = "bool apply_global_weight_decay=False, float gwd_lower_bound=0";

}  // namespace

TORCH_LIBRARY_FRAGMENT(fbgemm, m)
{
    m.def("split_embedding_codegen_forward_unweighted_cuda("
          "Tensor dev_weights, Tensor uvm_weights, Tensor lxu_cache_weights, Tensor weights_placements, "
          "Tensor weights_offsets, Tensor D_offsets, SymInt total_D, SymInt max_D, Tensor indices, Tensor offsets, "
          "int pooling_mode, Tensor lxu_cache_locations, Tensor uvm_cache_stats, int output_dtype, bool is_experimental, "
          "Tensor hash_indices = None, Tensor offset_per_key = None) -> Tensor");
    m.def(("split_embedding_backward_codegen_adagrad_unweighted_exact_cuda(" + kBackwardHead + kMomentum1 + kBackwardTail +
           "float eps = 0, float learning_rate = 0) -> Tensor")
              .c_str());
    m.def(("split_embedding_backward_codegen_adam_unweighted_exact_cuda(" + kBackwardHead + kMomentum1 + kMomentum2 +
           kBackwardTail + "float eps = 0, float learning_rate = 0, float beta1 = 0, float beta2 = 0, int iter = 0) -> Tensor")
              .c_str());
    m.def(("split_embedding_backward_codegen_sgd_unweighted_exact_cuda(" + kBackwardHead + kBackwardTail +
           "float learning_rate = 0) -> Tensor")
              .c_str());
    m.def(("split_embedding_codegen_lookup_adagrad_function(" + kLookupHead + kMomentum1 + kLookupUnique +
           "float eps = 0, float learning_rate = 0, " + kLookupVbe + "int iter=0, " + kGwd + ") -> Tensor")
              .c_str());
    m.def(("split_embedding_codegen_lookup_adam_function(" + kLookupHead + kMomentum1 + kMomentum2 + kLookupUnique +
           "float eps = 0, float learning_rate = 0, float beta1 = 0, float beta2 = 0, float weight_decay = 0, int iter = 0, " +
           kLookupVbe + kGwd + ") -> Tensor")
              .c_str());
    m.def(("split_embedding_codegen_lookup_sgd_function(" + kLookupHead + kLookupUnique + "float learning_rate = 0, " +
           kLookupVbe + "int iter=0, " + kGwd + ") -> Tensor")
              .c_str());
}

// ROCm tensors carry the CUDA dispatch key.
TORCH_LIBRARY_IMPL(fbgemm, CUDA, m)
{
    m.impl("split_embedding_codegen_forward_unweighted_cuda", TORCH_FN(forward_op));
    m.impl("split_embedding_backward_codegen_adagrad_unweighted_exact_cuda", TORCH_FN(backward_adagrad_op));
    m.impl("split_embedding_backward_codegen_adam_unweighted_exact_cuda", TORCH_FN(backward_adam_op));
    m.impl("split_embedding_backward_codegen_sgd_unweighted_exact_cuda", TORCH_FN(backward_sgd_op));
    m.impl("split_embedding_codegen_lookup_adagrad_function", TORCH_FN(lookup_adagrad));
    m.impl("split_embedding_codegen_lookup_adam_function", TORCH_FN(lookup_adam));
    m.impl("split_embedding_codegen_lookup_sgd_function", TORCH_FN(lookup_sgd));
}

TORCH_LIBRARY_IMPL(fbgemm, Autograd, m)
{
    m.impl("split_embedding_codegen_lookup_adagrad_function", TORCH_FN(lookup_adagrad));
    m.impl("split_embedding_codegen_lookup_adam_function", TORCH_FN(lookup_adam));
    m.impl("split_embedding_codegen_lookup_sgd_function", TORCH_FN(lookup_sgd));
}
