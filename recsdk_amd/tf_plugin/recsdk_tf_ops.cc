// Device kernels for the reference's four TensorFlow custom ops, over librecsdk_hip.so.
//
// The reference registers the ops (cust_op/framework/tf_plugin/src/cust_embedding_by_address.cpp:19-51, lazy_adam.cpp:20-34,
// sgd.cpp:19-26) together with a CPU kernel that only prints "Cust opp not installed"
// (include/mxrec_tf_plugin.h:34-47); the arithmetic lives in its Ascend C operators.  This file registers, for the
// SAME op names and signatures, kernels for DEVICE_GPU (TensorFlow-ROCm) that forward to the C ABI on the op's own
// stream.  A graph built by mx_rec then places the four ops on the GPU unchanged.
//
// Built only where TensorFlow's headers are installed (recsdk_amd/tf_plugin/build.py); nothing else in this repository
// depends on it.  Load with tf.load_op_library(<librecsdk_tf_ops.so>) in place of the reference's
// mx_rec/libasc library (training/tf_rec_v1/python/util/ops.py:30-48).
#include "tensorflow/core/framework/op.h"
#include "tensorflow/core/framework/op_kernel.h"
#include "tensorflow/core/framework/shape_inference.h"
#include "tensorflow/core/framework/tensor.h"
#include "tensorflow/core/platform/stream_executor.h"

#include "recsdk_hip.h"

namespace tensorflow {
namespace {

using shape_inference::DimensionHandle;
using shape_inference::InferenceContext;
using shape_inference::ShapeHandle;

// the hipStream_t TensorFlow runs this op's device work on
void* OpStream(OpKernelContext* ctx)
{
    auto* stream = ctx->op_device_context()->stream();
    return stream->implementation()->GpuStreamHack();
}

Status FromRc(int rc)
{
    return rc == RECSDK_OK ? Status() : errors::Internal("recsdk: ", recsdk_last_error());
}

// embedding_type of the reference's op prototype (cust_op_by_addr/v220/emb_custom.json:22-25): 0 int32, 1 float, 2 half
int ElementType(int embeddingType)
{
    return embeddingType == 0 ? RECSDK_DT_I32 : (embeddingType == 2 ? RECSDK_DT_F16 : RECSDK_DT_F32);
}

class EmbeddingLookupByAddressOp : public OpKernel {
public:
    explicit EmbeddingLookupByAddressOp(OpKernelConstruction* c) : OpKernel(c)
    {
        OP_REQUIRES_OK(c, c->GetAttr("embedding_dim", &dim_));
        OP_REQUIRES_OK(c, c->GetAttr("embedding_type", &type_));
    }

    void Compute(OpKernelContext* ctx) override
    {
        const Tensor& address = ctx->input(0);
        OP_REQUIRES(ctx, address.dims() == 1, errors::InvalidArgument("address must be a vector"));
        const int64_t n = address.NumElements();
        Tensor* y = nullptr;
        OP_REQUIRES_OK(ctx, ctx->allocate_output(0, TensorShape({n, dim_}), &y));
        if (n == 0) {
            return;
        }
        // the op's output is declared float; other element types travel as raw 4- or 2-byte values in it
        OP_REQUIRES_OK(ctx, FromRc(recsdk_lookup_by_addr(reinterpret_cast<const int64_t*>(address.flat<int64>().data()),
                                                         n, dim_, ElementType(type_), y->flat<float>().data(),
                                                         OpStream(ctx))));
    }

private:
    int dim_ = 0;
    int type_ = 1;
};

class EmbeddingUpdateByAddressOp : public OpKernel {
public:
    explicit EmbeddingUpdateByAddressOp(OpKernelConstruction* c) : OpKernel(c)
    {
        OP_REQUIRES_OK(c, c->GetAttr("update_type", &updateType_));
    }

    void Compute(OpKernelContext* ctx) override
    {
        const Tensor& address = ctx->input(0);
        const Tensor& embedding = ctx->input(1);
        OP_REQUIRES(ctx, address.dims() == 1 && embedding.dims() == 2 && embedding.dim_size(0) == address.NumElements(),
                    errors::InvalidArgument("embedding must be [len(address), D]"));
        // the op returns its embedding input (the reference's graph only uses it as a control dependency)
        ctx->set_output(0, embedding);
        const int64_t n = address.NumElements();
        if (n == 0) {
            return;
        }
        OP_REQUIRES_OK(ctx, FromRc(recsdk_update_by_addr(reinterpret_cast<const int64_t*>(address.flat<int64>().data()),
                                                         n, static_cast<int32_t>(embedding.dim_size(1)), RECSDK_DT_F32,
                                                         embedding.flat<float>().data(), updateType_, OpStream(ctx))));
    }

private:
    int updateType_ = 0;
};

// LazyAdam: m, v, var rows named by indices are updated in place; the outputs alias the inputs, as on the reference's
// device.  lr arrives already bias-corrected (training/tf_rec_v1/python/optimizers/lazy_adam.py:172,185-195).
class LazyAdamOp : public OpKernel {
public:
    explicit LazyAdamOp(OpKernelConstruction* c) : OpKernel(c)
    {
        OP_REQUIRES_OK(c, c->GetAttr("beta1", &beta1_));
        OP_REQUIRES_OK(c, c->GetAttr("beta2", &beta2_));
        OP_REQUIRES_OK(c, c->GetAttr("epsilon", &epsilon_));
    }

    void Compute(OpKernelContext* ctx) override
    {
        const Tensor& grad = ctx->input(0);
        const Tensor& indices = ctx->input(1);
        Tensor m = ctx->input(2);
        Tensor v = ctx->input(3);
        Tensor var = ctx->input(4);
        const Tensor& lr = ctx->input(5);   // host memory, see the kernel registration
        OP_REQUIRES(ctx, grad.dims() == 2 && m.dims() == 2 && m.shape() == v.shape() && m.shape() == var.shape() &&
                             grad.dim_size(1) == m.dim_size(1),
                    errors::InvalidArgument("gradient [n, dim]; input_m, input_v, input_var [rows, dim]"));
        ctx->set_output(0, m);
        ctx->set_output(1, v);
        ctx->set_output(2, var);
        const int64_t n = indices.NumElements();
        if (n == 0) {
            return;
        }
        OP_REQUIRES_OK(ctx, FromRc(recsdk_lazy_adam(grad.flat<float>().data(), indices.flat<int32>().data(), n,
                                                    static_cast<int32_t>(m.dim_size(1)), m.flat<float>().data(),
                                                    v.flat<float>().data(), var.flat<float>().data(),
                                                    lr.flat<float>()(0), beta1_, beta2_, epsilon_, OpStream(ctx))));
    }

private:
    float beta1_ = 0.9f;
    float beta2_ = 0.999f;
    float epsilon_ = 1e-8f;
};

class SgdOp : public OpKernel {
public:
    explicit SgdOp(OpKernelConstruction* c) : OpKernel(c) { OP_REQUIRES_OK(c, c->GetAttr("weightDecay", &weightDecay_)); }

    void Compute(OpKernelContext* ctx) override
    {
        const Tensor& grad = ctx->input(0);
        const Tensor& indices = ctx->input(1);
        Tensor var = ctx->input(2);
        const Tensor& lr = ctx->input(3);   // host memory
        OP_REQUIRES(ctx, grad.dims() == 2 && var.dims() == 2 && grad.dim_size(1) == var.dim_size(1),
                    errors::InvalidArgument("gradient [n, dim]; input_var [rows, dim]"));
        ctx->set_output(0, var);
        const int64_t n = indices.NumElements();
        if (n == 0) {
            return;
        }
        OP_REQUIRES_OK(ctx, FromRc(recsdk_sgd(grad.flat<float>().data(), indices.flat<int32>().data(), n,
                                              static_cast<int32_t>(var.dim_size(1)), var.flat<float>().data(),
                                              lr.flat<float>()(0), weightDecay_, OpStream(ctx))));
    }

private:
    float weightDecay_ = 0.0f;
};

}  // namespace

// The op definitions are the reference's, attribute for attribute, so that either library can be loaded.
REGISTER_OP("EmbeddingLookupByAddress")
    .Input("address: int64")
    .Attr("embedding_dim: int")
    .Attr("embedding_type: int")
    .Output("y: float")
    .SetIsStateful()
    .SetShapeFn([](InferenceContext* c) {
        ShapeHandle address;
        TF_RETURN_IF_ERROR(c->WithRank(c->input(0), 1, &address));
        int dim = 0;
        TF_RETURN_IF_ERROR(c->GetAttr("embedding_dim", &dim));
        c->set_output(0, c->Matrix(c->Dim(address, 0), dim));
        return Status();
    });
REGISTER_OP("EmbeddingUpdateByAddress")
    .Input("address: int64")
    .Input("embedding: float")
    .Attr("update_type: int")
    .Output("y: float")
    .SetIsStateful()
    .SetShapeFn([](InferenceContext* c) {
        ShapeHandle address;
        ShapeHandle embedding;
        TF_RETURN_IF_ERROR(c->WithRank(c->input(0), 1, &address));
        TF_RETURN_IF_ERROR(c->WithRank(c->input(1), 2, &embedding));
        c->set_output(0, c->Matrix(c->Dim(address, 0), c->Dim(embedding, 1)));
        return Status();
    });
REGISTER_OP("LazyAdam")
    .Input("gradient: float32")
    .Input("indices: int32")
    .Input("input_m: float32")
    .Input("input_v: float32")
    .Input("input_var: float32")
    .Input("lr: float32")
    .Attr("beta1: float")
    .Attr("beta2: float")
    .Attr("epsilon: float")
    .Output("output_m: float32")
    .Output("output_v: float32")
    .Output("output_var: float32")
    .SetIsStateful()
    .SetShapeFn(shape_inference::UnknownShape);
REGISTER_OP("Sgd")
    .Input("gradient: float32")
    .Input("indices: int32")
    .Input("input_var: float32")
    .Input("lr: float32")
    .Attr("weightDecay: float = 0.0")
    .Output("output_var: float32")
    .SetIsStateful()
    .SetShapeFn(shape_inference::UnknownShape);

REGISTER_KERNEL_BUILDER(Name("EmbeddingLookupByAddress").Device(DEVICE_GPU), EmbeddingLookupByAddressOp);
REGISTER_KERNEL_BUILDER(Name("EmbeddingUpdateByAddress").Device(DEVICE_GPU), EmbeddingUpdateByAddressOp);
REGISTER_KERNEL_BUILDER(Name("LazyAdam").Device(DEVICE_GPU).HostMemory("lr"), LazyAdamOp);
REGISTER_KERNEL_BUILDER(Name("Sgd").Device(DEVICE_GPU).HostMemory("lr"), SgdOp);

}  // namespace tensorflow
