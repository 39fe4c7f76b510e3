// Shared declarations of the row-update kernels (segment-reduce gradients + fused optimizer).
#ifndef RECSDK_CSRC_APPLY_H
#define RECSDK_CSRC_APPLY_H

#include "common.h"
#include "dedup.h"

namespace recsdk {

// Where one table's rows live.  w is fp32 or bf16 (see ApplyCtx::wBf16); optimizer state is fp32.
struct RowsDesc {
    void* w;
    float* s1;
    float* s2;
    int64_t stride;   // elements between consecutive rows (same for w, s1, s2)
    int32_t dim;      // row width of this table
    int32_t gradCol;  // first column of this table inside a gradient row (pooled-lookup layout), else 0
};

// optimizer codes of the kernels: the public RECSDK_OPT_* values plus the split-embedding variants
constexpr int kOptSgd = RECSDK_OPT_SGD;
constexpr int kOptAdagrad = RECSDK_OPT_ADAGRAD;
constexpr int kOptAdam = RECSDK_OPT_ADAM;
constexpr int kOptTbeSgd = 10;
constexpr int kOptTbeAdagrad = 11;
constexpr int kOptTbeAdam = 12;
constexpr int kOptStoreSum = 20;  // no update: the summed gradient itself is stored (chunk sums)

struct OptParams {
    int optim;
    float lr;
    float beta1;
    float beta2;
    float eps;
    float weightDecay;
    float stepSize;  // split-embedding Adam: -lr*sqrt(1-beta2^iter)/(1-beta1^iter)
    const float* lrDev;  // when set, the kernels read `lr` from here (a rate that changes between replays of a graph)
};

inline bool opt_uses_s1(int optim) { return optim != kOptSgd && optim != kOptTbeSgd; }
inline bool opt_uses_s2(int optim) { return optim == kOptAdam || optim == kOptTbeAdam; }

// Where the gradient row of list entry p comes from: base + p * stride (+ the table's gradCol).  For the by-key
// lookup p is the lookup position; the pooled lookup rewrites its lists to bag samples before the update.
struct GradSrc {
    const float* base;
    int64_t stride;
};

struct ApplyCtx {
    const RowsDesc* d_rows = nullptr;
    int T = 0;
    int maxDim = 0;
    bool wBf16 = false;
    bool gradShared = false;  // one gradient row serves several list entries (pooled lookup)
    const UniqueView* v = nullptr;
    recsdk_unique* uq = nullptr;  // the handle behind v (the two-level sums allocate their workspace through it)
    const int64_t* d_slots = nullptr;
    GradSrc g{};
    OptParams prm{};
    hipStream_t stream = nullptr;
    hipStream_t side = nullptr;   // optional second stream for the long-list kernels
    hipEvent_t evFork = nullptr;
    hipEvent_t evJoin = nullptr;
    hipEvent_t evMeta = nullptr;   // optional: lets the long lists that need no chunk sums start before the join
};

// Enqueue the update of every distinct key of ctx.v with slot >= 0.
int apply_launch(const ApplyCtx& ctx);

}  // namespace recsdk

#endif
