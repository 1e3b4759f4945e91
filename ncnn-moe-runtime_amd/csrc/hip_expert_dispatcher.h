// Host-side C++ face of the gfx950 expert router, shaped like the runtime's own ExpertDispatcher
// (include/ncnn/moe/expert_dispatcher.h:15-63) so that it can stand in for it:
//
//   ExpertRoute / ExpertBatch / ExpertDispatchOptions / ExpertDispatchPlan   the runtime's public
//       types.  When this header is compiled inside the runtime (NCNN_MOE_EXPERT_DISPATCHER_H already
//       defined) the runtime's own are used; a stand-alone build defines equivalents with the same
//       names and defaults.
//   HipExpertDispatcher   dispatch() / dispatch_into() with the CPU dispatcher's results (the same
//       batches in ascending expert id, the same routes by token then rank, the same fp32 weights)
//       and its errors (src/graph/expert_dispatcher.cpp:78-103, :122, :133).  dispatch_into() refills
//       the caller's plan without releasing its storage, as the CPU one does for decode steps.
//
// Everything runs on the device through the C ABI of include/ncnn_moe_hip_router.h.  There is no CPU
// fallback: without a usable GPU create() returns null.
#ifndef NCNN_MOE_HIP_EXPERT_DISPATCHER_H
#define NCNN_MOE_HIP_EXPERT_DISPATCHER_H

#include "hip_session_sampler.h" // Result<T>, Error, ErrorCode (the runtime's, or the stand-alone equivalents)

#include <cstddef>
#include <cstdint>
#include <memory>
#include <mutex>
#include <span>
#include <vector>

#ifndef NCNN_MOE_EXPERT_DISPATCHER_H

namespace ncnn {
namespace moe {

// include/ncnn/moe/types.h:216-228
enum class RouterScoreFunction
{
    Softmax,
    Sigmoid,
    SqrtSoftplus
};

enum class RouterNormalization
{
    None,
    SelectedExperts
};

struct ExpertRoute
{
    uint32_t token_index = 0;
    uint32_t rank = 0;
    float weight = 0.0f;
};

struct ExpertBatch
{
    uint32_t expert_id = 0;
    std::vector<ExpertRoute> routes;
};

enum ExpertDispatchOptionFlag : uint32_t
{
    ExpertDispatchNormalizeTopKWeights = UINT32_C(1) << 0
};

struct ExpertDispatchOptions
{
    uint32_t expert_count = 0;
    uint32_t top_k = 0;
    RouterScoreFunction score_function = RouterScoreFunction::Softmax;
    RouterNormalization normalization = RouterNormalization::SelectedExperts;
    float routed_scaling_factor = 1.0f;
    std::span<const float> selection_bias;
    std::span<const uint32_t> explicit_expert_ids;
    uint32_t flags = ExpertDispatchNormalizeTopKWeights;
};

struct ExpertDispatchPlan
{
    std::vector<ExpertBatch> batches;
    size_t assignment_count = 0;
};

} // namespace moe
} // namespace ncnn

#endif // NCNN_MOE_EXPERT_DISPATCHER_H

namespace ncnn {
namespace moe {

class HipExpertDispatcher
{
public:
    // Null when no GPU is usable, a limit is exceeded (1024 experts, Top-64) or the device buffers for
    // max_tokens x max_experts logits cannot be allocated.
    static std::shared_ptr<HipExpertDispatcher> create(int device, uint32_t max_tokens, uint32_t max_experts, uint32_t max_top_k);
    ~HipExpertDispatcher();
    HipExpertDispatcher(const HipExpertDispatcher&) = delete;
    HipExpertDispatcher& operator=(const HipExpertDispatcher&) = delete;

    // Input is token-major; output is stable and ordered by expert id (ExpertDispatcher::dispatch).
    [[nodiscard]] Result<ExpertDispatchPlan> dispatch(std::span<const float> router_logits, uint32_t token_count, const ExpertDispatchOptions& options);

    // Reuses caller storage across decode steps (ExpertDispatcher::dispatch_into).  The stand-alone
    // Result has no void form: the value is true.
    [[nodiscard]] Result<bool> dispatch_into(std::span<const float> router_logits, uint32_t token_count, const ExpertDispatchOptions& options, ExpertDispatchPlan& result);

private:
    HipExpertDispatcher();
    struct Impl;
    std::unique_ptr<Impl> impl_;
    std::mutex mutex_;
};

using HipExpertDispatcherPtr = std::shared_ptr<HipExpertDispatcher>;

} // namespace moe
} // namespace ncnn

#endif // NCNN_MOE_HIP_EXPERT_DISPATCHER_H
