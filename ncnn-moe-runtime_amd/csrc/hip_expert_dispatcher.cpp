// Host-side C++ face of the gfx950 expert router (see hip_expert_dispatcher.h).
#include "hip_expert_dispatcher.h"

#include "ncnn_moe_hip_router.h"

#include <cmath>

namespace ncnn {
namespace moe {

struct HipExpertDispatcher::Impl
{
    ncnn_moe_hip_router* handle = nullptr;
    uint32_t max_tokens = 0;
    uint32_t max_experts = 0;
    uint32_t max_top_k = 0;
    std::vector<uint32_t> offsets;
    std::vector<ncnn_moe_expert_route> routes;

    ~Impl()
    {
        if (handle != nullptr)
            ncnn_moe_hip_router_destroy(handle);
    }
};

HipExpertDispatcher::HipExpertDispatcher() : impl_(std::make_unique<Impl>()) {}

HipExpertDispatcher::~HipExpertDispatcher() = default;

std::shared_ptr<HipExpertDispatcher> HipExpertDispatcher::create(int device, uint32_t max_tokens, uint32_t max_experts, uint32_t max_top_k)
{
    std::shared_ptr<HipExpertDispatcher> dispatcher(new HipExpertDispatcher());
    if (ncnn_moe_hip_router_create(device, max_tokens, max_experts, max_top_k, &dispatcher->impl_->handle) != NCNN_MOE_ROUTER_SUCCESS)
        return nullptr;
    dispatcher->impl_->max_tokens = max_tokens;
    dispatcher->impl_->max_experts = max_experts;
    dispatcher->impl_->max_top_k = max_top_k;
    return dispatcher;
}

Result<ExpertDispatchPlan> HipExpertDispatcher::dispatch(std::span<const float> router_logits, uint32_t token_count, const ExpertDispatchOptions& options)
{
    ExpertDispatchPlan plan;
    auto dispatched = dispatch_into(router_logits, token_count, options, plan);
    if (!dispatched)
        return dispatched.error();
    return plan;
}

Result<bool> HipExpertDispatcher::dispatch_into(std::span<const float> router_logits, uint32_t token_count, const ExpertDispatchOptions& options, ExpertDispatchPlan& result)
{
    // the checks of src/graph/expert_dispatcher.cpp:78-97, in its order; the C ABI sees bare pointers,
    // so the three shape checks are made here
    if (token_count == 0)
        return Error{ErrorCode::InvalidArgument, ncnn_moe_hip_router_status_message(NCNN_MOE_ROUTER_NO_TOKENS)};
    if (options.expert_count == 0 || options.top_k == 0 || options.top_k > options.expert_count)
        return Error{ErrorCode::InvalidArgument, ncnn_moe_hip_router_status_message(NCNN_MOE_ROUTER_BAD_TOP_K)};
    if (router_logits.size() / options.expert_count != token_count || router_logits.size() % options.expert_count != 0)
        return Error{ErrorCode::InvalidArgument, "router logits shape does not match token and expert counts"};
    if (!options.selection_bias.empty() && options.selection_bias.size() != options.expert_count)
        return Error{ErrorCode::InvalidArgument, "router selection bias must match expert_count"};
    if (!options.explicit_expert_ids.empty() && options.explicit_expert_ids.size() != static_cast<size_t>(token_count) * options.top_k)
        return Error{ErrorCode::InvalidArgument, "explicit expert ids must match token_count * top_k"};

    ncnn_moe_router_options flat{};
    flat.expert_count = options.expert_count;
    flat.top_k = options.top_k;
    flat.score_function = static_cast<uint32_t>(options.score_function);
    flat.renormalize = ((options.flags & ExpertDispatchNormalizeTopKWeights) != 0u || options.normalization == RouterNormalization::SelectedExperts) ? 1u : 0u;
    flat.routed_scaling_factor = options.routed_scaling_factor;

    const std::lock_guard<std::mutex> lock(mutex_);
    Impl& impl = *impl_;
    const size_t assignments = static_cast<size_t>(token_count) * options.top_k;
    impl.offsets.resize(static_cast<size_t>(options.expert_count) + 1);
    impl.routes.resize(assignments);
    uint32_t status = NCNN_MOE_ROUTER_OK;
    const int rc = ncnn_moe_hip_router_dispatch(
        impl.handle, router_logits.data(), token_count, &flat,
        options.selection_bias.empty() ? nullptr : options.selection_bias.data(),
        options.explicit_expert_ids.empty() ? nullptr : options.explicit_expert_ids.data(),
        impl.offsets.data(), impl.routes.data(), &status);
    if (rc != NCNN_MOE_ROUTER_SUCCESS)
    {
        return Error{rc == NCNN_MOE_ROUTER_INVALID_ARGUMENT ? ErrorCode::InvalidArgument : ErrorCode::InternalError,
                     std::string("hip router: ") + ncnn_moe_hip_router_last_error(impl.handle)};
    }
    if (status != NCNN_MOE_ROUTER_OK)
    {
        return Error{status == NCNN_MOE_ROUTER_NON_POSITIVE_SUM ? ErrorCode::InvalidModel : ErrorCode::InvalidArgument,
                     ncnn_moe_hip_router_status_message(static_cast<int>(status))};
    }

    // ExpertDispatchPlan::batches is the non-empty groups; elements and their route vectors are reused
    size_t used = 0;
    for (uint32_t expert = 0; expert < options.expert_count; ++expert)
    {
        const uint32_t begin = impl.offsets[expert];
        const uint32_t end = impl.offsets[expert + 1];
        if (begin == end)
            continue;
        if (used == result.batches.size())
            result.batches.emplace_back();
        ExpertBatch& batch = result.batches[used++];
        batch.expert_id = expert;
        batch.routes.clear();
        for (uint32_t i = begin; i < end; ++i)
            batch.routes.push_back(ExpertRoute{impl.routes[i].token_index, impl.routes[i].rank, impl.routes[i].weight});
    }
    result.batches.resize(used);
    result.assignment_count = assignments;
    return true;
}

} // namespace moe
} // namespace ncnn
