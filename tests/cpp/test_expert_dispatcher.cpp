// Tests of the C++ host face of the HIP expert router, written in the manner of the runtime's own
// dispatcher tests (tests/test_runtime.cpp:3366-3540: grouping, weights, storage reuse of
// dispatch_into, tied scores, wide Top-K, caller-named experts, the sqrt-softplus router with a
// selection bias), plus the error texts and their order.
//
//   test_expert_dispatcher            all tests (needs a GPU)
//   test_expert_dispatcher --host     only the tests that need no GPU
#include "hip_expert_dispatcher.h"

#include <array>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <limits>
#include <stdexcept>
#include <string>
#include <vector>

using namespace ncnn::moe;

#define check(condition)                                                                              \
    do                                                                                                \
    {                                                                                                 \
        if (!(condition))                                                                             \
            throw std::runtime_error(std::string(__FILE__) + ":" + std::to_string(__LINE__) + ": check failed: " #condition); \
    } while (0)

static void check_near(float actual, float expected, float tolerance)
{
    if (!(std::fabs(actual - expected) <= tolerance))
        throw std::runtime_error("check_near failed: " + std::to_string(actual) + " vs " + std::to_string(expected));
}

static void test_defaults_match_the_runtime()
{
    const ExpertDispatchOptions options;
    check(options.expert_count == 0 && options.top_k == 0);
    check(options.score_function == RouterScoreFunction::Softmax);
    check(options.normalization == RouterNormalization::SelectedExperts);
    check(options.routed_scaling_factor == 1.0f);
    check(options.flags == ExpertDispatchNormalizeTopKWeights);
    check(options.selection_bias.empty() && options.explicit_expert_ids.empty());
    check(sizeof(ExpertRoute) == 12);
    // limits of the device router are refused at creation, with or without a GPU
    check(HipExpertDispatcher::create(0, 16, 2048, 8) == nullptr);
    check(HipExpertDispatcher::create(0, 16, 64, 65) == nullptr);
    check(HipExpertDispatcher::create(0, 0, 64, 8) == nullptr);
}

static void test_groups_routes(HipExpertDispatcher& dispatcher)
{
    ExpertDispatchOptions options;
    options.expert_count = 6;
    options.top_k = 1;
    const std::vector<float> logits = {
        0.0f, 5.0f, 0.0f, 0.0f, 0.0f, 1.0f,
        0.0f, 1.0f, 0.0f, 0.0f, 0.0f, 5.0f,
        0.0f, 4.0f, 0.0f, 0.0f, 0.0f, 1.0f,
        0.0f, 1.0f, 0.0f, 0.0f, 0.0f, 4.0f,
    };
    auto dispatch = dispatcher.dispatch(logits, 4, options);
    check(static_cast<bool>(dispatch));
    check(dispatch.value().assignment_count == 4);
    check(dispatch.value().batches.size() == 2);
    check(dispatch.value().batches[0].expert_id == 1);
    check(dispatch.value().batches[0].routes.size() == 2);
    check(dispatch.value().batches[0].routes[0].token_index == 0);
    check(dispatch.value().batches[0].routes[1].token_index == 2);
    check_near(dispatch.value().batches[0].routes[0].weight, 1.0f, 1e-6f);
    check(dispatch.value().batches[1].expert_id == 5);
    check(dispatch.value().batches[1].routes.size() == 2);
    check(dispatch.value().batches[1].routes[0].token_index == 1);
    check(dispatch.value().batches[1].routes[1].token_index == 3);

    options.expert_count = 3;
    options.top_k = 2;
    const std::vector<float> weighted_logits = {2.0f, 1.0f, 0.0f};
    auto weighted = dispatcher.dispatch(weighted_logits, 1, options);
    check(static_cast<bool>(weighted));
    check(weighted.value().assignment_count == 2);
    check(weighted.value().batches.size() == 2);
    check(weighted.value().batches[0].routes[0].rank == 0);
    check(weighted.value().batches[1].routes[0].rank == 1);
    check_near(weighted.value().batches[0].routes[0].weight + weighted.value().batches[1].routes[0].weight, 1.0f, 1e-6f);

    // dispatch_into gives the same plan and keeps the caller's storage across steps
    ExpertDispatchPlan reusable;
    auto dispatched_into = dispatcher.dispatch_into(weighted_logits, 1, options, reusable);
    check(static_cast<bool>(dispatched_into));
    check(reusable.assignment_count == weighted.value().assignment_count);
    check(reusable.batches.size() == weighted.value().batches.size());
    for (size_t index = 0; index < reusable.batches.size(); ++index)
    {
        check(reusable.batches[index].expert_id == weighted.value().batches[index].expert_id);
        check(reusable.batches[index].routes.front().rank == weighted.value().batches[index].routes.front().rank);
        check(reusable.batches[index].routes.front().weight == weighted.value().batches[index].routes.front().weight);
    }
    const ExpertBatch* reused_batches = reusable.batches.data();
    const ExpertRoute* reused_first_route = reusable.batches.front().routes.data();
    const std::vector<float> next_logits = {0.0f, 1.0f, 2.0f};
    dispatched_into = dispatcher.dispatch_into(next_logits, 1, options, reusable);
    check(static_cast<bool>(dispatched_into));
    check(reusable.batches.data() == reused_batches);
    check(reusable.batches.front().routes.data() == reused_first_route);
    check(reusable.batches[0].expert_id == 1 && reusable.batches[1].expert_id == 2);
    check(reusable.batches[1].routes[0].rank == 0);
}

static void check_dispatch_into_matches(HipExpertDispatcher& dispatcher, std::span<const float> logits, const ExpertDispatchOptions& options)
{
    auto expected = dispatcher.dispatch(logits, 1, options);
    check(static_cast<bool>(expected));
    ExpertDispatchPlan actual;
    auto status = dispatcher.dispatch_into(logits, 1, options, actual);
    check(static_cast<bool>(status));
    check(actual.assignment_count == expected.value().assignment_count);
    check(actual.batches.size() == expected.value().batches.size());
    size_t routes = 0;
    for (size_t b = 0; b < actual.batches.size(); ++b)
    {
        check(actual.batches[b].expert_id == expected.value().batches[b].expert_id);
        check(actual.batches[b].routes.size() == expected.value().batches[b].routes.size());
        for (size_t r = 0; r < actual.batches[b].routes.size(); ++r)
        {
            check(actual.batches[b].routes[r].token_index == expected.value().batches[b].routes[r].token_index);
            check(actual.batches[b].routes[r].rank == expected.value().batches[b].routes[r].rank);
            check(actual.batches[b].routes[r].weight == expected.value().batches[b].routes[r].weight);
        }
        routes += actual.batches[b].routes.size();
    }
    check(routes == options.top_k);
}

static void test_ties_wide_windows_and_named_experts(HipExpertDispatcher& dispatcher)
{
    ExpertDispatchOptions sigmoid_options;
    sigmoid_options.expert_count = 4;
    sigmoid_options.top_k = 2;
    sigmoid_options.score_function = RouterScoreFunction::Sigmoid;
    sigmoid_options.normalization = RouterNormalization::None;
    sigmoid_options.routed_scaling_factor = 2.0f;
    sigmoid_options.flags = 0;
    const std::array<float, 4> tied_sigmoid_logits = {0.0f, 0.0f, -1.0f, -1.0f};
    check_dispatch_into_matches(dispatcher, tied_sigmoid_logits, sigmoid_options);
    auto tied = dispatcher.dispatch(tied_sigmoid_logits, 1, sigmoid_options);
    check(tied.value().batches[0].expert_id == 0 && tied.value().batches[1].expert_id == 1); // the lower ids of the tie
    check(tied.value().batches[0].routes[0].weight == 1.0f);                                  // sigmoid(0) * 2, not renormalised

    ExpertDispatchOptions wide_options;
    wide_options.expert_count = 20;
    std::array<float, 20> wide_logits;
    for (size_t index = 0; index < wide_logits.size(); ++index)
        wide_logits[index] = static_cast<float>(static_cast<int>(index % 7) - 3);
    wide_options.top_k = 16;
    check_dispatch_into_matches(dispatcher, wide_logits, wide_options);
    wide_options.top_k = 17;
    check_dispatch_into_matches(dispatcher, wide_logits, wide_options);

    ExpertDispatchOptions duplicate_options;
    duplicate_options.expert_count = 4;
    duplicate_options.top_k = 2;
    const std::array<uint32_t, 2> duplicate_experts = {1, 1};
    duplicate_options.explicit_expert_ids = duplicate_experts;
    const std::array<float, 4> duplicate_logits = {0.0f, 1.0f, 2.0f, 3.0f};
    check_dispatch_into_matches(dispatcher, duplicate_logits, duplicate_options);
    auto duplicated = dispatcher.dispatch(duplicate_logits, 1, duplicate_options);
    check(duplicated.value().batches.size() == 1 && duplicated.value().batches[0].routes.size() == 2);
    check(duplicated.value().batches[0].routes[0].rank == 0 && duplicated.value().batches[0].routes[1].rank == 1);
}

static void test_sqrt_softplus_router(HipExpertDispatcher& dispatcher)
{
    ExpertDispatchOptions options;
    options.expert_count = 4;
    options.top_k = 2;
    options.score_function = RouterScoreFunction::SqrtSoftplus;
    options.routed_scaling_factor = 1.5f;
    const std::array<float, 4> selection_bias = {0.0f, 100.0f, 0.0f, 0.0f};
    options.selection_bias = selection_bias;
    const std::array<float, 4> logits = {4.0f, -4.0f, 3.0f, 2.0f};
    auto routed = dispatcher.dispatch(logits, 1, options);
    check(static_cast<bool>(routed));
    check(routed.value().batches.size() == 2);
    check(routed.value().batches[0].expert_id == 0);
    check(routed.value().batches[1].expert_id == 1);
    check_near(routed.value().batches[0].routes[0].weight + routed.value().batches[1].routes[0].weight, 1.5f, 1e-5f);
    // the weights come from the unbiased scores: sqrt(softplus(4)) and sqrt(softplus(-4))
    const float high = std::sqrt(std::log1p(std::exp(4.0f)));
    const float low = std::sqrt(std::log1p(std::exp(-4.0f)));
    check(routed.value().batches[0].routes[0].weight == high / (low + high) * 1.5f); // rank order: expert 1 (biased) first
    check(routed.value().batches[1].routes[0].rank == 0 && routed.value().batches[0].routes[0].rank == 1);

    const std::array<uint32_t, 2> explicit_experts = {3, 2};
    options.selection_bias = {};
    options.explicit_expert_ids = explicit_experts;
    routed = dispatcher.dispatch(logits, 1, options);
    check(static_cast<bool>(routed));
    check(routed.value().batches[0].expert_id == 2);
    check(routed.value().batches[1].expert_id == 3);
    check(routed.value().batches[0].routes[0].rank == 1 && routed.value().batches[1].routes[0].rank == 0);
}

static void test_errors(HipExpertDispatcher& dispatcher)
{
    ExpertDispatchOptions options;
    options.expert_count = 3;
    options.top_k = 2;
    const std::vector<float> logits = {2.0f, 1.0f, 0.0f};
    const auto expect = [&](const Result<ExpertDispatchPlan>& result, ErrorCode code, const char* message) {
        check(!result);
        check(result.error().code == code);
        check(result.error().message == message);
    };
    expect(dispatcher.dispatch(logits, 0, options), ErrorCode::InvalidArgument, "expert dispatch requires at least one token");
    ExpertDispatchOptions bad = options;
    bad.top_k = 4;
    expect(dispatcher.dispatch(logits, 1, bad), ErrorCode::InvalidArgument, "expert dispatch requires 0 < top_k <= expert_count");
    bad.top_k = 0;
    expect(dispatcher.dispatch(logits, 1, bad), ErrorCode::InvalidArgument, "expert dispatch requires 0 < top_k <= expert_count");
    const std::vector<float> invalid_logits = {1.0f, 2.0f};
    expect(dispatcher.dispatch(invalid_logits, 1, options), ErrorCode::InvalidArgument, "router logits shape does not match token and expert counts");
    expect(dispatcher.dispatch(logits, 2, options), ErrorCode::InvalidArgument, "router logits shape does not match token and expert counts");
    const std::array<float, 2> short_bias = {0.0f, 0.0f};
    bad = options;
    bad.selection_bias = short_bias;
    expect(dispatcher.dispatch(logits, 1, bad), ErrorCode::InvalidArgument, "router selection bias must match expert_count");
    const std::array<uint32_t, 3> long_ids = {0, 1, 2};
    bad = options;
    bad.explicit_expert_ids = long_ids;
    expect(dispatcher.dispatch(logits, 1, bad), ErrorCode::InvalidArgument, "explicit expert ids must match token_count * top_k");
    bad = options;
    bad.routed_scaling_factor = 0.0f;
    expect(dispatcher.dispatch(logits, 1, bad), ErrorCode::InvalidArgument, "routed scaling factor must be finite and positive");
    bad.routed_scaling_factor = std::numeric_limits<float>::infinity();
    expect(dispatcher.dispatch(logits, 1, bad), ErrorCode::InvalidArgument, "routed scaling factor must be finite and positive");
    const std::vector<float> nan_logits = {2.0f, std::numeric_limits<float>::quiet_NaN(), 0.0f};
    expect(dispatcher.dispatch(nan_logits, 1, options), ErrorCode::InvalidArgument, "router logits must be finite");
    const std::array<uint32_t, 2> out_of_range = {0, 3};
    bad = options;
    bad.explicit_expert_ids = out_of_range;
    expect(dispatcher.dispatch(logits, 1, bad), ErrorCode::InvalidArgument, "explicit expert id is out of range");
    // a non-finite logit is reported before a bad expert id (the CPU dispatcher scans the logits first)
    expect(dispatcher.dispatch(nan_logits, 1, bad), ErrorCode::InvalidArgument, "router logits must be finite");
    // sigmoid scores of exactly zero selected by name: the only InvalidModel of the dispatcher
    const std::vector<float> low_logits = {-200.0f, -200.0f, 0.0f};
    const std::array<uint32_t, 2> low_experts = {0, 1};
    bad = options;
    bad.score_function = RouterScoreFunction::Sigmoid;
    bad.explicit_expert_ids = low_experts;
    expect(dispatcher.dispatch(low_logits, 1, bad), ErrorCode::InvalidModel, "selected router weights have a non-positive sum");
    // a failed call leaves the caller's plan as it was
    ExpertDispatchPlan plan;
    check(static_cast<bool>(dispatcher.dispatch_into(logits, 1, options, plan)));
    const size_t batches = plan.batches.size();
    check(!dispatcher.dispatch_into(nan_logits, 1, options, plan));
    check(plan.batches.size() == batches && plan.assignment_count == 2);
    // the limits of this dispatcher object
    ExpertDispatchOptions large;
    large.expert_count = 512;
    large.top_k = 2;
    const std::vector<float> large_logits(512, 0.0f);
    auto refused = dispatcher.dispatch(large_logits, 1, large);
    check(!refused && refused.error().code == ErrorCode::InvalidArgument);
}

static void test_many_tokens(HipExpertDispatcher& dispatcher)
{
    // 1000 tokens over 128 experts, Top-8: every token appears K times, ranks 0..K-1 once each, every
    // batch ordered by token, weights of a token sum to the scaling factor
    ExpertDispatchOptions options;
    options.expert_count = 128;
    options.top_k = 8;
    options.routed_scaling_factor = 2.5f;
    const uint32_t tokens = 1000;
    std::vector<float> logits(static_cast<size_t>(tokens) * 128);
    uint32_t state = 12345u;
    for (float& value : logits)
    {
        state = state * 1664525u + 1013904223u;
        value = static_cast<float>(state >> 8) * (1.0f / 16777216.0f) * 8.0f - 4.0f;
    }
    auto plan = dispatcher.dispatch(logits, tokens, options);
    check(static_cast<bool>(plan));
    check(plan.value().assignment_count == static_cast<size_t>(tokens) * 8);
    std::vector<uint32_t> rank_mask(tokens, 0);
    std::vector<double> weight_sum(tokens, 0.0);
    uint32_t previous_expert = 0;
    bool first = true;
    size_t routes = 0;
    for (const ExpertBatch& batch : plan.value().batches)
    {
        check(first || batch.expert_id > previous_expert);
        first = false;
        previous_expert = batch.expert_id;
        check(!batch.routes.empty());
        for (size_t r = 0; r < batch.routes.size(); ++r)
        {
            const ExpertRoute& route = batch.routes[r];
            check(route.token_index < tokens && route.rank < 8);
            check(r == 0 || batch.routes[r - 1].token_index < route.token_index); // distinct experts per token: strictly ascending
            check((rank_mask[route.token_index] & (1u << route.rank)) == 0);
            rank_mask[route.token_index] |= 1u << route.rank;
            weight_sum[route.token_index] += route.weight;
        }
        routes += batch.routes.size();
    }
    check(routes == static_cast<size_t>(tokens) * 8);
    for (uint32_t token = 0; token < tokens; ++token)
    {
        check(rank_mask[token] == 0xffu);
        check_near(static_cast<float>(weight_sum[token]), 2.5f, 1e-5f);
    }
}

int main(int argc, char** argv)
{
    const bool host_only = argc > 1 && std::strcmp(argv[1], "--host") == 0;
    try
    {
        test_defaults_match_the_runtime();
        if (host_only)
        {
            std::printf("all host-side expert dispatcher tests passed\n");
            return 0;
        }
        HipExpertDispatcherPtr dispatcher = HipExpertDispatcher::create(0, 1024, 256, 32);
        if (!dispatcher)
        {
            std::fprintf(stderr, "HipExpertDispatcher::create failed: no usable GPU\n");
            return 2;
        }
        test_groups_routes(*dispatcher);
        test_ties_wide_windows_and_named_experts(*dispatcher);
        test_sqrt_softplus_router(*dispatcher);
        test_errors(*dispatcher);
        test_many_tokens(*dispatcher);
    }
    catch (const std::exception& error)
    {
        std::fprintf(stderr, "FAILED: %s\n", error.what());
        return 1;
    }
    std::printf("all expert dispatcher tests passed\n");
    return 0;
}
