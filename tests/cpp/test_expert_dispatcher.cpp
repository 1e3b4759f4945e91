// Tests of the C++ host face of the HIP expert router: a table of known plans (the vectors of the
// runtime's own dispatcher tests, tests/test_runtime.cpp:3366-3540: grouping, weights, tied scores, wide
// Top-K, caller-named experts, the sqrt-softplus router with a selection bias) run by one loop that also
// checks the plan's invariants and dispatch_into against dispatch; the error texts and their order; a
// large random call.
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

// ---- known plans.  The inputs and the facts checked are those of the runtime's dispatcher tests
// (tests/test_runtime.cpp:3366-3540), kept here as data: one record per call, the expected plan as the
// flat list of routes in plan order (expert ascending, then token, then rank).  A weight below zero is
// not compared; token_weight_sum below zero likewise.
struct ExpectedRoute
{
    uint32_t expert;
    uint32_t token;
    uint32_t rank;
    double weight;
};

struct PlanCase
{
    const char* name;
    uint32_t tokens;
    uint32_t experts;
    uint32_t top_k;
    RouterScoreFunction score;
    RouterNormalization normalization;
    float scaling;
    uint32_t flags;
    std::vector<float> bias;
    std::vector<uint32_t> named_experts;
    std::vector<float> logits;
    std::vector<ExpectedRoute> routes; // empty: only the invariants and dispatch == dispatch_into are checked
    double token_weight_sum;
};

static std::vector<float> cyclic_logits(size_t count)
{
    std::vector<float> logits(count);
    for (size_t i = 0; i < count; ++i)
        logits[i] = static_cast<float>(static_cast<int>(i % 7) - 3);
    return logits;
}

static std::vector<PlanCase> known_plans()
{
    const auto softmax = RouterScoreFunction::Softmax;
    const auto selected = RouterNormalization::SelectedExperts;
    const uint32_t renormalize = ExpertDispatchNormalizeTopKWeights;
    const double e = std::exp(1.0);
    const double high = std::sqrt(std::log1p(std::exp(4.0)));  // sqrt(softplus(4))
    const double low = std::sqrt(std::log1p(std::exp(-4.0)));  // sqrt(softplus(-4))
    return {
        {"four tokens, two experts in use (:3366-3391)", 4, 6, 1, softmax, selected, 1.0f, renormalize, {}, {},
         {0, 5, 0, 0, 0, 1, 0, 1, 0, 0, 0, 5, 0, 4, 0, 0, 0, 1, 0, 1, 0, 0, 0, 4},
         {{1, 0, 0, 1.0}, {1, 2, 0, 1.0}, {5, 1, 0, 1.0}, {5, 3, 0, 1.0}}, 1.0},
        {"Top-2 of three, renormalised (:3393-3404)", 1, 3, 2, softmax, selected, 1.0f, renormalize, {}, {},
         {2, 1, 0}, {{0, 0, 0, e / (1.0 + e)}, {1, 0, 1, 1.0 / (1.0 + e)}}, 1.0},
        {"the next step's logits (:3425-3435)", 1, 3, 2, softmax, selected, 1.0f, renormalize, {}, {},
         {0, 1, 2}, {{1, 0, 1, 1.0 / (1.0 + e)}, {2, 0, 0, e / (1.0 + e)}}, 1.0},
        {"tied sigmoid scores keep the lower ids, no renormalisation, scale 2 (:3437-3446)", 1, 4, 2,
         RouterScoreFunction::Sigmoid, RouterNormalization::None, 2.0f, 0, {}, {},
         {0, 0, -1, -1}, {{0, 0, 0, 1.0}, {1, 0, 1, 1.0}}, -1.0},
        {"Top-16 of twenty (:3448-3456)", 1, 20, 16, softmax, selected, 1.0f, renormalize, {}, {}, cyclic_logits(20), {}, 1.0},
        {"Top-17 of twenty (:3457-3458)", 1, 20, 17, softmax, selected, 1.0f, renormalize, {}, {}, cyclic_logits(20), {}, 1.0},
        {"one expert named twice (:3460-3468)", 1, 4, 2, softmax, selected, 1.0f, renormalize, {}, {1, 1},
         {0, 1, 2, 3}, {{1, 0, 0, 0.5}, {1, 0, 1, 0.5}}, 1.0},
        {"sqrt-softplus with a selection bias: the bias picks, the unbiased scores weigh (:3499-3518)", 1, 4, 2,
         RouterScoreFunction::SqrtSoftplus, selected, 1.5f, renormalize, {0, 100, 0, 0}, {},
         {4, -4, 3, 2}, {{0, 0, 1, high / (low + high) * 1.5}, {1, 0, 0, low / (low + high) * 1.5}}, 1.5},
        {"sqrt-softplus, experts named by the caller (:3520-3533)", 1, 4, 2,
         RouterScoreFunction::SqrtSoftplus, selected, 1.5f, renormalize, {}, {3, 2},
         {4, -4, 3, 2}, {{2, 0, 1, -1.0}, {3, 0, 0, -1.0}}, 1.5},
    };
}

static ExpertDispatchOptions options_of(const PlanCase& c)
{
    ExpertDispatchOptions options;
    options.expert_count = c.experts;
    options.top_k = c.top_k;
    options.score_function = c.score;
    options.normalization = c.normalization;
    options.routed_scaling_factor = c.scaling;
    options.flags = c.flags;
    options.selection_bias = c.bias;
    options.explicit_expert_ids = c.named_experts;
    return options;
}

static std::vector<ExpectedRoute> flatten(const ExpertDispatchPlan& plan)
{
    std::vector<ExpectedRoute> flat;
    for (const ExpertBatch& batch : plan.batches)
    {
        check(!batch.routes.empty());
        for (const ExpertRoute& route : batch.routes)
            flat.push_back({batch.expert_id, route.token_index, route.rank, static_cast<double>(route.weight)});
    }
    return flat;
}

static void test_known_plans(HipExpertDispatcher& dispatcher)
{
    ExpertDispatchPlan reused; // one plan object through every case: dispatch_into keeps the caller's storage
    for (const PlanCase& c : known_plans())
    {
        try
        {
            const ExpertDispatchOptions options = options_of(c);
            auto result = dispatcher.dispatch(c.logits, c.tokens, options);
            check(static_cast<bool>(result));
            const ExpertDispatchPlan& plan = result.value();
            const std::vector<ExpectedRoute> flat = flatten(plan);
            check(plan.assignment_count == static_cast<size_t>(c.tokens) * c.top_k);
            check(flat.size() == plan.assignment_count);
            std::vector<double> sums(c.tokens, 0.0);
            for (size_t i = 0; i < flat.size(); ++i)
            {
                check(flat[i].expert < c.experts && flat[i].token < c.tokens && flat[i].rank < c.top_k);
                if (i > 0) // plan order
                    check(flat[i - 1].expert < flat[i].expert ||
                          (flat[i - 1].expert == flat[i].expert &&
                           (flat[i - 1].token < flat[i].token || (flat[i - 1].token == flat[i].token && flat[i - 1].rank < flat[i].rank))));
                sums[flat[i].token] += flat[i].weight;
            }
            if (c.token_weight_sum >= 0.0)
            {
                for (double sum : sums)
                    check_near(static_cast<float>(sum), static_cast<float>(c.token_weight_sum), 1e-5f);
            }
            if (!c.routes.empty())
            {
                check(flat.size() == c.routes.size());
                for (size_t i = 0; i < flat.size(); ++i)
                {
                    check(flat[i].expert == c.routes[i].expert && flat[i].token == c.routes[i].token && flat[i].rank == c.routes[i].rank);
                    if (c.routes[i].weight >= 0.0)
                        check_near(static_cast<float>(flat[i].weight), static_cast<float>(c.routes[i].weight), 1e-6f);
                }
            }
            // dispatch_into: the same plan, bit for bit, in storage that it does not reallocate when it fits
            const ExpertBatch* batches_before = reused.batches.data();
            const size_t capacity_before = reused.batches.capacity();
            auto status = dispatcher.dispatch_into(c.logits, c.tokens, options, reused);
            check(static_cast<bool>(status));
            if (plan.batches.size() <= capacity_before)
                check(reused.batches.data() == batches_before);
            const std::vector<ExpectedRoute> again = flatten(reused);
            check(reused.assignment_count == plan.assignment_count && again.size() == flat.size());
            for (size_t i = 0; i < flat.size(); ++i)
            {
                check(again[i].expert == flat[i].expert && again[i].token == flat[i].token && again[i].rank == flat[i].rank);
                const float a = static_cast<float>(again[i].weight), b = static_cast<float>(flat[i].weight);
                check(std::memcmp(&a, &b, sizeof(a)) == 0);
            }
        }
        catch (const std::exception& error)
        {
            throw std::runtime_error(std::string("known plan \"") + c.name + "\": " + error.what());
        }
    }
    // a route's storage is kept as well: the same call twice leaves every vector where it was
    const PlanCase c = known_plans()[1];
    const ExpertDispatchOptions options = options_of(c);
    check(static_cast<bool>(dispatcher.dispatch_into(c.logits, c.tokens, options, reused)));
    const ExpertBatch* batches = reused.batches.data();
    const ExpertRoute* first_routes = reused.batches.front().routes.data();
    check(static_cast<bool>(dispatcher.dispatch_into(c.logits, c.tokens, options, reused)));
    check(reused.batches.data() == batches && reused.batches.front().routes.data() == first_routes);
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
        test_known_plans(*dispatcher);
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
