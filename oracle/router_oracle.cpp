/*
 * CPU oracle for the expert router -- TEST INFRASTRUCTURE ONLY, never shipped or measured as the
 * product.  It restates src/graph/expert_dispatcher.cpp:12-157 of the reference in the same
 * evaluation order: libm expf / log1pf / sqrtf, a sequential fp32 softmax sum in expert order,
 * ordered insertion of the Top-K routes by (score + bias descending, expert id ascending), a
 * sequential fp32 sum of the selected scores in rank order.  Build with -ffp-contract=off.
 *
 * What pins it (tests/test_oracle_router.py):
 *   oracle_router_scores, oracle_router_dispatch   the reference's own ExpertDispatcher::dispatch and
 *       dispatch_into (public API, called through the harness where the reference builds): random
 *       shapes, the three score functions, bias, explicit ids, bit-exact weights, same grouping and
 *       errors; the reference's own test vectors (tests/test_runtime.cpp:3362-3540); a float64
 *       model of the scores; committed golden vectors (tests/golden/router_golden.npz).
 */
#include "router_oracle.h"

#include <algorithm>
#include <cmath>
#include <vector>

namespace {

struct RouteCandidate
{
    uint32_t expert_id;
    float score;
};

/* src/graph/expert_dispatcher.cpp:19-22 */
bool route_precedes(const RouteCandidate& left, const RouteCandidate& right)
{
    return left.score > right.score || (left.score == right.score && left.expert_id < right.expert_id);
}

/* src/graph/expert_dispatcher.cpp:24-31 */
float stable_softplus(float value)
{
    if (value > 20.0f)
        return value;
    if (value < -20.0f)
        return std::exp(value);
    return std::log1p(std::exp(value));
}

/* src/graph/expert_dispatcher.cpp:33-38 */
float score_router_logit(float logit, uint32_t score_function)
{
    if (score_function == ORACLE_ROUTER_SIGMOID)
        return 1.0f / (1.0f + std::exp(-logit));
    return std::sqrt(stable_softplus(logit));
}

/* src/graph/expert_dispatcher.cpp:40-59 */
void router_scores(const float* logits, uint32_t size, uint32_t score_function, std::vector<float>& scores)
{
    scores.resize(size);
    if (score_function == ORACLE_ROUTER_SOFTMAX)
    {
        const float maximum = *std::max_element(logits, logits + size);
        float sum = 0.0f;
        for (uint32_t index = 0; index < size; ++index)
        {
            scores[index] = std::exp(logits[index] - maximum);
            sum += scores[index];
        }
        for (float& score : scores)
            score /= sum;
        return;
    }
    for (uint32_t index = 0; index < size; ++index)
        scores[index] = score_router_logit(logits[index], score_function);
}

/* src/graph/expert_dispatcher.cpp:61-77 */
void select_topk_routes(const float* scores, const float* selection_bias, uint32_t expert_count, uint32_t top_k,
                        std::vector<RouteCandidate>& selected)
{
    selected.clear();
    for (uint32_t expert_id = 0; expert_id < expert_count; ++expert_id)
    {
        const RouteCandidate candidate{expert_id, scores[expert_id] + (selection_bias == nullptr ? 0.0f : selection_bias[expert_id])};
        const auto insertion = std::lower_bound(selected.begin(), selected.end(), candidate, route_precedes);
        if (selected.size() == top_k && insertion == selected.end())
            continue;
        selected.insert(insertion, candidate);
        if (selected.size() > top_k)
            selected.pop_back();
    }
}

} // namespace

extern "C" {

const char* oracle_router_status_message(int status)
{
    switch (status)
    {
    case ORACLE_ROUTER_OK: return "";
    case ORACLE_ROUTER_NO_TOKENS: return "expert dispatch requires at least one token";
    case ORACLE_ROUTER_BAD_TOP_K: return "expert dispatch requires 0 < top_k <= expert_count";
    case ORACLE_ROUTER_BAD_SCALING: return "routed scaling factor must be finite and positive";
    case ORACLE_ROUTER_NON_FINITE_LOGIT: return "router logits must be finite";
    case ORACLE_ROUTER_EXPERT_OUT_OF_RANGE: return "explicit expert id is out of range";
    case ORACLE_ROUTER_NON_POSITIVE_SUM: return "selected router weights have a non-positive sum";
    default: return "unknown router status";
    }
}

void oracle_router_scores(const float* logits, uint32_t expert_count, uint32_t score_function, float* scores)
{
    std::vector<float> out;
    router_scores(logits, expert_count, score_function, out);
    std::copy(out.begin(), out.end(), scores);
}

/* src/graph/expert_dispatcher.cpp:76-157 */
int oracle_router_dispatch(
    const float* router_logits, uint32_t token_count, const oracle_router_options* options,
    const float* selection_bias, const uint32_t* explicit_expert_ids,
    uint32_t* expert_offsets, oracle_expert_route* routes)
{
    if (token_count == 0)
        return ORACLE_ROUTER_NO_TOKENS;
    if (options->expert_count == 0 || options->top_k == 0 || options->top_k > options->expert_count)
        return ORACLE_ROUTER_BAD_TOP_K;
    if (!std::isfinite(options->routed_scaling_factor) || options->routed_scaling_factor <= 0.0f)
        return ORACLE_ROUTER_BAD_SCALING;
    const size_t logit_count = static_cast<size_t>(token_count) * options->expert_count;
    for (size_t i = 0; i < logit_count; ++i)
    {
        if (!std::isfinite(router_logits[i]))
            return ORACLE_ROUTER_NON_FINITE_LOGIT;
    }
    std::vector<std::vector<oracle_expert_route>> batches(options->expert_count);
    std::vector<float> scores;
    std::vector<RouteCandidate> selected;
    for (uint32_t token_index = 0; token_index < token_count; ++token_index)
    {
        const float* logits = router_logits + static_cast<size_t>(token_index) * options->expert_count;
        router_scores(logits, options->expert_count, options->score_function, scores);
        if (explicit_expert_ids == nullptr)
            select_topk_routes(scores.data(), selection_bias, options->expert_count, options->top_k, selected);
        else
        {
            selected.clear();
            for (uint32_t route_index = 0; route_index < options->top_k; ++route_index)
            {
                const uint32_t expert_id = explicit_expert_ids[static_cast<size_t>(token_index) * options->top_k + route_index];
                if (expert_id >= options->expert_count)
                    return ORACLE_ROUTER_EXPERT_OUT_OF_RANGE;
                selected.push_back({expert_id, scores[expert_id]});
            }
        }
        float selected_sum = 0.0f;
        for (const RouteCandidate& candidate : selected)
            selected_sum += scores[candidate.expert_id];
        if (options->renormalize && selected_sum <= 0.0f)
            return ORACLE_ROUTER_NON_POSITIVE_SUM;
        for (uint32_t rank = 0; rank < selected.size(); ++rank)
        {
            const float score = scores[selected[rank].expert_id];
            const float weight = (options->renormalize ? score / selected_sum : score) * options->routed_scaling_factor;
            batches[selected[rank].expert_id].push_back({token_index, rank, weight});
        }
    }
    uint32_t written = 0;
    for (uint32_t expert_id = 0; expert_id < options->expert_count; ++expert_id)
    {
        expert_offsets[expert_id] = written;
        for (const oracle_expert_route& route : batches[expert_id])
            routes[written++] = route;
    }
    expert_offsets[options->expert_count] = written;
    return ORACLE_ROUTER_OK;
}

void oracle_log1pf_libm_array(const float* in, float* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = std::log1p(in[i]);
}

} // extern "C"
