/*
 * CPU oracle for the expert router (MoE token dispatch) -- TEST INFRASTRUCTURE ONLY.
 *
 * A CPU restatement of src/graph/expert_dispatcher.cpp:12-157 of the reference (router scores,
 * Top-K route selection, weight normalisation, grouping by expert), written to be the checker of
 * the HIP router.  Never part of the shipped path: only tests, the smoke check and the benchmark's
 * cpu_baseline leg may load it.  What pins each function is listed in router_oracle.cpp.
 */
#ifndef ROUTER_ORACLE_H
#define ROUTER_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* include/ncnn/moe/types.h:216-221 (RouterScoreFunction) */
enum oracle_router_score
{
    ORACLE_ROUTER_SOFTMAX = 0,
    ORACLE_ROUTER_SIGMOID = 1,
    ORACLE_ROUTER_SQRT_SOFTPLUS = 2
};

/* One value per error message of src/graph/expert_dispatcher.cpp:80-103, :122, :133. */
enum oracle_router_status
{
    ORACLE_ROUTER_OK = 0,
    ORACLE_ROUTER_NO_TOKENS = 1,          /* "expert dispatch requires at least one token" */
    ORACLE_ROUTER_BAD_TOP_K = 2,          /* "expert dispatch requires 0 < top_k <= expert_count" */
    ORACLE_ROUTER_BAD_SCALING = 3,        /* "routed scaling factor must be finite and positive" */
    ORACLE_ROUTER_NON_FINITE_LOGIT = 4,   /* "router logits must be finite" */
    ORACLE_ROUTER_EXPERT_OUT_OF_RANGE = 5,/* "explicit expert id is out of range" */
    ORACLE_ROUTER_NON_POSITIVE_SUM = 6    /* "selected router weights have a non-positive sum" (InvalidModel) */
};

/* ExpertDispatchOptions (include/ncnn/moe/expert_dispatcher.h:36-46) without the two spans. */
typedef struct oracle_router_options
{
    uint32_t expert_count;
    uint32_t top_k;
    uint32_t score_function;   /* enum oracle_router_score */
    uint32_t renormalize;      /* flags & NormalizeTopKWeights, or normalization == SelectedExperts */
    float routed_scaling_factor;
} oracle_router_options;

/* ExpertRoute (include/ncnn/moe/expert_dispatcher.h:15-20) */
typedef struct oracle_expert_route
{
    uint32_t token_index;
    uint32_t rank;
    float weight;
} oracle_expert_route;

const char* oracle_router_status_message(int status);

/* router_scores (src/graph/expert_dispatcher.cpp:40-59) for one token. */
void oracle_router_scores(const float* logits, uint32_t expert_count, uint32_t score_function, float* scores);

/*
 * ExpertDispatcher::dispatch (src/graph/expert_dispatcher.cpp:76-157).  router_logits is token-major
 * [token_count][expert_count]; selection_bias (expert_count floats) and explicit_expert_ids
 * (token_count * top_k ids) may be null.  The plan comes back flat: routes[] holds the
 * token_count * top_k routes grouped by expert id in ascending order (each group in the order the
 * reference pushed them: by token, then by rank), expert_offsets[e] .. expert_offsets[e + 1] is
 * expert e's group (expert_count + 1 entries).  Returns the status.
 */
int oracle_router_dispatch(
    const float* router_logits, uint32_t token_count, const oracle_router_options* options,
    const float* selection_bias, const uint32_t* explicit_expert_ids,
    uint32_t* expert_offsets, oracle_expert_route* routes);

/* libm's log1pf over an array: what the device restatement of it is compared with. */
void oracle_log1pf_libm_array(const float* in, float* out, size_t n);

#ifdef __cplusplus
}
#endif

#endif /* ROUTER_ORACLE_H */
