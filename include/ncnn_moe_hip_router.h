/*
 * C ABI of the MI355X expert router: the token-to-expert dispatch of a MoE layer (router scores,
 * Top-K route selection, weight normalisation, grouping of the routes by expert) on one GPU.
 *
 * Drop-in boundary for ncnn::moe::ExpertDispatcher::dispatch / dispatch_into
 * (include/ncnn/moe/expert_dispatcher.h:55-63, src/graph/expert_dispatcher.cpp:76-301): the same plan
 * (experts in ascending id order, an expert's routes by token then rank, the same fp32 weights bit for
 * bit), the same errors.  Plain C, POD structs, no exceptions across the boundary.
 */
#ifndef NCNN_MOE_HIP_ROUTER_H
#define NCNN_MOE_HIP_ROUTER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ncnn_moe_hip_router ncnn_moe_hip_router;

/* RouterScoreFunction (include/ncnn/moe/types.h:216-221) */
enum ncnn_moe_router_score
{
    NCNN_MOE_ROUTER_SOFTMAX = 0,
    NCNN_MOE_ROUTER_SIGMOID = 1,
    NCNN_MOE_ROUTER_SQRT_SOFTPLUS = 2
};

/* One value per error message of src/graph/expert_dispatcher.cpp:80-103, :122, :133 that a flat call
 * can raise (the shape checks of :88-95 are the caller's: the arrays have no size here). */
enum ncnn_moe_router_status
{
    NCNN_MOE_ROUTER_OK = 0,
    NCNN_MOE_ROUTER_NO_TOKENS = 1,           /* "expert dispatch requires at least one token" */
    NCNN_MOE_ROUTER_BAD_TOP_K = 2,           /* "expert dispatch requires 0 < top_k <= expert_count" */
    NCNN_MOE_ROUTER_BAD_SCALING = 3,         /* "routed scaling factor must be finite and positive" */
    NCNN_MOE_ROUTER_NON_FINITE_LOGIT = 4,    /* "router logits must be finite" */
    NCNN_MOE_ROUTER_EXPERT_OUT_OF_RANGE = 5, /* "explicit expert id is out of range" */
    NCNN_MOE_ROUTER_NON_POSITIVE_SUM = 6     /* "selected router weights have a non-positive sum" (ErrorCode::InvalidModel) */
};

/* Call-level return codes (as for the sampler: everything but INVALID_ARGUMENT maps to InternalError). */
enum ncnn_moe_router_rc
{
    NCNN_MOE_ROUTER_SUCCESS = 0,
    NCNN_MOE_ROUTER_INVALID_ARGUMENT = 1,
    NCNN_MOE_ROUTER_HIP_ERROR = 2,
    NCNN_MOE_ROUTER_NO_DEVICE = 3
};

/* ExpertDispatchOptions (include/ncnn/moe/expert_dispatcher.h:36-46) without its two spans. */
typedef struct ncnn_moe_router_options
{
    uint32_t expert_count;
    uint32_t top_k;
    uint32_t score_function;      /* enum ncnn_moe_router_score */
    uint32_t renormalize;         /* (flags & ExpertDispatchNormalizeTopKWeights) || normalization == SelectedExperts */
    float routed_scaling_factor;
} ncnn_moe_router_options;

/* ExpertRoute (include/ncnn/moe/expert_dispatcher.h:15-20) */
typedef struct ncnn_moe_expert_route
{
    uint32_t token_index;
    uint32_t rank;
    float weight;
} ncnn_moe_expert_route;

enum { NCNN_MOE_ROUTER_MAX_EXPERTS = 1024, NCNN_MOE_ROUTER_MAX_TOP_K = 64 };

/* Plays the role of constructing an ExpertDispatcher (which holds no state on the CPU): allocates
 * the device buffers for max_tokens x max_experts logits and max_tokens x max_top_k routes.
 * max_experts <= NCNN_MOE_ROUTER_MAX_EXPERTS, max_top_k <= NCNN_MOE_ROUTER_MAX_TOP_K. */
int ncnn_moe_hip_router_create(int device, uint32_t max_tokens, uint32_t max_experts, uint32_t max_top_k,
                               ncnn_moe_hip_router** out);
void ncnn_moe_hip_router_destroy(ncnn_moe_hip_router* router);

/* ExpertDispatcher::dispatch (src/graph/expert_dispatcher.cpp:76-157) with host operands; returns when
 * the plan is written.  router_logits is token-major [token_count][expert_count]; selection_bias
 * (expert_count floats) and explicit_expert_ids (token_count * top_k ids) may be null.  The plan is
 * flat: routes[] holds the token_count * top_k routes grouped by expert id in ascending order (an
 * expert's group by token, then rank, as ExpertBatch::routes), expert_offsets[e] ..
 * expert_offsets[e + 1] is expert e's group (expert_count + 1 entries); ExpertDispatchPlan::batches is
 * the non-empty groups.  *status receives an ncnn_moe_router_status; the plan is valid only for OK. */
int ncnn_moe_hip_router_dispatch(
    ncnn_moe_hip_router* router, const float* router_logits, uint32_t token_count,
    const ncnn_moe_router_options* options, const float* selection_bias, const uint32_t* explicit_expert_ids,
    uint32_t* expert_offsets, ncnn_moe_expert_route* routes, uint32_t* status);

/* The same computation with every array in device memory and no host synchronisation: kernels are
 * enqueued on `stream` (a hipStream_t, or null) and the call returns at once.  This is the entry a
 * device-resident gate GEMM feeds.  device_status receives the status word.  The argument checks
 * that need no data (token count, top_k, scaling factor) are made on the host and reported through
 * the return value's companion *host_status. */
int ncnn_moe_hip_router_dispatch_device(
    ncnn_moe_hip_router* router, const float* device_router_logits, uint32_t token_count,
    const ncnn_moe_router_options* options, const float* device_selection_bias,
    const uint32_t* device_explicit_expert_ids,
    uint32_t* device_expert_offsets, ncnn_moe_expert_route* device_routes, uint32_t* device_status,
    uint32_t* host_status, void* stream);

/* The dispatcher's fixed message for a status (src/graph/expert_dispatcher.cpp:80-103, :122, :133). */
const char* ncnn_moe_hip_router_status_message(int status);
const char* ncnn_moe_hip_router_last_error(const ncnn_moe_hip_router* router);

/* Test hook (no counterpart in the runtime): evaluates the device log1pf on n host values. */
int ncnn_moe_hip_router_debug_log1pf(ncnn_moe_hip_router* router, const float* in, float* out, size_t n);

#ifdef __cplusplus
}
#endif

#endif /* NCNN_MOE_HIP_ROUTER_H */
