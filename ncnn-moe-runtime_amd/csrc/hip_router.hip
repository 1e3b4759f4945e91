// C ABI of the gfx950 expert router: handle, device buffers and kernel launches.
#include "ncnn_moe_hip_router.h"

#include "router_kernels.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <new>
#include <string>

using namespace ncnn_moe_hip;

struct ncnn_moe_hip_router
{
    int device = 0;
    uint32_t max_tokens = 0;
    uint32_t max_experts = 0;
    uint32_t max_top_k = 0;
    hipStream_t stream = nullptr;

    float* logits = nullptr;
    float* bias = nullptr;
    uint32_t* explicit_ids = nullptr;
    uint32_t* selected_experts = nullptr;
    float* selected_weights = nullptr;
    uint32_t* chunk_counts = nullptr;
    uint32_t* scratch_words = nullptr; // error words [2], finished workgroups of the two kernels [2]
    uint32_t* expert_offsets = nullptr;
    ncnn_moe_expert_route* routes = nullptr;
    uint32_t* status = nullptr;
    uint32_t* host_status = nullptr; // pinned

    std::string last_error;
};

namespace {

int fail(ncnn_moe_hip_router* r, int rc, const std::string& message)
{
    if (r != nullptr)
        r->last_error = message;
    return rc;
}

#define ROUTER_HIP_CHECK(r, call)                                                                        \
    do                                                                                                   \
    {                                                                                                    \
        const hipError_t error_ = (call);                                                                \
        if (error_ != hipSuccess)                                                                        \
            return fail((r), NCNN_MOE_ROUTER_HIP_ERROR, std::string(#call) + ": " + hipGetErrorString(error_)); \
    } while (0)

// The checks of src/graph/expert_dispatcher.cpp:78-97 that need no data.
uint32_t check_options(uint32_t token_count, const ncnn_moe_router_options& o)
{
    if (token_count == 0)
        return NCNN_MOE_ROUTER_NO_TOKENS;
    if (o.expert_count == 0 || o.top_k == 0 || o.top_k > o.expert_count)
        return NCNN_MOE_ROUTER_BAD_TOP_K;
    if (!std::isfinite(o.routed_scaling_factor) || o.routed_scaling_factor <= 0.0f)
        return NCNN_MOE_ROUTER_BAD_SCALING;
    return NCNN_MOE_ROUTER_OK;
}

template <int SLOTS>
void launch_select(const RouterArgs& args, hipStream_t stream)
{
    const unsigned blocks = (args.tokens + kRouterWavesPerBlock - 1) / kRouterWavesPerBlock;
    if (args.tokens <= static_cast<uint32_t>(kRouterChunkTokens))
    {
        // one chunk of tokens: the select kernel's last workgroup places the routes itself, and the
        // scores are computed by all threads of a workgroup of few tokens
        const unsigned staged_blocks = (args.tokens + kStagedTokensPerBlock - 1) / kStagedTokensPerBlock;
        hipLaunchKernelGGL((router_select_kernel<SLOTS, true, true>), dim3(staged_blocks), dim3(kRouterThreads), 0, stream, args);
        return;
    }
    hipLaunchKernelGGL((router_select_kernel<SLOTS, false, false>), dim3(blocks), dim3(kRouterThreads), 0, stream, args);
    const unsigned chunks = (args.tokens + kRouterChunkTokens - 1) / kRouterChunkTokens;
    hipLaunchKernelGGL(router_group_kernel, dim3(chunks), dim3(kRouterThreads), 0, stream, args);
}

int enqueue(ncnn_moe_hip_router* r, const RouterArgs& args, hipStream_t stream)
{
    const uint32_t slots = (args.experts + kWaveSize - 1) / kWaveSize;
    if (slots <= 1)
        launch_select<1>(args, stream);
    else if (slots <= 2)
        launch_select<2>(args, stream);
    else if (slots <= 4)
        launch_select<4>(args, stream);
    else if (slots <= 8)
        launch_select<8>(args, stream);
    else
        launch_select<16>(args, stream);
    ROUTER_HIP_CHECK(r, hipGetLastError());
    return NCNN_MOE_ROUTER_SUCCESS;
}

int check_shape(ncnn_moe_hip_router* r, uint32_t token_count, const ncnn_moe_router_options& o)
{
    if (token_count > r->max_tokens)
        return fail(r, NCNN_MOE_ROUTER_INVALID_ARGUMENT, "token_count exceeds the handle's max_tokens");
    if (o.expert_count > r->max_experts)
        return fail(r, NCNN_MOE_ROUTER_INVALID_ARGUMENT, "expert_count exceeds the handle's max_experts");
    if (o.top_k > r->max_top_k && o.top_k <= o.expert_count)
        return fail(r, NCNN_MOE_ROUTER_INVALID_ARGUMENT, "top_k exceeds the handle's max_top_k");
    if (o.score_function > NCNN_MOE_ROUTER_SQRT_SOFTPLUS)
        return fail(r, NCNN_MOE_ROUTER_INVALID_ARGUMENT, "unknown router score function");
    return NCNN_MOE_ROUTER_SUCCESS;
}

} // namespace

extern "C" {

int ncnn_moe_hip_router_create(int device, uint32_t max_tokens, uint32_t max_experts, uint32_t max_top_k,
                               ncnn_moe_hip_router** out)
{
    if (out == nullptr)
        return NCNN_MOE_ROUTER_INVALID_ARGUMENT;
    *out = nullptr;
    if (max_tokens == 0 || max_experts == 0 || max_experts > NCNN_MOE_ROUTER_MAX_EXPERTS || max_top_k == 0 ||
        max_top_k > NCNN_MOE_ROUTER_MAX_TOP_K)
        return NCNN_MOE_ROUTER_INVALID_ARGUMENT;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count == 0)
        return NCNN_MOE_ROUTER_NO_DEVICE;
    if (device < 0 || device >= count)
        return NCNN_MOE_ROUTER_INVALID_ARGUMENT;
    ncnn_moe_hip_router* r = new (std::nothrow) ncnn_moe_hip_router();
    if (r == nullptr)
        return NCNN_MOE_ROUTER_HIP_ERROR;
    r->device = device;
    r->max_tokens = max_tokens;
    r->max_experts = max_experts;
    r->max_top_k = max_top_k;
    const size_t tokens = max_tokens;
    const size_t assignments = tokens * max_top_k;
    bool ok = hipSetDevice(device) == hipSuccess && hipStreamCreate(&r->stream) == hipSuccess;
    ok = ok && hipMalloc(&r->logits, tokens * max_experts * sizeof(float)) == hipSuccess;
    ok = ok && hipMalloc(&r->bias, max_experts * sizeof(float)) == hipSuccess;
    ok = ok && hipMalloc(&r->explicit_ids, assignments * sizeof(uint32_t)) == hipSuccess;
    ok = ok && hipMalloc(&r->selected_experts, assignments * sizeof(uint32_t)) == hipSuccess;
    ok = ok && hipMalloc(&r->selected_weights, assignments * sizeof(float)) == hipSuccess;
    const size_t chunk_counters = ((tokens + kRouterChunkTokens - 1) / kRouterChunkTokens) * max_experts;
    ok = ok && hipMalloc(&r->chunk_counts, chunk_counters * sizeof(uint32_t)) == hipSuccess;
    ok = ok && hipMalloc(&r->scratch_words, 4 * sizeof(uint32_t)) == hipSuccess;
    // the kernels find these zeroed (no failing token: all ones) and leave them so
    const uint32_t words[4] = {0u, 0xffffffffu, 0u, 0u};
    ok = ok && hipMemset(r->chunk_counts, 0, chunk_counters * sizeof(uint32_t)) == hipSuccess;
    ok = ok && hipMemcpy(r->scratch_words, words, sizeof(words), hipMemcpyHostToDevice) == hipSuccess;
    ok = ok && hipMalloc(&r->expert_offsets, (static_cast<size_t>(max_experts) + 1) * sizeof(uint32_t)) == hipSuccess;
    ok = ok && hipMalloc(&r->routes, assignments * sizeof(ncnn_moe_expert_route)) == hipSuccess;
    ok = ok && hipMalloc(&r->status, sizeof(uint32_t)) == hipSuccess;
    ok = ok && hipHostMalloc(&r->host_status, sizeof(uint32_t), hipHostMallocDefault) == hipSuccess;
    if (!ok)
    {
        std::fprintf(stderr, "ncnn_moe_hip_router_create: %s\n", hipGetErrorString(hipGetLastError()));
        ncnn_moe_hip_router_destroy(r);
        return NCNN_MOE_ROUTER_HIP_ERROR;
    }
    *out = r;
    return NCNN_MOE_ROUTER_SUCCESS;
}

void ncnn_moe_hip_router_destroy(ncnn_moe_hip_router* r)
{
    if (r == nullptr)
        return;
    (void)hipSetDevice(r->device);
    if (r->stream != nullptr)
    {
        (void)hipStreamSynchronize(r->stream);
        (void)hipStreamDestroy(r->stream);
    }
    void* buffers[] = {r->logits, r->bias, r->explicit_ids, r->selected_experts, r->selected_weights, r->chunk_counts,
                       r->scratch_words, r->expert_offsets, r->routes, r->status};
    for (void* buffer : buffers)
    {
        if (buffer != nullptr)
            (void)hipFree(buffer);
    }
    if (r->host_status != nullptr)
        (void)hipHostFree(r->host_status);
    delete r;
}

int ncnn_moe_hip_router_dispatch_device(
    ncnn_moe_hip_router* r, const float* device_router_logits, uint32_t token_count,
    const ncnn_moe_router_options* options, const float* device_selection_bias,
    const uint32_t* device_explicit_expert_ids,
    uint32_t* device_expert_offsets, ncnn_moe_expert_route* device_routes, uint32_t* device_status,
    uint32_t* host_status, void* stream)
{
    if (r == nullptr || options == nullptr || host_status == nullptr)
        return NCNN_MOE_ROUTER_INVALID_ARGUMENT;
    *host_status = check_options(token_count, *options);
    if (*host_status != NCNN_MOE_ROUTER_OK)
        return NCNN_MOE_ROUTER_SUCCESS;
    if (device_router_logits == nullptr || device_expert_offsets == nullptr || device_routes == nullptr || device_status == nullptr)
        return NCNN_MOE_ROUTER_INVALID_ARGUMENT;
    const int rc = check_shape(r, token_count, *options);
    if (rc != NCNN_MOE_ROUTER_SUCCESS)
        return rc;
    ROUTER_HIP_CHECK(r, hipSetDevice(r->device));
    RouterArgs args;
    args.logits = device_router_logits;
    args.selection_bias = device_selection_bias;
    args.explicit_ids = device_explicit_expert_ids;
    args.tokens = token_count;
    args.experts = options->expert_count;
    args.top_k = options->top_k;
    args.score_function = options->score_function;
    args.renormalize = options->renormalize;
    args.scaling = options->routed_scaling_factor;
    args.selected_experts = r->selected_experts;
    args.selected_weights = r->selected_weights;
    args.chunk_counts = r->chunk_counts;
    args.error_words = r->scratch_words;
    args.finished_chunks = r->scratch_words + 2;
    args.finished_selects = r->scratch_words + 3;
    args.expert_offsets = device_expert_offsets;
    args.routes = device_routes;
    args.status = device_status;
    return enqueue(r, args, static_cast<hipStream_t>(stream));
}

int ncnn_moe_hip_router_dispatch(
    ncnn_moe_hip_router* r, const float* router_logits, uint32_t token_count,
    const ncnn_moe_router_options* options, const float* selection_bias, const uint32_t* explicit_expert_ids,
    uint32_t* expert_offsets, ncnn_moe_expert_route* routes, uint32_t* status)
{
    if (r == nullptr || options == nullptr || status == nullptr)
        return NCNN_MOE_ROUTER_INVALID_ARGUMENT;
    *status = check_options(token_count, *options);
    if (*status != NCNN_MOE_ROUTER_OK)
        return NCNN_MOE_ROUTER_SUCCESS;
    if (router_logits == nullptr || expert_offsets == nullptr || routes == nullptr)
        return NCNN_MOE_ROUTER_INVALID_ARGUMENT;
    const int shape = check_shape(r, token_count, *options);
    if (shape != NCNN_MOE_ROUTER_SUCCESS)
        return shape;
    ROUTER_HIP_CHECK(r, hipSetDevice(r->device));
    const size_t logits_bytes = static_cast<size_t>(token_count) * options->expert_count * sizeof(float);
    const size_t assignments = static_cast<size_t>(token_count) * options->top_k;
    ROUTER_HIP_CHECK(r, hipMemcpyAsync(r->logits, router_logits, logits_bytes, hipMemcpyHostToDevice, r->stream));
    if (selection_bias != nullptr)
        ROUTER_HIP_CHECK(r, hipMemcpyAsync(r->bias, selection_bias, options->expert_count * sizeof(float), hipMemcpyHostToDevice, r->stream));
    if (explicit_expert_ids != nullptr)
        ROUTER_HIP_CHECK(r, hipMemcpyAsync(r->explicit_ids, explicit_expert_ids, assignments * sizeof(uint32_t), hipMemcpyHostToDevice, r->stream));
    uint32_t host_status = NCNN_MOE_ROUTER_OK;
    const int rc = ncnn_moe_hip_router_dispatch_device(
        r, r->logits, token_count, options, selection_bias != nullptr ? r->bias : nullptr,
        explicit_expert_ids != nullptr ? r->explicit_ids : nullptr, r->expert_offsets, r->routes, r->status, &host_status,
        r->stream);
    if (rc != NCNN_MOE_ROUTER_SUCCESS)
        return rc;
    ROUTER_HIP_CHECK(r, hipMemcpyAsync(r->host_status, r->status, sizeof(uint32_t), hipMemcpyDeviceToHost, r->stream));
    ROUTER_HIP_CHECK(r, hipMemcpyAsync(expert_offsets, r->expert_offsets, (static_cast<size_t>(options->expert_count) + 1) * sizeof(uint32_t), hipMemcpyDeviceToHost, r->stream));
    ROUTER_HIP_CHECK(r, hipMemcpyAsync(routes, r->routes, assignments * sizeof(ncnn_moe_expert_route), hipMemcpyDeviceToHost, r->stream));
    ROUTER_HIP_CHECK(r, hipStreamSynchronize(r->stream));
    *status = *r->host_status;
    return NCNN_MOE_ROUTER_SUCCESS;
}

const char* ncnn_moe_hip_router_status_message(int status)
{
    switch (status)
    {
    case NCNN_MOE_ROUTER_OK: return "";
    case NCNN_MOE_ROUTER_NO_TOKENS: return "expert dispatch requires at least one token";
    case NCNN_MOE_ROUTER_BAD_TOP_K: return "expert dispatch requires 0 < top_k <= expert_count";
    case NCNN_MOE_ROUTER_BAD_SCALING: return "routed scaling factor must be finite and positive";
    case NCNN_MOE_ROUTER_NON_FINITE_LOGIT: return "router logits must be finite";
    case NCNN_MOE_ROUTER_EXPERT_OUT_OF_RANGE: return "explicit expert id is out of range";
    case NCNN_MOE_ROUTER_NON_POSITIVE_SUM: return "selected router weights have a non-positive sum";
    default: return "unknown router status";
    }
}

const char* ncnn_moe_hip_router_last_error(const ncnn_moe_hip_router* r)
{
    return r == nullptr ? "" : r->last_error.c_str();
}

int ncnn_moe_hip_router_debug_log1pf(ncnn_moe_hip_router* r, const float* in, float* out, size_t n)
{
    if (r == nullptr || in == nullptr || out == nullptr)
        return NCNN_MOE_ROUTER_INVALID_ARGUMENT;
    if (n == 0)
        return NCNN_MOE_ROUTER_SUCCESS;
    ROUTER_HIP_CHECK(r, hipSetDevice(r->device));
    float* device_in = nullptr;
    float* device_out = nullptr;
    ROUTER_HIP_CHECK(r, hipMalloc(&device_in, n * sizeof(float)));
    hipError_t error = hipMalloc(&device_out, n * sizeof(float));
    if (error == hipSuccess)
        error = hipMemcpy(device_in, in, n * sizeof(float), hipMemcpyHostToDevice);
    if (error == hipSuccess)
    {
        hipLaunchKernelGGL(log1pf_probe_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, r->stream, device_in, device_out, n);
        error = hipGetLastError();
    }
    if (error == hipSuccess)
        error = hipStreamSynchronize(r->stream);
    if (error == hipSuccess)
        error = hipMemcpy(out, device_out, n * sizeof(float), hipMemcpyDeviceToHost);
    (void)hipFree(device_in);
    if (device_out != nullptr)
        (void)hipFree(device_out);
    if (error != hipSuccess)
        return fail(r, NCNN_MOE_ROUTER_HIP_ERROR, std::string("debug_log1pf: ") + hipGetErrorString(error));
    return NCNN_MOE_ROUTER_SUCCESS;
}

} // extern "C"
