// Expert router kernels (src/graph/expert_dispatcher.cpp:12-157 of the runtime, on the device):
//   router_select_kernel  one wave per token: scores, Top-K routes, normalised weights
//   router_group_kernel   one wave per expert: the expert's routes, by token then rank
#ifndef NCNN_MOE_HIP_ROUTER_KERNELS_H
#define NCNN_MOE_HIP_ROUTER_KERNELS_H

#include "ncnn_moe_hip_router.h"
#include "sampler_device.h"

namespace ncnn_moe_hip {

constexpr int kRouterWavesPerBlock = 4;
constexpr int kRouterThreads = kRouterWavesPerBlock * kWaveSize;

// log1pf bit-identical to glibc 2.35's (sysdeps/ieee754/flt-32/s_log1pf.c) for finite x > 0, which is
// all stable_softplus hands it (an exponential).  Plain fp32 operations in the library's order; built
// without contraction, so every one rounds once.  Compared with libm on every positive float.
__device__ __forceinline__ float log1pf_libm_positive(float x)
{
    const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f;
    const float Lp1 = 6.6666668653e-01f, Lp2 = 4.0000000596e-01f, Lp3 = 2.8571429849e-01f, Lp4 = 2.2222198546e-01f,
                Lp5 = 1.8183572590e-01f, Lp6 = 1.5313838422e-01f, Lp7 = 1.4798198640e-01f;
    float f = 0.0f, c = 0.0f, u;
    int32_t k = 1, hu = 0;
    const int32_t hx = static_cast<int32_t>(__float_as_uint(x));
    if (hx < 0x3ed413d7) // x < 0.41422
    {
        if (hx < 0x31000000) // x < 2^-29
        {
            if (hx < 0x24800000) // x < 2^-54
                return x;
            return x - x * x * 0.5f;
        }
        k = 0;
        f = x;
        hu = 1;
    }
    if (hx >= 0x7f800000)
        return x + x;
    if (k != 0)
    {
        if (hx < 0x5a000000)
        {
            u = 1.0f + x;
            hu = static_cast<int32_t>(__float_as_uint(u));
            k = (hu >> 23) - 127;
            c = (k > 0) ? 1.0f - (u - x) : x - (u - 1.0f); // correction term
            c /= u;
        }
        else
        {
            u = x;
            hu = static_cast<int32_t>(__float_as_uint(u));
            k = (hu >> 23) - 127;
            c = 0.0f;
        }
        hu &= 0x007fffff;
        if (hu < 0x3504f7)
            u = __uint_as_float(static_cast<uint32_t>(hu) | 0x3f800000u); // normalise u
        else
        {
            k += 1;
            u = __uint_as_float(static_cast<uint32_t>(hu) | 0x3f000000u); // normalise u / 2
            hu = (0x00800000 - hu) >> 2;
        }
        f = u - 1.0f;
    }
    const float hfsq = 0.5f * f * f;
    const float kf = static_cast<float>(k);
    if (hu == 0) // |f| < 2^-20
    {
        if (f == 0.0f)
        {
            if (k == 0)
                return 0.0f;
            c += kf * ln2_lo;
            return kf * ln2_hi + c;
        }
        const float R = hfsq * (1.0f - 0.66666666666666666f * f);
        if (k == 0)
            return f - R;
        return kf * ln2_hi - ((R - (kf * ln2_lo + c)) - f);
    }
    const float s = f / (2.0f + f);
    const float z = s * s;
    const float R = z * (Lp1 + z * (Lp2 + z * (Lp3 + z * (Lp4 + z * (Lp5 + z * (Lp6 + z * Lp7))))));
    if (k == 0)
        return f - (hfsq - s * (hfsq + R));
    return kf * ln2_hi - ((hfsq - (s * (hfsq + R) + (kf * ln2_lo + c))) - f);
}

// score_router_logit (src/graph/expert_dispatcher.cpp:24-38)
__device__ __forceinline__ float router_score_of_logit(float logit, uint32_t score_function)
{
    if (score_function == NCNN_MOE_ROUTER_SIGMOID)
        return 1.0f / (1.0f + expf_libm(-logit));
    float softplus;
    if (logit > 20.0f)
        softplus = logit;
    else if (logit < -20.0f)
        softplus = expf_libm(logit);
    else
        softplus = log1pf_libm_positive(expf_libm(logit));
    return __builtin_sqrtf(softplus); // correctly rounded: built with -fhip-fp32-correctly-rounded-divide-sqrt
}

struct RouterArgs
{
    const float* logits;          // [tokens][experts]
    const float* selection_bias;  // [experts] or null
    const uint32_t* explicit_ids; // [tokens][top_k] or null
    uint32_t tokens;
    uint32_t experts;
    uint32_t top_k;
    uint32_t score_function;
    uint32_t renormalize;
    float scaling;
    uint32_t* selected_experts;   // [tokens][top_k], rank order
    float* selected_weights;      // [tokens][top_k]
    uint32_t* expert_counts;      // [experts], zero at launch
    uint32_t* error_words;        // [0]: non-finite logit seen, [1]: min over failing tokens of (token << 3 | status), ~0 if none
    uint32_t* expert_offsets;     // [experts + 1]
    ncnn_moe_expert_route* routes; // [tokens * top_k]
    uint32_t* status;             // the call's ncnn_moe_router_status
};

struct RouterShared
{
    float scores[kRouterWavesPerBlock][NCNN_MOE_ROUTER_MAX_EXPERTS];
    uint32_t chosen[kRouterWavesPerBlock][NCNN_MOE_ROUTER_MAX_TOP_K];
};

// One wave per token.  Expert e lives in slot e / 64 of lane e % 64, so a loop over slots, then lanes,
// visits the experts in index order: the softmax sum and the sum of the selected scores are the CPU
// loops themselves, one fp32 addition at a time.
template <int SLOTS>
__global__ __launch_bounds__(kRouterThreads) void router_select_kernel(RouterArgs r)
{
    __shared__ RouterShared shared;
    const int lane = threadIdx.x & (kWaveSize - 1);
    const int wave = threadIdx.x >> 6;
    const uint32_t token = blockIdx.x * kRouterWavesPerBlock + wave;
    if (token >= r.tokens)
        return;
    const int experts = static_cast<int>(r.experts);
    const float* logits = r.logits + static_cast<size_t>(token) * r.experts;

    float logit[SLOTS];
    bool finite = true;
    float maximum = -__builtin_inff();
#pragma unroll
    for (int s = 0; s < SLOTS; ++s)
    {
        const int e = s * kWaveSize + lane;
        logit[s] = e < experts ? logits[e] : 0.0f;
        if (e < experts)
        {
            finite = finite && is_finite_f32(logit[s]);
            maximum = fmaxf(maximum, logit[s]);
        }
    }
    if (__ballot(!finite) != 0)
    {
        // src/graph/expert_dispatcher.cpp:98-102: any non-finite logit of the call fails it
        if (lane == 0)
            atomicOr(&r.error_words[0], 1u);
        return;
    }

    // ---- router_scores (src/graph/expert_dispatcher.cpp:40-59)
    float score[SLOTS];
    if (r.score_function == NCNN_MOE_ROUTER_SOFTMAX)
    {
#pragma unroll
        for (int step = 1; step < kWaveSize; step <<= 1)
            maximum = fmaxf(maximum, __shfl_xor(maximum, step, kWaveSize));
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
            score[s] = (s * kWaveSize + lane) < experts ? expf_libm(logit[s] - maximum) : 0.0f;
        float sum = 0.0f;
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
        {
            const int slot_count = min(kWaveSize, experts - s * kWaveSize);
            for (int l = 0; l < slot_count; ++l)
                sum += read_lane(score[s], l);
        }
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
            score[s] = score[s] / sum;
    }
    else
    {
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
            score[s] = (s * kWaveSize + lane) < experts ? router_score_of_logit(logit[s], r.score_function) : 0.0f;
    }
#pragma unroll
    for (int s = 0; s < SLOTS; ++s)
    {
        const int e = s * kWaveSize + lane;
        if (e < experts)
            shared.scores[wave][e] = score[s];
    }

    const int top_k = static_cast<int>(r.top_k);
    if (r.explicit_ids != nullptr)
    {
        // src/graph/expert_dispatcher.cpp:124-135: the caller names the experts; rank = position
        bool in_range = true;
        if (lane < top_k)
        {
            const uint32_t expert = r.explicit_ids[static_cast<size_t>(token) * r.top_k + lane];
            in_range = expert < r.experts;
            shared.chosen[wave][lane] = expert;
        }
        if (__ballot(!in_range) != 0)
        {
            if (lane == 0)
                atomicMin(&r.error_words[1], (token << 3) | NCNN_MOE_ROUTER_EXPERT_OUT_OF_RANGE);
            return;
        }
    }
    else
    {
        // ---- select_topk_routes (src/graph/expert_dispatcher.cpp:61-77): the best top_k by
        // (score + bias descending, expert id ascending), found one per round
        float keyed[SLOTS];
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
        {
            const int e = s * kWaveSize + lane;
            keyed[s] = score[s] + ((r.selection_bias == nullptr || e >= experts) ? 0.0f : r.selection_bias[e]);
        }
        uint32_t taken = 0; // this lane's slots already selected
        for (int round = 0; round < top_k; ++round)
        {
            float best = 0.0f;
            int best_expert = 0x7fffffff; // none
#pragma unroll
            for (int s = 0; s < SLOTS; ++s)
            {
                const int e = s * kWaveSize + lane;
                const bool available = e < experts && ((taken >> s) & 1u) == 0u;
                if (available && (best_expert == 0x7fffffff || keyed[s] > best))
                {
                    best = keyed[s];
                    best_expert = e;
                }
            }
#pragma unroll
            for (int step = 1; step < kWaveSize; step <<= 1)
            {
                const float other = __shfl_xor(best, step, kWaveSize);
                const int other_expert = __shfl_xor(best_expert, step, kWaveSize);
                const bool other_wins = other_expert != 0x7fffffff &&
                    (best_expert == 0x7fffffff || other > best || (other == best && other_expert < best_expert));
                if (other_wins)
                {
                    best = other;
                    best_expert = other_expert;
                }
            }
            if ((best_expert & (kWaveSize - 1)) == lane)
                taken |= 1u << (best_expert >> 6);
            if (lane == 0)
                shared.chosen[wave][round] = static_cast<uint32_t>(best_expert);
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f); // this wave's LDS writes, before its lanes read them back
    __builtin_amdgcn_wave_barrier();

    // ---- src/graph/expert_dispatcher.cpp:137-150: the selected scores are summed in rank order
    float selected_sum = 0.0f;
    for (int rank = 0; rank < top_k; ++rank)
        selected_sum += shared.scores[wave][shared.chosen[wave][rank]];
    if (r.renormalize != 0u && selected_sum <= 0.0f)
    {
        if (lane == 0)
            atomicMin(&r.error_words[1], (token << 3) | NCNN_MOE_ROUTER_NON_POSITIVE_SUM);
        return;
    }
    if (lane < top_k)
    {
        const uint32_t expert = shared.chosen[wave][lane];
        const float expert_score = shared.scores[wave][expert];
        const float weight = (r.renormalize != 0u ? expert_score / selected_sum : expert_score) * r.scaling;
        r.selected_experts[static_cast<size_t>(token) * r.top_k + lane] = expert;
        r.selected_weights[static_cast<size_t>(token) * r.top_k + lane] = weight;
        atomicAdd(&r.expert_counts[expert], 1u);
    }
}

// One wave per expert: its offset is the sum of the counts of the experts before it; its routes are
// the assignments that name it, in (token, rank) order, which is the order of the flat array.
// Wave 0 of the grid also settles the call's status.
__global__ __launch_bounds__(kRouterThreads) void router_group_kernel(RouterArgs r)
{
    const int lane = threadIdx.x & (kWaveSize - 1);
    const uint32_t expert = blockIdx.x * kRouterWavesPerBlock + (threadIdx.x >> 6);
    if (expert > r.experts)
        return;
    const uint32_t non_finite = r.error_words[0];
    const uint32_t first_bad = r.error_words[1];
    uint32_t status = NCNN_MOE_ROUTER_OK;
    if (non_finite != 0u)
        status = NCNN_MOE_ROUTER_NON_FINITE_LOGIT;
    else if (first_bad != 0xffffffffu)
        status = first_bad & 7u;
    uint32_t before = 0;
    for (uint32_t e = lane; e < expert; e += kWaveSize)
        before += r.expert_counts[e];
#pragma unroll
    for (int step = 1; step < kWaveSize; step <<= 1)
        before += __shfl_xor(before, step, kWaveSize);
    if (expert == r.experts)
    {
        // the extra wave writes the end of the last group and the status
        if (lane == 0)
        {
            r.expert_offsets[r.experts] = status == NCNN_MOE_ROUTER_OK ? before : 0u;
            *r.status = status;
        }
        return;
    }
    if (lane == 0)
        r.expert_offsets[expert] = status == NCNN_MOE_ROUTER_OK ? before : 0u;
    if (status != NCNN_MOE_ROUTER_OK)
        return;
    const uint32_t assignments = r.tokens * r.top_k;
    uint32_t written = before;
    for (uint32_t first = 0; first < assignments; first += 4u * kWaveSize)
    {
        uint32_t named[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
        {
            const uint32_t i = first + static_cast<uint32_t>(k * kWaveSize + lane);
            named[k] = i < assignments ? r.selected_experts[i] : 0xffffffffu;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
        {
            const uint32_t i = first + static_cast<uint32_t>(k * kWaveSize + lane);
            const bool mine = named[k] == expert;
            const uint64_t matches = __ballot(mine);
            if (mine)
            {
                ncnn_moe_expert_route route;
                route.token_index = i / r.top_k;
                route.rank = i - route.token_index * r.top_k;
                route.weight = r.selected_weights[i];
                r.routes[written + static_cast<uint32_t>(lanes_below(matches))] = route;
            }
            written += static_cast<uint32_t>(__popcll(matches));
        }
    }
}

__global__ void router_clear_kernel(uint32_t* expert_counts, uint32_t experts, uint32_t* error_words)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < experts)
        expert_counts[i] = 0u;
    if (i == 0)
    {
        error_words[0] = 0u;
        error_words[1] = 0xffffffffu;
    }
}

__global__ void log1pf_probe_kernel(const float* in, float* out, size_t n)
{
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n)
        out[i] = log1pf_libm_positive(in[i]);
}

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_ROUTER_KERNELS_H
