// Expert router kernels (src/graph/expert_dispatcher.cpp:12-157 of the runtime, on the device):
//   router_select_kernel  one wave per token: scores, Top-K routes, normalised weights
//   router_group_kernel   one workgroup per 256 tokens: their routes to their places in the plan
#ifndef NCNN_MOE_HIP_ROUTER_KERNELS_H
#define NCNN_MOE_HIP_ROUTER_KERNELS_H

#include "ncnn_moe_hip_router.h"
#include "sampler_device.h"

namespace ncnn_moe_hip {

constexpr int kRouterWavesPerBlock = 8;
constexpr int kRouterThreads = kRouterWavesPerBlock * kWaveSize;
constexpr int kRouterChunkTokens = 256; // tokens whose routes one workgroup of the grouping kernel places

// log1pf bit-identical to glibc 2.35's (sysdeps/ieee754/flt-32/s_log1pf.c) for finite x > 0, which is
// all stable_softplus hands it (an exponential).  Plain fp32 operations in the library's order; built
// without contraction, so every one rounds once.  Compared with libm on every positive float.
__device__ __forceinline__ float log1pf_libm_positive(float x)
{
    const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f;
    const float Lp1 = 6.6666668653e-01f, Lp2 = 4.0000000596e-01f, Lp3 = 2.8571429849e-01f, Lp4 = 2.2222198546e-01f,
                Lp5 = 1.8183572590e-01f, Lp6 = 1.5313838422e-01f, Lp7 = 1.4798198640e-01f;
    const int32_t hx = static_cast<int32_t>(__float_as_uint(x));
    if (hx < 0x31000000) // x < 2^-29
    {
        if (hx < 0x24800000) // x < 2^-54
            return x;
        return x - x * x * 0.5f;
    }
    if (hx >= 0x7f800000)
        return x + x;
    // The library's three range cases (x < 0.41422: no reduction; x < 2^53: reduce 1 + x and keep the
    // rounding error of the sum as a correction; above: reduce x itself) as selects, so that lanes in
    // different ranges share one instruction stream.
    const bool direct = hx < 0x3ed413d7;
    const bool huge = hx >= 0x5a000000;
    float u = huge ? x : 1.0f + x;
    int32_t hu = static_cast<int32_t>(__float_as_uint(u));
    int32_t k = (hu >> 23) - 127;
    float c = (k > 0) ? 1.0f - (u - x) : x - (u - 1.0f); // correction term
    c = huge ? 0.0f : c / u;
    hu &= 0x007fffff;
    const bool low_half = hu < 0x3504f7;
    u = __uint_as_float(static_cast<uint32_t>(hu) | (low_half ? 0x3f800000u : 0x3f000000u)); // u, or u / 2
    k = low_half ? k : k + 1;
    hu = low_half ? hu : (0x00800000 - hu) >> 2;
    float f = u - 1.0f;
    k = direct ? 0 : k;
    f = direct ? x : f;
    hu = direct ? 1 : hu;
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
    const float near = f - (hfsq - s * (hfsq + R));
    const float far = kf * ln2_hi - ((hfsq - (s * (hfsq + R) + (kf * ln2_lo + c))) - f);
    return k == 0 ? near : far;
}

// Wave-wide reductions through the data-parallel primitives: four exchanges inside each row of 16
// lanes (lane pairs at distance 1 and 2, then the two mirrors), then the four rows through scalar reads.
template <int CONTROL>
__device__ __forceinline__ int dpp_move(int value)
{
    return __builtin_amdgcn_mov_dpp(value, CONTROL, 0xf, 0xf, true);
}

constexpr int kDppSwapPairs = 0xB1;   // quad_perm:[1,0,3,2]
constexpr int kDppSwapHalves = 0x4E;  // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // row_half_mirror
constexpr int kDppMirror = 0x140;     // row_mirror

__device__ __forceinline__ float wave_max(float value)
{
    value = fmaxf(value, __int_as_float(dpp_move<kDppSwapPairs>(__float_as_int(value))));
    value = fmaxf(value, __int_as_float(dpp_move<kDppSwapHalves>(__float_as_int(value))));
    value = fmaxf(value, __int_as_float(dpp_move<kDppHalfMirror>(__float_as_int(value))));
    value = fmaxf(value, __int_as_float(dpp_move<kDppMirror>(__float_as_int(value))));
    return fmaxf(fmaxf(read_lane(value, 0), read_lane(value, 16)), fmaxf(read_lane(value, 32), read_lane(value, 48)));
}

__device__ __forceinline__ int wave_min(int value)
{
    value = min(value, dpp_move<kDppSwapPairs>(value));
    value = min(value, dpp_move<kDppSwapHalves>(value));
    value = min(value, dpp_move<kDppHalfMirror>(value));
    value = min(value, dpp_move<kDppMirror>(value));
    return min(min(read_lane(value, 0), read_lane(value, 16)), min(read_lane(value, 32), read_lane(value, 48)));
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
    uint32_t* chunk_counts;       // [chunks][experts] assignments per chunk of 256 tokens and expert, zero at launch
    uint32_t* error_words;        // [0]: non-finite logit seen, [1]: min over failing tokens of (token << 3 | status), ~0 if none
    uint32_t* finished_chunks;    // workgroups of the grouping kernel that are done, zero at launch
    uint32_t* finished_selects;   // workgroups of the fused select kernel that are done, zero at launch
    uint32_t* expert_offsets;     // [experts + 1]
    ncnn_moe_expert_route* routes; // [tokens * top_k]
    uint32_t* status;             // the call's ncnn_moe_router_status
};

struct RouterShared
{
    float scores[kRouterWavesPerBlock][NCNN_MOE_ROUTER_MAX_EXPERTS]; // a token's scores: for the caller-named experts, or staged
    uint32_t non_finite[kRouterWavesPerBlock];                       // staged scoring: the token holds a non-finite logit
    float staged_maximum[kRouterWavesPerBlock];                      // staged softmax: the waves' maxima
};

// Decode-sized calls (STAGED): a workgroup takes kStagedTokensPerBlock tokens instead of one per wave
// and all its threads compute the scores, one or a few experts each, into LDS; a wave per token then
// selects from there.  The scores of a token (exp, log1p, sqrt per expert) are two fifths of a lone
// wave's time for it; spread over four waves they take a quarter as long.  (The softmax sum is the CPU's
// loop, one addition at a time in expert order, and stays with the selecting wave.)
constexpr int kStagedTokensPerBlock = 2;
constexpr int kStagedThreadsPerToken = kRouterThreads / kStagedTokensPerBlock;

__device__ __forceinline__ float router_score_of_logit(float logit, uint32_t score_function);

__device__ __forceinline__ void stage_token_scores(const RouterArgs& r, RouterShared& shared, uint32_t first_token)
{
    const int slot = threadIdx.x / kStagedThreadsPerToken;
    const int member = threadIdx.x % kStagedThreadsPerToken;
    const uint32_t token = first_token + static_cast<uint32_t>(slot);
    if (threadIdx.x < kStagedTokensPerBlock)
        shared.non_finite[threadIdx.x] = 0u;
    __syncthreads();
    constexpr int kPerThread = NCNN_MOE_ROUTER_MAX_EXPERTS / kStagedThreadsPerToken;
    float logit[kPerThread];
    bool finite = true;
    float maximum = -__builtin_inff();
    const float* logits = r.logits + static_cast<size_t>(token < r.tokens ? token : 0u) * r.experts;
#pragma unroll
    for (int k = 0; k < kPerThread; ++k)
    {
        const uint32_t e = static_cast<uint32_t>(k * kStagedThreadsPerToken + member);
        logit[k] = (token < r.tokens && e < r.experts) ? logits[e] : -__builtin_inff();
        finite = finite && (e >= r.experts || is_finite_f32(logit[k]));
        maximum = fmaxf(maximum, logit[k]);
    }
    if (token < r.tokens && !finite)
        shared.non_finite[slot] = 1u;
    if (r.score_function == NCNN_MOE_ROUTER_SOFTMAX)
    {
        // the row maximum first (src/graph/expert_dispatcher.cpp:44-46); the sum stays with the selecting wave
        maximum = wave_max(maximum);
        if ((threadIdx.x & (kWaveSize - 1)) == 0)
            shared.staged_maximum[threadIdx.x >> 6] = maximum;
        __syncthreads();
        constexpr int kWavesPerToken = kStagedThreadsPerToken / kWaveSize;
        maximum = shared.staged_maximum[slot * kWavesPerToken];
#pragma unroll
        for (int w = 1; w < kWavesPerToken; ++w)
            maximum = fmaxf(maximum, shared.staged_maximum[slot * kWavesPerToken + w]);
    }
#pragma unroll
    for (int k = 0; k < kPerThread; ++k)
    {
        const uint32_t e = static_cast<uint32_t>(k * kStagedThreadsPerToken + member);
        if (token < r.tokens && e < r.experts)
            shared.scores[slot][e] = r.score_function == NCNN_MOE_ROUTER_SOFTMAX ? expf_libm(logit[k] - maximum)
                                                                                : router_score_of_logit(logit[k], r.score_function);
    }
    __syncthreads();
}

// One wave per token.  Expert e lives in slot e / 64 of lane e % 64, so a loop over slots, then lanes,
// visits the experts in index order: the softmax sum is the CPU loop itself, one fp32 addition at a
// time.  The routes are chosen one per round and stay in registers: lane r keeps the route of rank r.
template <int SLOTS, bool COUNT_CHUNKS, bool STAGED>
__device__ __forceinline__ void select_token_routes(const RouterArgs& r, RouterShared& shared, uint32_t token, int lane, int wave)
{
    const int experts = static_cast<int>(r.experts);
    const int top_k = static_cast<int>(r.top_k);
    const float* logits = r.logits + static_cast<size_t>(token) * r.experts;
    const bool explicit_routes = r.explicit_ids != nullptr;

    // every load of the token up front
    float logit[SLOTS];
    float bias[SLOTS];
#pragma unroll
    for (int s = 0; s < SLOTS; ++s)
    {
        const int e = s * kWaveSize + lane;
        logit[s] = (e < experts && !STAGED) ? logits[e] : 0.0f;
        bias[s] = (e < experts && r.selection_bias != nullptr && !explicit_routes) ? r.selection_bias[e] : 0.0f;
    }
    uint32_t my_expert = (explicit_routes && lane < top_k) ? r.explicit_ids[static_cast<size_t>(token) * r.top_k + lane] : 0u;

    bool finite = true;
    float maximum = -__builtin_inff();
#pragma unroll
    for (int s = 0; s < SLOTS; ++s)
    {
        const int e = s * kWaveSize + lane;
        if (e < experts)
        {
            finite = finite && is_finite_f32(logit[s]);
            maximum = fmaxf(maximum, logit[s]);
        }
    }
    if (STAGED ? shared.non_finite[wave] != 0u : __ballot(!finite) != 0)
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
        maximum = wave_max(maximum);
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
        {
            if constexpr (STAGED)
                score[s] = (s * kWaveSize + lane) < experts ? shared.scores[wave][s * kWaveSize + lane] : 0.0f;
            else
                score[s] = (s * kWaveSize + lane) < experts ? expf_libm(logit[s] - maximum) : 0.0f;
        }
        float sum = 0.0f;
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
        {
            // in trips of eight (a loop trip of a lone wave costs as much as a dozen additions); the
            // lanes past the last expert hold 0, which leaves the sum as it is
            const int slot_count = min(kWaveSize, experts - s * kWaveSize);
            for (int trip = 0; trip * 8 < slot_count; ++trip)
            {
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    sum += read_lane(score[s], trip * 8 + k);
            }
        }
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
            score[s] = score[s] / sum;
    }
    else if constexpr (STAGED)
    {
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
            score[s] = (s * kWaveSize + lane) < experts ? shared.scores[wave][s * kWaveSize + lane] : 0.0f;
    }
    else
    {
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
            score[s] = (s * kWaveSize + lane) < experts ? router_score_of_logit(logit[s], r.score_function) : 0.0f;
    }

    float my_score = 0.0f;
    float selected_sum = 0.0f;
    if (explicit_routes)
    {
        // src/graph/expert_dispatcher.cpp:124-135: the caller names the experts; rank = position
        const bool in_range = lane >= top_k || my_expert < r.experts;
        if (__ballot(!in_range) != 0)
        {
            if (lane == 0)
                atomicMin(&r.error_words[1], (token << 3) | NCNN_MOE_ROUTER_EXPERT_OUT_OF_RANGE);
            return;
        }
        // (staged scores are in LDS already, but a softmax row only before its division by the sum)
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
        {
            const int e = s * kWaveSize + lane;
            if (e < experts)
                shared.scores[wave][e] = score[s];
        }
        __builtin_amdgcn_s_waitcnt(0xc07f); // this wave's LDS writes, before its lanes read them back
        __builtin_amdgcn_wave_barrier();
        if (lane < top_k)
            my_score = shared.scores[wave][my_expert];
        for (int rank = 0; rank < top_k; ++rank)
            selected_sum += read_lane(my_score, rank);
    }
    else
    {
        // ---- select_topk_routes (src/graph/expert_dispatcher.cpp:61-77): the best top_k by
        // (score + bias descending, expert id ascending), one per round; the selected scores are
        // summed in rank order (src/graph/expert_dispatcher.cpp:137-143)
        float keyed[SLOTS];
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
            keyed[s] = score[s] + bias[s];
        uint32_t taken = 0; // this lane's slots already selected
        for (int round = 0; round < top_k; ++round)
        {
            // this lane's best remaining expert: the lowest slot (lowest id) among equals
            float lane_best = -__builtin_inff();
            float lane_score = 0.0f;
            int lane_expert = 0x7fffffff; // none
#pragma unroll
            for (int s = 0; s < SLOTS; ++s)
            {
                const int e = s * kWaveSize + lane;
                const bool available = e < experts && ((taken >> s) & 1u) == 0u;
                if (available && (lane_expert == 0x7fffffff || keyed[s] > lane_best))
                {
                    lane_best = keyed[s];
                    lane_score = score[s];
                    lane_expert = e;
                }
            }
            const float best = wave_max(lane_best);
            int winner = wave_min((lane_expert != 0x7fffffff && lane_best == best) ? lane_expert : 0x7fffffff);
            if (winner == 0x7fffffff) // selection scores that compare unordered: any remaining expert
                winner = wave_min(lane_expert);
            const int winner_lane = winner & (kWaveSize - 1);
            const float winner_score = read_lane(lane_score, winner_lane);
            if (lane == winner_lane)
                taken |= 1u << (winner >> 6);
            selected_sum += winner_score;
            if (lane == round)
            {
                my_expert = static_cast<uint32_t>(winner);
                my_score = winner_score;
            }
        }
    }

    // ---- src/graph/expert_dispatcher.cpp:144-150
    if (r.renormalize != 0u && selected_sum <= 0.0f)
    {
        if (lane == 0)
            atomicMin(&r.error_words[1], (token << 3) | NCNN_MOE_ROUTER_NON_POSITIVE_SUM);
        return;
    }
    if (lane < top_k)
    {
        const float weight = (r.renormalize != 0u ? my_score / selected_sum : my_score) * r.scaling;
        // written through the per-XCD L2: the workgroup that groups the routes may sit on another XCD
        store_agent(&r.selected_experts[static_cast<size_t>(token) * r.top_k + lane], my_expert);
        store_agent(reinterpret_cast<uint32_t*>(&r.selected_weights[static_cast<size_t>(token) * r.top_k + lane]), __float_as_uint(weight));
        if (COUNT_CHUNKS) // a call of one chunk is counted by the workgroup that groups it
            atomicAdd(&r.chunk_counts[static_cast<size_t>(token / kRouterChunkTokens) * r.experts + my_expert], 1u);
    }
}

// Grouping is a stable counting sort of the flat assignment array (token-major, so already in
// (token, rank) order) by expert id.  The select kernel counts assignments per (chunk of 256 tokens,
// expert); one workgroup per chunk then places its chunk's routes:
//   position = routes of lower experts (all chunks) + this expert's routes in earlier chunks
//              + this expert's routes earlier in the chunk.
// The last workgroup to finish returns the scratch counters to zero for the next call.
struct GroupShared
{
    uint32_t wave_base[kRouterWavesPerBlock][NCNN_MOE_ROUTER_MAX_EXPERTS];
    uint32_t wave_totals[kRouterWavesPerBlock];
    uint32_t is_last;
};

constexpr int kGroupExpertsPerThread = NCNN_MOE_ROUTER_MAX_EXPERTS / kRouterThreads; // experts one thread owns, at most
constexpr int kGroupBatch = 8;                                                       // loads in flight per lane

__device__ __forceinline__ void place_chunk_routes(const RouterArgs& r, GroupShared& shared, uint32_t chunk, uint32_t chunks)
{
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    const uint32_t experts = r.experts;

    // this wave's tokens of the chunk: consecutive ones, an equal share of the chunk's (a short chunk is
    // spread over all waves: placing is sequential inside a wave); the first loads go out before anything waits
    const uint32_t chunk_first = chunk * kRouterChunkTokens;
    const uint32_t chunk_tokens = min(static_cast<uint32_t>(kRouterChunkTokens), r.tokens - chunk_first);
    const uint32_t share = (chunk_tokens + kRouterWavesPerBlock - 1) / kRouterWavesPerBlock;
    const uint32_t wave_first = static_cast<uint32_t>(wave) * share;
    const uint32_t first_token = chunk_first + wave_first;
    const uint32_t wave_tokens = wave_first < chunk_tokens ? min(share, chunk_tokens - wave_first) : 0u;
    const uint32_t first_assignment = first_token * r.top_k;
    const uint32_t count = wave_tokens * r.top_k;
    uint32_t first_named[kGroupBatch];
    float first_weight[kGroupBatch];
#pragma unroll
    for (int k = 0; k < kGroupBatch; ++k)
    {
        const uint32_t i = static_cast<uint32_t>(k * kWaveSize + lane);
        first_named[k] = i < count ? load_agent(&r.selected_experts[first_assignment + i]) : 0xffffffffu;
        first_weight[k] = i < count ? __uint_as_float(load_agent(reinterpret_cast<const uint32_t*>(&r.selected_weights[first_assignment + i]))) : 0.0f;
    }
    const uint32_t non_finite = load_agent(&r.error_words[0]);
    const uint32_t first_bad = load_agent(&r.error_words[1]);
    uint32_t status = NCNN_MOE_ROUTER_OK;
    if (non_finite != 0u)
        status = NCNN_MOE_ROUTER_NON_FINITE_LOGIT;
    else if (first_bad != 0xffffffffu)
        status = first_bad & 7u;
    if (chunk == 0 && tid == 0)
        *r.status = status;

    if (status != NCNN_MOE_ROUTER_OK)
    {
        if (chunk == 0)
        {
            for (uint32_t e = tid; e <= experts; e += kRouterThreads)
                r.expert_offsets[e] = 0u;
        }
    }
    else
    {
        // ---- a histogram of the experts of this wave's tokens
        const auto build_histogram = [&]() {
            for (uint32_t e = lane; e < experts; e += kWaveSize)
                shared.wave_base[wave][e] = 0u;
            lds_barrier();
            for (uint32_t first = 0; first < count; first += kGroupBatch * kWaveSize)
            {
                uint32_t named[kGroupBatch];
#pragma unroll
                for (int k = 0; k < kGroupBatch; ++k)
                {
                    const uint32_t i = first + static_cast<uint32_t>(k * kWaveSize + lane);
                    named[k] = first_named[k];
                    if (first != 0u)
                        named[k] = i < count ? load_agent(&r.selected_experts[first_assignment + i]) : 0xffffffffu;
                }
#pragma unroll
                for (int k = 0; k < kGroupBatch; ++k)
                {
                    if (named[k] != 0xffffffffu)
                        atomicAdd(&shared.wave_base[wave][named[k]], 1u);
                }
            }
            __syncthreads();
        };
        // ---- this thread's experts: their routes in all chunks, and in the chunks before this one.
        // A call of one chunk has no chunk counters: the totals are the sums of the waves' histograms.
        const uint32_t per_thread = (experts + kRouterThreads - 1) / kRouterThreads;
        uint32_t total[kGroupExpertsPerThread];
        uint32_t before[kGroupExpertsPerThread];
#pragma unroll
        for (int j = 0; j < kGroupExpertsPerThread; ++j)
        {
            total[j] = 0u;
            before[j] = 0u;
        }
        if (chunks == 1u)
        {
            build_histogram();
#pragma unroll
            for (int j = 0; j < kGroupExpertsPerThread; ++j)
            {
                const uint32_t e = tid * per_thread + j;
                if (static_cast<uint32_t>(j) < per_thread && e < experts)
                {
#pragma unroll
                    for (int w = 0; w < kRouterWavesPerBlock; ++w)
                        total[j] += shared.wave_base[w][e];
                }
            }
        }
        else
        {
#pragma unroll 8
            for (uint32_t c = 0; c < chunks; ++c)
            {
#pragma unroll
                for (int j = 0; j < kGroupExpertsPerThread; ++j)
                {
                    const uint32_t e = tid * per_thread + j;
                    const uint32_t routed = (static_cast<uint32_t>(j) < per_thread && e < experts) ? load_agent(&r.chunk_counts[c * experts + e]) : 0u;
                    total[j] += routed;
                    before[j] += c < chunk ? routed : 0u;
                }
            }
        }
        uint32_t thread_sum = 0u;
#pragma unroll
        for (int j = 0; j < kGroupExpertsPerThread; ++j)
            thread_sum += total[j];
        uint32_t inclusive = thread_sum;
#pragma unroll
        for (int step = 1; step < kWaveSize; step <<= 1)
        {
            const uint32_t other = __shfl_up(inclusive, step, kWaveSize);
            inclusive += lane >= step ? other : 0u;
        }
        if (lane == kWaveSize - 1)
            shared.wave_totals[wave] = inclusive;
        if (chunks == 1u)
            __syncthreads();
        else
            build_histogram();
        uint32_t exclusive = inclusive - thread_sum;
        for (int w = 0; w < wave; ++w)
            exclusive += shared.wave_totals[w];
        // ---- first position of each of this thread's experts for each wave of this chunk
#pragma unroll
        for (int j = 0; j < kGroupExpertsPerThread; ++j)
        {
            const uint32_t e = tid * per_thread + j;
            if (static_cast<uint32_t>(j) < per_thread && e < experts)
            {
                if (chunk == 0)
                    r.expert_offsets[e] = exclusive;
                uint32_t running = exclusive + before[j];
#pragma unroll
                for (int w = 0; w < kRouterWavesPerBlock; ++w)
                {
                    const uint32_t here = shared.wave_base[w][e];
                    shared.wave_base[w][e] = running;
                    running += here;
                }
            }
            exclusive += total[j];
        }
        if (chunk == 0 && tid == 0)
            r.expert_offsets[experts] = r.tokens * r.top_k;
        __syncthreads();

        // ---- place the wave's routes, 64 at a time in assignment order
        const int bits = 32 - __clz(static_cast<int>(experts - 1u) | 1);
        for (uint32_t first = 0; first < count; first += kGroupBatch * kWaveSize)
        {
            uint32_t named[kGroupBatch];
            float weight[kGroupBatch];
#pragma unroll
            for (int k = 0; k < kGroupBatch; ++k)
            {
                const uint32_t i = first + static_cast<uint32_t>(k * kWaveSize + lane);
                named[k] = first_named[k];
                weight[k] = first_weight[k];
                if (first != 0u)
                {
                    named[k] = i < count ? load_agent(&r.selected_experts[first_assignment + i]) : 0xffffffffu;
                    weight[k] = i < count ? __uint_as_float(load_agent(reinterpret_cast<const uint32_t*>(&r.selected_weights[first_assignment + i]))) : 0.0f;
                }
            }
#pragma unroll
            for (int k = 0; k < kGroupBatch; ++k)
            {
                if (first + static_cast<uint32_t>(k * kWaveSize) >= count)
                    break;
                const bool valid = named[k] != 0xffffffffu;
                uint64_t same = __ballot(valid);
                for (int b = 0; b < bits; ++b)
                {
                    const bool set = ((named[k] >> b) & 1u) != 0u;
                    const uint64_t vote = __ballot(set);
                    same &= set ? vote : ~vote;
                }
                if (valid)
                {
                    const uint32_t earlier = static_cast<uint32_t>(lanes_below(same));
                    const uint32_t position = shared.wave_base[wave][named[k]] + earlier;
                    if (earlier == 0u)
                        shared.wave_base[wave][named[k]] = position + static_cast<uint32_t>(__popcll(same));
                    const uint32_t i = first_assignment + first + static_cast<uint32_t>(k * kWaveSize + lane);
                    ncnn_moe_expert_route route;
                    route.token_index = i / r.top_k;
                    route.rank = i - route.token_index * r.top_k;
                    route.weight = weight[k];
                    r.routes[position] = route;
                }
                // the group leaders' updates, before this wave's next 64 read them (waves run different
                // numbers of rounds: nothing here may wait for another wave)
                __builtin_amdgcn_s_waitcnt(0xc07f);
                __builtin_amdgcn_wave_barrier();
            }
        }
    }

    // ---- the last workgroup to get here clears the counters for the next call
    __syncthreads();
    if (tid == 0)
    {
        const uint32_t finished =
            chunks == 1u ? 0u : __hip_atomic_fetch_add(r.finished_chunks, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        shared.is_last = finished == chunks - 1u ? 1u : 0u;
    }
    __syncthreads();
    if (shared.is_last != 0u)
    {
        for (uint32_t i = tid; chunks > 1u && i < chunks * experts; i += kRouterThreads)
            r.chunk_counts[i] = 0u;
        if (tid == 0)
        {
            r.error_words[0] = 0u;
            r.error_words[1] = 0xffffffffu;
            *r.finished_chunks = 0u;
        }
    }
}

__global__ __launch_bounds__(kRouterThreads) void router_group_kernel(RouterArgs r)
{
    __shared__ GroupShared shared;
    place_chunk_routes(r, shared, blockIdx.x, gridDim.x);
}

// FUSED (calls of at most one chunk of tokens): the workgroup that finishes last also places the
// routes, so the whole dispatch is one launch.
template <int SLOTS, bool FUSED, bool STAGED>
__global__ __launch_bounds__(kRouterThreads) void router_select_kernel(RouterArgs r)
{
    static_assert(FUSED || !STAGED, "staged scoring serves the single-launch calls");
    __shared__ RouterShared shared;
    const int lane = threadIdx.x & (kWaveSize - 1);
    const int wave = threadIdx.x >> 6;
    constexpr int kTokensPerBlock = STAGED ? kStagedTokensPerBlock : kRouterWavesPerBlock;
    const uint32_t token = blockIdx.x * kTokensPerBlock + wave;
    if constexpr (STAGED)
        stage_token_scores(r, shared, blockIdx.x * kTokensPerBlock);
    if (wave < kTokensPerBlock && token < r.tokens)
        select_token_routes<SLOTS, !FUSED, STAGED>(r, shared, token, lane, wave);
    if constexpr (FUSED)
    {
        __shared__ GroupShared group_shared;
        // this workgroup's routes (written through), counts and error words (atomics) have landed once
        // its waves have waited for them; then the workgroup is counted, and whoever counts last reads
        // every other workgroup's around its own L2: no cache write-back or invalidate is needed
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (threadIdx.x == 0)
        {
            const uint32_t finished = __hip_atomic_fetch_add(r.finished_selects, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            group_shared.is_last = finished == gridDim.x - 1u ? 1u : 0u;
        }
        __syncthreads();
        if (group_shared.is_last == 0u)
            return;
        if (threadIdx.x == 0)
            *r.finished_selects = 0u;
        __syncthreads(); // is_last is read by all before place_chunk_routes writes it again
        place_chunk_routes(r, group_shared, 0u, 1u);
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
