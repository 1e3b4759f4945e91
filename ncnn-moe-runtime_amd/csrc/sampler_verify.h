// Speculative verification (src/engine/session.cpp:776-874): the accept loop over the drafted
// tokens and the draw of the token that follows them, from the filtered distributions that the
// sampling kernels exported for the target and draft rows.  One wave.
#ifndef NCNN_MOE_HIP_SAMPLER_VERIFY_H
#define NCNN_MOE_HIP_SAMPLER_VERIFY_H

#include "sampler_common.h"

namespace ncnn_moe_hip {

struct VerifyArgs
{
    uint32_t draft_count;
    float temperature;
    const ncnn_moe_sample_result* row_results; // [2 * draft_count + 1]: target rows, then draft rows
    const int32_t* distribution_ids;           // [rows][distribution_cap], cap <= 64
    const float* distribution_probabilities;
    const uint32_t* distribution_count;        // [rows]
    uint32_t distribution_cap;
    const int32_t* proposed;                   // [draft_count]
    const float* uniforms;                     // [draft_count + 1]
    float* accepted_probabilities;             // [draft_count]
    ncnn_moe_verify_result* result;
};

struct VerifyShared
{
    float residual[kWaveSize];
    int32_t token[kWaveSize];
};

// candidate_probability (src/engine/session.cpp:138-148): the probability the row's filtered
// distribution gives `token`, 0 when it is not a candidate.  Lane l holds candidate l of the row.
__device__ __forceinline__ float candidate_probability_wave(int32_t candidate_id, float probability, bool valid, int32_t token)
{
    const uint64_t match = __ballot(valid && candidate_id == token);
    if (match == 0)
        return 0.0f;
    return read_lane(probability, __builtin_ctzll(match));
}

__device__ __forceinline__ void write_verify_result(
    const VerifyArgs& v, uint32_t accepted, int32_t token, float probability, uint32_t status, uint32_t row_status,
    uint32_t accept_draws, uint32_t final_draw, uint32_t residual)
{
    ncnn_moe_verify_result r;
    r.accepted = accepted;
    r.next_token_id = status == NCNN_MOE_VERIFY_OK ? token : -1;
    r.next_probability = status == NCNN_MOE_VERIFY_OK ? probability : 0.0f;
    r.status = status;
    r.row_status = row_status;
    r.accept_draws = accept_draws;
    r.final_draw_consumed = final_draw;
    r.next_is_residual = residual;
    *v.result = r;
}

__global__ __launch_bounds__(kWaveSize) void speculative_verify_kernel(VerifyArgs v)
{
    __shared__ VerifyShared shared;
    const int lane = threadIdx.x;
    const uint32_t drafts = v.draft_count;
    uint32_t accepted = 0;
    uint32_t accept_draws = 0;

    if (v.temperature == 0.0f)
    {
        // ---- greedy (session.cpp:778-796): a drafted token stands while it is the target's own choice
        for (; accepted < drafts; ++accepted)
        {
            const ncnn_moe_sample_result target = v.row_results[accepted];
            if (target.status != NCNN_MOE_ROW_OK)
            {
                if (lane == 0)
                    write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_ROW_ERROR, target.status, 0, 0, 0);
                return;
            }
            if (target.token_id != v.proposed[accepted])
                break;
            if (lane == 0)
                v.accepted_probabilities[accepted] = 1.0f;
        }
    }
    else
    {
        // ---- session.cpp:797-842: accept with probability min(1, target / draft)
        for (; accepted < drafts; ++accepted)
        {
            const uint32_t target_row = accepted;
            const uint32_t draft_row = drafts + 1u + accepted;
            const ncnn_moe_sample_result target = v.row_results[target_row];
            const ncnn_moe_sample_result draft = v.row_results[draft_row];
            if (target.status != NCNN_MOE_ROW_OK || draft.status != NCNN_MOE_ROW_OK)
            {
                const uint32_t row_status = target.status != NCNN_MOE_ROW_OK ? target.status : draft.status;
                if (lane == 0)
                    write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_ROW_ERROR, row_status, accept_draws, 0, 0);
                return;
            }
            const int32_t token = v.proposed[accepted];
            const uint32_t target_count = min(v.distribution_count[target_row], v.distribution_cap);
            const uint32_t draft_count = min(v.distribution_count[draft_row], v.distribution_cap);
            const bool target_valid = static_cast<uint32_t>(lane) < target_count;
            const bool draft_valid = static_cast<uint32_t>(lane) < draft_count;
            const int32_t target_id = target_valid ? v.distribution_ids[target_row * v.distribution_cap + lane] : -1;
            const float target_p = target_valid ? v.distribution_probabilities[target_row * v.distribution_cap + lane] : 0.0f;
            const int32_t draft_id = draft_valid ? v.distribution_ids[draft_row * v.distribution_cap + lane] : -1;
            const float draft_p = draft_valid ? v.distribution_probabilities[draft_row * v.distribution_cap + lane] : 0.0f;
            const float target_probability = candidate_probability_wave(target_id, target_p, target_valid, token);
            const float draft_probability = candidate_probability_wave(draft_id, draft_p, draft_valid, token);
            if (draft_probability <= 0.0f)
            {
                if (lane == 0)
                    write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_ZERO_DRAFT_PROBABILITY, 0, accept_draws, 0, 0);
                return;
            }
            const float ratio = target_probability / draft_probability;
            const float acceptance = ratio < 1.0f ? ratio : 1.0f; // std::min(1.0f, ratio)
            const float uniform = v.uniforms[accept_draws];
            ++accept_draws;
            if (uniform >= acceptance)
            {
                // ---- rejected: sample_residual_distribution (session.cpp:150-202) over
                // max(0, target - draft), summed and walked in token-id order
                float residual = target_p;
                for (uint32_t j = 0; j < draft_count; ++j)
                {
                    const int32_t other_id = read_lane(draft_id, static_cast<int>(j));
                    const float other_p = read_lane(draft_p, static_cast<int>(j));
                    if (target_valid && other_id == target_id)
                    {
                        const float difference = residual - other_p;
                        residual = 0.0f < difference ? difference : 0.0f; // std::max(0.0f, difference)
                    }
                }
                int rank = 0;
                for (uint32_t j = 0; j < target_count; ++j)
                    rank += read_lane(target_id, static_cast<int>(j)) < target_id ? 1 : 0;
                if (target_valid)
                {
                    shared.residual[rank] = residual;
                    shared.token[rank] = target_id;
                }
                __syncthreads();
                const float ordered_residual = target_valid ? shared.residual[lane] : 0.0f;
                const int32_t ordered_token = target_valid ? shared.token[lane] : -1;
                float normalizer = 0.0f; // std::accumulate over the dense vector: zeros leave the sum as it is
                for (uint32_t j = 0; j < target_count; ++j)
                    normalizer += read_lane(ordered_residual, static_cast<int>(j));
                if (!is_finite_f32(normalizer) || !(normalizer > 0.0f))
                {
                    if (lane == 0)
                        write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_RESIDUAL_EMPTY, 0, accept_draws, 0, 1);
                    return;
                }
                // uniform_real_distribution<float>(0, normalizer): canonical draw times the range
                const float sample_value = v.uniforms[accept_draws] * normalizer;
                float cumulative = 0.0f;
                int selected = -1;
                for (uint32_t j = 0; j < target_count; ++j)
                {
                    cumulative += read_lane(ordered_residual, static_cast<int>(j));
                    if (sample_value < cumulative)
                    {
                        selected = static_cast<int>(j);
                        break;
                    }
                }
                if (selected < 0)
                {
                    // session.cpp:189-198: the last token that has any residual mass
                    const uint64_t positive = __ballot(target_valid && ordered_residual > 0.0f);
                    if (positive != 0)
                        selected = 63 - __builtin_clzll(positive);
                }
                if (selected < 0)
                {
                    if (lane == 0)
                        write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_RESIDUAL_FAILED, 0, accept_draws, 1, 1);
                    return;
                }
                const float chosen_residual = read_lane(ordered_residual, selected);
                const int32_t chosen_token = read_lane(ordered_token, selected);
                if (lane == 0)
                    write_verify_result(v, accepted, chosen_token, chosen_residual / normalizer, NCNN_MOE_VERIFY_OK, 0,
                                        accept_draws, 1, 1);
                return;
            }
            if (lane == 0)
                v.accepted_probabilities[accepted] = target_probability;
        }
    }

    // ---- session.cpp:871-873: the target's own sample at the first position that was not accepted
    // (greedy mismatch) or after the last drafted token (everything accepted)
    const ncnn_moe_sample_result next = v.row_results[accepted];
    if (lane == 0)
    {
        if (next.status != NCNN_MOE_ROW_OK)
            write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_ROW_ERROR, next.status, accept_draws, 0, 0);
        else
            write_verify_result(v, accepted, next.token_id, next.probability, NCNN_MOE_VERIFY_OK, 0, accept_draws,
                                next.draw_consumed, 0);
    }
}

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_SAMPLER_VERIFY_H
