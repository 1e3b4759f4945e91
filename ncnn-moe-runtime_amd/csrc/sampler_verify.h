// Speculative verification (src/engine/session.cpp:776-874): the accept loop over the drafted
// tokens and the draw of the token that follows them, from the filtered distributions that the
// sampling kernels exported for the target and draft rows.  One workgroup.
#ifndef NCNN_MOE_HIP_SAMPLER_VERIFY_H
#define NCNN_MOE_HIP_SAMPLER_VERIFY_H

#include "sampler_common.h"
#include "sampler_exact_sum.h"

namespace ncnn_moe_hip {

constexpr int kVerifyThreads = 512;
static_assert(kSumThreads <= kVerifyThreads, "the exact running sums need kSumThreads threads of the workgroup that calls them");
constexpr int kVerifyCap = kSelectTopK; // candidates of a row's filtered distribution the step can use
constexpr int kVerifySlots = kVerifyCap / kWaveSize;

struct VerifyArgs
{
    uint32_t draft_count;
    float temperature;
    const ncnn_moe_sample_result* row_results; // [2 * draft_count + 1]: target rows, then draft rows
    const int32_t* distribution_ids;           // [rows][kVerifyCap]
    const float* distribution_probabilities;
    const uint32_t* distribution_count;        // [rows]: the full kept length, which may exceed kVerifyCap
    const int32_t* proposed;                   // [draft_count]
    const float* uniforms;                     // [draft_count + 1]
    float* accepted_probabilities;             // [draft_count]
    ncnn_moe_verify_result* result;
};

struct VerifyShared
{
    int32_t target_ids[kVerifyCap];
    float target_probabilities[kVerifyCap];
    int32_t draft_ids[kVerifyCap];
    float draft_probabilities[kVerifyCap];
    float ordered_residual[kVerifyCap]; // the residual in token-id order
    int32_t ordered_token[kVerifyCap];
    float found[2];                     // candidate_probability of the proposed token: target, draft
    // the step's small operands, fetched once (proposed tokens and uniforms may lie in host memory)
    ncnn_moe_sample_result row_results[2 * NCNN_MOE_MAX_DRAFT_TOKENS + 1];
    uint32_t counts[2 * NCNN_MOE_MAX_DRAFT_TOKENS + 1];
    int32_t proposed[NCNN_MOE_MAX_DRAFT_TOKENS];
    float uniforms[NCNN_MOE_MAX_DRAFT_TOKENS + 1];
};

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

__global__ __launch_bounds__(kVerifyThreads) void speculative_verify_kernel(VerifyArgs v)
{
    __shared__ VerifyShared shared;
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    const uint32_t drafts = v.draft_count;
    uint32_t accepted = 0;
    uint32_t accept_draws = 0;
    if (static_cast<uint32_t>(tid) < 2u * drafts + 1u)
    {
        shared.row_results[tid] = v.row_results[tid];
        shared.counts[tid] = v.distribution_count[tid];
    }
    if (static_cast<uint32_t>(tid) < drafts)
        shared.proposed[tid] = v.proposed[tid];
    if (static_cast<uint32_t>(tid) <= drafts)
        shared.uniforms[tid] = v.uniforms[tid];
    __syncthreads();

    if (v.temperature == 0.0f)
    {
        // ---- greedy (session.cpp:778-796): a drafted token stands while it is the target's own choice
        for (; accepted < drafts; ++accepted)
        {
            const ncnn_moe_sample_result target = shared.row_results[accepted];
            if (target.status != NCNN_MOE_ROW_OK)
            {
                if (tid == 0)
                    write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_ROW_ERROR, target.status, 0, 0, 0);
                return;
            }
            if (target.token_id != shared.proposed[accepted])
                break;
            if (tid == 0)
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
            const ncnn_moe_sample_result target = shared.row_results[target_row];
            const ncnn_moe_sample_result draft = shared.row_results[draft_row];
            if (target.status != NCNN_MOE_ROW_OK || draft.status != NCNN_MOE_ROW_OK)
            {
                const uint32_t row_status = target.status != NCNN_MOE_ROW_OK ? target.status : draft.status;
                if (tid == 0)
                    write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_ROW_ERROR, row_status, accept_draws, 0, 0);
                return;
            }
            const uint32_t target_count = __builtin_amdgcn_readfirstlane(shared.counts[target_row]);
            const uint32_t draft_count = __builtin_amdgcn_readfirstlane(shared.counts[draft_row]);
            if (target_count > static_cast<uint32_t>(kVerifyCap) || draft_count > static_cast<uint32_t>(kVerifyCap))
            {
                // a filtered distribution longer than the step holds: reported, never approximated
                if (tid == 0)
                    write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_UNSUPPORTED_WINDOW, 0, accept_draws, 0, 0);
                return;
            }
            const int32_t token = shared.proposed[accepted];
            // ---- candidate_probability (session.cpp:138-148) of the proposed token in both lists; the
            // lists go to LDS on the way, for the residual that a rejection needs
            if (tid < 2)
                shared.found[tid] = 0.0f;
            __syncthreads();
            for (uint32_t j = tid; j < target_count; j += kVerifyThreads)
            {
                const int32_t id = v.distribution_ids[static_cast<size_t>(target_row) * kVerifyCap + j];
                const float probability = v.distribution_probabilities[static_cast<size_t>(target_row) * kVerifyCap + j];
                shared.target_ids[j] = id;
                shared.target_probabilities[j] = probability;
                if (id == token)
                    shared.found[0] = probability; // ids are distinct: at most one writer
            }
            for (uint32_t j = tid; j < draft_count; j += kVerifyThreads)
            {
                const int32_t id = v.distribution_ids[static_cast<size_t>(draft_row) * kVerifyCap + j];
                const float probability = v.distribution_probabilities[static_cast<size_t>(draft_row) * kVerifyCap + j];
                shared.draft_ids[j] = id;
                shared.draft_probabilities[j] = probability;
                if (id == token)
                    shared.found[1] = probability;
            }
            __syncthreads();
            const float target_probability = shared.found[0];
            const float draft_probability = shared.found[1];
            if (draft_probability <= 0.0f)
            {
                if (tid == 0)
                    write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_ZERO_DRAFT_PROBABILITY, 0, accept_draws, 0, 0);
                return;
            }
            const float ratio = target_probability / draft_probability;
            const float acceptance = ratio < 1.0f ? ratio : 1.0f; // std::min(1.0f, ratio)
            const float uniform = shared.uniforms[accept_draws];
            ++accept_draws;
            if (uniform >= acceptance)
            {
                // ---- rejected: sample_residual_distribution (session.cpp:150-202) over
                // max(0, target - draft), summed and walked in token-id order
                for (uint32_t j = tid; j < target_count; j += kVerifyThreads)
                {
                    const int32_t id = shared.target_ids[j];
                    float residual = shared.target_probabilities[j];
                    int rank = 0;
                    for (uint32_t q = 0; q < draft_count; ++q)
                    {
                        if (shared.draft_ids[q] == id)
                        {
                            const float difference = residual - shared.draft_probabilities[q];
                            residual = 0.0f < difference ? difference : 0.0f; // std::max(0.0f, difference)
                        }
                    }
                    for (uint32_t q = 0; q < target_count; ++q)
                        rank += shared.target_ids[q] < id ? 1 : 0;
                    shared.ordered_residual[rank] = residual;
                    shared.ordered_token[rank] = id;
                }
                __syncthreads();
                if (wave != 0)
                    return;
                // one wave walks the ordered residual: entry i in slot i / 64 of lane i % 64, one fp32
                // addition per entry in order, as std::accumulate over the dense vector does (zeros
                // leave an fp32 sum as it is)
                const int n = static_cast<int>(target_count);
                float residual[kVerifySlots];
#pragma unroll
                for (int s = 0; s < kVerifySlots; ++s)
                {
                    const int i = s * kWaveSize + lane;
                    residual[s] = i < n ? shared.ordered_residual[i] : 0.0f;
                }
                // the sums run in trips of eight entries (a loop trip of a lone wave costs as much as a
                // dozen additions); an entry past the end holds +0.0, which leaves a sum as it is
                float normalizer = 0.0f;
#pragma unroll
                for (int s = 0; s < kVerifySlots; ++s)
                {
                    const int slot_count = min(kWaveSize, n - s * kWaveSize);
                    for (int trip = 0; trip * 8 < slot_count; ++trip)
                    {
#pragma unroll
                        for (int k = 0; k < 8; ++k)
                            normalizer += read_lane(residual[s], trip * 8 + k);
                    }
                }
                if (!is_finite_f32(normalizer) || !(normalizer > 0.0f))
                {
                    if (lane == 0)
                        write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_RESIDUAL_EMPTY, 0, accept_draws, 0, 1);
                    return;
                }
                // uniform_real_distribution<float>(0, normalizer): canonical draw times the range
                const float sample_value = shared.uniforms[accept_draws] * normalizer;
                float cumulative = 0.0f;
                int selected = -1;
                int last_positive = -1;
#pragma unroll
                for (int s = 0; s < kVerifySlots; ++s)
                {
                    // every lane keeps the running sum at its own entry; one ballot per trip tells
                    // whether the draw has been passed (the first entry that passes it holds mass)
                    float cumulative_here = 0.0f;
                    const int slot_count = selected >= 0 ? 0 : min(kWaveSize, n - s * kWaveSize);
                    for (int trip = 0; trip * 8 < slot_count; ++trip)
                    {
#pragma unroll
                        for (int k = 0; k < 8; ++k)
                        {
                            cumulative += read_lane(residual[s], trip * 8 + k);
                            cumulative_here = lane == trip * 8 + k ? cumulative : cumulative_here;
                        }
                        const uint64_t passed = __ballot(lane < (trip + 1) * 8 && sample_value < cumulative_here);
                        if (passed != 0)
                        {
                            selected = s * kWaveSize + __builtin_ctzll(passed);
                            break;
                        }
                    }
                    const uint64_t positive = __ballot(residual[s] > 0.0f);
                    if (selected < 0 && slot_count > 0 && positive != 0)
                        last_positive = s * kWaveSize + 63 - __builtin_clzll(positive);
                }
                if (selected < 0)
                    selected = last_positive; // session.cpp:189-198: the last token that has any residual mass
                if (selected < 0)
                {
                    if (lane == 0)
                        write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_RESIDUAL_FAILED, 0, accept_draws, 1, 1);
                    return;
                }
                if (lane == 0)
                    write_verify_result(v, accepted, shared.ordered_token[selected],
                                        shared.ordered_residual[selected] / normalizer, NCNN_MOE_VERIFY_OK, 0,
                                        accept_draws, 1, 1);
                return;
            }
            if (tid == 0)
                v.accepted_probabilities[accepted] = target_probability;
            __syncthreads(); // found[] is reset by the next position
        }
    }

    // ---- session.cpp:871-873: the target's own sample at the first position that was not accepted
    // (greedy mismatch) or after the last drafted token (everything accepted)
    const ncnn_moe_sample_result next = shared.row_results[accepted];
    if (tid == 0)
    {
        if (next.status != NCNN_MOE_ROW_OK)
            write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_ROW_ERROR, next.status, accept_draws, 0, 0);
        else
            write_verify_result(v, accepted, next.token_id, next.probability, NCNN_MOE_VERIFY_OK, 0, accept_draws,
                                next.draw_consumed, 0);
    }
}

// The same step for filtered distributions of any length (a row without a Top-K window whose Top-P
// keeps more than kVerifyCap tokens): the lists stay in global memory, `list_cap` entries per row, and
// a rejection builds the residual as the CPU does, as a dense vector over the vocabulary
// (session.cpp:150-202): the draft's probabilities are scattered into one vector, max(0, target - draft)
// into another, and the sequential fp32 sum and the walk to the draw over that vector (zeros leave an
// fp32 sum as it is) come from the exact parallel running sum.  One workgroup of kReplayThreads threads.
struct VerifyDenseArgs
{
    VerifyArgs step;       // distribution_ids / distribution_probabilities hold list_cap entries per row
    uint32_t list_cap;
    uint32_t vocab;
    float* dense_draft;    // [vocab]
    float* dense_residual; // [vocab]
};

struct VerifyDenseShared
{
    ReplayScratch replay;
    float found[2];
    int last_positive;
    ncnn_moe_sample_result row_results[2 * NCNN_MOE_MAX_DRAFT_TOKENS + 1];
    uint32_t counts[2 * NCNN_MOE_MAX_DRAFT_TOKENS + 1];
    int32_t proposed[NCNN_MOE_MAX_DRAFT_TOKENS];
    float uniforms[NCNN_MOE_MAX_DRAFT_TOKENS + 1];
};

__global__ __launch_bounds__(kReplayThreads) void speculative_verify_dense_kernel(VerifyDenseArgs d)
{
    __shared__ VerifyDenseShared shared;
    const VerifyArgs& v = d.step;
    const int tid = threadIdx.x;
    const uint32_t drafts = v.draft_count;
    uint32_t accepted = 0;
    uint32_t accept_draws = 0;
    if (static_cast<uint32_t>(tid) < 2u * drafts + 1u)
    {
        shared.row_results[tid] = v.row_results[tid];
        shared.counts[tid] = v.distribution_count[tid];
    }
    if (static_cast<uint32_t>(tid) < drafts)
        shared.proposed[tid] = v.proposed[tid];
    if (static_cast<uint32_t>(tid) <= drafts)
        shared.uniforms[tid] = v.uniforms[tid];
    __syncthreads();

    // ---- session.cpp:797-842 (a greedy step never needs the lists and is served by the kernel above)
    for (; accepted < drafts; ++accepted)
    {
        const uint32_t target_row = accepted;
        const uint32_t draft_row = drafts + 1u + accepted;
        const ncnn_moe_sample_result target = shared.row_results[target_row];
        const ncnn_moe_sample_result draft = shared.row_results[draft_row];
        if (target.status != NCNN_MOE_ROW_OK || draft.status != NCNN_MOE_ROW_OK)
        {
            const uint32_t row_status = target.status != NCNN_MOE_ROW_OK ? target.status : draft.status;
            if (tid == 0)
                write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_ROW_ERROR, row_status, accept_draws, 0, 0);
            return;
        }
        const uint32_t target_count = __builtin_amdgcn_readfirstlane(shared.counts[target_row]);
        const uint32_t draft_count = __builtin_amdgcn_readfirstlane(shared.counts[draft_row]);
        if (target_count > d.list_cap || draft_count > d.list_cap)
        {
            if (tid == 0)
                write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_UNSUPPORTED_WINDOW, 0, accept_draws, 0, 0);
            return;
        }
        const int32_t* const target_ids = v.distribution_ids + static_cast<size_t>(target_row) * d.list_cap;
        const float* const target_probabilities = v.distribution_probabilities + static_cast<size_t>(target_row) * d.list_cap;
        const int32_t* const draft_ids = v.distribution_ids + static_cast<size_t>(draft_row) * d.list_cap;
        const float* const draft_probabilities = v.distribution_probabilities + static_cast<size_t>(draft_row) * d.list_cap;
        const int32_t token = shared.proposed[accepted];
        // ---- candidate_probability (session.cpp:138-148) of the proposed token in both lists
        if (tid < 2)
            shared.found[tid] = 0.0f;
        __syncthreads();
        for (uint32_t j = tid; j < target_count; j += kReplayThreads)
        {
            if (target_ids[j] == token)
                shared.found[0] = target_probabilities[j]; // ids are distinct: at most one writer
        }
        for (uint32_t j = tid; j < draft_count; j += kReplayThreads)
        {
            if (draft_ids[j] == token)
                shared.found[1] = draft_probabilities[j];
        }
        __syncthreads();
        const float target_probability = shared.found[0];
        const float draft_probability = shared.found[1];
        if (draft_probability <= 0.0f)
        {
            if (tid == 0)
                write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_ZERO_DRAFT_PROBABILITY, 0, accept_draws, 0, 0);
            return;
        }
        const float ratio = target_probability / draft_probability;
        const float acceptance = ratio < 1.0f ? ratio : 1.0f; // std::min(1.0f, ratio)
        const float uniform = shared.uniforms[accept_draws];
        ++accept_draws;
        if (uniform >= acceptance)
        {
            // ---- rejected: sample_residual_distribution (session.cpp:150-202), dense over the vocabulary
            for (uint32_t i = tid; i < d.vocab; i += kReplayThreads)
            {
                d.dense_draft[i] = 0.0f;
                d.dense_residual[i] = 0.0f;
            }
            if (tid == 0)
                shared.last_positive = -1;
            __syncthreads();
            for (uint32_t j = tid; j < draft_count; j += kReplayThreads)
                d.dense_draft[draft_ids[j]] = draft_probabilities[j];
            __syncthreads();
            for (uint32_t j = tid; j < target_count; j += kReplayThreads)
            {
                const int32_t id = target_ids[j];
                const float difference = target_probabilities[j] - d.dense_draft[id];
                const float residual = 0.0f < difference ? difference : 0.0f; // std::max(0.0f, difference)
                d.dense_residual[id] = residual;
                if (residual > 0.0f)
                    atomicMax(&shared.last_positive, id);
            }
            __syncthreads();
            const float* const residual = d.dense_residual;
            const RunningSum total = exact_running_sum_of_array<false, false>(residual, 1.0f, 1.0f, d.vocab, kStopNever, 0.0f, shared.replay, tid);
            const float normalizer = total.sum;
            if (!is_finite_f32(normalizer) || !(normalizer > 0.0f))
            {
                if (tid == 0)
                    write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_RESIDUAL_EMPTY, 0, accept_draws, 0, 1);
                return;
            }
            // uniform_real_distribution<float>(0, normalizer): canonical draw times the range
            const float sample_value = shared.uniforms[accept_draws] * normalizer;
            __syncthreads();
            const RunningSum walk = exact_running_sum_of_array<false, false>(residual, 1.0f, 1.0f, d.vocab, kStopAbove, sample_value, shared.replay, tid);
            // session.cpp:189-198: past the end, the last token that has any residual mass
            const int selected = walk.stopped ? static_cast<int>(walk.stop_index) : shared.last_positive;
            if (selected < 0)
            {
                if (tid == 0)
                    write_verify_result(v, accepted, -1, 0.0f, NCNN_MOE_VERIFY_RESIDUAL_FAILED, 0, accept_draws, 1, 1);
                return;
            }
            if (tid == 0)
                write_verify_result(v, accepted, selected, residual[selected] / normalizer, NCNN_MOE_VERIFY_OK, 0, accept_draws, 1, 1);
            return;
        }
        if (tid == 0)
            v.accepted_probabilities[accepted] = target_probability;
        __syncthreads(); // found[] is reset by the next position
    }

    // ---- session.cpp:871-873: the target's own sample after the last drafted token
    const ncnn_moe_sample_result next = shared.row_results[accepted];
    if (tid == 0)
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
