// Exact reproduction of the CPU sampler's sequential fp32 sums over a sorted window, in parallel,
// and the sampler's walk over such a window (normaliser, Min-P, Top-P, renormaliser, draw).
#ifndef NCNN_MOE_HIP_SAMPLER_EXACT_SUM_H
#define NCNN_MOE_HIP_SAMPLER_EXACT_SUM_H

#include "sampler_common.h"

namespace ncnn_moe_hip {

// ---------------------------------------------------------------------------------------------
// Exact sequential fp32 sums, computed in parallel.
//
// The CPU sampler adds probabilities one at a time in sorted order (session.cpp:100, :123, :131,
// :437), so every partial sum is rounded to fp32 before the next term is added.  While the running
// sum s stays inside one binade [2^k, 2^(k+1)) its 24-bit mantissa N is an integer in units of
// ulp(s), and adding a non-negative term t moves it by
//     floor(t/ulp) + [frac > 1/2] + [frac == 1/2 and N + floor(t/ulp) is odd]      (round to nearest even)
// which depends on the sum only through the parity of N.  A term is therefore a pair
// (step if N is even, step if N is odd); pairs compose associatively, so a block-wide scan gives
// every partial sum of a chunk exactly.  The first step that would leave the binade is carried
// out as one real fp32 addition and the scan restarts behind it with the wider ulp.
// ---------------------------------------------------------------------------------------------

struct ParityStep
{
    uint32_t even; // mantissa increment when the mantissa is even before the step
    uint32_t odd;  // ... when it is odd
};

constexpr uint32_t kBinadeFull = 1u << 24;
constexpr uint32_t kStepCap = 1u << 28; // sums past the binade are only compared against 2^24

__device__ __forceinline__ ParityStep compose_steps(const ParityStep& first, const ParityStep& second)
{
    ParityStep r;
    r.even = first.even + ((first.even & 1u) ? second.odd : second.even);
    r.odd = first.odd + ((first.odd & 1u) ? second.even : second.odd);
    r.even = min(r.even, kStepCap);
    r.odd = min(r.odd, kStepCap);
    return r;
}

// Biased exponent (denormals and zero share exponent 1) and integer mantissa of a non-negative float:
// value = mantissa * 2^(exponent - 150).
__device__ __forceinline__ void decode_sum(float value, int& exponent, uint32_t& mantissa)
{
    const uint32_t bits = __float_as_uint(value);
    exponent = static_cast<int>(bits >> 23);
    mantissa = bits & 0x7fffffu;
    if (exponent == 0)
        exponent = 1;
    else
        mantissa |= 0x800000u;
}

__device__ __forceinline__ float encode_sum(int exponent, uint32_t mantissa)
{
    return __uint_as_float((static_cast<uint32_t>(exponent - 1) << 23) + mantissa);
}

// The step a term causes on a sum with biased exponent `exponent`.
__device__ __forceinline__ ParityStep step_of_term(float term, int exponent)
{
    int term_exponent;
    uint32_t term_mantissa;
    decode_sum(term, term_exponent, term_mantissa);
    ParityStep step;
    const int shift = exponent - term_exponent;
    if (term_mantissa == 0u || shift >= 25)
    {
        step.even = 0u;
        step.odd = 0u;
    }
    else if (shift <= 0)
    {
        step.even = kBinadeFull; // at least half the sum: the addition leaves the binade
        step.odd = kBinadeFull;
    }
    else
    {
        const uint32_t whole = term_mantissa >> shift;
        const uint32_t rest = term_mantissa & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1);
        if (rest > half)
        {
            step.even = whole + 1u;
            step.odd = whole + 1u;
        }
        else if (rest < half)
        {
            step.even = whole;
            step.odd = whole;
        }
        else
        {
            step.even = whole + (whole & 1u);
            step.odd = whole + 1u - (whole & 1u);
        }
    }
    return step;
}

enum StopMode : int
{
    kStopNever = 0,
    kStopAtOrAbove = 1, // first partial sum s with s >= bound
    kStopAbove = 2      // first partial sum s with s > bound
};

// Smallest mantissa (at biased exponent `exponent`) whose sum satisfies the stop condition.
__device__ __forceinline__ uint32_t stop_mantissa(int mode, float bound, int exponent)
{
    if (mode == kStopNever)
        return 0xffffffffu;
    int bound_exponent;
    uint32_t bound_mantissa;
    decode_sum(bound, bound_exponent, bound_mantissa);
    if (bound_exponent > exponent)
        return 0xffffffffu; // not inside this binade
    const int shift = exponent - bound_exponent;
    if (shift == 0)
        return mode == kStopAtOrAbove ? bound_mantissa : bound_mantissa + 1u;
    if (shift >= 25)
        return (mode == kStopAtOrAbove && bound_mantissa == 0u) ? 0u : 1u;
    const uint32_t whole = bound_mantissa >> shift;
    const uint32_t rest = bound_mantissa & ((1u << shift) - 1u);
    if (mode == kStopAtOrAbove)
        return whole + (rest != 0u ? 1u : 0u);
    return whole + 1u;
}

constexpr int kReplayWaves = kReplayThreads / kWaveSize;

struct ReplayScratch
{
    ParityStep wave_totals[kReplayWaves];
    uint32_t first_event; // (index << 1 | kind) of the earliest event of the round, kind 0 = leaves the binade, 1 = stop
    uint32_t final_mantissa;
    float event_sum;
    int absorbed;
};

struct RunningSum
{
    float sum;          // the sum after the last term processed (after the stopping term if stopped)
    uint32_t stop_index; // index of the term at which the stop condition first held
    bool stopped;
};

// One sorted row seen as a sequence of terms; `phase` selects what the CPU loop adds:
//   0  exp(logit/T - maximum)                                  (session.cpp:98-100)
//   1  the above divided by the normaliser                     (session.cpp:105, :123)
//   2  the above divided by the renormaliser                   (session.cpp:134, :437)
struct SortedRow
{
    const uint32_t* keys;
    float temperature;
    float maximum;
    float normalizer;
    float renormalizer;
};

template <int PHASE>
__device__ __forceinline__ float row_term(const SortedRow& row, uint32_t i)
{
    float t = expf_libm(value_from_descending_key(row.keys[i]) / row.temperature - row.maximum);
    if (PHASE >= 1)
        t = t / row.normalizer;
    if (PHASE >= 2)
        t = t / row.renormalizer;
    return t;
}

// The running fp32 sum of terms [0, count) of the row, starting from 0, exactly as a sequential
// loop produces it.  PHASE 0 also stops (without `stopped`) once the sum no longer moves, which
// is final because the terms are non-increasing.  Every thread of the workgroup must call it.
template <int PHASE>
__device__ __forceinline__ RunningSum exact_running_sum(
    const SortedRow& row, uint32_t count, int mode, float bound, ReplayScratch& scratch, int tid)
{
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    float sum = 0.0f;
    for (uint32_t base = 0; base < count; base += kReplayChunk)
    {
        const uint32_t chunk_end = min(count, base + static_cast<uint32_t>(kReplayChunk));
        const uint32_t thread_first = base + static_cast<uint32_t>(tid) * kReplayPerThread;
        float terms[kReplayPerThread];
#pragma unroll
        for (int j = 0; j < kReplayPerThread; ++j)
        {
            const uint32_t i = thread_first + j;
            terms[j] = i < chunk_end ? row_term<PHASE>(row, i) : 0.0f;
        }
        uint32_t start = base;
        while (start < chunk_end)
        {
            int exponent;
            uint32_t mantissa;
            decode_sum(sum, exponent, mantissa);
            const uint32_t stop_at = stop_mantissa(mode, bound, exponent);

            ParityStep thread_total{0u, 0u};
            ParityStep first_step{0u, 0u};
#pragma unroll
            for (int j = 0; j < kReplayPerThread; ++j)
            {
                const uint32_t i = thread_first + j;
                ParityStep step{0u, 0u};
                if (i >= start && i < chunk_end)
                    step = step_of_term(terms[j], exponent);
                if (j == 0)
                    first_step = step;
                thread_total = compose_steps(thread_total, step);
            }
            if (tid == 0)
            {
                scratch.first_event = 0xffffffffu;
                // the largest remaining term of the row does not move the sum: nothing later can
                scratch.absorbed = (PHASE == 0 && start == base && base > 0 && first_step.even == 0u && first_step.odd == 0u) ? 1 : 0;
            }
            // inclusive scan of the per-thread totals across the wave, then across waves
            ParityStep inclusive = thread_total;
#pragma unroll
            for (int step = 1; step < kWaveSize; step <<= 1)
            {
                ParityStep earlier;
                earlier.even = __shfl_up(inclusive.even, step, kWaveSize);
                earlier.odd = __shfl_up(inclusive.odd, step, kWaveSize);
                if (lane >= step)
                    inclusive = compose_steps(earlier, inclusive);
            }
            ParityStep exclusive;
            exclusive.even = __shfl_up(inclusive.even, 1, kWaveSize);
            exclusive.odd = __shfl_up(inclusive.odd, 1, kWaveSize);
            if (lane == 0)
                exclusive = ParityStep{0u, 0u};
            if (lane == kWaveSize - 1)
                scratch.wave_totals[wave] = inclusive;
            __syncthreads();
            if (scratch.absorbed)
                return RunningSum{sum, 0u, false};
            ParityStep before{0u, 0u};
            for (int w = 0; w < wave; ++w)
                before = compose_steps(before, scratch.wave_totals[w]);
            before = compose_steps(before, exclusive);
            uint32_t current = mantissa + ((mantissa & 1u) ? before.odd : before.even);

            // walk this thread's terms with the true mantissa; remember the first event
            bool have_event = false;
            uint32_t event_key = 0;
            uint32_t event_mantissa = 0;
            float event_term = 0.0f;
#pragma unroll
            for (int j = 0; j < kReplayPerThread; ++j)
            {
                const uint32_t i = thread_first + j;
                const bool active = i >= start && i < chunk_end;
                ParityStep step{0u, 0u};
                if (active)
                    step = step_of_term(terms[j], exponent);
                const uint32_t next = current + ((current & 1u) ? step.odd : step.even);
                if (active && !have_event)
                {
                    if (next >= kBinadeFull)
                    {
                        have_event = true;
                        event_key = i << 1;
                        event_mantissa = current;
                        event_term = terms[j];
                    }
                    else if (next >= stop_at)
                    {
                        have_event = true;
                        event_key = (i << 1) | 1u;
                        event_mantissa = next;
                    }
                }
                current = next;
            }
            if (have_event)
                atomicMin(&scratch.first_event, event_key);
            if (tid == kReplayThreads - 1)
                scratch.final_mantissa = current;
            __syncthreads();
            const uint32_t event = scratch.first_event;
            if (event == 0xffffffffu)
            {
                sum = encode_sum(exponent, scratch.final_mantissa);
                __syncthreads();
                break;
            }
            if (have_event && event_key == event)
            {
                const float at_event = encode_sum(exponent, event_mantissa);
                scratch.event_sum = (event & 1u) ? at_event : at_event + event_term;
            }
            __syncthreads();
            sum = scratch.event_sum;
            const uint32_t event_index = event >> 1;
            __syncthreads();
            if (event & 1u)
                return RunningSum{sum, event_index, true};
            if ((mode == kStopAtOrAbove && sum >= bound) || (mode == kStopAbove && sum > bound))
                return RunningSum{sum, event_index, true};
            start = event_index + 1u;
        }
    }
    return RunningSum{sum, 0u, false};
}

// The CPU sampler from the sorted Top-K window onwards (src/engine/session.cpp:89-134, :429-442) for a
// window of any length: `keys` holds the descending keys of the window's n finite logits in
// (logit descending, index ascending) order (global memory or LDS).  token_at(rank) yields the token
// index of a position of the window and is called by every thread of the workgroup; sorted_indices
// (may be null) lists all token indices and is only needed to export the distribution.
// Every running sum is reproduced exactly by exact_running_sum.  All threads must call it.
template <typename TokenAt>
__device__ __forceinline__ void replay_sorted_window(
    const SamplerArgs& a, uint32_t row, const ncnn_moe_sample_params& p,
    const uint32_t* keys, uint32_t n, const uint32_t* sorted_indices, uint8_t flags,
    ReplayScratch& scratch, int tid, TokenAt token_at)
{
    SortedRow sorted;
    sorted.keys = keys;
    sorted.temperature = p.temperature;
    sorted.maximum = value_from_descending_key(keys[0]) / p.temperature;
    sorted.normalizer = 1.0f;
    sorted.renormalizer = 1.0f;

    // ---- normaliser (session.cpp:92-103).  A first term that is not finite poisons the sum.
    const float first_term = row_term<0>(sorted, 0);
    float normalizer = first_term;
    if (is_finite_f32(first_term))
        normalizer = exact_running_sum<0>(sorted, n, kStopNever, 0.0f, scratch, tid).sum;
    if (!is_finite_f32(normalizer) || !(normalizer > 0.0f))
    {
        if (tid == 0)
            write_error(a, row, NCNN_MOE_ROW_INVALID_DISTRIBUTION, flags);
        return;
    }
    sorted.normalizer = normalizer;

    // ---- Min-P (session.cpp:107-117): probabilities are non-increasing, so the survivors are a prefix
    uint32_t candidates = n;
    if (p.min_p > 0.0f)
    {
        const float threshold = row_term<1>(sorted, 0) * p.min_p;
        uint32_t first = 0, last = n; // first position whose probability is below the threshold
        while (first < last)
        {
            const uint32_t middle = (first + last) >> 1;
            if (row_term<1>(sorted, middle) >= threshold)
                first = middle + 1;
            else
                last = middle;
        }
        candidates = first;
    }

    // ---- Top-P (session.cpp:119-128) and the renormaliser (:130-132), which adds the same values
    const RunningSum nucleus = exact_running_sum<1>(sorted, candidates, kStopAtOrAbove, p.top_p, scratch, tid);
    const uint32_t kept = nucleus.stopped ? nucleus.stop_index + 1u : candidates;
    sorted.renormalizer = nucleus.sum;

    if (a.distribution_count != nullptr && sorted_indices != nullptr)
    {
        const size_t first = static_cast<size_t>(row) * a.distribution_cap;
        const uint32_t limit = kept < a.distribution_cap ? kept : a.distribution_cap;
        for (uint32_t i = tid; i < limit; i += kReplayThreads)
        {
            a.distribution_ids[first + i] = static_cast<int32_t>(sorted_indices[i]);
            a.distribution_probabilities[first + i] = row_term<2>(sorted, i);
        }
        if (tid == 0)
            a.distribution_count[row] = kept;
    }

    if (kept == 1)
    {
        const int32_t token = token_at(0u);
        if (tid == 0)
            write_token(a, row, p, token, 1.0f, 1u, 0, flags);
        return;
    }

    // ---- inverse-CDF draw over the kept prefix (session.cpp:432-442)
    const RunningSum draw = exact_running_sum<2>(sorted, kept, kStopAbove, a.uniforms[row], scratch, tid);
    const uint32_t selected = draw.stopped ? draw.stop_index : kept - 1u;
    const int32_t token = token_at(selected);
    if (tid == 0)
        write_token(a, row, p, token, row_term<2>(sorted, selected), kept, 1, flags);
}

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_SAMPLER_EXACT_SUM_H
