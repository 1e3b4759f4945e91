// Exact reproduction of the CPU sampler's sequential fp32 sums over a sorted window, in parallel,
// and the sampler's walk over such a window (normaliser, Min-P, Top-P, renormaliser, draw).
#ifndef NCNN_MOE_HIP_SAMPLER_EXACT_SUM_H
#define NCNN_MOE_HIP_SAMPLER_EXACT_SUM_H

#include "sampler_common.h"

#include <type_traits>

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
constexpr int kSequentialHead = 64; // terms a running sum adds one by one before it scans
constexpr int kHeadSlots = (kSequentialHead + kWaveSize - 1) / kWaveSize;
constexpr int kSequentialHeadOfRuns = 16; // ... of a row stored as runs
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

// The mantissa increment of `count` successive additions of one term (step `s`) to a mantissa of the
// given parity.  An even step keeps the parity, so the same step repeats; an odd step flips it, and
// the flipped parity either stays (even step there) or flips back (the two steps alternate).
__device__ __forceinline__ uint32_t repeated_step(bool odd, const ParityStep& s, uint32_t count)
{
    if (count == 0u)
        return 0u;
    const uint64_t first = odd ? s.odd : s.even;
    uint64_t total;
    if ((first & 1u) == 0u)
        total = first * count;
    else
    {
        const uint64_t flipped = odd ? s.even : s.odd;
        if ((flipped & 1u) == 0u)
            total = first + flipped * (count - 1u);
        else
            total = first * ((count + 1u) >> 1) + flipped * (count >> 1);
    }
    return total > kStepCap ? kStepCap : static_cast<uint32_t>(total);
}

__device__ __forceinline__ ParityStep repeat_steps(const ParityStep& s, uint32_t count)
{
    return ParityStep{repeated_step(false, s, count), repeated_step(true, s, count)};
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
    const uint32_t* keys;     // one key per element, or one per run of equal keys
    const uint32_t* run_ends; // runs only: position behind the last element of each run (null otherwise)
    uint32_t run_count;
    float temperature;
    float maximum;
    float normalizer;
    float renormalizer;
};

// Runs: a sorted row stored as (key, end position) per run of equal keys.  Element e belongs to the
// first run whose end lies behind it.
__device__ __forceinline__ uint32_t run_first_element(const SortedRow& row, uint32_t run)
{
    return run == 0u ? 0u : row.run_ends[run - 1u];
}

__device__ __forceinline__ uint32_t run_of_element(const SortedRow& row, uint32_t element)
{
    uint32_t low = 0, high = row.run_count;
    while (low < high)
    {
        const uint32_t middle = (low + high) >> 1;
        if (row.run_ends[middle] <= element)
            low = middle + 1;
        else
            high = middle;
    }
    return low;
}

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

// The running fp32 sum of the non-negative terms term_at(0) ... term_at(count - 1), starting from 0,
// exactly as a sequential loop produces it.  With NON_INCREASING (the terms never grow) it also stops
// (without `stopped`) once the sum no longer moves, which is then final.  Every thread of the
// workgroup (kReplayThreads threads) must call it.
template <bool NON_INCREASING, class TermAt>
__device__ __forceinline__ RunningSum exact_running_sum_of_terms(
    TermAt term_at, uint32_t count, int mode, float bound, ReplayScratch& scratch, int tid)
{
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    float sum = 0.0f;
    // The first kSequentialHead terms are added one by one, as the CPU does (every thread runs the same
    // loop on wave-uniform values): the sum climbs through most of its binades here, each of which
    // would cost the scan below a round, and a stop condition usually holds this early.
    const uint32_t head = min(count, static_cast<uint32_t>(kSequentialHead));
    {
        float head_terms[kHeadSlots];
#pragma unroll
        for (int slot = 0; slot < kHeadSlots; ++slot)
        {
            const uint32_t i = static_cast<uint32_t>(slot * kWaveSize + lane);
            head_terms[slot] = i < head ? term_at(i) : 0.0f;
        }
#pragma unroll
        for (int slot = 0; slot < kHeadSlots; ++slot)
        {
            const uint32_t slot_first = static_cast<uint32_t>(slot * kWaveSize);
            const uint32_t slot_count = head > slot_first ? min(head - slot_first, static_cast<uint32_t>(kWaveSize)) : 0u;
            for (uint32_t l = 0; l < slot_count; ++l)
            {
                sum += read_lane(head_terms[slot], static_cast<int>(l));
                if ((mode == kStopAtOrAbove && sum >= bound) || (mode == kStopAbove && sum > bound))
                    return RunningSum{sum, slot_first + l, true};
            }
        }
        if (head >= count)
            return RunningSum{sum, 0u, false};
    }
    for (uint32_t base = 0; base < count; base += kReplayChunk)
    {
        const uint32_t chunk_end = min(count, base + static_cast<uint32_t>(kReplayChunk));
        const uint32_t thread_first = base + static_cast<uint32_t>(tid) * kReplayPerThread;
        float terms[kReplayPerThread];
#pragma unroll
        for (int j = 0; j < kReplayPerThread; ++j)
        {
            const uint32_t i = thread_first + j;
            terms[j] = i < chunk_end ? term_at(i) : 0.0f;
        }
        uint32_t start = max(base, head);
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
                scratch.absorbed = (NON_INCREASING && start == base && base > 0 && first_step.even == 0u && first_step.odd == 0u) ? 1 : 0;
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
            // every wave's total is read at once (independent LDS loads); the composition stays in registers
            ParityStep totals[kReplayWaves];
#pragma unroll
            for (int w = 0; w < kReplayWaves; ++w)
                totals[w] = scratch.wave_totals[w];
            ParityStep before{0u, 0u};
#pragma unroll
            for (int w = 0; w < kReplayWaves - 1; ++w)
            {
                if (w < wave)
                    before = compose_steps(before, totals[w]);
            }
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

// The running sum of terms [0, count) of a sorted row.  PHASE 0 (terms that never grow) also stops
// once the sum no longer moves.  Every thread of the workgroup must call it.
template <int PHASE>
__device__ __forceinline__ RunningSum exact_running_sum(
    const SortedRow& row, uint32_t count, int mode, float bound, ReplayScratch& scratch, int tid)
{
    return exact_running_sum_of_terms<PHASE == 0>(
        [&row](uint32_t i) { return row_term<PHASE>(row, i); }, count, mode, bound, scratch, tid);
}

// The same running sum over a row stored as runs: `count` elements are added, run after run.  A run of
// m equal terms is one step (repeat_steps); when an event (the sum leaves its binade, or the stop
// condition first holds) falls inside a run, the thread that owns the run finds the addition it
// falls on by bisection over repeated_step, which is monotone in the number of additions.
template <int PHASE>
__device__ __forceinline__ RunningSum exact_running_sum_runs(
    const SortedRow& row, uint32_t count, int mode, float bound, ReplayScratch& scratch, int tid)
{
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    float sum = 0.0f;
    if (count == 0u)
        return RunningSum{sum, 0u, false};
    const uint32_t runs = run_of_element(row, count - 1u) + 1u;
    uint32_t start = 0; // elements before this one have been added

    // The first kSequentialHeadOfRuns elements are added one by one, as the CPU does (every thread runs the
    // same loop on wave-uniform values): the sum climbs through most of its binades here, each of
    // which would cost the scan below a round, and a stop condition usually holds this early.
    {
        const uint32_t head_runs = min(runs, static_cast<uint32_t>(kWaveSize));
        const float head_term = static_cast<uint32_t>(lane) < head_runs ? row_term<PHASE>(row, static_cast<uint32_t>(lane)) : 0.0f;
        const uint32_t head_end = static_cast<uint32_t>(lane) < head_runs ? min(row.run_ends[lane], count) : 0u;
        const uint32_t head_limit = min(count, static_cast<uint32_t>(kSequentialHeadOfRuns));
        for (uint32_t run = 0; run < head_runs && start < head_limit; ++run)
        {
            const float term = read_lane(head_term, static_cast<int>(run));
            const uint32_t run_end = min(static_cast<uint32_t>(read_lane(static_cast<int>(head_end), static_cast<int>(run))), head_limit);
            for (; start < run_end; ++start)
            {
                sum += term;
                if ((mode == kStopAtOrAbove && sum >= bound) || (mode == kStopAbove && sum > bound))
                    return RunningSum{sum, start, true};
            }
        }
        if (start >= count)
            return RunningSum{sum, 0u, false};
    }
    const uint32_t first_run = run_of_element(row, start);
    for (uint32_t base = first_run; base < runs; base += kReplayChunk)
    {
        const uint32_t chunk_end = min(runs, base + static_cast<uint32_t>(kReplayChunk));
        const uint32_t thread_first = base + static_cast<uint32_t>(tid) * kReplayPerThread;
        float terms[kReplayPerThread];
        uint32_t firsts[kReplayPerThread]; // first and one-past-last element of each run, clipped to count
        uint32_t lasts[kReplayPerThread];
#pragma unroll
        for (int j = 0; j < kReplayPerThread; ++j)
        {
            const uint32_t i = thread_first + j;
            const bool valid = i < chunk_end;
            terms[j] = valid ? row_term<PHASE>(row, i) : 0.0f;
            firsts[j] = valid ? run_first_element(row, i) : 0u;
            lasts[j] = valid ? min(row.run_ends[i], count) : 0u;
        }
        bool fresh = true; // no event in this chunk yet
        while (true)
        {
            int exponent;
            uint32_t mantissa;
            decode_sum(sum, exponent, mantissa);
            const uint32_t stop_at = stop_mantissa(mode, bound, exponent);
            const uint32_t limit = min(stop_at, kBinadeFull);

            ParityStep thread_total{0u, 0u};
            ParityStep first_step{0u, 0u};
#pragma unroll
            for (int j = 0; j < kReplayPerThread; ++j)
            {
                const uint32_t low = max(firsts[j], start);
                const uint32_t multiplicity = lasts[j] > low ? lasts[j] - low : 0u;
                const ParityStep single = step_of_term(terms[j], exponent);
                if (j == 0)
                    first_step = multiplicity > 0u ? single : ParityStep{0u, 0u};
                thread_total = compose_steps(thread_total, repeat_steps(single, multiplicity));
            }
            if (tid == 0)
            {
                scratch.first_event = 0xffffffffu;
                // the largest remaining term of the row does not move the sum: nothing later can
                scratch.absorbed = (PHASE == 0 && fresh && base > first_run && first_step.even == 0u && first_step.odd == 0u) ? 1 : 0;
            }
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
            // every wave's total is read at once (independent LDS loads); the composition stays in registers
            ParityStep totals[kReplayWaves];
#pragma unroll
            for (int w = 0; w < kReplayWaves; ++w)
                totals[w] = scratch.wave_totals[w];
            ParityStep before{0u, 0u};
#pragma unroll
            for (int w = 0; w < kReplayWaves - 1; ++w)
            {
                if (w < wave)
                    before = compose_steps(before, totals[w]);
            }
            before = compose_steps(before, exclusive);
            uint32_t current = mantissa + ((mantissa & 1u) ? before.odd : before.even);

            bool have_event = false;
            uint32_t event_key = 0;
            uint32_t event_mantissa = 0;
            float event_term = 0.0f;
#pragma unroll
            for (int j = 0; j < kReplayPerThread; ++j)
            {
                const uint32_t low = max(firsts[j], start);
                const uint32_t multiplicity = lasts[j] > low ? lasts[j] - low : 0u;
                const ParityStep single = step_of_term(terms[j], exponent);
                const bool odd = (current & 1u) != 0u;
                const uint32_t next = current + repeated_step(odd, single, multiplicity);
                // A thread that starts at or beyond the limit comes after the round's first event (the
                // mantissa never decreases and began below the limit), so its own cannot be the first:
                // it skips the search.  (A round that begins at the limit keeps every thread's event.)
                if (multiplicity > 0u && !have_event && next >= limit && (current < limit || mantissa >= limit))
                {
                    // the first addition of the run after which the mantissa reaches the limit
                    uint32_t none = 0u, some = multiplicity; // repeated additions: `none` stay below, `some` reach it
                    while (some - none > 1u)
                    {
                        const uint32_t middle = none + ((some - none) >> 1);
                        if (current + repeated_step(odd, single, middle) >= limit)
                            some = middle;
                        else
                            none = middle;
                    }
                    const uint32_t before_event = current + repeated_step(odd, single, none);
                    const uint32_t after_event = before_event + ((before_event & 1u) ? single.odd : single.even);
                    const uint32_t element = low + none;
                    have_event = true;
                    if (after_event >= kBinadeFull)
                    {
                        event_key = element << 1;
                        event_mantissa = before_event;
                        event_term = terms[j];
                    }
                    else
                    {
                        event_key = (element << 1) | 1u;
                        event_mantissa = after_event;
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
            const uint32_t event_element = event >> 1;
            __syncthreads();
            if (event & 1u)
                return RunningSum{sum, event_element, true};
            if ((mode == kStopAtOrAbove && sum >= bound) || (mode == kStopAbove && sum > bound))
                return RunningSum{sum, event_element, true};
            start = event_element + 1u;
            fresh = false;
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
// With RUNS the row is stored as runs of equal keys (`keys` and `run_ends` hold one entry per run,
// run_count of them) and n still counts elements.
template <bool RUNS, typename TokenAt>
__device__ __forceinline__ void replay_sorted_window(
    const SamplerArgs& a, uint32_t row, const ncnn_moe_sample_params& p,
    const uint32_t* keys, const uint32_t* run_ends, uint32_t run_count, uint32_t n,
    const uint32_t* sorted_indices, uint8_t flags, ReplayScratch& scratch, int tid, TokenAt token_at)
{
    SortedRow sorted;
    sorted.keys = keys;
    sorted.run_ends = run_ends;
    sorted.run_count = run_count;
    sorted.temperature = p.temperature;
    sorted.maximum = value_from_descending_key(keys[0]) / p.temperature;
    sorted.normalizer = 1.0f;
    sorted.renormalizer = 1.0f;
    auto running_sum = [&](auto phase, uint32_t count, int mode, float bound) -> RunningSum {
        constexpr int kPhase = decltype(phase)::value;
        if constexpr (RUNS)
            return exact_running_sum_runs<kPhase>(sorted, count, mode, bound, scratch, tid);
        else
            return exact_running_sum<kPhase>(sorted, count, mode, bound, scratch, tid);
    };
    // the item (element, or run) that holds an element
    auto item_of = [&](uint32_t element) -> uint32_t {
        if constexpr (RUNS)
            return run_of_element(sorted, element);
        else
            return element;
    };

    // ---- normaliser (session.cpp:92-103).  A first term that is not finite poisons the sum.
    const float first_term = row_term<0>(sorted, 0);
    float normalizer = first_term;
    if (is_finite_f32(first_term))
        normalizer = running_sum(std::integral_constant<int, 0>{}, n, kStopNever, 0.0f).sum;
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
        uint32_t first = 0, last = RUNS ? item_of(n - 1u) + 1u : n; // first item whose probability is below the threshold
        while (first < last)
        {
            const uint32_t middle = (first + last) >> 1;
            if (row_term<1>(sorted, middle) >= threshold)
                first = middle + 1;
            else
                last = middle;
        }
        if constexpr (RUNS)
            candidates = min(n, run_first_element(sorted, first));
        else
            candidates = first;
    }

    // ---- Top-P (session.cpp:119-128) and the renormaliser (:130-132), which adds the same values
    const RunningSum nucleus = running_sum(std::integral_constant<int, 1>{}, candidates, kStopAtOrAbove, p.top_p);
    const uint32_t kept = nucleus.stopped ? nucleus.stop_index + 1u : candidates;
    sorted.renormalizer = nucleus.sum;

    if (a.distribution_count != nullptr && sorted_indices != nullptr)
    {
        const size_t first = static_cast<size_t>(row) * a.distribution_cap;
        const uint32_t limit = kept < a.distribution_cap ? kept : a.distribution_cap;
        for (uint32_t i = tid; i < limit; i += kReplayThreads)
        {
            a.distribution_ids[first + i] = static_cast<int32_t>(sorted_indices[i]);
            a.distribution_probabilities[first + i] = row_term<2>(sorted, item_of(i));
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
    const RunningSum draw = running_sum(std::integral_constant<int, 2>{}, kept, kStopAbove, a.uniforms[row]);
    const uint32_t selected = draw.stopped ? draw.stop_index : kept - 1u;
    const int32_t token = token_at(selected);
    if (tid == 0)
        write_token(a, row, p, token, row_term<2>(sorted, item_of(selected)), kept, 1, flags);
}

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_SAMPLER_EXACT_SUM_H
