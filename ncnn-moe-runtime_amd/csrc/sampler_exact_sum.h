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
constexpr int kSequentialHead = 256; // terms a running sum adds one by one before it scans
constexpr int kHeadSlots = (kSequentialHead + kWaveSize - 1) / kWaveSize;
constexpr int kSequentialHeadOfRuns = 64; // ... of a row stored as runs
constexpr uint32_t kStepCap = 1u << 28; // sums past the binade are only compared against 2^24

// `odd` where the lowest bit of `parity_of` is set, else `even`.  (Written on the values: a choice between
// the two members of a ParityStep that the compiler sees as two loads becomes one load at a computed
// address, which moves the struct from registers into scratch memory, a trip to memory per use.)
__device__ __forceinline__ uint32_t pick_by_parity(uint32_t parity_of, uint32_t even, uint32_t odd)
{
    const uint32_t mask = 0u - (parity_of & 1u);
    return even ^ ((even ^ odd) & mask);
}

__device__ __forceinline__ ParityStep compose_steps(const ParityStep first, const ParityStep second)
{
    ParityStep r;
    r.even = first.even + pick_by_parity(first.even, second.even, second.odd);
    r.odd = first.odd + pick_by_parity(first.odd, second.odd, second.even);
    r.even = min(r.even, kStepCap);
    r.odd = min(r.odd, kStepCap);
    return r;
}

// The mantissa increment of `count` successive additions of one term (step `s`) to a mantissa of the
// given parity.  An even step keeps the parity, so the same step repeats; an odd step flips it, and
// the flipped parity either stays (even step there) or flips back (the two steps alternate).
__device__ __forceinline__ uint32_t repeated_step(bool odd, const ParityStep s, uint32_t count)
{
    if (count == 0u)
        return 0u;
    const uint64_t first = pick_by_parity(odd ? 1u : 0u, s.even, s.odd);
    uint64_t total;
    if ((first & 1u) == 0u)
        total = first * count;
    else
    {
        const uint64_t flipped = pick_by_parity(odd ? 1u : 0u, s.odd, s.even);
        if ((flipped & 1u) == 0u)
            total = first + flipped * (count - 1u);
        else
            total = first * ((count + 1u) >> 1) + flipped * (count >> 1);
    }
    return total > kStepCap ? kStepCap : static_cast<uint32_t>(total);
}

__device__ __forceinline__ ParityStep repeat_steps(const ParityStep s, uint32_t count)
{
    // The two steps differ only for a term that ends exactly half an ulp above a multiple of it; when no lane
    // of the wave holds such a term, every addition moves the mantissa by the same step.
    if (__builtin_amdgcn_ballot_w64(s.even != s.odd) == 0ull)
    {
        const uint64_t total = static_cast<uint64_t>(s.even) * count;
        const uint32_t capped = total > kStepCap ? kStepCap : static_cast<uint32_t>(total);
        return ParityStep{capped, capped};
    }
    return ParityStep{repeated_step(false, s, count), repeated_step(true, s, count)};
}

// Inclusive scan of the lanes' steps in lane order (lane i: the composition of lanes 0 .. i), by DPP shifts
// inside rows of 16 lanes and two broadcasts across rows; a lane without a source composes with the
// identity (a step of zero).
__device__ __forceinline__ ParityStep wave_scan_steps(ParityStep v)
{
#define NCNN_MOE_SCAN_STAGE(CONTROL, ROW_MASK)                                                              \
    {                                                                                                        \
        const ParityStep earlier{dpp_source<CONTROL, ROW_MASK>(v.even), dpp_source<CONTROL, ROW_MASK>(v.odd)}; \
        v = compose_steps(earlier, v);                                                                       \
    }
    NCNN_MOE_SCAN_STAGE(0x111, 0xf) // row_shr:1
    NCNN_MOE_SCAN_STAGE(0x112, 0xf) // row_shr:2
    NCNN_MOE_SCAN_STAGE(0x114, 0xf) // row_shr:4
    NCNN_MOE_SCAN_STAGE(0x118, 0xf) // row_shr:8
    NCNN_MOE_SCAN_STAGE(0x142, 0xa) // row_bcast15: rows 1 and 3 compose with the row before
    NCNN_MOE_SCAN_STAGE(0x143, 0xc) // row_bcast31: rows 2 and 3 compose with rows 0 + 1
#undef NCNN_MOE_SCAN_STAGE
    return v;
}

__device__ __forceinline__ uint32_t apply_step(uint32_t mantissa, const ParityStep step)
{
    return mantissa + pick_by_parity(mantissa, step.even, step.odd);
}

// First index in [0, count) at which a predicate that holds on a prefix stops holding; the wave probes
// 64 places per step (three dependent loads for 2^18 items where a bisection takes eighteen).  The
// arguments must be the same in every lane of the wave; every lane receives the result.
template <class Holds>
__device__ __forceinline__ uint32_t wave_partition_point(uint32_t count, Holds holds)
{
    const uint32_t lane = static_cast<uint32_t>(lane_id());
    uint32_t low = 0, high = count;
    while (low < high)
    {
        const uint32_t step = (high - low + kWaveSize - 1u) / kWaveSize;
        const uint32_t probe = low + lane * step;
        const bool ok = probe < high && holds(probe);
        const uint32_t passed = static_cast<uint32_t>(__popcll(__builtin_amdgcn_ballot_w64(ok)));
        if (passed == 0u)
            break;
        high = min(high, low + passed * step);
        low = low + (passed - 1u) * step + 1u;
    }
    return low;
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

// The step a term causes on a sum with biased exponent `exponent`: with the term's mantissa split at
// the sum's ulp into `whole` ulps and a rest, the sum moves by whole ulps, one more when the rest is
// above half an ulp, and on a rest of exactly half to the even neighbour: up when the mantissa and
// `whole` differ in parity.  Adding (half - 1 + [whole odd]) before the shift rounds that way for an
// even mantissa, (half - [whole odd]) for an odd one.
__device__ __forceinline__ ParityStep step_of_term(float term, int exponent)
{
    // Without branches (a workgroup runs this for every term of every round).  A shift of 25 or more, or a
    // term of zero, gives zero by the arithmetic itself: mantissa + half stays below 2^shift.
    const uint32_t bits = __float_as_uint(term);
    const int stored_exponent = static_cast<int>(bits >> 23);
    const int term_exponent = max(stored_exponent, 1);
    const uint32_t term_mantissa = (bits & 0x7fffffu) | (stored_exponent != 0 ? 0x800000u : 0u);
    const int difference = exponent - term_exponent;
    const uint32_t shift = static_cast<uint32_t>(min(max(difference, 1), 25));
    const uint32_t half = 1u << (shift - 1u);
    const uint32_t whole_odd = (term_mantissa >> shift) & 1u;
    const uint32_t even = (term_mantissa + half - 1u + whole_odd) >> shift;
    const uint32_t odd = (term_mantissa + half - whole_odd) >> shift;
    const bool leaves = difference <= 0 && term_mantissa != 0u; // at least half the sum: the addition leaves the binade
    return ParityStep{leaves ? kBinadeFull : even, leaves ? kBinadeFull : odd};
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

// Two copies of everything, used by alternate rounds: a round's values are read after one of its barriers
// and written again two rounds later, with barriers in between, so that a round needs two barriers (three
// with an event) and none at its end.
struct ReplayScratch
{
    ParityStep wave_totals[2][kReplayWaves];
    uint32_t first_event[2]; // (index << 1 | kind) of the earliest event of the round, kind 0 = leaves the binade, 1 = stop
    uint32_t final_mantissa[2];
    float event_sum[2];
    int absorbed[2];
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
    uint32_t known_runs;      // runs only, 0 = unknown: the first known_runs runs hold ...
    uint32_t known_elements;  // ... exactly this many elements
    const float* terms0;      // exp(logit/T - maximum) of every item (element or run), computed beforehand
    const uint4* chunk_steps; // elements only, may be null: (exponent, even step, odd step, valid) of every chunk of terms0 ...
    uint32_t chunk_steps_cover; // ... up to this element (the last chunk may be a partial one)
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

// ... the same for an element that every lane of the wave asks for
__device__ __forceinline__ uint32_t run_of_element_uniform(const SortedRow& row, uint32_t element)
{
    const uint32_t* run_ends = row.run_ends;
    return wave_partition_point(row.run_count, [run_ends, element](uint32_t run) { return run_ends[run] <= element; });
}

// The term of item i that the CPU loop of `PHASE` adds.
template <int PHASE>
__device__ __forceinline__ float row_term(const SortedRow& row, uint32_t i)
{
    float t = row.terms0[i];
    if (PHASE >= 1)
        t = t / row.normalizer;
    if (PHASE >= 2)
        t = t / row.renormalizer;
    return t;
}

// What the rounds of the two running sums below share.  A round has every thread compose the steps of its
// own terms; this turns the threads' totals into the mantissa in front of each thread, finds the first
// event (the sum leaves its binade, or the stop condition first holds) and hands it to every thread.
//   thread_total   composition of the calling thread's steps
//   find_event     called in a thread whose range holds an event, with the mantissa in front of the thread:
//                  fills the event's key (index << 1 | kind), mantissa and term
// Returns kRoundPlain when the round ended without an event: `sum` is then the sum behind the round's last
// term.  With an event (kRoundEvent), `sum` is the sum behind the event's term and event_key names it.
// With CHECK_ABSORBED, thread 0 has written scratch.absorbed[slot] before the call: when set, the round
// is abandoned (kRoundAbsorbed, `sum` unchanged).
enum RoundOutcome : int
{
    kRoundPlain = 0,
    kRoundEvent = 1,
    kRoundAbsorbed = 2
};

struct RoundEvent
{
    uint32_t key;
    uint32_t mantissa; // kind 0: before the term is added; kind 1: behind it
    float term;
};

// The first half of a round: the mantissa in front of the calling thread's terms, and whether the round's
// first event lies among them.
struct RoundFront
{
    uint32_t current;
    bool have_event;
    bool absorbed; // (CHECK_ABSORBED) the round is abandoned; the caller returns at once
};

template <int WAVES, bool CHECK_ABSORBED>
__device__ __forceinline__ RoundFront begin_round(
    const ParityStep& thread_total, uint32_t mantissa, uint32_t limit, ReplayScratch& scratch, uint32_t slot, int tid)
{
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    const bool summing = wave < WAVES; // the other waves only follow the round's barriers and its outcome
    ParityStep exclusive{0u, 0u};
    if (summing)
    {
        const ParityStep inclusive = wave_scan_steps(thread_total);
        exclusive.even = __shfl_up(inclusive.even, 1, kWaveSize);
        exclusive.odd = __shfl_up(inclusive.odd, 1, kWaveSize);
        if (lane == 0)
            exclusive = ParityStep{0u, 0u};
        if (lane == kWaveSize - 1)
            scratch.wave_totals[slot][wave] = inclusive;
    }
    lds_barrier();
    if (tid == 0)
        scratch.first_event[slot ^ 1u] = 0xffffffffu; // for the next round: its readers are behind the barrier
    if (CHECK_ABSORBED)
    {
        if (scratch.absorbed[slot])
        {
            lds_barrier(); // every thread has read the flag before a later call writes it
            return RoundFront{0u, false, true};
        }
    }
    RoundFront front{0u, false, false};
    if (summing)
    {
        ParityStep before{0u, 0u};
        if constexpr (WAVES > 8)
        {
            // many waves: lane w takes wave w's total, and four DPP stages (the lanes share a row of sixteen)
            // compose them in order; the waves in front of this one end at lane wave - 1
            static_assert(WAVES <= 16, "the waves' totals must fit one DPP row");
            ParityStep v = lane < WAVES ? scratch.wave_totals[slot][lane] : ParityStep{0u, 0u};
#define NCNN_MOE_SCAN_STAGE(CONTROL)                                                                         \
    {                                                                                                        \
        const ParityStep earlier{dpp_source<CONTROL, 0xf>(v.even), dpp_source<CONTROL, 0xf>(v.odd)};         \
        v = compose_steps(earlier, v);                                                                       \
    }
            NCNN_MOE_SCAN_STAGE(0x111) // row_shr:1
            NCNN_MOE_SCAN_STAGE(0x112) // row_shr:2
            NCNN_MOE_SCAN_STAGE(0x114) // row_shr:4
            NCNN_MOE_SCAN_STAGE(0x118) // row_shr:8
#undef NCNN_MOE_SCAN_STAGE
            const int source = wave > 0 ? wave - 1 : 0;
            const uint32_t even_there = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v.even), source));
            const uint32_t odd_there = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v.odd), source));
            before = ParityStep{wave > 0 ? even_there : 0u, wave > 0 ? odd_there : 0u};
        }
        else
        {
            // every wave's total is read at once (independent LDS loads); the composition stays in registers
            ParityStep totals[WAVES];
#pragma unroll
            for (int w = 0; w < WAVES; ++w)
                totals[w] = scratch.wave_totals[slot][w];
#pragma unroll
            for (int w = 0; w < WAVES - 1; ++w)
            {
                const ParityStep with = compose_steps(before, totals[w]);
                before = ParityStep{w < wave ? with.even : before.even, w < wave ? with.odd : before.odd};
            }
        }
        before = compose_steps(before, exclusive);
        front.current = apply_step(mantissa, before);
        const uint32_t behind = apply_step(front.current, thread_total);
        // The mantissa never decreases: the first event lies in the thread whose range takes it to the limit.
        // (A round that begins at the limit - a stop bound of zero - has its event at its first term.)
        front.have_event = behind >= limit && (front.current < limit || mantissa >= limit);
        if (tid == WAVES * kWaveSize - 1)
            scratch.final_mantissa[slot] = behind;
    }
    return front;
}

// The second half: `reported` threads have found an event in their range (`found`); the first of them wins.
__device__ __forceinline__ RoundOutcome end_round(
    bool reported, const RoundEvent& found, int exponent, ReplayScratch& scratch, uint32_t slot, float& sum, uint32_t& event_key)
{
    if (reported)
        atomicMin(&scratch.first_event[slot], found.key);
    lds_barrier();
    const uint32_t event = scratch.first_event[slot];
    if (event == 0xffffffffu)
    {
        sum = encode_sum(exponent, scratch.final_mantissa[slot]);
        return kRoundPlain;
    }
    if (reported && found.key == event)
    {
        const float at_event = encode_sum(exponent, found.mantissa);
        scratch.event_sum[slot] = (event & 1u) ? at_event : at_event + found.term;
    }
    lds_barrier();
    sum = scratch.event_sum[slot];
    event_key = event;
    return kRoundEvent;
}

template <int WAVES, bool CHECK_ABSORBED, class FindEvent>
__device__ __forceinline__ RoundOutcome finish_round(
    const ParityStep& thread_total, int exponent, uint32_t mantissa, uint32_t limit, FindEvent find_event,
    ReplayScratch& scratch, uint32_t slot, int tid, float& sum, uint32_t& event_key)
{
    const RoundFront front = begin_round<WAVES, CHECK_ABSORBED>(thread_total, mantissa, limit, scratch, slot, tid);
    if (CHECK_ABSORBED && front.absorbed)
        return kRoundAbsorbed;
    RoundEvent found{0u, 0u, 0.0f};
    bool reported = false;
    if (front.have_event)
        reported = find_event(front.current, found);
    return end_round(reported, found, exponent, scratch, slot, sum, event_key);
}

// The running fp32 sum of the non-negative terms term(0) ... term(count - 1), starting from 0, exactly as
// a sequential loop produces it; term(i) = terms[i], divided by `divisor` and then by `second_divisor` with
// DIVIDED (a divisor of one leaves a term as it is).  With NON_INCREASING (the terms never grow) it also
// stops (without `stopped`) once the sum no longer moves, which is then final.  Every thread of the
// workgroup (kSumThreads or more) must call it.
// CHECK_FIRST: a first term that is not finite is returned as the sum at once (it poisons the sum; the caller need
// not load it beforehand to find out).
template <bool NON_INCREASING, bool DIVIDED, bool CHECK_FIRST = false>
__device__ __forceinline__ RunningSum exact_running_sum_of_array_inline(
    const float* terms_array, float divisor, float second_divisor, uint32_t count, int mode, float bound,
    ReplayScratch& scratch, int tid, const uint4* chunk_steps = nullptr, uint32_t chunk_steps_cover = 0u)
{
    const auto scaled = [divisor, second_divisor](float t) { return DIVIDED ? (t / divisor) / second_divisor : t; };
    const auto term_at = [&](uint32_t i) { return scaled(terms_array[i]); };
    const int lane = tid & (kWaveSize - 1);
    float sum = 0.0f;
    const uint32_t head = min(count, static_cast<uint32_t>(kSequentialHead));
    // the terms of the next chunk are asked for while this one is summed
    float upcoming[kReplayPerThread];
    const bool summing = tid < kSumThreads;
    const bool aligned = (reinterpret_cast<uintptr_t>(terms_array) & 15u) == 0u;
    const auto fetch = [&](uint32_t base) {
        const uint32_t chunk_end = min(count, base + static_cast<uint32_t>(kReplayChunk));
        const uint32_t first = base + static_cast<uint32_t>(tid) * kReplayPerThread;
        if (aligned && first + kReplayPerThread <= chunk_end)
        {
            // (only whole groups: nothing is read behind `count`)
#pragma unroll
            for (int j = 0; j < kReplayPerThread; j += 4)
            {
                const float4 four = *reinterpret_cast<const float4*>(terms_array + first + j);
                upcoming[j + 0] = four.x;
                upcoming[j + 1] = four.y;
                upcoming[j + 2] = four.z;
                upcoming[j + 3] = four.w;
            }
        }
        else
        {
#pragma unroll
            for (int j = 0; j < kReplayPerThread; ++j)
                upcoming[j] = (summing && first + j < chunk_end) ? terms_array[first + j] : 0.0f;
        }
    };
    // A sum that runs over the whole row (the normaliser) asks for everything it will need first - the composed
    // steps of the first 64 whole chunks, one per lane, and the first chunk's terms - so that the loads of the
    // head below are not the first of three trips to memory, one behind the other.
    uint4 own_chunk_steps{0u, 0u, 0u, 0u};
    if (NON_INCREASING && !DIVIDED && chunk_steps != nullptr &&
        static_cast<uint32_t>(lane) < (chunk_steps_cover + static_cast<uint32_t>(kReplayChunk) - 1u) / kReplayChunk)
        own_chunk_steps = chunk_steps[lane];
    if (NON_INCREASING && count > head)
        fetch(0);
    // The first kSequentialHead terms are added in order, as the CPU does, 64 at a time with a term per lane
    // (every wave does the same): the sum climbs through most of its binades here, each of which would cost
    // the scan below a round, and a stop condition usually holds this early.
    {
        float head_terms[kHeadSlots];
#pragma unroll
        for (int slot = 0; slot < kHeadSlots; ++slot)
        {
            const uint32_t i = static_cast<uint32_t>(slot * kWaveSize + lane);
            head_terms[slot] = i < head ? term_at(i) : 0.0f;
        }
        if (CHECK_FIRST)
        {
            const float first_term = read_lane(head_terms[0], 0);
            if (!is_finite_f32(first_term))
                return RunningSum{first_term, 0u, false};
        }
#pragma unroll
        for (int slot = 0; slot < kHeadSlots; ++slot)
        {
            const uint32_t slot_first = static_cast<uint32_t>(slot * kWaveSize);
            if (slot > 0 && slot_first >= head)
                break;
            // (the sum so far goes in front of the slot's first term: one addition, the one the loop would make)
            const float own = (slot > 0 && lane == 0) ? sum + head_terms[slot] : head_terms[slot];
            const float sums = wave_sequential_sums(own); // (lanes behind the head add zero: they hold the head's sum)
            const bool stops = slot_first + static_cast<uint32_t>(lane) < head &&
                ((mode == kStopAtOrAbove && sums >= bound) || (mode == kStopAbove && sums > bound));
            const uint64_t stopping = __builtin_amdgcn_ballot_w64(stops);
            if (stopping != 0ull)
            {
                const int first = __builtin_ctzll(stopping);
                return RunningSum{read_lane(sums, first), slot_first + static_cast<uint32_t>(first), true};
            }
            sum = read_lane(sums, kWaveSize - 1);
        }
        if (head >= count)
            return RunningSum{sum, 0u, false};
    }
    if (tid == 0)
        scratch.first_event[0] = 0xffffffffu;
    uint32_t round = 0;
    if (!NON_INCREASING)
        fetch(0);
    bool fetched = true; // `upcoming` holds the terms of the chunk at `base`
    for (uint32_t base = 0; base < count; base += kReplayChunk)
    {
        const uint32_t chunk_end = min(count, base + static_cast<uint32_t>(kReplayChunk));
        if (NON_INCREASING && !DIVIDED && chunk_steps != nullptr && mode == kStopNever && head == static_cast<uint32_t>(kSequentialHead))
        {
            // Chunks whose composed step was worked out beforehand for the exponent that the sum has now: if that
            // step leaves the mantissa inside the binade, nothing inside the chunk left it either (the mantissa
            // never decreases), and the chunk is this one addition.  A chunk's step is usable when the sum's
            // terms cover the chunk as far as the step does.
            const uint32_t chunk = base / kReplayChunk;
            int exponent;
            uint32_t mantissa;
            decode_sum(sum, exponent, mantissa);
            if (chunk < static_cast<uint32_t>(kWaveSize))
            {
                // lane c holds the step of chunk c: all the chunks from this one on that can be added so, at once
                // (a scan over the lanes; a row's flat tail is some dozens of such chunks, one after the other)
                const uint32_t lane_base = static_cast<uint32_t>(lane) * kReplayChunk;
                const bool usable = static_cast<uint32_t>(lane) >= chunk && lane_base < count &&
                    min(count, lane_base + static_cast<uint32_t>(kReplayChunk)) == min(chunk_steps_cover, lane_base + static_cast<uint32_t>(kReplayChunk)) &&
                    own_chunk_steps.w != 0u && own_chunk_steps.x == static_cast<uint32_t>(exponent);
                const ParityStep through = wave_scan_steps(ParityStep{usable ? own_chunk_steps.y : 0u, usable ? own_chunk_steps.z : 0u});
                const uint32_t behind = apply_step(mantissa, through);
                const uint64_t not_so = __builtin_amdgcn_ballot_w64(static_cast<uint32_t>(lane) >= chunk && !(usable && behind < kBinadeFull));
                const uint64_t still = __builtin_amdgcn_ballot_w64(usable && own_chunk_steps.y == 0u && own_chunk_steps.z == 0u);
                const uint32_t first_not_so = not_so != 0ull ? static_cast<uint32_t>(__builtin_ctzll(not_so)) : static_cast<uint32_t>(kWaveSize);
                const uint32_t first_still = still != 0ull ? static_cast<uint32_t>(__builtin_ctzll(still)) : static_cast<uint32_t>(kWaveSize);
                const uint32_t stop = min(first_not_so, first_still);
                if (stop > chunk)
                    sum = encode_sum(exponent, static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(behind), static_cast<int>(stop - 1u))));
                if (first_still < first_not_so)
                    return RunningSum{sum, 0u, false}; // no term of that chunk moves the sum: none behind it can
                if (stop > chunk)
                {
                    base = (stop - 1u) * kReplayChunk; // (the loop moves on to chunk `stop`)
                    fetched = false;
                    continue;
                }
            }
            else if (chunk_end == min(chunk_steps_cover, base + static_cast<uint32_t>(kReplayChunk)))
            {
                const uint4 composed = chunk_steps[chunk];
                if (composed.w != 0u && composed.x == static_cast<uint32_t>(exponent))
                {
                    const uint32_t behind = apply_step(mantissa, ParityStep{composed.y, composed.z});
                    if (behind < kBinadeFull)
                    {
                        if (composed.y == 0u && composed.z == 0u)
                            return RunningSum{sum, 0u, false}; // no term of the chunk moves the sum: none behind it can
                        sum = encode_sum(exponent, behind);
                        fetched = false;
                        continue;
                    }
                }
            }
        }
        if (!fetched)
            fetch(base);
        fetched = true;
        const uint32_t thread_first = base + static_cast<uint32_t>(tid) * kReplayPerThread;
        float terms[kReplayPerThread];
#pragma unroll
        for (int j = 0; j < kReplayPerThread; ++j)
            terms[j] = DIVIDED ? upcoming[j] / divisor : upcoming[j];
        // (a second divisor of one, the Top-P walk's, leaves the quotients as they are: eight divisions not made)
        if (DIVIDED && second_divisor != 1.0f)
        {
#pragma unroll
            for (int j = 0; j < kReplayPerThread; ++j)
                terms[j] = terms[j] / second_divisor;
        }
        if (base + kReplayChunk < count)
            fetch(base + kReplayChunk);
        uint32_t start = max(base, head);
        while (start < chunk_end)
        {
            int exponent;
            uint32_t mantissa;
            decode_sum(sum, exponent, mantissa);
            const uint32_t stop_at = stop_mantissa(mode, bound, exponent);
            const uint32_t limit = min(stop_at, kBinadeFull);
            const uint32_t slot = round & 1u;
            ++round;
            NCNN_MOE_COUNT(blockIdx.x, 15, 12);
        
            const auto step_at = [&](int j) {
                const uint32_t i = thread_first + j;
                const ParityStep step = step_of_term(terms[j], exponent);
                const bool active = i >= start && i < chunk_end;
                return ParityStep{active ? step.even : 0u, active ? step.odd : 0u};
            };
            ParityStep steps[kReplayPerThread];
            ParityStep thread_total{0u, 0u};
#pragma unroll
            for (int j = 0; j < kReplayPerThread; ++j)
            {
                steps[j] = summing ? step_at(j) : ParityStep{0u, 0u};
                thread_total = compose_steps(thread_total, steps[j]);
            }
            if (NON_INCREASING)
            {
                // the largest remaining term of the row does not move the sum: nothing later can
                if (tid == 0)
                {
                    const ParityStep first_step = steps[0];
                    scratch.absorbed[slot] = (start == base && base > 0 && first_step.even == 0u && first_step.odd == 0u) ? 1 : 0;
                }
            }
            const RoundFront front = begin_round<kSumWaves, NON_INCREASING>(thread_total, mantissa, limit, scratch, slot, tid);
            if (NON_INCREASING && front.absorbed)
                return RunningSum{sum, 0u, false};
            // The thread whose range holds the round's first event walks its terms from the mantissa in front of
            // them, with the steps worked out above and without a branch (every other thread waits for it).
            RoundEvent found{0u, 0u, 0.0f};
            bool hit = false;
            if (front.have_event)
            {
                uint32_t current = front.current;
#pragma unroll
                for (int j = 0; j < kReplayPerThread; ++j)
                {
                    const uint32_t i = thread_first + static_cast<uint32_t>(j);
                    const bool active = i >= start && i < chunk_end;
                    const uint32_t next = apply_step(current, steps[j]); // (a term that is not active has no step)
                    const bool leaves = next >= kBinadeFull;
                    const bool here = active && !hit && (leaves || next >= stop_at);
                    found.key = here ? ((i << 1) | (leaves ? 0u : 1u)) : found.key;
                    found.mantissa = here ? (leaves ? current : next) : found.mantissa;
                    found.term = here ? (leaves ? terms[j] : 0.0f) : found.term;
                    hit = hit || here;
                    current = next;
                }
            }
            uint32_t event = 0;
            const RoundOutcome outcome = end_round(hit, found, exponent, scratch, slot, sum, event);
            if (outcome == kRoundAbsorbed)
                return RunningSum{sum, 0u, false};
            if (outcome == kRoundPlain)
                break;
            const uint32_t event_index = event >> 1;
            if (event & 1u)
                return RunningSum{sum, event_index, true};
            if ((mode == kStopAtOrAbove && sum >= bound) || (mode == kStopAbove && sum > bound))
                return RunningSum{sum, event_index, true};
            start = event_index + 1u;
        }
    }
    return RunningSum{sum, 0u, false};
}

// ... as a function of its own: a kernel that sums several times (Top-P walk, draw, the verification's residual)
// holds one copy of it.
template <bool NON_INCREASING, bool DIVIDED>
__device__ __noinline__ RunningSum exact_running_sum_of_array(
    const float* terms_array, float divisor, float second_divisor, uint32_t count, int mode, float bound,
    ReplayScratch& scratch, int tid, const uint4* chunk_steps = nullptr, uint32_t chunk_steps_cover = 0u)
{
    return exact_running_sum_of_array_inline<NON_INCREASING, DIVIDED>(terms_array, divisor, second_divisor, count, mode, bound, scratch, tid, chunk_steps, chunk_steps_cover);
}

// The running sum of terms [0, count) of a sorted row.  PHASE 0 (terms that never grow) also stops
// once the sum no longer moves.  Every thread of the workgroup must call it.
template <int PHASE>
__device__ __forceinline__ RunningSum exact_running_sum(
    const SortedRow& row, uint32_t count, int mode, float bound, ReplayScratch& scratch, int tid)
{
    if constexpr (PHASE == 0) // the normaliser: one call per kernel, inlined (a call saves and restores its registers through memory)
        return exact_running_sum_of_array_inline<true, false, true>(row.terms0, 1.0f, 1.0f, count, mode, bound, scratch, tid, row.chunk_steps, row.chunk_steps_cover);
    else
        return exact_running_sum_of_array<false, true>(
            row.terms0, row.normalizer, PHASE == 2 ? row.renormalizer : 1.0f, count, mode, bound, scratch, tid, nullptr);
}

// The same running sum over a row stored as runs: `count` elements are added, run after run.  A run of
// m equal terms is one step (repeat_steps); when an event (the sum leaves its binade, or the stop
// condition first holds) falls inside a run, the thread that owns the run finds the addition it
// falls on by bisection over repeated_step, which is monotone in the number of additions.
template <bool FIRST>
__device__ __noinline__ RunningSum exact_running_sum_runs_scaled(
    const SortedRow& row, float divisor, float second_divisor, uint32_t count, int mode, float bound, ReplayScratch& scratch, int tid)
{
    // FIRST: the terms as they are (they never grow: the sum also stops once it no longer moves); else
    // divided by the two divisors, one after the other (a divisor of one leaves a term as it is)
    const float* const terms0 = row.terms0;
    const uint32_t* const run_ends = row.run_ends;
    const auto term_of_run = [terms0, divisor, second_divisor](uint32_t run) {
        const float t = terms0[run];
        return FIRST ? t : (t / divisor) / second_divisor;
    };
    const int lane = tid & (kWaveSize - 1);
    float sum = 0.0f;
    if (count == 0u)
        return RunningSum{sum, 0u, false};
    // runs that hold the elements in front of `count` (the caller may know it for its whole row)
    const uint32_t runs = (row.known_runs != 0u && count == row.known_elements) ? row.known_runs
                                                                               : run_of_element_uniform(row, count - 1u) + 1u;
    uint32_t start = 0; // elements before this one have been added
    uint32_t first_run; // the run that holds element `start`

    // The first kSequentialHeadOfRuns elements are added in order, as the CPU does, an element per lane (every
    // wave does the same): the sum climbs through most of its binades here, each of which would cost the
    // scan below a round, and a stop condition usually holds this early.
    {
        static_assert(kSequentialHeadOfRuns == kWaveSize, "the head is one element per lane");
        const uint32_t head_runs = min(runs, static_cast<uint32_t>(kWaveSize));
        const float head_term = static_cast<uint32_t>(lane) < head_runs ? term_of_run(static_cast<uint32_t>(lane)) : 0.0f;
        // (a lane without a run: an end that no element lies behind)
        const uint32_t head_end = static_cast<uint32_t>(lane) < head_runs ? min(run_ends[lane], count) : 0xffffffffu;
        const uint32_t head_limit = min(count, static_cast<uint32_t>(kSequentialHeadOfRuns));
        // Bit b of `last_elements`: a run ends with element b.  The run of element `lane` is the number of runs that
        // end in front of it: the bits below `lane`.  (The ends ascend, one run per lane: no bit is set twice.)
        const bool ends_in_head = head_end <= static_cast<uint32_t>(kWaveSize);
        const uint32_t last_element = head_end - 1u;
        const uint32_t low_bits = wave_or_u32(ends_in_head && last_element < 32u ? 1u << last_element : 0u);
        const uint32_t high_bits = wave_or_u32(ends_in_head && last_element >= 32u ? 1u << (last_element - 32u) : 0u);
        const uint64_t last_elements = (static_cast<uint64_t>(high_bits) << 32) | low_bits;
        const uint32_t run = static_cast<uint32_t>(__popcll(last_elements & ((1ull << lane) - 1ull)));
        const float term_there = __shfl(head_term, static_cast<int>(run), kWaveSize);
        const float own = static_cast<uint32_t>(lane) < head_limit ? term_there : 0.0f;
        const float sums = wave_sequential_sums(own); // (lanes behind the head add zero: they hold the head's sum)
        const bool stops = static_cast<uint32_t>(lane) < head_limit &&
            ((mode == kStopAtOrAbove && sums >= bound) || (mode == kStopAbove && sums > bound));
        const uint64_t stopping = __builtin_amdgcn_ballot_w64(stops);
        if (stopping != 0ull)
        {
            const int first = __builtin_ctzll(stopping);
            return RunningSum{read_lane(sums, first), static_cast<uint32_t>(first), true};
        }
        sum = read_lane(sums, kWaveSize - 1);
        start = head_limit;
        if (start >= count)
            return RunningSum{sum, 0u, false};
        // (start is 64 here: every run that ends inside the head ends in front of it)
        first_run = static_cast<uint32_t>(__popcll(last_elements));
    }
    if (tid == 0)
        scratch.first_event[0] = 0xffffffffu;
    uint32_t round = 0;
    // A thread takes kRunsPerThread consecutive runs and the workgroup kRunsChunk; a chunk costs a round, and one
    // more for each binade the sum leaves inside it (measured on 256 rows of 201,088 bf16 logits, ~5,500 runs each:
    // 2 runs x 8 waves 67.3 us, 2 x 4 68.5, 4 x 8 69.5, 1 x 16 69.7, 4 x 16 69.9, 2 x 16 70.1, 1 x 8 71.1, 8 x 16 74.3:
    // a round over a long chunk repeats more work after every event than the rounds of short chunks cost).
    // The chunks start at a multiple of kRunsPerThread, so that a thread's runs are whole groups of the arrays
    // (runs in front of `start` add nothing: their elements are clipped away below).
    static_assert((kRunsPerThread & (kRunsPerThread - 1)) == 0, "the chunks start at a multiple of a thread's runs");
    constexpr bool kGroups = kRunsPerThread % 4 == 0; // a thread's runs are loaded in groups of four
    const uint32_t first_base = first_run & ~static_cast<uint32_t>(kRunsPerThread - 1);
    const bool groups_aligned = kGroups &&
        ((reinterpret_cast<uintptr_t>(terms0) | reinterpret_cast<uintptr_t>(run_ends)) & 15u) == 0u;
    for (uint32_t base = first_base; base < runs; base += kRunsChunk)
    {
        const uint32_t chunk_end = min(runs, base + static_cast<uint32_t>(kRunsChunk));
        const uint32_t thread_first = base + static_cast<uint32_t>(tid) * kRunsPerThread;
        float terms[kRunsPerThread];
        uint32_t firsts[kRunsPerThread]; // first and one-past-last element of each run, clipped to count
        uint32_t lasts[kRunsPerThread];
        const bool summing = tid < kRunsWaves * kWaveSize;
        if (groups_aligned && summing && thread_first + kRunsPerThread <= chunk_end)
        {
            float loaded[kRunsPerThread];
            uint32_t ends[kRunsPerThread];
#pragma unroll
            for (int g = 0; g + 4 <= kRunsPerThread; g += 4)
            {
                const float4 t = *reinterpret_cast<const float4*>(terms0 + thread_first + g);
                const uint4 e = *reinterpret_cast<const uint4*>(run_ends + thread_first + g);
                loaded[g + 0] = t.x, loaded[g + 1] = t.y, loaded[g + 2] = t.z, loaded[g + 3] = t.w;
                ends[g + 0] = e.x, ends[g + 1] = e.y, ends[g + 2] = e.z, ends[g + 3] = e.w;
            }
            const uint32_t before = thread_first == 0u ? 0u : run_ends[thread_first - 1u];
#pragma unroll
            for (int j = 0; j < kRunsPerThread; ++j)
            {
                terms[j] = FIRST ? loaded[j] : (loaded[j] / divisor) / second_divisor;
                firsts[j] = j == 0 ? before : ends[j - 1];
                lasts[j] = min(ends[j], count);
            }
        }
        else
        {
#pragma unroll
            for (int j = 0; j < kRunsPerThread; ++j)
            {
                const uint32_t i = thread_first + j;
                const bool valid = summing && i < chunk_end;
                terms[j] = valid ? term_of_run(i) : 0.0f;
                firsts[j] = valid ? run_first_element(row, i) : 0u;
                lasts[j] = valid ? min(run_ends[i], count) : 0u;
            }
        }
        bool fresh = true; // no event in this chunk yet
        while (true)
        {
            int exponent;
            uint32_t mantissa;
            decode_sum(sum, exponent, mantissa);
            const uint32_t stop_at = stop_mantissa(mode, bound, exponent);
            const uint32_t limit = min(stop_at, kBinadeFull);
            const uint32_t slot = round & 1u;
            ++round;
            NCNN_MOE_COUNT(blockIdx.x, 15, 13);

            // A run of m equal terms moves the mantissa m times by the term's step - unless the term ends exactly
            // half an ulp above a multiple of the ulp (its two steps differ): where a lane of the wave holds such
            // a run, the wave works that run's two totals out the long way.  A wave none of whose runs has an
            // element left (all in front of `start`, or behind `count`) composes nothing.
            ParityStep thread_total{0u, 0u};
            ParityStep run_totals[kRunsPerThread]; // of each run's additions, for the search for an event
            ParityStep first_single{0u, 0u};
            uint32_t first_multiplicity = 0;
            bool live = false;
#pragma unroll
            for (int j = 0; j < kRunsPerThread; ++j)
                run_totals[j] = ParityStep{0u, 0u};
#pragma unroll
            for (int j = 0; j < kRunsPerThread; ++j)
                live = live || lasts[j] > max(firsts[j], start);
            if (__builtin_amdgcn_ballot_w64(live) != 0ull)
            {
#pragma unroll
                for (int j = 0; j < kRunsPerThread; ++j)
                {
                    const uint32_t low = max(firsts[j], start);
                    const uint32_t multiplicity = lasts[j] > low ? lasts[j] - low : 0u;
                    const ParityStep single = step_of_term(terms[j], exponent);
                    if (j == 0)
                    {
                        first_single = single;
                        first_multiplicity = multiplicity;
                    }
                    const uint64_t product = static_cast<uint64_t>(single.even) * multiplicity;
                    const uint32_t repeated = product > kStepCap ? kStepCap : static_cast<uint32_t>(product);
                    ParityStep run_total{repeated, repeated};
                    if (__builtin_amdgcn_ballot_w64(single.even != single.odd && multiplicity != 0u) != 0ull)
                        run_total = ParityStep{repeated_step(false, single, multiplicity), repeated_step(true, single, multiplicity)};
                    run_totals[j] = run_total;
                    thread_total = compose_steps(thread_total, run_total);
                }
            }
            if (FIRST)
            {
                // the largest remaining term of the row does not move the sum: nothing later can
                if (tid == 0)
                    scratch.absorbed[slot] =
                        (fresh && base > first_base && (first_multiplicity == 0u || (first_single.even == 0u && first_single.odd == 0u))) ? 1 : 0;
            }
            const auto find_event = [&](uint32_t current, RoundEvent& found) -> bool {
                // The thread's first run whose additions take the mantissa to the limit (from the registers: no
                // branch, no load), then the first such addition of that run.
                bool hit = false;
                uint32_t hit_low = 0, hit_multiplicity = 0, hit_current = 0;
                float hit_term = 0.0f;
#pragma unroll
                for (int j = 0; j < kRunsPerThread; ++j)
                {
                    const uint32_t low = max(firsts[j], start);
                    const uint32_t multiplicity = lasts[j] > low ? lasts[j] - low : 0u;
                    const uint32_t next = apply_step(current, run_totals[j]);
                    const bool here = !hit && multiplicity > 0u && next >= limit;
                    hit_low = here ? low : hit_low;
                    hit_multiplicity = here ? multiplicity : hit_multiplicity;
                    hit_current = here ? current : hit_current;
                    hit_term = here ? terms[j] : hit_term;
                    hit = hit || here;
                    current = next;
                }
                if (!hit)
                    return false;
                const ParityStep single = step_of_term(hit_term, exponent);
                const bool odd = (hit_current & 1u) != 0u;
                // repeated additions: `none` of them stay below the limit, one more reaches it
                uint32_t none = 0u;
                if (single.even == single.odd)
                {
                    // every addition moves the mantissa by the same step: a division finds the first that arrives
                    // (a mantissa at the limit already - a stop bound of zero - has its event at the first addition)
                    if (hit_current < limit && single.even != 0u)
                        none = (limit - 1u - hit_current) / single.even;
                }
                else
                {
                    uint32_t some = hit_multiplicity; // this many reach it
                    while (some - none > 1u)
                    {
                        const uint32_t middle = none + ((some - none) >> 1);
                        if (hit_current + repeated_step(odd, single, middle) >= limit)
                            some = middle;
                        else
                            none = middle;
                    }
                }
                const uint32_t before_event = hit_current + repeated_step(odd, single, none);
                const uint32_t after_event = apply_step(before_event, single);
                const uint32_t element = hit_low + none;
                if (after_event >= kBinadeFull)
                    found = RoundEvent{element << 1, before_event, hit_term};
                else
                    found = RoundEvent{(element << 1) | 1u, after_event, 0.0f};
                return true;
            };
            uint32_t event = 0;
            const RoundOutcome outcome =
                finish_round<kRunsWaves, FIRST>(thread_total, exponent, mantissa, limit, find_event, scratch, slot, tid, sum, event);
            if (outcome == kRoundAbsorbed)
                return RunningSum{sum, 0u, false};
            if (outcome == kRoundPlain)
                break;
            const uint32_t event_element = event >> 1;
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

template <int PHASE>
__device__ __forceinline__ RunningSum exact_running_sum_runs(
    const SortedRow& row, uint32_t count, int mode, float bound, ReplayScratch& scratch, int tid)
{
    return exact_running_sum_runs_scaled<PHASE == 0>(
        row, row.normalizer, PHASE == 2 ? row.renormalizer : 1.0f, count, mode, bound, scratch, tid);
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
    const uint32_t* sorted_indices, uint8_t flags, ReplayScratch& scratch, int tid, TokenAt token_at,
    const float* terms0 = nullptr, const uint4* chunk_steps = nullptr, uint32_t chunk_steps_cover = 0u,
    uint32_t known_runs = 0u, uint32_t known_elements = 0u, uint32_t sorted_elements = 0xffffffffu, uint32_t tail_key = 0u,
    bool* tail_matters = nullptr)
{
#ifdef NCNN_MOE_TIMELINE
    const uint32_t stamp_row = a.only_pending ? 0xffffffffu : row; // the full-order rows' stamps (not the wide select's)
#endif
    SortedRow sorted;
    sorted.keys = keys;
    sorted.run_ends = run_ends;
    sorted.run_count = run_count;
    sorted.known_runs = RUNS ? known_runs : 0u;
    sorted.known_elements = known_elements;
    sorted.terms0 = terms0;
    sorted.chunk_steps = RUNS ? nullptr : chunk_steps;
    sorted.chunk_steps_cover = chunk_steps_cover;
    sorted.temperature = p.temperature;
    sorted.maximum = value_from_descending_key(keys[0]) / p.temperature;
    sorted.normalizer = 1.0f;
    sorted.renormalizer = 1.0f;
    // A row sorted in part (elements only): `keys` holds its first sorted_elements elements in sorted order, and
    // every element behind them has a key of tail_key or more, a term of at most tail_term.  A sum that runs
    // past the sorted elements is the sum over those, as long as the largest term of the tail does not move it
    // (neither does any smaller one, and a sum that does not move meets no stop condition that it has not met);
    // where it could, *tail_matters is set and the caller has the row sorted whole.
    const bool sorted_in_part = !RUNS && sorted_elements < n;
    // (the exp may be off its neighbours' by an ulp: the bound is taken a little above it)
    const float tail_term =
        sorted_in_part ? expf_libm(value_from_descending_key(tail_key) / p.temperature - sorted.maximum) * 1.00001f : 0.0f;
    bool tail_moves = false;
    auto running_sum = [&](auto phase, uint32_t count, int mode, float bound) -> RunningSum {
        constexpr int kPhase = decltype(phase)::value;
        if constexpr (RUNS)
            return exact_running_sum_runs<kPhase>(sorted, count, mode, bound, scratch, tid);
        else
        {
            const uint32_t covered = min(count, sorted_elements);
            const RunningSum result = exact_running_sum<kPhase>(sorted, covered, mode, bound, scratch, tid);
            if (covered < count && !result.stopped)
            {
                float largest = tail_term;
                if (kPhase >= 1)
                    largest = largest / sorted.normalizer;
                if (kPhase >= 2)
                    largest = largest / sorted.renormalizer;
                int exponent;
                uint32_t mantissa;
                decode_sum(result.sum, exponent, mantissa);
                const ParityStep step = step_of_term(largest, exponent);
                tail_moves = tail_moves || step.even != 0u || step.odd != 0u || !is_finite_f32(result.sum);
            }
            return result;
        }
    };
    const auto leave_to_whole_sort = [&]() {
        if (tail_matters != nullptr)
            *tail_matters = true;
    };
    // the item (element, or run) that holds an element
    auto item_of = [&](uint32_t element) -> uint32_t { // for an element that the whole wave asks for
        if constexpr (RUNS)
            return run_of_element_uniform(sorted, element);
        else
            return element;
    };

    // ---- normaliser (session.cpp:92-103).  A first term that is not finite poisons the sum.
    float normalizer;
    if constexpr (RUNS)
    {
        const float first_term = row_term<0>(sorted, 0);
        normalizer = first_term;
        if (is_finite_f32(first_term))
            normalizer = running_sum(std::integral_constant<int, 0>{}, n, kStopNever, 0.0f).sum;
    }
    else
        normalizer = running_sum(std::integral_constant<int, 0>{}, n, kStopNever, 0.0f).sum; // (checks the first term itself)
    if (tail_moves)
        return leave_to_whole_sort();
    if (!is_finite_f32(normalizer) || !(normalizer > 0.0f))
    {
        if (tid == 0)
            write_error(a, row, NCNN_MOE_ROW_INVALID_DISTRIBUTION, flags);
        return;
    }
    sorted.normalizer = normalizer;
    NCNN_MOE_STAMP(stamp_row, 15, 3);

    // ---- Min-P (session.cpp:107-117): probabilities are non-increasing, so the survivors are a prefix
    uint32_t candidates = n;
    if (p.min_p > 0.0f)
    {
        const float threshold = row_term<1>(sorted, 0) * p.min_p;
        // first item whose probability is below the threshold
        const uint32_t first = wave_partition_point(
            RUNS ? item_of(n - 1u) + 1u : min(n, sorted_elements),
            [&sorted, threshold](uint32_t item) { return row_term<1>(sorted, item) >= threshold; });
        if constexpr (RUNS)
            candidates = min(n, run_first_element(sorted, first));
        else
        {
            candidates = first;
            // every sorted element survives: the cut lies in the tail unless the tail's largest term is below it
            if (sorted_in_part && first == sorted_elements && tail_term / sorted.normalizer >= threshold)
                return leave_to_whole_sort();
        }
    }

    NCNN_MOE_STAMP(stamp_row, 15, 4);
    // ---- Top-P (session.cpp:119-128) and the renormaliser (:130-132), which adds the same values
    const RunningSum nucleus = running_sum(std::integral_constant<int, 1>{}, candidates, kStopAtOrAbove, p.top_p);
    if (tail_moves)
        return leave_to_whole_sort();
    const uint32_t kept = nucleus.stopped ? nucleus.stop_index + 1u : candidates;
    sorted.renormalizer = nucleus.sum;
    NCNN_MOE_STAMP(stamp_row, 15, 5);

    if (a.distribution_count != nullptr && sorted_indices != nullptr)
    {
        const size_t first = static_cast<size_t>(row) * a.distribution_cap;
        const uint32_t limit = kept < a.distribution_cap ? kept : a.distribution_cap;
        for (uint32_t i = tid; i < limit; i += blockDim.x)
        {
            a.distribution_ids[first + i] = static_cast<int32_t>(sorted_indices[i]);
            a.distribution_probabilities[first + i] = row_term<2>(sorted, RUNS ? run_of_element(sorted, i) : i);
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
    // (a draw that no partial sum exceeds takes the last kept element, which a row sorted in part may not hold)
    if (tail_moves || (sorted_in_part && selected >= sorted_elements))
        return leave_to_whole_sort();
    NCNN_MOE_STAMP(stamp_row, 15, 6);
    const int32_t token = token_at(selected);
    NCNN_MOE_STAMP(stamp_row, 15, 7);
    const float probability = row_term<2>(sorted, item_of(selected)); // (item_of: every lane takes part)
    if (tid == 0)
        write_token(a, row, p, token, probability, kept, 1, flags);
}

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_SAMPLER_EXACT_SUM_H
