// Shared pieces of the sampler kernels: launch arguments, result writers, logits vector traits,
// agent-scope accesses, integer keys, wave-level selection, and the one-wave epilogue.
#ifndef NCNN_MOE_HIP_SAMPLER_COMMON_H
#define NCNN_MOE_HIP_SAMPLER_COMMON_H

#include "sampler_device.h"

namespace ncnn_moe_hip {

struct SamplerArgs
{
    const void* logits;
    uint64_t row_stride; // elements
    uint32_t rows;
    uint32_t vocab;
    uint32_t segments;           // workgroups per row in the select kernel
    uint32_t chunks_per_segment; // chunks (512 x 5 fp32 / 3 bf16 vectors) one workgroup streams
    uint32_t max_select_top_k;   // widest Top-K window the select kernel of this launch serves
    int force_general;
    int only_pending;            // wide select: 1 = serve the rows an earlier launch of the call left pending; 2 = serve the rows
                                 // whose options ask for a window of 65 to 1024, whatever their state (it runs beside the first select)
    int leave_wide_rows;         // first select and full-order kernels: rows that the wide select serves are another stream's

    const ncnn_moe_sample_params* params;
    const float* uniforms;
    const int32_t* stop_ids;
    ncnn_moe_sample_result* results;

    // select-path scratch
    float* segment_values;     // [rows][segments][kSegmentRecordSlots]
    int32_t* segment_indices;  // [rows][segments][kSegmentRecordSlots]
    uint32_t* segment_counts;  // [rows][segments]
    // [rows], zero between launches: bits 0-7 count the row's finished segments, bits 8 + 6 x count
    // those that ran on XCD x
    unsigned long long* row_counter;
    uint32_t xcd_grouped;      // the grid is one-dimensional and puts the segments of a row on one XCD
    uint32_t* row_flags;       // [rows], zero between launches
    uint32_t* row_state;       // [rows], written by every launch
    // split path: [rows][kSplitMaxSegments][kSplitRecordSlots] entries of (key, epoch | token index), and the
    // row's epoch (1 .. 8191; the row's last workgroup moves it on in every launch)
    unsigned long long* split_records;
    uint32_t* row_epoch;

    // general-path scratch, [rows][sort_stride] each
    uint32_t* sort_keys[2];
    uint32_t* sort_indices[2];
    uint64_t sort_stride;
    // full-order path with a row's sort spread over several workgroups: [rows][sort_parts][256] digit counts
    // of the pass in flight, the number of parts, tiles (kSortTile keys) per part, and the pass
    uint32_t* sort_part_counts;
    uint32_t sort_parts;
    uint32_t sort_tiles_per_part;
    uint32_t sort_pass;
    // full_order_terms_kernel has run: sort_keys[0] holds exp(logit/T - maximum) of the sorted rows' elements
    uint32_t terms_precomputed;
    // ... and what every whole chunk of kReplayChunk of them does to a running sum of a guessed exponent:
    // term_sums [rows][term_sum_parts] (fp64 sums of the terms kernel's blocks), chunk_steps [rows][chunk_capacity]
    // (exponent, step on an even mantissa, step on an odd one, valid); chunk_steps_ready: the kernels that fill them have run
    double* term_sums;
    uint4* chunk_steps;
    uint32_t term_sum_parts;
    uint32_t chunk_capacity;
    uint32_t chunk_steps_ready;

    // optional filtered-distribution output: row r writes at most distribution_cap (id, probability)
    // entries from r * distribution_cap on, and its full kept length to distribution_count[r]
    int32_t* distribution_ids;
    float* distribution_probabilities;
    uint32_t distribution_cap;
    uint32_t* distribution_count;

    // the rows that the full-order kernels serve, listed by full_order_row_list_kernel: [0] their number, then
    // the rows in ascending order.  Kernels over a (parts, rows) grid look their row up here (null: in row_state).
    // (The struct's last member: what the select kernels read keeps its place among the kernel's arguments.)
    const uint32_t* row_list;

    // Full-order fp32 rows sorted only as far as their terms can move a sum (full_order_cut_kernel), all [rows]
    // (null: every row is sorted whole): the last key among the elements that are sorted (every element with a
    // larger key is left out; 0xffffffff: none is), their number, and the row's finite logits (with kRowHoldsNan).
    uint32_t* sort_lengths;
    uint32_t* sort_last_keys;
    uint32_t* finite_counts;
    // The spread sort of such rows may leave out the keys' lowest byte (sort_low_digit_skipped = 1: three passes,
    // over bits 8 to 31, which end in sort_keys[0]).  full_order_terms_kernel then puts the few neighbours that
    // agree in their upper 24 bits in order on its way through the keys (into sort_keys[1]; the terms go to
    // sort_indices[0]), and notes in disordered_rows [rows] a row in which it cannot (such keys too many in a
    // row to see them all, and out of order): that row is sorted whole by the launch behind this one.
    uint32_t* disordered_rows;
    uint32_t sort_low_digit_skipped;
    // full_order_row_list_kernel, full_order_cut_kernel and the sort's first counting pass run beside the first
    // select: they take the rows that no select pass serves by their options (widest window: max_select_top_k),
    // not by row_state, which that select is still writing.  The cut kernel then marks every other row in
    // disordered_rows (bit 1): should a select kernel hand such a row on after all (ties beyond its list), it is in
    // no list, and the replay (rows_listed_by_options = 1) leaves it to the launch behind it like a disordered one.
    uint32_t cut_by_options;
    uint32_t rows_listed_by_options;
    // ... and the list is written by one more workgroup of full_order_cut_kernel (the one behind the rows'), beside the others
    uint32_t* row_list_out;
    // The wide select takes the bound of a window wider than kTwoKeyBoundTopK from a sample of the whole row (1)
    // or from the row's first chunk alone (0); same results either way.
    uint32_t wide_sampled_bound;
};

// Where the terms of the sorted rows' elements are kept (see sort_low_digit_skipped).
__device__ __forceinline__ float* sorted_terms(const SamplerArgs& a, uint32_t row)
{
    uint32_t* const base = a.sort_low_digit_skipped != 0u ? a.sort_indices[0] : a.sort_keys[0];
    return reinterpret_cast<float*>(base + row * a.sort_stride);
}

// Elements of the row that the full-order sort orders (the row's first ones in sorted order).
__device__ __forceinline__ uint32_t sorted_length(const SamplerArgs& a, uint32_t row)
{
    return a.sort_lengths == nullptr ? a.vocab : a.sort_lengths[row];
}

constexpr uint32_t kRowHoldsNan = 0x80000000u; // in finite_counts: the row holds a NaN (a row has fewer than 2^31 logits)

__device__ __forceinline__ uint8_t stop_flag(const SamplerArgs& a, const ncnn_moe_sample_params& p, int32_t token)
{
    if (a.stop_ids == nullptr)
        return 0;
    for (uint32_t i = 0; i < p.stop_count; ++i)
    {
        if (a.stop_ids[p.stop_begin + i] == token)
            return 1;
    }
    return 0;
}

__device__ __forceinline__ void write_error(const SamplerArgs& a, uint32_t row, int status, uint8_t flags)
{
    ncnn_moe_sample_result r;
    r.token_id = -1;
    r.probability = 0.0f;
    r.kept_count = 0;
    r.status = static_cast<uint8_t>(status);
    r.is_stop = 0;
    r.draw_consumed = 0;
    r.flags = flags;
    a.results[row] = r;
    if (a.distribution_count != nullptr)
        a.distribution_count[row] = 0;
}

// Marks a row that still has to go through the full-order kernels.
__device__ __forceinline__ void write_pending(const SamplerArgs& a, uint32_t row)
{
    ncnn_moe_sample_result r;
    r.token_id = -1;
    r.probability = 0.0f;
    r.kept_count = 0;
    r.status = NCNN_MOE_ROW_NEEDS_FULL_ORDER;
    r.is_stop = 0;
    r.draw_consumed = 0;
    r.flags = 0;
    a.results[row] = r;
}

__device__ __forceinline__ void write_token(
    const SamplerArgs& a, uint32_t row, const ncnn_moe_sample_params& p,
    int32_t token, float probability, uint32_t kept, uint8_t draw_consumed, uint8_t flags)
{
    ncnn_moe_sample_result r;
    r.token_id = token;
    r.probability = probability;
    r.kept_count = kept;
    r.status = NCNN_MOE_ROW_OK;
    r.is_stop = stop_flag(a, p, token);
    r.draw_consumed = draw_consumed;
    r.flags = flags;
    a.results[row] = r;
}

// The CPU sampler from the sorted Top-K window onwards (src/engine/session.cpp:89-134, :429-442),
// executed by one wave: lane i holds candidate i of n <= 64 candidates in (logit descending, index
// ascending) order.  Sums run in candidate order on every lane redundantly.  uniform is the row's draw
// (a.uniforms[row], loaded by the caller long before: a load here would sit on the row's critical path).
__device__ __forceinline__ void finish_row_wave(
    const SamplerArgs& a, uint32_t row, const ncnn_moe_sample_params& p,
    float value, int32_t index, int n, int lane, uint8_t flags, float uniform, const uint64_t* exp2_table)
{
    NCNN_MOE_STAMP_ROW(row, 0);
    n = __builtin_amdgcn_readfirstlane(n); // the same in every lane: the loops over it stay scalar
    const float temperature = p.temperature;
    const float top_value = read_lane(value, 0);
    const float maximum = top_value / temperature;
    float term = 0.0f;
    if (lane < n)
        term = expf_libm(value / temperature - maximum, exp2_table);

    // The three walks below are the CPU's sequential fp32 sums.  Each is a chain of DPP shifts over the lanes
    // (wave_sequential_sums_of_first): every lane ends up with the running sum at its own position, without a
    // data-dependent exit; a lane past the end (or a filtered candidate) adds +0.0, which leaves a
    // non-negative sum as it is, and where the CPU loop would have stopped is read off afterwards with one ballot.
    NCNN_MOE_STAMP_ROW(row, 1);
    const float normalizer = read_lane(wave_sequential_sums_of_first(term, n), n - 1);
    if (!is_finite_f32(normalizer) || !(normalizer > 0.0f))
    {
        if (lane == 0)
            write_error(a, row, NCNN_MOE_ROW_INVALID_DISTRIBUTION, flags);
        return;
    }
    NCNN_MOE_STAMP_ROW(row, 2);
    const float probability = term / normalizer;

    bool keep = lane < n;
    if (p.min_p > 0.0f)
    {
        const float threshold = read_lane(probability, 0) * p.min_p;
        keep = keep && (probability >= threshold);
    }
    const uint64_t keep_mask = __ballot(keep);

    // Top-P: the cumulative sum over the kept candidates in order, up to the first that reaches top_p
    const float contribution = keep ? probability : 0.0f;
    const float cumulative_here = wave_sequential_sums_of_first(contribution, n);
    NCNN_MOE_STAMP_ROW(row, 3);
    const uint64_t reached = __ballot(keep && cumulative_here >= p.top_p);
    const int last = reached != 0 ? __builtin_ctzll(reached) : 63 - __builtin_clzll(keep_mask);
    const uint64_t kept_mask = keep_mask & ((2ull << last) - 1ull);
    const int kept = __popcll(kept_mask);
    // The renormaliser of session.cpp:130-132 adds the same values in the same order as the Top-P scan.
    const float renormalizer = read_lane(cumulative_here, last);
    const float final_probability = probability / renormalizer;

    if (a.distribution_count != nullptr)
    {
        const size_t first = static_cast<size_t>(row) * a.distribution_cap;
        if ((kept_mask >> lane) & 1ull)
        {
            const int position = lanes_below(kept_mask);
            if (static_cast<uint32_t>(position) < a.distribution_cap)
            {
                a.distribution_ids[first + position] = index;
                a.distribution_probabilities[first + position] = final_probability;
            }
        }
        if (lane == 0)
            a.distribution_count[row] = static_cast<uint32_t>(kept);
    }

    NCNN_MOE_STAMP_ROW(row, 4);
    int selected = 0;
    uint8_t draw_consumed = 0;
    float selected_probability = 1.0f;
    if (kept == 1)
    {
        selected = __builtin_ctzll(kept_mask);
    }
    else
    {
        draw_consumed = 1;
        const bool is_kept = ((kept_mask >> lane) & 1ull) != 0ull;
        const float share = is_kept ? final_probability : 0.0f;
        const float running_here = wave_sequential_sums_of_first(share, last + 1); // positions 0 .. last
        const uint64_t passed = __ballot(is_kept && uniform < running_here);
        selected = passed != 0 ? __builtin_ctzll(passed) : last; // past the last sum: the last kept candidate
        selected_probability = read_lane(final_probability, selected);
    }
    NCNN_MOE_STAMP_ROW(row, 5);
    const int32_t token = read_lane(index, selected);
    if (lane == 0)
        write_token(a, row, p, token, selected_probability, static_cast<uint32_t>(kept), draw_consumed, flags);
    NCNN_MOE_STAMP_ROW(row, 6);
}

template <int DTYPE>
struct LogitsVector;

template <>
struct LogitsVector<NCNN_MOE_LOGITS_F32>
{
    static constexpr int kWidth = 4;
    static constexpr int kElementBytes = 4;
    static constexpr int kVectorsPerLane = kVectorsPerLaneF32;
    __device__ static __forceinline__ void unpack(const uint4& raw, float* out)
    {
        out[0] = __uint_as_float(raw.x);
        out[1] = __uint_as_float(raw.y);
        out[2] = __uint_as_float(raw.z);
        out[3] = __uint_as_float(raw.w);
    }
};

template <>
struct LogitsVector<NCNN_MOE_LOGITS_BF16>
{
    static constexpr int kWidth = 8;
    static constexpr int kElementBytes = 2;
    static constexpr int kVectorsPerLane = kVectorsPerLaneBF16;
    // bf16 -> fp32 is bits << 16 (src/kernels/cpu_ops.cpp:26-32); element 2i is the low half of word i.
    __device__ static __forceinline__ void unpack(const uint4& raw, float* out)
    {
        out[0] = __uint_as_float(raw.x << 16);
        out[1] = __uint_as_float(raw.x & 0xffff0000u);
        out[2] = __uint_as_float(raw.y << 16);
        out[3] = __uint_as_float(raw.y & 0xffff0000u);
        out[4] = __uint_as_float(raw.z << 16);
        out[5] = __uint_as_float(raw.z & 0xffff0000u);
        out[6] = __uint_as_float(raw.w << 16);
        out[7] = __uint_as_float(raw.w & 0xffff0000u);
    }
};

// Ascending integer key of a float for bitwise selection (larger logit, larger key); never 0 for a
// finite logit, so 0 can mark an empty slot.
__device__ __forceinline__ uint32_t ascending_key(float value)
{
    uint32_t bits = __float_as_uint(value);
    if (bits == 0x80000000u)
        bits = 0u; // -0 ties with +0
    return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}

__device__ __forceinline__ float value_from_ascending_key(uint32_t key)
{
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

// The quota-th largest of the wave's 64 keys (one per lane), found bit by bit with wave-wide counts.
__device__ __forceinline__ uint32_t wave_select_key(uint32_t key, int quota)
{
    uint32_t prefix = 0;
#pragma unroll
    for (int bit = 31; bit >= 0; --bit)
    {
        const uint32_t trial = prefix | (1u << bit);
        if (__popcll(__ballot(key >= trial)) >= quota)
            prefix = trial;
    }
    return prefix;
}

// The top_k-th largest of m <= 64 * R keys in LDS (0 if fewer than top_k are non-zero), by one wave:
// keys in registers, the answer built bit by bit from wave-wide counts.
template <int R>
__device__ __forceinline__ uint32_t select_kth_key(const uint32_t* keys_in_lds, int m, int top_k, int lane)
{
    uint32_t keys[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
    {
        const int q = r * kWaveSize + lane;
        keys[r] = q < m ? keys_in_lds[q] : 0u;
    }
    uint32_t prefix = 0;
    for (int bit = 31; bit >= 0; --bit)
    {
        const uint32_t trial = prefix | (1u << bit);
        int count = 0;
#pragma unroll
        for (int r = 0; r < R; ++r)
            count += __popcll(__ballot(keys[r] >= trial));
        if (count >= top_k)
            prefix = trial;
    }
    return prefix;
}

// Exact top_k-th largest of m keys in LDS, by one wave; m <= 64 * MAX_SLOTS (MAX_SLOTS 8 or 16).
template <int MAX_SLOTS>
__device__ __forceinline__ uint32_t select_kth_key_dispatch(const uint32_t* keys_in_lds, int m, int top_k, int lane)
{
    if (m <= kWaveSize)
        return select_kth_key<1>(keys_in_lds, m, top_k, lane);
    if (m <= 2 * kWaveSize)
        return select_kth_key<2>(keys_in_lds, m, top_k, lane);
    if (m <= 4 * kWaveSize)
        return select_kth_key<4>(keys_in_lds, m, top_k, lane);
    if (MAX_SLOTS <= 8 || m <= 8 * kWaveSize)
        return select_kth_key<8>(keys_in_lds, m, top_k, lane);
    return select_kth_key<16>(keys_in_lds, m, top_k, lane);
}

constexpr int kQuadMaxima = kScanThreads / 4; // one per quad of lanes
static_assert(kQuadMaxima == 2 * kWaveSize, "a wave searches the quad maxima two per lane");

struct BoundScratch
{
    uint32_t quad_maxima[kQuadMaxima];
    uint32_t wave_bounds[kScanWaves];
    uint32_t hot_keys[2 * kScanThreads];
    uint32_t hot_total;
    uint32_t result;
};

// A cheap lower bound of the top_k-th largest of the workgroup's keys (one per thread, each standing
// for a distinct logit; 0 = no key) that at least top_k keys reach: the top_k-th largest of the 128
// maxima of the quads of lanes, every maximum being one of the keys.  0 when top_k exceeds three
// quarters of the quads that hold a key (a short row fills few of them; beyond that the smallest
// maxima decide): the caller then takes the exact routine below.  Slightly looser than the exact
// top_k-th largest (for top_k = 20 of 10,240 values about 22 reach it, for top_k = 50 about 63), at a
// third of the cost: two exchanges inside the quads, an LDS round trip, a 16-step search by one wave,
// a second LDS round trip.  All threads of the workgroup must call it.
__device__ __forceinline__ uint32_t workgroup_kth_of_quad_maxima(
    uint32_t key, int top_k, int tid, BoundScratch& scratch, uint32_t* maximum_out = nullptr)
{
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    uint32_t quad_max = key;
    quad_max = max(quad_max, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(quad_max), 0xB1, 0xf, 0xf, true))); // lanes 1 apart
    quad_max = max(quad_max, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(quad_max), 0x4E, 0xf, 0xf, true))); // lanes 2 apart
    if ((lane & 3) == 0)
        scratch.quad_maxima[wave * (kWaveSize / 4) + (lane >> 2)] = quad_max;
    lds_barrier();
    // One wave searches the 128 maxima (two per lane) bit by bit, counting with ballots, while the others
    // wait: the steps are scalar, and eight waves searching side by side (which would save the second
    // barrier) queue for the one scalar unit of their SIMDs and take 0.2 to 0.7 us longer per batch.
    // The lowest 16 bits are left at zero: a step costs a VALU-to-scalar round trip, and a bound that
    // is half a percent lower lets hardly any more keys through.
    if (wave == 0)
    {
        const uint32_t first = scratch.quad_maxima[lane];
        const uint32_t second = scratch.quad_maxima[kWaveSize + lane];
        const auto reaching = [&](uint32_t trial) { return __popcll(__ballot(first >= trial)) + __popcll(__ballot(second >= trial)); };
        if (maximum_out != nullptr)
        {
            // the largest key of the workgroup (an address in LDS), for callers that want the range of the keys
            const uint32_t largest = wave_max_u32(max(first, second));
            if (lane == 0)
                *maximum_out = largest;
        }
        uint32_t prefix = 0;
        if (top_k * 4 <= reaching(1u) * 3)
        {
#pragma unroll
            for (int bit = 31; bit >= 16; --bit)
            {
                const uint32_t trial = prefix | (1u << bit);
                if (reaching(trial) >= top_k)
                    prefix = trial;
            }
        }
        if (lane == 0)
            scratch.result = prefix;
    }
    lds_barrier();
    return scratch.result;
}

// The top_k-th largest of the workgroup's keys (KEYS per thread, each standing for a distinct
// logit; 0 = no key), or with exact == false a lower bound of it that at least top_k keys still
// reach; 0 when fewer than top_k keys exist.  top_k <= 512 * KEYS.  All threads of the workgroup must call it.
//   A  every wave finds a lower bound of the ceil(top_k/8)-th largest of its 64 * KEYS keys (upper 16 bits
//      only); the smallest of the eight bounds is reached by at least top_k keys of the workgroup;
//   B  the keys at or above that bound are gathered in LDS;
//   C  wave 0 selects the exact top_k-th largest of the gathered keys.
template <int KEYS>
__device__ __forceinline__ uint32_t workgroup_kth_largest_key(
    const uint32_t (&keys)[KEYS], int top_k, int tid, BoundScratch& scratch, bool exact)
{
    static_assert(KEYS == 1 || KEYS == 2, "the gather buffer holds two keys per thread");
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    const int quota = (top_k + kScanWaves - 1) / kScanWaves;
    uint32_t prefix = 0;
#pragma unroll
    for (int bit = 31; bit >= 16; --bit)
    {
        const uint32_t trial = prefix | (1u << bit);
        int reached = 0;
#pragma unroll
        for (int slot = 0; slot < KEYS; ++slot)
            reached += __popcll(__ballot(keys[slot] >= trial));
        if (reached >= quota)
            prefix = trial;
    }
    if (lane == 0)
        scratch.wave_bounds[wave] = prefix;
    if (tid == 0)
        scratch.hot_total = 0;
    __syncthreads();
    uint32_t loose_bound = scratch.wave_bounds[0];
#pragma unroll
    for (int w = 1; w < kScanWaves; ++w)
        loose_bound = min(loose_bound, scratch.wave_bounds[w]);
    if (!exact)
    {
        __syncthreads();
        return loose_bound;
    }
#pragma unroll
    for (int slot = 0; slot < KEYS; ++slot)
    {
        const uint32_t key = keys[slot];
        const bool hot = key != 0u && key >= loose_bound;
        const uint64_t hot_mask = __ballot(hot);
        if (hot_mask != 0)
        {
            uint32_t base = 0;
            if (lane == 0)
                base = atomicAdd(&scratch.hot_total, static_cast<uint32_t>(__popcll(hot_mask)));
            base = __builtin_amdgcn_readfirstlane(base);
            if (hot)
                scratch.hot_keys[base + lanes_below(hot_mask)] = key;
        }
    }
    __syncthreads();
    if (wave == 0)
    {
        const uint32_t kth = select_kth_key_dispatch<8 * KEYS>(scratch.hot_keys, static_cast<int>(scratch.hot_total), top_k, lane);
        if (lane == 0)
            scratch.result = kth;
    }
    __syncthreads();
    return scratch.result;
}

// The top_k-th largest of the workgroup's N keys per thread (0 = no key), found bit by bit over the
// upper BITS bits of the key with workgroup-wide counts: BITS == 32 gives the exact key, fewer bits a
// lower bound that at least top_k keys reach (and only as many more as share those bits with the
// top_k-th largest).  0 when fewer than top_k keys exist.  All threads of the workgroup must call it.
template <int BITS, int N>
__device__ __forceinline__ uint32_t workgroup_kth_of_keys(
    const uint32_t (&keys)[N], int top_k, int tid, BoundScratch& scratch)
{
    static_assert(BITS >= 1 && BITS <= 32, "one counter per bit lives in the gather buffer");
    if (tid < BITS)
        scratch.hot_keys[tid] = 0; // one counter per bit
    __syncthreads();
    uint32_t prefix = 0;
    for (int bit = 31; bit > 31 - BITS; --bit)
    {
        const uint32_t trial = prefix | (1u << bit);
        int wave_count = 0;
#pragma unroll
        for (int i = 0; i < N; ++i)
            wave_count += __popcll(__ballot(keys[i] >= trial));
        if ((tid & (kWaveSize - 1)) == 0)
            atomicAdd(&scratch.hot_keys[31 - bit], static_cast<uint32_t>(wave_count));
        __syncthreads();
        if (scratch.hot_keys[31 - bit] >= static_cast<uint32_t>(top_k))
            prefix = trial;
    }
    __syncthreads();
    return prefix;
}

// The exact top_k-th largest of the workgroup's N keys per thread (0 = no key; 0 when fewer than top_k keys
// exist), digit by digit: four rounds of a 256-bin histogram of the keys that share the digits found so
// far, from which every wave reads off the digit at which the count from the top reaches the wanted rank
// (lane l takes bins 255 - 4 l down to 252 - 4 l, so a prefix sum over the lanes counts from the largest
// digit down).  A tenth of the barriers of the bit-by-bit search above.  The keys of a candidate list
// share their upper digits: a wave first counts the lanes that hold its first lane's digit and adds them
// with one atomic (twice), and only what is left goes to the histogram lane by lane.
// LEVELS < 4: only the upper LEVELS digits are worked out, the rest left at zero: a lower bound that at least
// top_k keys reach (and only as many more as share those digits with the top_k-th largest).
// All threads of the workgroup must call it.
template <int N, int LEVELS = 4>
__device__ __forceinline__ uint32_t workgroup_kth_of_keys_by_digits(
    const uint32_t (&keys)[N], int top_k, int tid, BoundScratch& scratch)
{
    static_assert(LEVELS >= 1 && LEVELS <= 4, "a key has four digits");
    const int lane = tid & (kWaveSize - 1);
    uint32_t prefix = 0;     // the digits found so far, in place
    uint32_t determined = 0; // the bits they occupy
    uint32_t wanted = static_cast<uint32_t>(top_k); // rank among the keys that share those digits
    for (int level = 0; level < LEVELS; ++level)
    {
        const int shift = 24 - 8 * level;
        uint32_t* const bins = scratch.hot_keys + 256 * (level & 1); // alternate levels, alternate bins: one barrier less
        if (tid < 256)
            bins[tid] = 0;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < N; ++i)
        {
            bool pending = keys[i] != 0u && (keys[i] & determined) == prefix;
            const uint32_t digit = (keys[i] >> shift) & 255u;
#pragma unroll
            for (int round = 0; round < 2; ++round)
            {
                const uint64_t holders = __ballot(pending);
                if (holders == 0ull)
                    break;
                const int leader = __builtin_ctzll(holders);
                const uint32_t leader_digit = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(digit), leader));
                const uint64_t same = __ballot(pending && digit == leader_digit);
                if (lane == leader)
                    atomicAdd(&bins[leader_digit], static_cast<uint32_t>(__popcll(same)));
                pending = pending && digit != leader_digit;
            }
            if (pending)
                atomicAdd(&bins[digit], 1u);
        }
        __syncthreads();
        const uint32_t top_bin = 255u - 4u * static_cast<uint32_t>(lane);
        const uint32_t c0 = bins[top_bin], c1 = bins[top_bin - 1u], c2 = bins[top_bin - 2u], c3 = bins[top_bin - 3u];
        const uint32_t inclusive = wave_prefix_sum_u32(c0 + c1 + c2 + c3);
        const uint32_t total = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(inclusive), kWaveSize - 1));
        if (total < wanted)
        {
            __syncthreads();
            return 0u; // (only at the first level: fewer keys than top_k)
        }
        const int crossing = __builtin_ctzll(__ballot(inclusive >= wanted));
        const uint32_t before = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(inclusive - (c0 + c1 + c2 + c3)), crossing));
        const uint32_t d0 = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(c0), crossing));
        const uint32_t d1 = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(c1), crossing));
        const uint32_t d2 = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(c2), crossing));
        uint32_t step = 0, above = before; // bins of the crossing lane in front of the one that holds the rank
        if (above + d0 < wanted)
        {
            above += d0;
            step = 1;
            if (above + d1 < wanted)
            {
                above += d1;
                step = 2;
                if (above + d2 < wanted)
                {
                    above += d2;
                    step = 3;
                }
            }
        }
        const uint32_t digit = 255u - 4u * static_cast<uint32_t>(crossing) - step;
        wanted -= above;
        prefix |= digit << shift;
        determined |= 255u << shift;
    }
    __syncthreads();
    return prefix;
}

// Exact best-K selection over m <= 64 * R candidates in LDS by one wave; keys live in registers.
// Selected candidates (at most top_k) are written, unordered, to final_values / final_indices.
template <int R>
__device__ __forceinline__ int select_best_wave(
    const uint32_t* staged_keys, const int32_t* staged_indices, int m, int top_k, int lane,
    float* final_values, int32_t* final_indices)
{
    m = __builtin_amdgcn_readfirstlane(m);
    top_k = __builtin_amdgcn_readfirstlane(top_k);
    uint32_t keys[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
    {
        const int q = r * kWaveSize + lane;
        keys[r] = q < m ? staged_keys[q] : 0u;
    }
    uint32_t key_cut = 1u; // every staged key qualifies
    uint32_t index_cut = 0xffffffffu;
    if (m > top_k)
    {
        uint32_t prefix = 0;
        for (int bit = 31; bit >= 0; --bit)
        {
            const uint32_t trial = prefix | (1u << bit);
            int count = 0;
#pragma unroll
            for (int r = 0; r < R; ++r)
                count += __popcll(__ballot(keys[r] >= trial));
            if (count >= top_k)
                prefix = trial;
        }
        key_cut = prefix;
        int above = 0;
        int ties = 0;
#pragma unroll
        for (int r = 0; r < R; ++r)
        {
            above += __popcll(__ballot(keys[r] > key_cut));
            ties += __popcll(__ballot(keys[r] == key_cut));
        }
        const int needed = top_k - above; // of the ties, the `needed` lowest indices stay
        if (ties > needed)
        {
            uint32_t index_prefix = 0;
            for (int bit = 31; bit >= 0; --bit)
            {
                const uint32_t trial = index_prefix | (1u << bit);
                int count = 0;
#pragma unroll
                for (int r = 0; r < R; ++r)
                {
                    const int q = r * kWaveSize + lane;
                    const bool tie = keys[r] == key_cut && key_cut != 0u && q < m;
                    const uint32_t index = tie ? static_cast<uint32_t>(staged_indices[q]) : 0xffffffffu;
                    count += __popcll(__ballot(tie && index < trial));
                }
                if (count < needed)
                    index_prefix = trial;
            }
            index_cut = index_prefix;
        }
    }
    int n = 0;
#pragma unroll
    for (int r = 0; r < R; ++r)
    {
        const int q = r * kWaveSize + lane;
        const uint32_t key = keys[r];
        bool selected = key != 0u && key >= key_cut;
        int32_t index = 0;
        if (selected)
        {
            index = staged_indices[q];
            if (key == key_cut && static_cast<uint32_t>(index) > index_cut)
                selected = false;
        }
        const uint64_t mask = __ballot(selected);
        if (mask != 0)
        {
            const int position = n + lanes_below(mask);
            if (selected && position < kFastTopK)
            {
                final_values[position] = value_from_ascending_key(key);
                final_indices[position] = index;
            }
            n += __popcll(mask);
        }
    }
    return n < kFastTopK ? n : kFastTopK;
}

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_SAMPLER_COMMON_H
