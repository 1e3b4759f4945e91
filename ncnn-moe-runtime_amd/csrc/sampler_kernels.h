// Kernels of the gfx950 generation sampler.
//
//   scan_select_kernel   one pass over the [rows, vocab] logits in HBM: every workgroup loads a
//                        10240-value segment of one row into registers with 16-byte loads, selects
//                        the segment's best K candidates in LDS, and the last workgroup to finish a
//                        row merges the segments and runs the softmax / Min-P / Top-P / draw
//                        epilogue.  Serves greedy rows and rows with an effective Top-K <= 64.
//   general_sort_kernel  full stable order of one row (LSD radix sort on descending keys) for rows
//   general_replay_kernel  whose Top-K window is wider than 64 or absent; the replay walks the
//                        sorted row exactly as the CPU sampler does (sequential fp32 sums).
#ifndef NCNN_MOE_HIP_SAMPLER_KERNELS_H
#define NCNN_MOE_HIP_SAMPLER_KERNELS_H

#include "sampler_device.h"

namespace ncnn_moe_hip {

struct SamplerArgs
{
    const void* logits;
    uint64_t row_stride; // elements
    uint32_t rows;
    uint32_t vocab;
    uint32_t segments;
    int force_general;

    const ncnn_moe_sample_params* params;
    const float* uniforms;
    const int32_t* stop_ids;
    ncnn_moe_sample_result* results;

    // select-path scratch
    float* segment_values;     // [rows][segments][kFastTopK]
    int32_t* segment_indices;  // [rows][segments][kFastTopK]
    uint32_t* segment_counts;  // [rows][segments]
    uint32_t* row_counter;     // [rows], zero between launches
    uint32_t* row_flags;       // [rows], zero between launches
    uint32_t* row_state;       // [rows], written by every launch

    // general-path scratch, [rows][sort_stride] each
    uint32_t* sort_keys[2];
    uint32_t* sort_indices[2];
    uint64_t sort_stride;

    // optional filtered-distribution output for row 0 of the launch
    int32_t* distribution_ids;
    float* distribution_probabilities;
    uint32_t distribution_cap;
    uint32_t* distribution_count;
};

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
    if (a.distribution_count != nullptr && row == 0)
        *a.distribution_count = 0;
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
// ascending) order.  Sums run in candidate order on every lane redundantly.
__device__ __forceinline__ void finish_row_wave(
    const SamplerArgs& a, uint32_t row, const ncnn_moe_sample_params& p,
    float value, int32_t index, int n, int lane, uint8_t flags)
{
    const float temperature = p.temperature;
    const float top_value = read_lane(value, 0);
    const float maximum = top_value / temperature;
    float term = 0.0f;
    if (lane < n)
        term = expf_libm(value / temperature - maximum);

    float normalizer = 0.0f;
    for (int i = 0; i < n; ++i)
        normalizer += read_lane(term, i);
    if (!is_finite_f32(normalizer) || !(normalizer > 0.0f))
    {
        if (lane == 0)
            write_error(a, row, NCNN_MOE_ROW_INVALID_DISTRIBUTION, flags);
        return;
    }
    const float probability = term / normalizer;

    bool keep = lane < n;
    if (p.min_p > 0.0f)
    {
        const float threshold = read_lane(probability, 0) * p.min_p;
        keep = keep && (probability >= threshold);
    }
    uint64_t pending = __ballot(keep);

    float cumulative = 0.0f;
    uint64_t kept_mask = 0;
    int kept = 0;
    while (pending != 0)
    {
        const int i = __builtin_ctzll(pending);
        pending &= pending - 1;
        cumulative += read_lane(probability, i);
        kept_mask |= 1ull << i;
        ++kept;
        if (cumulative >= p.top_p)
            break;
    }
    // The renormaliser of session.cpp:130-132 adds the same values in the same order as the Top-P scan.
    const float renormalizer = cumulative;
    const float final_probability = probability / renormalizer;

    if (a.distribution_count != nullptr && row == 0)
    {
        if ((kept_mask >> lane) & 1ull)
        {
            const int position = lanes_below(kept_mask);
            if (static_cast<uint32_t>(position) < a.distribution_cap)
            {
                a.distribution_ids[position] = index;
                a.distribution_probabilities[position] = final_probability;
            }
        }
        if (lane == 0)
            *a.distribution_count = static_cast<uint32_t>(kept);
    }

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
        const float uniform = a.uniforms[row];
        float running = 0.0f;
        uint64_t walk = kept_mask;
        selected = 63 - __builtin_clzll(kept_mask);
        while (walk != 0)
        {
            const int i = __builtin_ctzll(walk);
            walk &= walk - 1;
            running += read_lane(final_probability, i);
            if (uniform < running)
            {
                selected = i;
                break;
            }
        }
        selected_probability = read_lane(final_probability, selected);
    }
    const int32_t token = read_lane(index, selected);
    if (lane == 0)
        write_token(a, row, p, token, selected_probability, static_cast<uint32_t>(kept), draw_consumed, flags);
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

// Agent-scope relaxed accesses: they write through / read around the per-XCD L2, so data handed from
// one workgroup to another needs no L2 write-back or invalidate, only a wait for the stores to land.
__device__ __forceinline__ void store_agent(uint32_t* address, uint32_t value)
{
    __hip_atomic_store(address, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ uint32_t load_agent(const uint32_t* address)
{
    return __hip_atomic_load(address, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

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

__device__ __forceinline__ uint32_t select_kth_key_dispatch(const uint32_t* keys_in_lds, int m, int top_k, int lane)
{
    if (m <= kWaveSize)
        return select_kth_key<1>(keys_in_lds, m, top_k, lane);
    if (m <= 2 * kWaveSize)
        return select_kth_key<2>(keys_in_lds, m, top_k, lane);
    if (m <= 4 * kWaveSize)
        return select_kth_key<4>(keys_in_lds, m, top_k, lane);
    return select_kth_key<8>(keys_in_lds, m, top_k, lane);
}

struct BoundScratch
{
    uint32_t wave_bounds[kScanWaves];
    uint32_t hot_keys[kScanThreads];
    uint32_t hot_total;
    uint32_t result;
};

// The exact top_k-th largest of the workgroup's per-thread keys (one key per thread, 0 = no key);
// 0 when fewer than top_k threads hold a key.  All threads of the workgroup must call it.
//   A  every wave finds a lower bound of the ceil(top_k/8)-th largest of its 64 keys (upper 16 bits
//      only); the smallest of the eight bounds is reached by at least top_k keys of the workgroup;
//   B  the keys at or above that bound (a few dozen) are gathered in LDS;
//   C  wave 0 selects the exact top_k-th largest of the gathered keys.
__device__ __forceinline__ uint32_t workgroup_kth_largest_key(uint32_t key, int top_k, int tid, BoundScratch& scratch)
{
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    const int quota = (top_k + kScanWaves - 1) / kScanWaves;
    uint32_t prefix = 0;
#pragma unroll
    for (int bit = 31; bit >= 16; --bit)
    {
        const uint32_t trial = prefix | (1u << bit);
        if (__popcll(__ballot(key >= trial)) >= quota)
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
    __syncthreads();
    if (wave == 0)
    {
        const uint32_t kth = select_kth_key_dispatch(scratch.hot_keys, static_cast<int>(scratch.hot_total), top_k, lane);
        if (lane == 0)
            scratch.result = kth;
    }
    __syncthreads();
    return scratch.result;
}

// Exact best-K selection over m <= 64 * R candidates in LDS by one wave; keys live in registers.
// Selected candidates (at most top_k) are written, unordered, to final_values / final_indices.
template <int R>
__device__ __forceinline__ int select_best_wave(
    const uint32_t* staged_keys, const int32_t* staged_indices, int m, int top_k, int lane,
    float* final_values, int32_t* final_indices)
{
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

// One HBM pass of the select path.  CHUNKS * (5 fp32 | 3 bf16) vectors per lane are held in registers.
//
// Every workgroup: 16-byte loads -> per-vector and per-lane maxima -> the exact K-th largest lane
// maximum of the workgroup, a bound that at least K logits of the segment reach -> the logits at
// or above the bound (K and a few) go to the segment's record in HBM.  The last workgroup to finish
// a row loads every record of the row, prunes the candidates with the same kind of bound, selects
// the exact best K by (logit descending, index ascending), and runs the CPU sampler's epilogue.
template <int DTYPE, int CHUNKS>
__global__ __launch_bounds__(kScanThreads, (CHUNKS == 1 && DTYPE == NCNN_MOE_LOGITS_F32) ? 8 : 1) void scan_select_kernel(SamplerArgs a)
{
    using Vector = LogitsVector<DTYPE>;
    constexpr int kWidth = Vector::kWidth;
    constexpr int kVectors = Vector::kVectorsPerLane * CHUNKS;
    constexpr int kLaneValues = kVectors * kWidth;
    constexpr uint32_t kSegment = static_cast<uint32_t>(kScanThreads) * kLaneValues;
    constexpr uint32_t kNegativeInfinity = 0xff800000u;
    constexpr uint32_t kPositiveInfinity = 0x7f800000u;

    const uint32_t row = blockIdx.y;
    const uint32_t segment = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;

    __shared__ BoundScratch bound_scratch;
    __shared__ float candidate_values[kScanWaves][kWaveCandidateCap];
    __shared__ int32_t candidate_indices[kScanWaves][kWaveCandidateCap];
    __shared__ int candidate_counts[kScanWaves];
    __shared__ uint32_t block_flags;
    __shared__ int block_is_last;
    __shared__ uint32_t survivor_keys[kMergeSurvivorCap];
    __shared__ int32_t survivor_indices[kMergeSurvivorCap];
    __shared__ uint32_t survivor_total;
    __shared__ float final_values[kFastTopK];
    __shared__ int32_t final_indices[kFastTopK];

    const ncnn_moe_sample_params p = a.params[row];
    uint32_t effective_k = 0;
    int status = NCNN_MOE_ROW_OK;
    const int mode = resolve_row_mode(p, a.vocab, a.segments, a.force_general, effective_k, status);
    if (mode == kModeInvalid || mode == kModeGeneral)
    {
        if (segment == 0 && tid == 0)
        {
            if (mode == kModeInvalid)
            {
                write_error(a, row, status, 0);
                a.row_state[row] = kRowDone;
            }
            else
            {
                write_pending(a, row);
                a.row_state[row] = kRowNeedsGeneral;
            }
        }
        return;
    }
    const bool greedy = mode == kModeGreedy;
    const int top_k = static_cast<int>(effective_k);
    const uint32_t record_entries = segment_record_entries(effective_k);

    if (tid == 0)
    {
        block_flags = 0;
        survivor_total = 0;
    }

    // ---- load the segment: 16-byte loads from the 16-byte aligned address at or below the row start
    const char* row_pointer = static_cast<const char*>(a.logits) +
        static_cast<size_t>(row) * a.row_stride * Vector::kElementBytes;
    const uint32_t misalignment =
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row_pointer) & 15u) / Vector::kElementBytes;
    const char* aligned_base = row_pointer - static_cast<size_t>(misalignment) * Vector::kElementBytes;
    const uint32_t valid_begin = misalignment;
    const uint32_t valid_end = misalignment + a.vocab;
    const uint32_t segment_base = segment * kSegment;

    float values[kLaneValues];
    uint4 raw[kVectors];
#pragma unroll
    for (int v = 0; v < kVectors; ++v)
    {
        const uint32_t first = segment_base + static_cast<uint32_t>(v * kScanThreads + tid) * kWidth;
        if (first < valid_end && first + kWidth > valid_begin)
            raw[v] = *reinterpret_cast<const uint4*>(aligned_base + static_cast<size_t>(first) * Vector::kElementBytes);
        else
            raw[v] = make_uint4(kNegativeInfinity, kNegativeInfinity, kNegativeInfinity, kNegativeInfinity);
    }

    // ---- per-vector maxima, per-lane maximum (NaN ignored), NaN / +inf detection
    float group_max[kVectors];
    float lane_max = __uint_as_float(kNegativeInfinity);
    bool saw_nan = false;
#pragma unroll
    for (int v = 0; v < kVectors; ++v)
    {
        const uint32_t first = segment_base + static_cast<uint32_t>(v * kScanThreads + tid) * kWidth;
        const bool any_valid = first < valid_end && first + kWidth > valid_begin;
        if (any_valid)
            Vector::unpack(raw[v], &values[v * kWidth]);
        else
        {
#pragma unroll
            for (int c = 0; c < kWidth; ++c)
                values[v * kWidth + c] = __uint_as_float(kNegativeInfinity);
        }
        if (any_valid && (first < valid_begin || first + kWidth > valid_end))
        {
#pragma unroll
            for (int c = 0; c < kWidth; ++c)
            {
                const uint32_t position = first + c;
                if (position < valid_begin || position >= valid_end)
                    values[v * kWidth + c] = __uint_as_float(kNegativeInfinity);
            }
        }
        float vector_max = __uint_as_float(kNegativeInfinity);
#pragma unroll
        for (int c = 0; c < kWidth; ++c)
        {
            float x = values[v * kWidth + c];
            saw_nan = saw_nan || (x != x);
            if (greedy && x == __uint_as_float(kPositiveInfinity))
            {
                x = __uint_as_float(kNegativeInfinity); // greedy skips every non-finite logit (session.cpp:411-412)
                values[v * kWidth + c] = x;
            }
            vector_max = fmaxf(vector_max, x);
        }
        group_max[v] = vector_max;
        lane_max = fmaxf(lane_max, vector_max);
    }
    uint32_t local_flags = 0;
    if (saw_nan)
        local_flags |= kScanSawNan;
    if (lane_max == __uint_as_float(kPositiveInfinity))
        local_flags |= kScanSawPositiveInfinity;

    // ---- bound: the exact K-th largest lane maximum of the workgroup.  The lanes at or above it each
    // hold a distinct logit at least that large, so the K-th best logit of the row is no smaller.
    const uint32_t lane_key = lane_max == __uint_as_float(kNegativeInfinity) ? 0u : ascending_key(lane_max);
    const uint32_t bound_key = workgroup_kth_largest_key(lane_key, top_k, tid, bound_scratch);
    // fewer than K lanes hold a finite logit: every finite logit of the segment is a candidate
    const float threshold = bound_key == 0u ? -3.402823466e+38f : fmaxf(value_from_ascending_key(bound_key), -3.402823466e+38f);

    // ---- collect the values at or above the bound into this wave's LDS region; only vectors whose
    // maximum reaches the bound are looked at
    int wave_count = 0;
#pragma unroll
    for (int v = 0; v < kVectors; ++v)
    {
        const bool vector_hit = group_max[v] >= threshold;
        if (__ballot(vector_hit) != 0)
        {
#pragma unroll
            for (int c = 0; c < kWidth; ++c)
            {
                const float x = values[v * kWidth + c];
                const bool hit = vector_hit && x >= threshold;
                const uint64_t hits = __ballot(hit);
                if (hits != 0)
                {
                    const int position = wave_count + lanes_below(hits);
                    if (hit && position < kWaveCandidateCap)
                    {
                        const uint32_t element =
                            segment_base + static_cast<uint32_t>(v * kScanThreads + tid) * kWidth + c - misalignment;
                        candidate_values[wave][position] = x;
                        candidate_indices[wave][position] = static_cast<int32_t>(element);
                    }
                    wave_count += __popcll(hits);
                }
            }
        }
    }
    if (lane == 0)
        candidate_counts[wave] = wave_count;
    if (local_flags != 0)
        atomicOr(&block_flags, local_flags);
    __syncthreads();

    // ---- hand the candidates over: compact copy of the wave regions into the segment's record
    uint32_t* const out_values = reinterpret_cast<uint32_t*>(a.segment_values);
    uint32_t* const out_indices = reinterpret_cast<uint32_t*>(a.segment_indices);
    const size_t segment_slot = (static_cast<size_t>(row) * a.segments + segment);
    int offset = 0;
    int total = 0;
    bool overflow = false;
#pragma unroll
    for (int w = 0; w < kScanWaves; ++w)
    {
        const int count = candidate_counts[w];
        overflow = overflow || count > kWaveCandidateCap;
        if (w < wave)
            offset += count;
        total += count;
    }
    overflow = overflow || static_cast<uint32_t>(total) > record_entries;
    if (!overflow)
    {
        for (int j = lane; j < wave_count; j += kWaveSize)
        {
            store_agent(&out_values[segment_slot * kSegmentRecordSlots + offset + j], __float_as_uint(candidate_values[wave][j]));
            store_agent(&out_indices[segment_slot * kSegmentRecordSlots + offset + j], static_cast<uint32_t>(candidate_indices[wave][j]));
        }
    }
    if (tid == 0)
    {
        store_agent(&a.segment_counts[segment_slot], overflow ? 0u : static_cast<uint32_t>(total));
        uint32_t flags = block_flags;
        if (overflow)
            flags |= kScanOverflow;
        if (flags != 0)
            atomicOr(&a.row_flags[row], flags);
    }

    // ---- the last workgroup of the row merges the segments.  The barrier waits for this workgroup's
    // agent-scope stores; the counter is bumped only after that.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0)
    {
        const uint32_t previous = __hip_atomic_fetch_add(&a.row_counter[row], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        block_is_last = previous == a.segments - 1 ? 1 : 0;
    }
    __syncthreads();
    if (!block_is_last)
        return;

    // every load of the merge is issued before any is used: one trip to memory
    const size_t row_slot = static_cast<size_t>(row) * a.segments;
    const uint32_t row_entries = a.segments * record_entries;
    constexpr int kPerThread = kMergeStageSlots / kScanThreads;
    uint32_t loaded_keys[kPerThread];
    uint32_t loaded_indices[kPerThread];
    uint32_t loaded_counts[kPerThread];
    const uint32_t row_flags = load_agent(&a.row_flags[row]);
    const bool stageable = row_entries <= static_cast<uint32_t>(kMergeStageSlots);
#pragma unroll
    for (int j = 0; j < kPerThread; ++j)
    {
        const uint32_t q = static_cast<uint32_t>(j * kScanThreads + tid);
        loaded_keys[j] = 0;
        loaded_indices[j] = 0;
        loaded_counts[j] = 0;
        if (stageable && q < row_entries)
        {
            const uint32_t s = q / record_entries;
            const uint32_t r = q - s * record_entries;
            loaded_keys[j] = load_agent(&out_values[(row_slot + s) * kSegmentRecordSlots + r]);
            loaded_indices[j] = load_agent(&out_indices[(row_slot + s) * kSegmentRecordSlots + r]);
            loaded_counts[j] = load_agent(&a.segment_counts[row_slot + s]);
        }
    }
    uint8_t result_flags = (row_flags & kScanSawNan) ? NCNN_MOE_ROW_FLAG_HAS_NAN : 0;
    __syncthreads();
    if (tid == 0)
    {
        a.row_counter[row] = 0;
        a.row_flags[row] = 0;
    }
    if ((row_flags & kScanOverflow) || !stageable)
    {
        // ties (or a very long row) left more candidates than the records hold: the full-order kernels take the row
        if (tid == 0)
        {
            write_pending(a, row);
            a.row_state[row] = kRowNeedsGeneral;
        }
        return;
    }
    if (!greedy && (row_flags & kScanSawPositiveInfinity))
    {
        // the stable order puts +inf first and the CPU sampler rejects the row (session.cpp:84-85)
        if (tid == 0)
        {
            write_error(a, row, NCNN_MOE_ROW_NO_FINITE_LOGIT, result_flags);
            a.row_state[row] = kRowDone;
        }
        return;
    }
    // per-thread best key; slots past a segment's count hold nothing
    uint32_t thread_key = 0;
#pragma unroll
    for (int j = 0; j < kPerThread; ++j)
    {
        const uint32_t q = static_cast<uint32_t>(j * kScanThreads + tid);
        const uint32_t r = q % record_entries;
        loaded_keys[j] = (q < row_entries && r < loaded_counts[j]) ? ascending_key(__uint_as_float(loaded_keys[j])) : 0u;
        thread_key = max(thread_key, loaded_keys[j]);
    }
    // prune: at least K candidates reach the K-th largest per-thread best
    const uint32_t prune_key = workgroup_kth_largest_key(thread_key, top_k, tid, bound_scratch);
    {
        int survivors_here = 0;
#pragma unroll
        for (int j = 0; j < kPerThread; ++j)
            survivors_here += (loaded_keys[j] != 0u && loaded_keys[j] >= prune_key) ? 1 : 0;
        // wave-aggregated reservation of survivor slots
        int prefix = survivors_here;
#pragma unroll
        for (int step = 1; step < kWaveSize; step <<= 1)
        {
            const int up = __shfl_up(prefix, step, kWaveSize);
            if (lane >= step)
                prefix += up;
        }
        const int wave_total = __shfl(prefix, kWaveSize - 1, kWaveSize);
        uint32_t base = 0;
        if (lane == 0 && wave_total > 0)
            base = atomicAdd(&survivor_total, static_cast<uint32_t>(wave_total));
        base = __builtin_amdgcn_readfirstlane(base);
        uint32_t position = base + static_cast<uint32_t>(prefix - survivors_here);
#pragma unroll
        for (int j = 0; j < kPerThread; ++j)
        {
            if (loaded_keys[j] != 0u && loaded_keys[j] >= prune_key)
            {
                if (position < static_cast<uint32_t>(kMergeSurvivorCap))
                {
                    survivor_keys[position] = loaded_keys[j];
                    survivor_indices[position] = static_cast<int32_t>(loaded_indices[j]);
                }
                ++position;
            }
        }
    }
    __syncthreads();
    const int survivors = static_cast<int>(survivor_total);
    if (survivors > kMergeSurvivorCap)
    {
        if (tid == 0)
        {
            write_pending(a, row);
            a.row_state[row] = kRowNeedsGeneral;
        }
        return;
    }
    if (wave != 0)
        return;

    // ---- wave 0: exact best K of the survivors, then their order, then the epilogue
    int n = 0;
    if (survivors <= kWaveSize)
        n = select_best_wave<1>(survivor_keys, survivor_indices, survivors, top_k, lane, final_values, final_indices);
    else if (survivors <= 2 * kWaveSize)
        n = select_best_wave<2>(survivor_keys, survivor_indices, survivors, top_k, lane, final_values, final_indices);
    else
        n = select_best_wave<8>(survivor_keys, survivor_indices, survivors, top_k, lane, final_values, final_indices);
    if (lane == 0)
        a.row_state[row] = kRowDone;
    if (n == 0)
    {
        if (lane == 0)
            write_error(a, row, NCNN_MOE_ROW_NO_FINITE_LOGIT, result_flags);
        return;
    }
    float value = lane < n ? final_values[lane] : 0.0f;
    int32_t index = lane < n ? final_indices[lane] : -1;
    int rank = 0;
    for (int j = 0; j < n; ++j)
        rank += candidate_before(read_lane(value, j), read_lane(index, j), value, index) ? 1 : 0;
    if (lane < n)
    {
        final_values[rank] = value;
        final_indices[rank] = index;
    }
    value = lane < n ? final_values[lane] : 0.0f;
    index = lane < n ? final_indices[lane] : -1;
    if (greedy)
    {
        if (lane == 0)
        {
            write_token(a, row, p, index, 1.0f, 1u, 0, result_flags);
            if (a.distribution_count != nullptr && row == 0)
            {
                *a.distribution_count = 1;
                if (a.distribution_cap > 0)
                {
                    a.distribution_ids[0] = index;
                    a.distribution_probabilities[0] = 1.0f;
                }
            }
        }
        return;
    }
    finish_row_wave(a, row, p, value, index, n, lane, result_flags);
}

// ---------------------------------------------------------------------------------------------
// Full-order path
// ---------------------------------------------------------------------------------------------

template <int DTYPE>
__device__ __forceinline__ float load_logit(const void* row_pointer, uint32_t i);

template <>
__device__ __forceinline__ float load_logit<NCNN_MOE_LOGITS_F32>(const void* row_pointer, uint32_t i)
{
    return static_cast<const float*>(row_pointer)[i];
}

template <>
__device__ __forceinline__ float load_logit<NCNN_MOE_LOGITS_BF16>(const void* row_pointer, uint32_t i)
{
    return __uint_as_float(static_cast<uint32_t>(static_cast<const uint16_t*>(row_pointer)[i]) << 16);
}

// Stable LSD radix sort (8-bit digits) of one row by descending_key; one workgroup per row.
// fp32 rows take four passes; bf16 keys only differ in their upper 16 bits and take two.
// The sorted keys end in sort_keys[1].  With PAIRS the token indices travel with the keys and end in
// sort_indices[1] (needed only when the whole filtered distribution is exported); sampling sorts the
// keys alone and recovers the one index it needs from the logits afterwards.
template <int DTYPE, bool PAIRS>
__global__ __launch_bounds__(kSortThreads) void general_sort_kernel(SamplerArgs a)
{
    constexpr int kPasses = DTYPE == NCNN_MOE_LOGITS_F32 ? 4 : 2;
    constexpr int kFirstDigit = DTYPE == NCNN_MOE_LOGITS_F32 ? 0 : 2;
    const uint32_t row = blockIdx.x;
    if (a.row_state[row] != kRowNeedsGeneral)
        return;
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    const uint32_t n = a.vocab;

    __shared__ uint32_t histogram[kPasses][256];
    __shared__ uint32_t digit_base[256];
    __shared__ uint32_t wave_counts[kSortWaves][256];

    const char* row_pointer = static_cast<const char*>(a.logits) +
        static_cast<size_t>(row) * a.row_stride * LogitsVector<DTYPE>::kElementBytes;
    uint32_t* keys[2] = {a.sort_keys[0] + row * a.sort_stride, a.sort_keys[1] + row * a.sort_stride};
    uint32_t* indices[2] = {a.sort_indices[0] + row * a.sort_stride, a.sort_indices[1] + row * a.sort_stride};

    for (int i = tid; i < kPasses * 256; i += kSortThreads)
        (&histogram[0][0])[i] = 0;
    __syncthreads();
    for (uint32_t i = tid; i < n; i += kSortThreads)
    {
        const uint32_t key = descending_key(load_logit<DTYPE>(row_pointer, i));
#pragma unroll
        for (int pass = 0; pass < kPasses; ++pass)
            atomicAdd(&histogram[pass][(key >> (8 * (pass + kFirstDigit))) & 255u], 1u);
    }
    __syncthreads();
    // exclusive scan of each histogram by one wave (4 bins per lane)
    if (wave < kPasses)
    {
        uint32_t* h = histogram[wave];
        const uint32_t c0 = h[lane * 4 + 0], c1 = h[lane * 4 + 1], c2 = h[lane * 4 + 2], c3 = h[lane * 4 + 3];
        const uint32_t lane_total = c0 + c1 + c2 + c3;
        uint32_t inclusive = lane_total;
#pragma unroll
        for (int j = 1; j < kWaveSize; j <<= 1)
        {
            const uint32_t up = __shfl_up(inclusive, j, kWaveSize);
            if (lane >= j)
                inclusive += up;
        }
        const uint32_t exclusive = inclusive - lane_total;
        h[lane * 4 + 0] = exclusive;
        h[lane * 4 + 1] = exclusive + c0;
        h[lane * 4 + 2] = exclusive + c0 + c1;
        h[lane * 4 + 3] = exclusive + c0 + c1 + c2;
    }
    __syncthreads();

    // Every pass walks the row in tiles of 1024 x 8 elements.  A wave owns 512 consecutive elements of
    // the tile and ranks them in 8 rounds of 64 (one element per lane), so that the order inside the
    // wave is the input order; its per-digit running counts live in LDS.  A prefix over the 16 waves
    // and the digit bases then turns the ranks into output positions.
    for (int pass = 0; pass < kPasses; ++pass)
    {
        const int shift = 8 * (pass + kFirstDigit);
        const uint32_t* source_keys = keys[(pass + 1) & 1];   // pass 0 reads the logits instead
        const uint32_t* source_indices = indices[(pass + 1) & 1];
        uint32_t* target_keys = keys[pass & 1];
        uint32_t* target_indices = indices[pass & 1];
        if (tid < 256)
            digit_base[tid] = histogram[pass][tid];
        for (uint32_t tile = 0; tile < n; tile += kSortTile)
        {
            for (int i = tid; i < kSortWaves * 256; i += kSortThreads)
                (&wave_counts[0][0])[i] = 0;
            uint32_t tile_keys[kSortPerThread];
            uint32_t tile_indices[kSortPerThread];
            uint32_t tile_ranks[kSortPerThread];
            const uint32_t wave_first = tile + static_cast<uint32_t>(wave) * (kWaveSize * kSortPerThread);
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                const uint32_t i = wave_first + static_cast<uint32_t>(e * kWaveSize + lane);
                tile_keys[e] = 0xffffffffu;
                tile_indices[e] = i;
                if (i < n)
                {
                    if (pass == 0)
                        tile_keys[e] = descending_key(load_logit<DTYPE>(row_pointer, i));
                    else
                    {
                        tile_keys[e] = source_keys[i];
                        if (PAIRS)
                            tile_indices[e] = source_indices[i];
                    }
                }
            }
            __syncthreads();
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                const uint32_t i = wave_first + static_cast<uint32_t>(e * kWaveSize + lane);
                const bool valid = i < n;
                const uint32_t digit = (tile_keys[e] >> shift) & 255u;
                uint64_t peers = __ballot(valid);
#pragma unroll
                for (int b = 0; b < 8; ++b)
                {
                    const bool bit = (digit >> b) & 1u;
                    const uint64_t set = __ballot(valid && bit);
                    peers &= bit ? set : ~set;
                }
                const int rank_in_round = lanes_below(peers);
                uint32_t seen = 0;
                if (valid)
                    seen = wave_counts[wave][digit];
                tile_ranks[e] = seen + static_cast<uint32_t>(rank_in_round);
                if (valid && rank_in_round == 0)
                    wave_counts[wave][digit] = seen + static_cast<uint32_t>(__popcll(peers));
            }
            __syncthreads();
            if (tid < 256)
            {
                uint32_t running = digit_base[tid];
#pragma unroll
                for (int w = 0; w < kSortWaves; ++w)
                {
                    const uint32_t c = wave_counts[w][tid];
                    wave_counts[w][tid] = running;
                    running += c;
                }
                digit_base[tid] = running;
            }
            __syncthreads();
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                const uint32_t i = wave_first + static_cast<uint32_t>(e * kWaveSize + lane);
                if (i < n)
                {
                    const uint32_t digit = (tile_keys[e] >> shift) & 255u;
                    const uint32_t position = wave_counts[wave][digit] + tile_ranks[e];
                    target_keys[position] = tile_keys[e];
                    if (PAIRS)
                        target_indices[position] = tile_indices[e];
                }
            }
            __syncthreads();
        }
        __threadfence_block();
        __syncthreads();
    }
}

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

struct RecoverScratch
{
    uint32_t wave_counts[kReplayWaves];
    int32_t found;
};

// Token index of position `rank` of the sorted row, from the logits: the sort is stable, so it is
// the (rank - first position of that key)-th element, in index order, whose key equals keys[rank].
// Every thread of the workgroup must call it.
template <int DTYPE>
__device__ __forceinline__ int32_t recover_token_index(
    const void* row_pointer, uint32_t vocab, const uint32_t* keys, uint32_t rank, RecoverScratch& scratch, int tid)
{
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    const uint32_t key = keys[rank];
    uint32_t low = 0, high = rank; // first position holding this key
    while (low < high)
    {
        const uint32_t middle = (low + high) >> 1;
        if (keys[middle] < key)
            low = middle + 1;
        else
            high = middle;
    }
    const uint32_t ordinal = rank - low;
    uint32_t passed = 0; // matches before the current chunk
    if (tid == 0)
        scratch.found = -1;
    __syncthreads();
    for (uint32_t base = 0; base < vocab; base += kReplayChunk)
    {
        const uint32_t first = base + static_cast<uint32_t>(tid) * kReplayPerThread;
        uint32_t matches = 0;
        uint32_t count = 0;
#pragma unroll
        for (int j = 0; j < kReplayPerThread; ++j)
        {
            const uint32_t i = first + j;
            if (i < vocab && descending_key(load_logit<DTYPE>(row_pointer, i)) == key)
            {
                matches |= 1u << j;
                ++count;
            }
        }
        uint32_t inclusive = count;
#pragma unroll
        for (int step = 1; step < kWaveSize; step <<= 1)
        {
            const uint32_t up = __shfl_up(inclusive, step, kWaveSize);
            if (lane >= step)
                inclusive += up;
        }
        if (lane == kWaveSize - 1)
            scratch.wave_counts[wave] = inclusive;
        __syncthreads();
        uint32_t before = passed;
        uint32_t chunk_total = 0;
        for (int w = 0; w < kReplayWaves; ++w)
        {
            const uint32_t c = scratch.wave_counts[w];
            if (w < wave)
                before += c;
            chunk_total += c;
        }
        before += inclusive - count;
        if (ordinal >= before && ordinal < before + count)
        {
            uint32_t skip = ordinal - before;
#pragma unroll
            for (int j = 0; j < kReplayPerThread; ++j)
            {
                if (matches & (1u << j))
                {
                    if (skip == 0)
                        scratch.found = static_cast<int32_t>(first + j);
                    --skip;
                }
            }
        }
        __syncthreads();
        if (scratch.found >= 0)
            break;
        passed += chunk_total;
    }
    const int32_t found = scratch.found;
    __syncthreads();
    return found;
}

// Walks the sorted row as the CPU sampler does (src/engine/session.cpp:84-134, :429-442), with
// every running sum reproduced exactly by exact_running_sum.  One workgroup per row.
template <int DTYPE>
__global__ __launch_bounds__(kReplayThreads) void general_replay_kernel(SamplerArgs a)
{
    const uint32_t row = blockIdx.x;
    if (a.row_state[row] != kRowNeedsGeneral)
        return;
    const int tid = threadIdx.x;
    const ncnn_moe_sample_params p = a.params[row];
    const uint32_t* keys = a.sort_keys[1] + row * a.sort_stride;
    const uint32_t* indices = a.sort_indices[1] + row * a.sort_stride; // valid only when the distribution is exported
    const bool have_indices = a.distribution_count != nullptr;
    const uint32_t vocab = a.vocab;
    const char* row_pointer = static_cast<const char*>(a.logits) +
        static_cast<size_t>(row) * a.row_stride * LogitsVector<DTYPE>::kElementBytes;

    __shared__ ReplayScratch scratch;
    __shared__ RecoverScratch recover_scratch;

    uint8_t flags = NCNN_MOE_ROW_FLAG_GENERAL_PATH;
    {
        uint32_t effective_k = 0;
        int status = 0;
        if (resolve_row_mode(p, vocab, a.segments, 0, effective_k, status) != kModeGeneral)
            flags |= NCNN_MOE_ROW_FLAG_FALLBACK;
    }
    if (keys[vocab - 1] == 0xffffffffu)
        flags |= NCNN_MOE_ROW_FLAG_HAS_NAN;
    if (tid == 0)
        a.row_state[row] = kRowDone;

    if (p.temperature == 0.0f)
    {
        // a greedy row whose select overflowed (every logit tied): first finite logit in sorted order,
        // non-finite logits skipped (src/engine/session.cpp:404-424)
        uint32_t low = 0, high = vocab;
        while (low < high)
        {
            const uint32_t middle = (low + high) >> 1;
            if (keys[middle] <= kPositiveInfinityKey)
                low = middle + 1;
            else
                high = middle;
        }
        const bool any_finite = low < vocab && keys[low] <= kLastFiniteKey;
        int32_t token = -1;
        if (any_finite)
            token = have_indices ? static_cast<int32_t>(indices[low])
                                 : recover_token_index<DTYPE>(row_pointer, vocab, keys, low, recover_scratch, tid);
        if (tid == 0)
        {
            if (any_finite)
                write_token(a, row, p, token, 1.0f, 1u, 0, flags);
            else
                write_error(a, row, NCNN_MOE_ROW_NO_FINITE_LOGIT, flags);
        }
        return;
    }

    // finite logits form a prefix of the sorted row, after any +inf (which rejects the row)
    const uint32_t first_key = keys[0];
    if (first_key <= kPositiveInfinityKey || first_key > kLastFiniteKey)
    {
        if (tid == 0)
            write_error(a, row, NCNN_MOE_ROW_NO_FINITE_LOGIT, flags);
        return;
    }
    uint32_t low = 0, high = vocab; // first position whose key is not finite
    while (low < high)
    {
        const uint32_t middle = (low + high) >> 1;
        if (keys[middle] <= kLastFiniteKey)
            low = middle + 1;
        else
            high = middle;
    }
    uint32_t n = low;
    if (p.top_k > 0 && p.top_k < vocab && n > p.top_k)
        n = p.top_k;

    SortedRow sorted;
    sorted.keys = keys;
    sorted.temperature = p.temperature;
    sorted.maximum = value_from_descending_key(first_key) / p.temperature;
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

    if (a.distribution_count != nullptr && row == 0)
    {
        const uint32_t limit = kept < a.distribution_cap ? kept : a.distribution_cap;
        for (uint32_t i = tid; i < limit; i += kReplayThreads)
        {
            a.distribution_ids[i] = static_cast<int32_t>(indices[i]);
            a.distribution_probabilities[i] = row_term<2>(sorted, i);
        }
        if (tid == 0)
            *a.distribution_count = kept;
    }

    if (kept == 1)
    {
        const int32_t token = have_indices ? static_cast<int32_t>(indices[0])
                                           : recover_token_index<DTYPE>(row_pointer, vocab, keys, 0, recover_scratch, tid);
        if (tid == 0)
            write_token(a, row, p, token, 1.0f, 1u, 0, flags);
        return;
    }

    // ---- inverse-CDF draw over the kept prefix (session.cpp:432-442)
    const RunningSum draw = exact_running_sum<2>(sorted, kept, kStopAbove, a.uniforms[row], scratch, tid);
    const uint32_t selected = draw.stopped ? draw.stop_index : kept - 1u;
    const int32_t token = have_indices ? static_cast<int32_t>(indices[selected])
                                       : recover_token_index<DTYPE>(row_pointer, vocab, keys, selected, recover_scratch, tid);
    if (tid == 0)
        write_token(a, row, p, token, row_term<2>(sorted, selected), kept, 1, flags);
}

// Evaluates expf_libm on n values (test hook).
__global__ void expf_probe_kernel(const float* in, float* out, size_t n)
{
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n)
        out[i] = expf_libm(in[i]);
}

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_SAMPLER_KERNELS_H
