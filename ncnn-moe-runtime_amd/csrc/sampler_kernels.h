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
    int debug_stage; // TEMPORARY profiling knob

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

template <int DTYPE>
__global__ __launch_bounds__(kScanThreads) void scan_select_kernel(SamplerArgs a)
{
    using Vector = LogitsVector<DTYPE>;
    constexpr int kWidth = Vector::kWidth;
    constexpr int kVectors = kValuesPerLane / kWidth;
    constexpr uint32_t kNegativeInfinity = 0xff800000u;

    const uint32_t row = blockIdx.y;
    const uint32_t segment = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;

    __shared__ float lane_maxima[kScanWaves][kWaveSize];
    __shared__ float candidate_values[kScanWaves][kWaveCandidateCap];
    __shared__ int32_t candidate_indices[kScanWaves][kWaveCandidateCap];
    __shared__ int candidate_counts[kScanWaves];
    __shared__ uint32_t block_flags;
    __shared__ int block_is_last;
    __shared__ float survivor_values[kSurvivorCap];
    __shared__ int32_t survivor_indices[kSurvivorCap];
    __shared__ int survivor_count;
    __shared__ float reduce_scratch[kScanWaves];
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
                a.row_state[row] = kRowNeedsGeneral;
            }
        }
        return;
    }
    const bool greedy = mode == kModeGreedy;
    const int top_k = static_cast<int>(effective_k);

    if (tid == 0)
        block_flags = 0;

    // ---- load the segment: 16-byte loads from the 16-byte aligned address at or below the row start
    const char* row_pointer = static_cast<const char*>(a.logits) +
        static_cast<size_t>(row) * a.row_stride * Vector::kElementBytes;
    const uint32_t misalignment =
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row_pointer) & 15u) / Vector::kElementBytes;
    const char* aligned_base = row_pointer - static_cast<size_t>(misalignment) * Vector::kElementBytes;
    const uint32_t valid_begin = misalignment;
    const uint32_t valid_end = misalignment + a.vocab;
    const uint32_t segment_base = segment * static_cast<uint32_t>(kSegmentValues);

    float values[kValuesPerLane];
    uint4 raw[kVectors];
#pragma unroll
    for (int it = 0; it < kVectors; ++it)
    {
        const uint32_t first = segment_base + static_cast<uint32_t>(it * kScanThreads + tid) * kWidth;
        if (first < valid_end && first + kWidth > valid_begin)
            raw[it] = *reinterpret_cast<const uint4*>(aligned_base + static_cast<size_t>(first) * Vector::kElementBytes);
        else
            raw[it] = make_uint4(kNegativeInfinity, kNegativeInfinity, kNegativeInfinity, kNegativeInfinity);
    }
#pragma unroll
    for (int it = 0; it < kVectors; ++it)
    {
        const uint32_t first = segment_base + static_cast<uint32_t>(it * kScanThreads + tid) * kWidth;
        const bool any_valid = first < valid_end && first + kWidth > valid_begin;
        if (any_valid)
            Vector::unpack(raw[it], &values[it * kWidth]);
        else
        {
#pragma unroll
            for (int c = 0; c < kWidth; ++c)
                values[it * kWidth + c] = __uint_as_float(kNegativeInfinity);
        }
        if (any_valid && (first < valid_begin || first + kWidth > valid_end))
        {
#pragma unroll
            for (int c = 0; c < kWidth; ++c)
            {
                const uint32_t position = first + c;
                if (position < valid_begin || position >= valid_end)
                    values[it * kWidth + c] = __uint_as_float(kNegativeInfinity);
            }
        }
    }

    // ---- per-lane maximum (NaN ignored), NaN / +inf detection
    uint32_t local_flags = 0;
    float lane_max = __uint_as_float(kNegativeInfinity);
    bool saw_nan = false;
#pragma unroll
    for (int i = 0; i < kValuesPerLane; ++i)
    {
        float v = values[i];
        saw_nan = saw_nan || (v != v);
        if (greedy && v == __uint_as_float(0x7f800000u))
        {
            v = __uint_as_float(kNegativeInfinity); // greedy skips every non-finite logit (session.cpp:411-412)
            values[i] = v;
        }
        lane_max = fmaxf(lane_max, v);
    }
    if (saw_nan)
        local_flags |= kScanSawNan;
    if (lane_max == __uint_as_float(0x7f800000u))
        local_flags |= kScanSawPositiveInfinity;

    if (a.debug_stage == 1)
    {
        if (lane_max == 12345.678f)
            a.segment_values[0] = lane_max;
        return;
    }
    // ---- K-th largest lane maximum of the workgroup: a lower bound for the K-th best logit of the
    // row, because the lanes above it each hold a distinct logit at least that large.
    const float sorted_max = wave_sort_descending(lane_max, lane);
    lane_maxima[wave][lane] = sorted_max;
    __syncthreads();
    float merged = sorted_max;
#pragma unroll
    for (int other = 1; other < kScanWaves; ++other)
    {
        const int source = (wave + other) & (kScanWaves - 1);
        const float reversed = lane_maxima[source][kWaveSize - 1 - lane];
        merged = wave_bitonic_merge_descending(fmaxf(merged, reversed), lane);
    }
    float threshold = read_lane(merged, top_k - 1);
    threshold = fmaxf(threshold, -3.402823466e+38f); // -inf and padding never qualify

    if (a.debug_stage == 2)
    {
        if (threshold == 12345.678f)
            a.segment_values[0] = threshold;
        return;
    }
    // ---- collect the lane values at or above the bound into this wave's LDS region
    int wave_count = 0;
#pragma unroll
    for (int i = 0; i < kValuesPerLane; ++i)
    {
        const bool hit = values[i] >= threshold;
        const uint64_t hits = __ballot(hit);
        if (hits != 0)
        {
            const int position = wave_count + lanes_below(hits);
            if (hit && position < kWaveCandidateCap)
            {
                const int it = i / kWidth;
                const int c = i % kWidth;
                const uint32_t element = segment_base + static_cast<uint32_t>(it * kScanThreads + tid) * kWidth + c - misalignment;
                candidate_values[wave][position] = values[i];
                candidate_indices[wave][position] = static_cast<int32_t>(element);
            }
            wave_count += __popcll(hits);
        }
    }
    if (lane == 0)
        candidate_counts[wave] = wave_count;
    if (local_flags != 0)
        atomicOr(&block_flags, local_flags);
    __syncthreads();

    if (a.debug_stage == 3)
    {
        if (candidate_counts[0] == 12345)
            a.segment_values[0] = 1.0f;
        return;
    }
    // ---- exact rank of every candidate among the workgroup's candidates; the best K go to HBM
    int counts[kScanWaves];
    int total = 0;
    bool overflow = false;
#pragma unroll
    for (int w = 0; w < kScanWaves; ++w)
    {
        counts[w] = candidate_counts[w];
        overflow = overflow || counts[w] > kWaveCandidateCap;
        total += counts[w];
    }
    const size_t segment_slot = (static_cast<size_t>(row) * a.segments + segment);
    if (!overflow)
    {
        for (int slot = lane; slot < counts[wave]; slot += kWaveSize)
        {
            const float my_value = candidate_values[wave][slot];
            const int32_t my_index = candidate_indices[wave][slot];
            int rank = 0;
            for (int w = 0; w < kScanWaves; ++w)
            {
                for (int j = 0; j < counts[w]; ++j)
                    rank += candidate_before(candidate_values[w][j], candidate_indices[w][j], my_value, my_index) ? 1 : 0;
            }
            if (rank < top_k)
            {
                a.segment_values[segment_slot * kFastTopK + rank] = my_value;
                a.segment_indices[segment_slot * kFastTopK + rank] = my_index;
            }
        }
    }
    if (tid == 0)
    {
        a.segment_counts[segment_slot] = overflow ? 0u : static_cast<uint32_t>(total < top_k ? total : top_k);
        uint32_t flags = block_flags;
        if (overflow)
            flags |= kScanOverflow;
        if (flags != 0)
            atomicOr(&a.row_flags[row], flags);
    }

    if (a.debug_stage == 4)
        return;
    // ---- the last workgroup of the row merges the segments
    __threadfence();
    __syncthreads();
    if (tid == 0)
    {
        const uint32_t previous = atomicAdd(&a.row_counter[row], 1u);
        block_is_last = previous == a.segments - 1 ? 1 : 0;
        survivor_count = 0;
    }
    __syncthreads();
    if (!block_is_last)
        return;
    __threadfence();
    if (a.debug_stage == 5)
    {
        if (tid == 0)
        {
            a.row_counter[row] = 0;
            a.row_flags[row] = 0;
        }
        return;
    }

    const uint32_t row_flags = __hip_atomic_load(&a.row_flags[row], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint8_t result_flags = (row_flags & kScanSawNan) ? NCNN_MOE_ROW_FLAG_HAS_NAN : 0;
    __syncthreads();
    if (tid == 0)
    {
        a.row_counter[row] = 0;
        a.row_flags[row] = 0;
    }
    if (row_flags & kScanOverflow)
    {
        if (tid == 0)
            a.row_state[row] = kRowNeedsGeneral;
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

    const size_t row_slot = static_cast<size_t>(row) * a.segments;
    // prune bound: the best K-th value of any segment that holds K candidates
    float bound = __uint_as_float(kNegativeInfinity);
    for (uint32_t s = tid; s < a.segments; s += kScanThreads)
    {
        if (a.segment_counts[row_slot + s] == static_cast<uint32_t>(top_k))
            bound = fmaxf(bound, a.segment_values[(row_slot + s) * kFastTopK + top_k - 1]);
    }
#pragma unroll
    for (int j = kWaveSize >> 1; j > 0; j >>= 1)
        bound = fmaxf(bound, __shfl_xor(bound, j, kWaveSize));
    if (lane == 0)
        reduce_scratch[wave] = bound;
    __syncthreads();
    bound = fmaxf(fmaxf(reduce_scratch[0], reduce_scratch[1]), fmaxf(reduce_scratch[2], reduce_scratch[3]));

    const uint32_t slots = a.segments * kFastTopK;
    for (uint32_t slot = tid; slot < slots; slot += kScanThreads)
    {
        const uint32_t s = slot / kFastTopK;
        const uint32_t r = slot % kFastTopK;
        if (r < a.segment_counts[row_slot + s])
        {
            const float v = a.segment_values[(row_slot + s) * kFastTopK + r];
            if (v >= bound)
            {
                const int position = atomicAdd(&survivor_count, 1);
                if (position < kSurvivorCap)
                {
                    survivor_values[position] = v;
                    survivor_indices[position] = a.segment_indices[(row_slot + s) * kFastTopK + r];
                }
            }
        }
    }
    __syncthreads();
    const int survivors = survivor_count;
    if (survivors > kSurvivorCap)
    {
        if (tid == 0)
            a.row_state[row] = kRowNeedsGeneral;
        return;
    }
    for (int slot = tid; slot < survivors; slot += kScanThreads)
    {
        const float my_value = survivor_values[slot];
        const int32_t my_index = survivor_indices[slot];
        int rank = 0;
        for (int j = 0; j < survivors; ++j)
            rank += candidate_before(survivor_values[j], survivor_indices[j], my_value, my_index) ? 1 : 0;
        if (rank < top_k)
        {
            final_values[rank] = my_value;
            final_indices[rank] = my_index;
        }
    }
    __syncthreads();
    if (wave != 0)
        return;
    const int n = survivors < top_k ? survivors : top_k;
    if (lane == 0)
        a.row_state[row] = kRowDone;
    if (n == 0)
    {
        if (lane == 0)
            write_error(a, row, NCNN_MOE_ROW_NO_FINITE_LOGIT, result_flags);
        return;
    }
    const float value = lane < n ? final_values[lane] : 0.0f;
    const int32_t index = lane < n ? final_indices[lane] : -1;
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
// The sorted keys and indices end in sort_keys[1] / sort_indices[1].
template <int DTYPE>
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

    for (int pass = 0; pass < kPasses; ++pass)
    {
        const int shift = 8 * (pass + kFirstDigit);
        const uint32_t* source_keys = keys[(pass + 1) & 1];   // pass 0 reads the logits instead
        const uint32_t* source_indices = indices[(pass + 1) & 1];
        uint32_t* target_keys = keys[pass & 1];
        uint32_t* target_indices = indices[pass & 1];
        if (tid < 256)
            digit_base[tid] = histogram[pass][tid];
        for (uint32_t tile = 0; tile < n; tile += kSortThreads)
        {
            for (int i = tid; i < kSortWaves * 256; i += kSortThreads)
                (&wave_counts[0][0])[i] = 0;
            const uint32_t i = tile + tid;
            const bool valid = i < n;
            uint32_t key = 0xffffffffu;
            uint32_t index = i;
            if (valid)
            {
                if (pass == 0)
                    key = descending_key(load_logit<DTYPE>(row_pointer, i));
                else
                {
                    key = source_keys[i];
                    index = source_indices[i];
                }
            }
            const uint32_t digit = (key >> shift) & 255u;
            uint64_t peers = __ballot(valid);
#pragma unroll
            for (int b = 0; b < 8; ++b)
            {
                const bool bit = (digit >> b) & 1u;
                const uint64_t set = __ballot(valid && bit);
                peers &= bit ? set : ~set;
            }
            const int rank_in_wave = lanes_below(peers);
            __syncthreads();
            if (valid && rank_in_wave == 0)
                wave_counts[wave][digit] = static_cast<uint32_t>(__popcll(peers));
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
            if (valid)
            {
                const uint32_t position = wave_counts[wave][digit] + static_cast<uint32_t>(rank_in_wave);
                target_keys[position] = key;
                target_indices[position] = index;
            }
            __syncthreads();
        }
        __threadfence_block();
        __syncthreads();
    }
}

// Walks the sorted row as the CPU sampler does (src/engine/session.cpp:84-134, :429-442).
// Terms are computed by the whole workgroup a chunk at a time; thread 0 adds them in order.
__global__ __launch_bounds__(kReplayThreads) void general_replay_kernel(SamplerArgs a)
{
    const uint32_t row = blockIdx.x;
    if (a.row_state[row] != kRowNeedsGeneral)
        return;
    const int tid = threadIdx.x;
    const ncnn_moe_sample_params p = a.params[row];
    const uint32_t* keys = a.sort_keys[1] + row * a.sort_stride;
    const uint32_t* indices = a.sort_indices[1] + row * a.sort_stride;
    const uint32_t vocab = a.vocab;

    __shared__ float chunk[kReplayChunk];
    __shared__ float shared_value;
    __shared__ float shared_cumulative;
    __shared__ uint32_t shared_count;
    __shared__ int shared_stop;
    __shared__ int shared_selected;

    uint8_t flags = NCNN_MOE_ROW_FLAG_GENERAL_PATH;
    {
        uint32_t effective_k = 0;
        int status = 0;
        if (resolve_row_mode(p, vocab, a.segments, 0, effective_k, status) == kModeTopK && !a.force_general)
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
        if (tid == 0)
        {
            if (low < vocab && keys[low] <= kLastFiniteKey)
                write_token(a, row, p, static_cast<int32_t>(indices[low]), 1.0f, 1u, 0, flags);
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

    const float temperature = p.temperature;
    const float maximum = value_from_descending_key(first_key) / temperature;

    // ---- normaliser: sequential sum in sorted order; stops once the sum no longer moves, which is
    // exact because the terms are non-increasing
    if (tid == 0)
    {
        shared_value = 0.0f;
        shared_stop = 0;
    }
    __syncthreads();
    for (uint32_t base = 0; base < n; base += kReplayChunk)
    {
        for (int j = tid; j < kReplayChunk; j += kReplayThreads)
        {
            const uint32_t i = base + j;
            chunk[j] = i < n ? expf_libm(value_from_descending_key(keys[i]) / temperature - maximum) : 0.0f;
        }
        __syncthreads();
        if (tid == 0)
        {
            float sum = shared_value;
            const uint32_t count = n - base < kReplayChunk ? n - base : kReplayChunk;
            if (base > 0 && sum + chunk[0] == sum)
            {
                shared_stop = 1;
            }
            else
            {
                for (uint32_t j = 0; j < count; ++j)
                    sum += chunk[j];
                shared_value = sum;
            }
        }
        __syncthreads();
        if (shared_stop)
            break;
    }
    const float normalizer = shared_value;
    if (!is_finite_f32(normalizer) || !(normalizer > 0.0f))
    {
        if (tid == 0)
            write_error(a, row, NCNN_MOE_ROW_INVALID_DISTRIBUTION, flags);
        return;
    }

    // ---- Min-P and Top-P: probabilities are non-increasing, so both keep a prefix
    const float top_probability = expf_libm(value_from_descending_key(first_key) / temperature - maximum) / normalizer;
    const float min_p_threshold = top_probability * p.min_p;
    const bool use_min_p = p.min_p > 0.0f;
    __syncthreads();
    if (tid == 0)
    {
        shared_cumulative = 0.0f;
        shared_count = 0;
        shared_stop = 0;
    }
    __syncthreads();
    for (uint32_t base = 0; base < n; base += kReplayChunk)
    {
        for (int j = tid; j < kReplayChunk; j += kReplayThreads)
        {
            const uint32_t i = base + j;
            float probability = -1.0f;
            if (i < n)
            {
                probability = expf_libm(value_from_descending_key(keys[i]) / temperature - maximum) / normalizer;
                if (use_min_p && !(probability >= min_p_threshold))
                    probability = -1.0f;
            }
            chunk[j] = probability;
        }
        __syncthreads();
        if (tid == 0)
        {
            float cumulative = shared_cumulative;
            uint32_t count = shared_count;
            int stop = 0;
            for (int j = 0; j < kReplayChunk; ++j)
            {
                const float probability = chunk[j];
                if (probability < 0.0f)
                {
                    stop = 1; // end of the row or first candidate under the Min-P threshold
                    break;
                }
                cumulative += probability;
                ++count;
                if (cumulative >= p.top_p)
                {
                    stop = 1;
                    break;
                }
            }
            shared_cumulative = cumulative;
            shared_count = count;
            shared_stop = stop;
        }
        __syncthreads();
        if (shared_stop)
            break;
    }
    const uint32_t kept = shared_count;
    const float renormalizer = shared_cumulative;

    if (a.distribution_count != nullptr && row == 0)
    {
        const uint32_t limit = kept < a.distribution_cap ? kept : a.distribution_cap;
        for (uint32_t i = tid; i < limit; i += kReplayThreads)
        {
            const float probability = expf_libm(value_from_descending_key(keys[i]) / temperature - maximum) / normalizer;
            a.distribution_ids[i] = static_cast<int32_t>(indices[i]);
            a.distribution_probabilities[i] = probability / renormalizer;
        }
        if (tid == 0)
            *a.distribution_count = kept;
    }

    if (kept == 1)
    {
        if (tid == 0)
            write_token(a, row, p, static_cast<int32_t>(indices[0]), 1.0f, 1u, 0, flags);
        return;
    }

    // ---- inverse-CDF draw over the kept prefix
    const float uniform = a.uniforms[row];
    __syncthreads();
    if (tid == 0)
    {
        shared_cumulative = 0.0f;
        shared_selected = -1;
    }
    __syncthreads();
    for (uint32_t base = 0; base < kept; base += kReplayChunk)
    {
        for (int j = tid; j < kReplayChunk; j += kReplayThreads)
        {
            const uint32_t i = base + j;
            float probability = 0.0f;
            if (i < kept)
                probability = (expf_libm(value_from_descending_key(keys[i]) / temperature - maximum) / normalizer) / renormalizer;
            chunk[j] = probability;
        }
        __syncthreads();
        if (tid == 0)
        {
            float cumulative = shared_cumulative;
            const uint32_t count = kept - base < kReplayChunk ? kept - base : kReplayChunk;
            for (uint32_t j = 0; j < count; ++j)
            {
                cumulative += chunk[j];
                if (uniform < cumulative)
                {
                    shared_selected = static_cast<int>(base + j);
                    break;
                }
            }
            shared_cumulative = cumulative;
        }
        __syncthreads();
        if (shared_selected >= 0)
            break;
    }
    if (tid == 0)
    {
        const uint32_t selected = shared_selected >= 0 ? static_cast<uint32_t>(shared_selected) : kept - 1;
        const float probability =
            (expf_libm(value_from_descending_key(keys[selected]) / temperature - maximum) / normalizer) / renormalizer;
        write_token(a, row, p, static_cast<int32_t>(indices[selected]), probability, kept, 1, flags);
    }
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
