// Select path: the one HBM pass over the logits for greedy rows and rows with a Top-K window.
//
// A workgroup of 512 threads streams a contiguous range of chunks of one row (a chunk is 512 lanes x
// 5 fp32 or 3 bf16 16-byte vectors) and keeps the row's Top-K candidates of that range:
//   * per-vector and per-lane maxima of the chunk;
//   * a bound that at least K logits reach: for the first chunk the exact K-th largest of the 512
//     lane maxima, later the K-th best candidate collected so far (the list is tightened whenever
//     it grows past 2K + 64 entries);
//   * the logits at or above the bound are appended to a candidate list in LDS.
// One segment per row (large batches): the workgroup finishes the row itself.  Several segments per
// row (small batches, so that every CU streams): each hands its list over through HBM and the last
// workgroup to arrive merges them.  Either way the candidates are reduced to the exact best K by
// (logit descending, index ascending) and the CPU sampler's epilogue runs on them.
#ifndef NCNN_MOE_HIP_SAMPLER_SELECT_H
#define NCNN_MOE_HIP_SAMPLER_SELECT_H

#include "sampler_exact_sum.h"

namespace ncnn_moe_hip {

template <bool WIDE>
struct SelectShared
{
    static constexpr int kListCap = WIDE ? kWideListCap : kNarrowListCap;
    static constexpr int kSortedCap = WIDE ? kSelectTopK : 1;
    static_assert(kSelectTopK <= 2 * kScanThreads, "the ordered window is copied two entries per thread");
    static_assert(kSumThreads <= kScanThreads, "the exact running sums need kSumThreads threads of the workgroup that calls them");
    BoundScratch bound;
    alignas(16) uint32_t list_keys[kListCap]; // (the wide finish sorts the list as one array of 64-bit pairs over these two)
    int32_t list_indices[kListCap];
    uint32_t list_count;
    uint32_t block_flags;
    int block_is_last;
    int block_all_local;
    float final_values[kFastTopK];
    int32_t final_indices[kFastTopK];
    uint32_t sorted_keys[kSortedCap];    // descending keys of the ordered window when K > 64
    uint32_t sorted_indices[kSortedCap];
    ReplayScratch replay;                // of the exact running sums over such a window
};

// Appends the caller's candidate (if `hit`) to the workgroup's list.  Positions are reserved per
// wave with one LDS atomic; the order inside the list is irrelevant.  Called by whole waves.
template <bool WIDE>
__device__ __forceinline__ void append_candidate(SelectShared<WIDE>& shared, bool hit, uint32_t key, int32_t index, int lane)
{
    const uint64_t hits = __ballot(hit);
    if (hits == 0)
        return;
    uint32_t base = 0;
    if (lane == __builtin_ctzll(hits))
        base = atomicAdd(&shared.list_count, static_cast<uint32_t>(__popcll(hits)));
    base = __builtin_amdgcn_readlane(base, __builtin_ctzll(hits));
    const uint32_t position = base + static_cast<uint32_t>(lanes_below(hits));
    if (hit && position < static_cast<uint32_t>(SelectShared<WIDE>::kListCap))
    {
        shared.list_keys[position] = key;
        shared.list_indices[position] = index;
    }
}

// Raises the bound to (a lower bound of) the K-th best candidate of the list and drops the
// candidates below it.  All threads call it; returns the new bound key.  exact == false (lists of one
// entry per thread): the cheaper bound of the eight waves' own searches, which at least K entries
// reach and usually two to three times as many.
template <bool WIDE>
__device__ __forceinline__ uint32_t tighten_list(SelectShared<WIDE>& shared, uint32_t bound_key, int top_k, int tid, bool exact = true)
{
    constexpr int kPerThread = SelectShared<WIDE>::kListCap / kScanThreads;
    const int lane = tid & (kWaveSize - 1);
    const uint32_t count = min(shared.list_count, static_cast<uint32_t>(SelectShared<WIDE>::kListCap));
    uint32_t keys[kPerThread];
    int32_t indices[kPerThread];
    uint32_t best = 0;
#pragma unroll
    for (int j = 0; j < kPerThread; ++j)
    {
        // one entry per thread: entry q goes to wave q % 8, so that every wave holds its share of a short
        // list (the waves' own searches bound loosely where some waves hold nothing)
        const uint32_t q = kPerThread == 1 ? static_cast<uint32_t>(lane * kScanWaves + (tid >> 6))
                                           : static_cast<uint32_t>(j * kScanThreads + tid);
        keys[j] = q < count ? shared.list_keys[q] : 0u;
        indices[j] = q < count ? shared.list_indices[q] : 0;
        best = max(best, keys[j]);
    }
    uint32_t kth;
    if constexpr (kPerThread > 1)
    {
        // a long list: the exact K-th best of all its entries (a bound from per-thread maxima would keep
        // most of a list whose threads hold several members of a wide window each)
        kth = workgroup_kth_of_keys_by_digits(keys, top_k, tid, shared.bound);
    }
    else
    {
        const uint32_t thread_keys[1] = {best};
        kth = workgroup_kth_largest_key(thread_keys, top_k, tid, shared.bound, exact);
    }
    bound_key = max(bound_key, kth);
    if (tid == 0)
        shared.list_count = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kPerThread; ++j)
        append_candidate(shared, keys[j] != 0u && keys[j] >= bound_key, keys[j], indices[j], lane);
    __syncthreads();
    return bound_key;
}

// The ordered window (lane i holds candidate i of n <= 64) to the row's result; one wave.
__device__ __forceinline__ void finish_ordered_wave(
    const SamplerArgs& a, uint32_t row, const ncnn_moe_sample_params& p, bool greedy,
    float value, int32_t index, int n, int lane, uint8_t result_flags, float uniform, const uint64_t* exp2_table)
{
    if (greedy)
    {
        if (lane == 0)
        {
            write_token(a, row, p, index, 1.0f, 1u, 0, result_flags);
            if (a.distribution_count != nullptr)
            {
                a.distribution_count[row] = 1;
                if (a.distribution_cap > 0)
                {
                    a.distribution_ids[static_cast<size_t>(row) * a.distribution_cap] = index;
                    a.distribution_probabilities[static_cast<size_t>(row) * a.distribution_cap] = 1.0f;
                }
            }
        }
        return;
    }
    finish_row_wave(a, row, p, value, index, n, lane, result_flags, uniform, exp2_table);
}

// From the candidate list to the sampled token: exact best K, their order, the epilogue.
// All threads of the workgroup call it; n_list <= kListCap.
template <bool WIDE>
__device__ __forceinline__ void finish_from_list(
    const SamplerArgs& a, uint32_t row, const ncnn_moe_sample_params& p, bool greedy, int top_k,
    SelectShared<WIDE>& shared, uint8_t result_flags, int tid, float uniform, const uint64_t* exp2_table = kExp2Table)
{
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    // the count comes from LDS: telling the compiler that it is the same in every lane keeps the loops
    // over it scalar (a loop it takes for divergent costs several times as much per trip)
    int n_list = __builtin_amdgcn_readfirstlane(static_cast<int>(shared.list_count));
    if (top_k <= kFastTopK)
    {
        if constexpr (WIDE)
        {
            if (n_list > 8 * kWaveSize)
            {
                tighten_list(shared, 0u, top_k, tid);
                n_list = __builtin_amdgcn_readfirstlane(static_cast<int>(shared.list_count));
            }
        }
        else if (n_list > 2 * kWaveSize)
        {
            // A workgroup that streamed many chunks under its first chunk's bound ends with a few hundred
            // candidates.  All eight waves cut the list down to what the rankings below take (128); one
            // wave selecting among them bit by bit takes several times as long.
            tighten_list(shared, 0u, top_k, tid, false);
            n_list = __builtin_amdgcn_readfirstlane(static_cast<int>(shared.list_count));
            if (n_list > 2 * kWaveSize)
            {
                tighten_list(shared, 0u, top_k, tid, true);
                n_list = __builtin_amdgcn_readfirstlane(static_cast<int>(shared.list_count));
            }
        }
        if (n_list > 8 * kWaveSize)
        {
            // ties left more candidates than one wave orders: the full-order kernels take the row
            if (tid == 0)
            {
                write_pending(a, row);
                a.row_state[row] = kRowNeedsGeneral;
            }
            return;
        }
        int n = 0;
        if (n_list <= kWaveSize)
        {
            // one candidate per lane: its rank among all of them is its place in the window.  Every
            // wave counts the candidates of its eighth of the list that go before the lane's own;
            // wave 0 adds the eight counts up and goes on alone.
            const uint32_t key = lane < n_list ? shared.list_keys[lane] : 0u;
            const int32_t candidate_index = lane < n_list ? shared.list_indices[lane] : 0;
            constexpr int kShare = kWaveSize / kScanWaves;
            int partial = 0;
#pragma unroll
            for (int k = 0; k < kShare; ++k)
            {
                const int j = wave * kShare + k;
                const uint32_t other_key = shared.list_keys[j];
                const int32_t other_index = shared.list_indices[j];
                partial += (j < n_list && (other_key > key || (other_key == key && other_index < candidate_index))) ? 1 : 0;
            }
            uint32_t* const partial_counts = shared.bound.hot_keys; // kScanWaves x 64 counts
            partial_counts[wave * kWaveSize + lane] = static_cast<uint32_t>(partial);
            __syncthreads();
            if (wave != 0)
                return;
            int before = 0;
#pragma unroll
            for (int w = 0; w < kScanWaves; ++w)
                before += static_cast<int>(partial_counts[w * kWaveSize + lane]);
            if (lane < n_list && before < top_k)
            {
                shared.final_values[before] = value_from_ascending_key(key);
                shared.final_indices[before] = candidate_index;
            }
            n = n_list < top_k ? n_list : top_k;
            if (lane == 0)
                a.row_state[row] = kRowDone;
            if (n == 0)
            {
                if (lane == 0)
                    write_error(a, row, NCNN_MOE_ROW_NO_FINITE_LOGIT, result_flags);
                return;
            }
            const float value = lane < n ? shared.final_values[lane] : 0.0f;
            const int32_t index = lane < n ? shared.final_indices[lane] : -1;
            finish_ordered_wave(a, row, p, greedy, value, index, n, lane, result_flags, uniform, exp2_table);
            return;
        }
        if (n_list <= 2 * kWaveSize)
        {
            // two candidates per lane of wave 0: thread t counts, for candidate t % 128, the candidates of
            // its quarter of the list that go before it; wave 0 adds the four counts of its two up
            const int c = tid & (2 * kWaveSize - 1);
            const int part = tid >> 7;
            const uint32_t key = c < n_list ? shared.list_keys[c] : 0u;
            const int32_t candidate_index = c < n_list ? shared.list_indices[c] : 0;
            constexpr int kShare = 2 * kWaveSize / (kScanThreads / (2 * kWaveSize));
            int partial = 0;
#pragma unroll 8
            for (int k = 0; k < kShare; ++k)
            {
                const int j = part * kShare + k;
                const uint32_t other_key = shared.list_keys[j];
                const int32_t other_index = shared.list_indices[j];
                partial += (j < n_list && (other_key > key || (other_key == key && other_index < candidate_index))) ? 1 : 0;
            }
            uint32_t* const partial_counts = shared.bound.hot_keys; // 4 x 128 counts
            partial_counts[part * 2 * kWaveSize + c] = static_cast<uint32_t>(partial);
            __syncthreads();
            if (wave != 0)
                return;
#pragma unroll
            for (int half = 0; half < 2; ++half)
            {
                const int mine = half * kWaveSize + lane;
                int before = 0;
#pragma unroll
                for (int q = 0; q < kScanThreads / (2 * kWaveSize); ++q)
                    before += static_cast<int>(partial_counts[q * 2 * kWaveSize + mine]);
                if (mine < n_list && before < top_k)
                {
                    shared.final_values[before] = value_from_ascending_key(shared.list_keys[mine]);
                    shared.final_indices[before] = shared.list_indices[mine];
                }
            }
            n = n_list < top_k ? n_list : top_k;
            if (lane == 0)
                a.row_state[row] = kRowDone;
            const float value = lane < n ? shared.final_values[lane] : 0.0f;
            const int32_t index = lane < n ? shared.final_indices[lane] : -1;
            finish_ordered_wave(a, row, p, greedy, value, index, n, lane, result_flags, uniform, exp2_table);
            return;
        }
        if (wave != 0)
            return;
        if (n_list <= 4 * kWaveSize)
            n = select_best_wave<4>(shared.list_keys, shared.list_indices, n_list, top_k, lane, shared.final_values, shared.final_indices);
        else
            n = select_best_wave<8>(shared.list_keys, shared.list_indices, n_list, top_k, lane, shared.final_values, shared.final_indices);
        if (lane == 0)
            a.row_state[row] = kRowDone;
        if (n == 0)
        {
            if (lane == 0)
                write_error(a, row, NCNN_MOE_ROW_NO_FINITE_LOGIT, result_flags);
            return;
        }
        float value = lane < n ? shared.final_values[lane] : 0.0f;
        int32_t index = lane < n ? shared.final_indices[lane] : -1;
        int rank = 0;
        for (int trip = 0; trip < (n + 3) >> 2; ++trip)
        {
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                const int j = trip * 4 + k;
                rank += (j < n && candidate_before(read_lane(value, j), read_lane(index, j), value, index)) ? 1 : 0;
            }
        }
        if (lane < n)
        {
            shared.final_values[rank] = value;
            shared.final_indices[rank] = index;
        }
        value = lane < n ? shared.final_values[lane] : 0.0f;
        index = lane < n ? shared.final_indices[lane] : -1;
        finish_ordered_wave(a, row, p, greedy, value, index, n, lane, result_flags, uniform, exp2_table);
        return;
    }
    if constexpr (WIDE)
    {
        // ---- a window wider than one wave: exact K-th best key, then ranks by counting, then the
        // walk over the ordered window with exact running sums
        constexpr int kPerThread = SelectShared<WIDE>::kListCap / kScanThreads;
        if (n_list > top_k + 64)
            tighten_list(shared, 0u, top_k, tid); // fewer candidates to rank
        const int n_ranked = __builtin_amdgcn_readfirstlane(static_cast<int>(shared.list_count));
        uint32_t keys[kPerThread];
        int32_t indices[kPerThread];
#pragma unroll
        for (int j = 0; j < kPerThread; ++j)
        {
            const int q = j * kScanThreads + tid;
            keys[j] = q < n_ranked ? shared.list_keys[q] : 0u;
            indices[j] = q < n_ranked ? shared.list_indices[q] : 0;
        }
        // The candidates are put in order by a bitonic sort in LDS: (key, index) pairs as one 64-bit number,
        // larger = earlier, written over the list itself (its two arrays are one array of pairs), padded
        // with zeros to a power of two.  (Ranking every candidate by counting those ahead of it, a million
        // comparisons for a full window, took five times as long.)
        __syncthreads();
        NCNN_MOE_STAMP_NEXT(row, 12);
        uint64_t* const pairs = reinterpret_cast<uint64_t*>(shared.list_keys);
        int padded = kScanThreads * 2;
        while (padded < n_ranked)
            padded <<= 1;
#pragma unroll
        for (int j = 0; j < kPerThread; ++j)
        {
            const int q = j * kScanThreads + tid;
            if (q < padded)
                pairs[q] = (q < n_ranked && keys[j] != 0u)
                    ? (static_cast<uint64_t>(keys[j]) << 32) | (0xffffffffu - static_cast<uint32_t>(indices[j])) : 0ull;
        }
        __syncthreads();
        for (int k = 2; k <= padded; k <<= 1)
        {
            for (int j = k >> 1; j > 0; j >>= 1)
            {
                for (int pair = tid; pair < padded / 2; pair += kScanThreads)
                {
                    const int low = ((pair & ~(j - 1)) << 1) | (pair & (j - 1));
                    const int high = low | j;
                    const uint64_t first = pairs[low];
                    const uint64_t second = pairs[high];
                    const bool descending = (low & k) == 0; // the last merge (k == padded) is descending throughout
                    if (descending ? first < second : first > second)
                    {
                        pairs[low] = second;
                        pairs[high] = first;
                    }
                }
                __syncthreads();
            }
        }
        NCNN_MOE_STAMP_NEXT(row, 12);
        const int ordered = n_ranked < top_k ? n_ranked : top_k;
        uint64_t chosen[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) // top_k <= kSelectTopK = two per thread
        {
            const int rank = j * kScanThreads + tid;
            chosen[j] = rank < ordered ? pairs[rank] : 0ull;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j)
        {
            const int rank = j * kScanThreads + tid;
            if (rank < ordered && chosen[j] != 0ull)
            {
                shared.sorted_keys[rank] = descending_key(value_from_ascending_key(static_cast<uint32_t>(chosen[j] >> 32)));
                shared.sorted_indices[rank] = 0xffffffffu - static_cast<uint32_t>(chosen[j]);
            }
        }
        __syncthreads();
        const int n = n_ranked < top_k ? n_ranked : top_k;
        if (tid == 0)
            a.row_state[row] = kRowDone;
        if (n == 0)
        {
            if (tid == 0)
                write_error(a, row, NCNN_MOE_ROW_NO_FINITE_LOGIT, result_flags);
            return;
        }
        // the walk over the ordered window with exact running sums, as for a full-order row: the
        // window's exp terms go where the list was
        float* const terms = reinterpret_cast<float*>(shared.list_keys);
        const float maximum = value_from_descending_key(shared.sorted_keys[0]) / p.temperature;
        for (int i = tid; i < n; i += kScanThreads)
            terms[i] = expf_libm(value_from_descending_key(shared.sorted_keys[i]) / p.temperature - maximum, exp2_table);
        __syncthreads();
        const uint32_t* const sorted_indices = shared.sorted_indices;
        const auto token_at = [sorted_indices](uint32_t rank) { return static_cast<int32_t>(sorted_indices[rank]); };
        replay_sorted_window<false>(a, row, p, shared.sorted_keys, nullptr, static_cast<uint32_t>(n), static_cast<uint32_t>(n),
                                    shared.sorted_indices, result_flags, shared.replay, tid, token_at, terms);
    }
}

// Issues the chunk's loads.  A vector with no valid element reads the row's last vector instead (and is
// ignored later): the loads stay free of branches, so the next chunk's loads can be in flight while
// this chunk is processed.  vocab >= 1.
template <int DTYPE, int VECTORS>
__device__ __forceinline__ void load_chunk(
    uint4 (&raw)[VECTORS], const char* aligned_base, uint32_t chunk_base, uint32_t valid_begin, uint32_t segment_end,
    uint32_t valid_end, int tid)
{
    using Vector = LogitsVector<DTYPE>;
    const uint32_t last_vector = (valid_end - 1u) / Vector::kWidth * Vector::kWidth;
#pragma unroll
    for (int v = 0; v < VECTORS; ++v)
    {
        const uint32_t first = chunk_base + static_cast<uint32_t>(v * kScanThreads + tid) * Vector::kWidth;
        const bool any_valid = first < segment_end && first + Vector::kWidth > valid_begin;
        const uint32_t source = any_valid ? first : last_vector;
        // (a non-temporal load: the logits are read once, and marking them so took 0.5 us off a 39 MB batch)
        typedef uint32_t NativeVector __attribute__((ext_vector_type(4)));
        const NativeVector loaded = __builtin_nontemporal_load(
            reinterpret_cast<const NativeVector*>(aligned_base + static_cast<size_t>(source) * Vector::kElementBytes));
        raw[v] = make_uint4(loaded.x, loaded.y, loaded.z, loaded.w);
    }
}

// LOOPED: a workgroup streams several chunks (double-buffered).  WIDE: Top-K windows up to kSelectTopK
// (a long candidate list, more registers and LDS); otherwise up to kFastTopK.
template <int DTYPE, bool LOOPED, bool WIDE>
__global__ __launch_bounds__(kScanThreads, (!LOOPED && DTYPE == NCNN_MOE_LOGITS_F32) ? 8 : 4) void scan_select_kernel(SamplerArgs a)
{
    using Vector = LogitsVector<DTYPE>;
    static_assert(LOOPED || !WIDE, "wide windows are served by whole-row workgroups");
    using Shared = SelectShared<WIDE>;
    constexpr int kWidth = Vector::kWidth;
    constexpr int kVectors = Vector::kVectorsPerLane;
    constexpr int kLaneValues = kVectors * kWidth;
    constexpr uint32_t kChunk = static_cast<uint32_t>(kScanThreads) * kLaneValues;
    constexpr uint32_t kNegativeInfinity = 0xff800000u;
    constexpr uint32_t kPositiveInfinity = 0x7f800000u;

    // Workgroups are handed to the eight XCDs in turn.  A grouped grid numbers them so that the segments
    // of a row all land on one XCD: the row's merge can then read their records from that XCD's L2.
    // (Nothing relies on it: the counter below records where the segments really ran.)
    uint32_t row = blockIdx.y;
    uint32_t segment = blockIdx.x;
    if (a.xcd_grouped != 0u)
    {
        const uint32_t turn = blockIdx.x >> 3;
        row = (turn / a.segments) * 8u + (blockIdx.x & 7u);
        segment = turn % a.segments;
        if (row >= a.rows)
            return;
    }
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);

    __shared__ Shared shared;

    if (a.only_pending == 1 && a.row_state[row] != kRowNeedsGeneral)
        return;
    if (WIDE) { NCNN_MOE_STAMP_RESET(row, 12); NCNN_MOE_STAMP_NEXT(row, 12); }
    // The first chunk's loads go out before anything that waits for the row's options.
    const char* row_pointer = static_cast<const char*>(a.logits) +
        static_cast<size_t>(row) * a.row_stride * Vector::kElementBytes;
    const uint32_t misalignment =
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row_pointer) & 15u) / Vector::kElementBytes;
    const char* aligned_base = row_pointer - static_cast<size_t>(misalignment) * Vector::kElementBytes;
    const uint32_t valid_begin = misalignment;
    const uint32_t valid_end = misalignment + a.vocab;
    const uint32_t first_chunk = segment * a.chunks_per_segment;
    const uint32_t total_chunks = (valid_end + kChunk - 1) / kChunk;
    const uint32_t end_chunk = min(total_chunks, first_chunk + a.chunks_per_segment);
    // positions this workgroup covers end here; a chunk past end_chunk holds nothing valid
    const uint32_t segment_end = min(valid_end, end_chunk * kChunk);

    uint32_t bound_key = 0; // ascending key every Top-K member is known to reach; 0: none yet
    uint32_t local_flags = 0;
    bool overflow = false;

    uint4 raw[2][kVectors];
    load_chunk<DTYPE, kVectors>(raw[0], aligned_base, first_chunk * kChunk, valid_begin, segment_end, valid_end, tid);
    const ncnn_moe_sample_params p = a.params[row];
    const float uniform = a.uniforms[row];
    uint32_t effective_k = 0;
    int status = NCNN_MOE_ROW_OK;
    const int mode = resolve_row_mode(p, a.vocab, a.max_select_top_k, a.force_general, effective_k, status);
    if (mode == kModeInvalid || mode == kModeGeneral)
    {
        // A row that another launch of the call serves is not touched: a launch for pending rows finds a
        // full-order row marked already (the full-order kernels may be serving it at this moment on another
        // stream); a wide select that runs beside the first select leaves the marking of every row to that
        // one; and the first select leaves the wide select's rows alone when told that one runs beside it.
        const bool not_mine = a.only_pending == 2 || (a.only_pending == 1 && mode == kModeGeneral) ||
            (!WIDE && a.leave_wide_rows != 0 && mode == kModeGeneral && a.force_general == 0 &&
             effective_k <= static_cast<uint32_t>(kSelectTopK));
        if (segment == 0 && tid == 0 && !not_mine)
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
    if (WIDE && a.only_pending == 2 && (greedy || effective_k <= static_cast<uint32_t>(kFastTopK)))
        return; // the first select's row
    // the list is tightened when it grows past this; a wide list keeps room for a chunk's additions
    uint32_t tighten_limit = WIDE ? static_cast<uint32_t>(2 * top_k + 64) : static_cast<uint32_t>(kNarrowListCap - 192);
    uint32_t next_check = 0;      // chunk at which the list is looked at next
    uint32_t count_at_check = 0;  // list length at the last look
    uint32_t chunk_at_check = first_chunk;  // first chunk after the last look

    if (tid == 0)
    {
        shared.block_flags = 0;
        shared.list_count = 0;
    }

    // ---- a window wider than kTwoKeyBoundTopK over a long row: the bound comes from a sample of the whole row.
    // The K-th largest value of the first chunk is reached by a tenth of that chunk, and the bounds that the list's
    // cuts give after c chunks are still reached by K / c values of the next one: some 4 K candidates in all for a
    // row of thirteen chunks, and two or three cuts of the list on the way.  A sample of one chunk's size, in runs of
    // 64 bytes spread evenly over the row, says where the K-th largest of the row lies: with r = vocab / sample size,
    // the sample's m-th largest is reached by about m r values of the row, give or take r sqrt(m), and m is chosen
    // so that m r - kSampleSigmas r sqrt(m) = K.  For K = 1000 in 129,280 logits m = 146: some 1,840 candidates in
    // all (give or take 150), no cut on the way, and no bound to work out from the first chunk.  The sample can mislead (values in an
    // order that the runs' spacing resonates with): a list that ends with fewer than K candidates under such a
    // bound proves nothing, and the row is handed to the full-order kernels like a row whose list overflowed.
    bool sampled_bound = false;
    if constexpr (WIDE)
    {
        constexpr uint32_t kRunVectors = 4; // 64 bytes
        constexpr uint32_t kRuns = static_cast<uint32_t>(kScanThreads) * kVectors / kRunVectors;
        constexpr uint32_t kSampledBoundMinChunks = 4;
        constexpr float kSampleSigmas = 5.5f;
        static_assert(static_cast<uint32_t>(kScanThreads) * kVectors % kRunVectors == 0, "whole runs");
        if (a.wide_sampled_bound != 0u && top_k > kTwoKeyBoundTopK && total_chunks >= kSampledBoundMinChunks)
        {
            // vectors that lie inside the row as a whole: at least (kSampledBoundMinChunks - 1) chunks' worth - 2
            const uint32_t first_whole = (valid_begin + kWidth - 1) / kWidth;
            const uint32_t whole_vectors = valid_end / kWidth - first_whole;
            const uint32_t spacing = whole_vectors / kRuns; // >= 2 * kRunVectors
            uint32_t sample_keys[kLaneValues];
            uint4 sample[kVectors];
#pragma unroll
            for (int v = 0; v < kVectors; ++v)
            {
                const uint32_t g = static_cast<uint32_t>(v * kScanThreads + tid);
                const uint32_t vector = first_whole + (g / kRunVectors) * spacing + g % kRunVectors;
                // (an ordinary load: the line stays in the cache for the chunk that holds it)
                sample[v] = *reinterpret_cast<const uint4*>(aligned_base + static_cast<size_t>(vector) * 16u);
            }
#pragma unroll
            for (int v = 0; v < kVectors; ++v)
            {
                float x[kWidth];
                Vector::unpack(sample[v], x);
#pragma unroll
                for (int c = 0; c < kWidth; ++c)
                    sample_keys[v * kWidth + c] = x[c] > -__builtin_inff() ? ascending_key(x[c]) : 0u; // false for NaN as well
            }
            const float ratio = static_cast<float>(a.vocab) / static_cast<float>(kChunk);
            const float root = 0.5f * (kSampleSigmas + sqrtf(kSampleSigmas * kSampleSigmas + 4.0f * static_cast<float>(top_k) / ratio));
            const int sample_rank = static_cast<int>(root * root) + 1;
            // (the upper 16 bits of the sample's m-th largest: half the selection's rounds, and the few dozen values of
            // the row that share those bits with it are nothing beside the estimate's own spread)
            const uint32_t sample_bound = workgroup_kth_of_keys_by_digits<kLaneValues, 2>(sample_keys, sample_rank, tid, shared.bound);
            if (sample_bound != 0u)
            {
                bound_key = sample_bound;
                sampled_bound = true;
                // under such a bound a chunk adds a few hundred candidates at most: the list may grow further
                tighten_limit = max(tighten_limit, static_cast<uint32_t>(kWideListCap - 1024));
            }
        }
    }

    __syncthreads();

    // Processes the chunk held in `buffer`; all indexing is static after unrolling.
    auto process = [&](uint4 (&buffer)[kVectors], uint32_t chunk, bool first_of_segment) {
        const uint32_t chunk_base = chunk * kChunk;
        float values[kLaneValues];
        float group_max[kVectors];
        float lane_max = __uint_as_float(kNegativeInfinity);
        float half_max[2] = {__uint_as_float(kNegativeInfinity), __uint_as_float(kNegativeInfinity)};
        bool saw_nan = false;
#pragma unroll
        for (int v = 0; v < kVectors; ++v)
        {
            const uint32_t first = chunk_base + static_cast<uint32_t>(v * kScanThreads + tid) * kWidth;
            const bool any_valid = first < segment_end && first + kWidth > valid_begin;
            if (any_valid)
                Vector::unpack(buffer[v], &values[v * kWidth]);
            else
            {
#pragma unroll
                for (int c = 0; c < kWidth; ++c)
                    values[v * kWidth + c] = __uint_as_float(kNegativeInfinity);
            }
            if (any_valid && (first < valid_begin || first + kWidth > segment_end))
            {
#pragma unroll
                for (int c = 0; c < kWidth; ++c)
                {
                    const uint32_t position = first + c;
                    if (position < valid_begin || position >= segment_end)
                        values[v * kWidth + c] = __uint_as_float(kNegativeInfinity);
                }
            }
            float vector_max = __uint_as_float(kNegativeInfinity);
#pragma unroll
            for (int c = 0; c < kWidth; ++c)
            {
                const float x = values[v * kWidth + c];
                saw_nan = saw_nan || (x != x);
                vector_max = fmaxf(vector_max, x);
            }
            group_max[v] = vector_max;
            lane_max = fmaxf(lane_max, vector_max);
        }
        if (greedy && __ballot(lane_max == __uint_as_float(kPositiveInfinity)) != 0)
        {
            // greedy skips every non-finite logit (session.cpp:411-412): rare, so redone out of line
            lane_max = __uint_as_float(kNegativeInfinity);
#pragma unroll
            for (int v = 0; v < kVectors; ++v)
            {
                float vector_max = __uint_as_float(kNegativeInfinity);
#pragma unroll
                for (int c = 0; c < kWidth; ++c)
                {
                    if (values[v * kWidth + c] == __uint_as_float(kPositiveInfinity))
                        values[v * kWidth + c] = __uint_as_float(kNegativeInfinity);
                    vector_max = fmaxf(vector_max, values[v * kWidth + c]);
                }
                group_max[v] = vector_max;
                lane_max = fmaxf(lane_max, vector_max);
            }
        }
        if constexpr (WIDE)
        {
#pragma unroll
            for (int v = 0; v < kVectors; ++v)
                half_max[v < (kVectors + 1) / 2 ? 0 : 1] = fmaxf(half_max[v < (kVectors + 1) / 2 ? 0 : 1], group_max[v]);
        }
        if (saw_nan)
            local_flags |= kScanSawNan;
        if (lane_max == __uint_as_float(kPositiveInfinity))
            local_flags |= kScanSawPositiveInfinity;

        // ---- bound of the first chunk: the K-th largest lane maximum, or a cheaper bound below it.  The
        // lanes at or above it each hold a distinct logit at least that large, so the K-th best logit of
        // the row is no smaller.
        // (also a later chunk while there is no bound yet: a row that begins with a stretch of -inf, a masked
        // part of the vocabulary, must not pour its first chunk of finite logits into the list unfiltered)
        if ((first_of_segment && !sampled_bound) || (LOOPED && bound_key == 0u))
        {
            if (WIDE && top_k > kTwoKeyBoundTopK)
            {
                // a wide window: the lane maxima bound too loosely, so select over every value of the chunk
                uint32_t value_keys[kLaneValues];
#pragma unroll
                for (int i = 0; i < kLaneValues; ++i)
                    value_keys[i] = values[i] > -__builtin_inff() ? ascending_key(values[i]) : 0u; // false for NaN as well
                bound_key = max(bound_key, workgroup_kth_of_keys_by_digits(value_keys, top_k, tid, shared.bound));
            }
            else if constexpr (WIDE)
            {
                // two keys per lane (the maxima of the two halves of its vectors): 1024 distinct logits
                const uint32_t lane_keys[2] = {
                    half_max[0] == __uint_as_float(kNegativeInfinity) ? 0u : ascending_key(half_max[0]),
                    half_max[1] == __uint_as_float(kNegativeInfinity) ? 0u : ascending_key(half_max[1])};
                bound_key = max(bound_key, workgroup_kth_largest_key(lane_keys, top_k, tid, shared.bound, true));
            }
            else
            {
                const uint32_t lane_keys[1] = {lane_max == __uint_as_float(kNegativeInfinity) ? 0u : ascending_key(lane_max)};
                uint32_t chunk_bound = workgroup_kth_of_quad_maxima(lane_keys[0], top_k, tid, shared.bound);
                if (chunk_bound == 0u) // a chunk with few values: the exact K-th largest lane maximum
                    chunk_bound = workgroup_kth_largest_key(lane_keys, top_k, tid, shared.bound, true);
                bound_key = max(bound_key, chunk_bound);
            }
        }
        // no bound yet (fewer than K lanes hold a finite logit): every finite logit is a candidate
        const float threshold = bound_key == 0u ? -3.402823466e+38f : fmaxf(value_from_ascending_key(bound_key), -3.402823466e+38f);

        // ---- collect the values at or above the bound.  Nearly every lane that holds a candidate holds
        // exactly one, its maximum: each lane counts its candidates and locates its maximum without a
        // branch, and one append per wave takes the maxima.  The lanes that hold more hand the others
        // over one per round (a round per extra candidate of the fullest lane; usually none).
        // A looped workgroup's bound is tight after its first chunks: most waves then hold no candidate
        // at all and skip the counting.  (A single-chunk workgroup's waves nearly always hold some.)
        const bool wave_has_candidates = !LOOPED || __ballot(lane_max >= threshold) != 0;
        int lane_hits = 0;
        int best_at = 0;
        if (wave_has_candidates)
        {
#pragma unroll
            for (int i = 0; i < kLaneValues; ++i)
            {
                lane_hits += values[i] >= threshold ? 1 : 0;
                best_at = values[i] == lane_max ? i : best_at;
            }
        }
        const auto element_of = [&](int i) {
            return static_cast<int32_t>(chunk_base + static_cast<uint32_t>((i / kWidth) * kScanThreads + tid) * kWidth +
                                        static_cast<uint32_t>(i % kWidth) - misalignment);
        };
        if (wave_has_candidates)
            append_candidate(shared, lane_hits >= 1, ascending_key(lane_max), element_of(best_at), lane);
        if (wave_has_candidates && __ballot(lane_hits > 1) != 0)
        {
            uint32_t rest = 0; // bit i: value i is a candidate that has not been appended
#pragma unroll
            for (int i = 0; i < kLaneValues; ++i)
                rest |= (lane_hits > 1 && values[i] >= threshold && i != best_at) ? (1u << i) : 0u;
            while (__ballot(rest != 0u) != 0)
            {
                // the value is read back from the row (it sits in a register whose number is not known
                // until run time; this path is rare and the line is in the cache)
                const int i = rest != 0u ? __builtin_ctz(rest) : 0;
                const int32_t element = element_of(i);
                float x = 0.0f;
                if constexpr (WIDE)
                {
                    // under a wide window's bound most lanes hold several candidates: the value is picked out of
                    // the registers (a chain of selects) rather than waited for
#pragma unroll
                    for (int k = 0; k < kLaneValues; ++k)
                        x = i == k ? values[k] : x;
                }
                else if (rest != 0u)
                {
                    if constexpr (DTYPE == NCNN_MOE_LOGITS_F32)
                        x = reinterpret_cast<const float*>(row_pointer)[element];
                    else
                        x = __uint_as_float(static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(row_pointer)[element]) << 16);
                }
                append_candidate(shared, rest != 0u, ascending_key(x), element, lane);
                rest &= rest - 1u;
            }
        }
        if constexpr (!LOOPED)
        {
            __syncthreads();
            if (shared.list_count > static_cast<uint32_t>(Shared::kListCap))
                overflow = true; // candidates were dropped: only the full-order path can serve the row
        }
        else if (first_of_segment || chunk >= next_check)
        {
            // The list is looked at (a barrier) only as often as its growth asks for: once the bound is
            // tight a chunk adds next to nothing and the waves stream on without waiting for each other.
            __syncthreads();
            const uint32_t count = shared.list_count;
            if (count > static_cast<uint32_t>(Shared::kListCap))
                overflow = true;
            else
            {
                const uint32_t chunks = chunk - chunk_at_check + 1u;
                const uint32_t rate = (count - count_at_check + chunks - 1u) / chunks; // candidates per chunk
                if (count > tighten_limit)
                {
                    // the waves' own searches first (a third of the exact selection's time); what they
                    // leave is nearly always short enough
                    bound_key = tighten_list(shared, bound_key, top_k, tid, WIDE);
                    if (!WIDE && shared.list_count > tighten_limit / 4u * 3u)
                        bound_key = tighten_list(shared, bound_key, top_k, tid, true);
                }
                count_at_check = shared.list_count;
                chunk_at_check = chunk + 1u;
                const uint32_t slack = static_cast<uint32_t>(Shared::kListCap) - count_at_check;
                const uint32_t interval = slack / (2u * rate + 16u);
                next_check = chunk + (interval < 1u ? 1u : (interval > 8u ? 8u : interval));
            }
        }
    };

    if constexpr (LOOPED)
    {
        // Two chunks per trip, the loads of the next chunk always in flight while one is processed.  The
        // loop is free of branches around loads: a chunk past end_chunk reads the row's last vector and
        // counts nothing.
        for (uint32_t chunk = first_chunk; chunk < end_chunk; chunk += 2)
        {
            load_chunk<DTYPE, kVectors>(raw[1], aligned_base, (chunk + 1) * kChunk, valid_begin, segment_end, valid_end, tid);
            process(raw[0], chunk, chunk == first_chunk);
            load_chunk<DTYPE, kVectors>(raw[0], aligned_base, (chunk + 2) * kChunk, valid_begin, segment_end, valid_end, tid);
            process(raw[1], chunk + 1, false);
        }
        __syncthreads();
        if (shared.list_count > static_cast<uint32_t>(Shared::kListCap))
            overflow = true;
        if (sampled_bound && shared.list_count < static_cast<uint32_t>(top_k))
            overflow = true; // the sample misled: the list holds a part of the window only
    }
    else
    {
        process(raw[0], first_chunk, true);
    }

    if (local_flags != 0)
        atomicOr(&shared.block_flags, local_flags);
    __syncthreads();

    if (a.segments == 1)
    {
        // ---- the workgroup saw the whole row: finish it here
        const uint32_t flags = shared.block_flags;
        const uint8_t result_flags = (flags & kScanSawNan) ? NCNN_MOE_ROW_FLAG_HAS_NAN : 0;
        if (overflow)
        {
            if (tid == 0)
            {
                write_pending(a, row);
                a.row_state[row] = kRowNeedsGeneral;
            }
            return;
        }
        if (!greedy && (flags & kScanSawPositiveInfinity))
        {
            // the stable order puts +inf first and the CPU sampler rejects the row (session.cpp:84-85)
            if (tid == 0)
            {
                write_error(a, row, NCNN_MOE_ROW_NO_FINITE_LOGIT, result_flags);
                a.row_state[row] = kRowDone;
            }
            return;
        }
        if (WIDE) NCNN_MOE_STAMP_NEXT(row, 12);
        finish_from_list(a, row, p, greedy, top_k, shared, result_flags, tid, uniform);
        if (WIDE) NCNN_MOE_STAMP_NEXT(row, 12);
        return;
    }

    // ---- several segments per row: hand the list over through the segment's record in HBM
    uint32_t* const out_values = reinterpret_cast<uint32_t*>(a.segment_values);
    uint32_t* const out_indices = reinterpret_cast<uint32_t*>(a.segment_indices);
    const size_t segment_slot = static_cast<size_t>(row) * a.segments + segment;
    const uint32_t record_entries = segment_record_entries(effective_k);
    // the record holds 2K + 16 candidates: a longer list (a loose bound, ties) is cut to the exact window first
    if (!overflow && shared.list_count > record_entries)
        bound_key = tighten_list(shared, bound_key, top_k, tid);
    const uint32_t handed = shared.list_count;
    overflow = overflow || handed > record_entries;
    if (!overflow)
    {
        for (uint32_t j = tid; j < handed; j += kScanThreads)
        {
            store_agent(&out_values[segment_slot * kSegmentRecordSlots + j], shared.list_keys[j]);
            store_agent(&out_indices[segment_slot * kSegmentRecordSlots + j], static_cast<uint32_t>(shared.list_indices[j]));
        }
    }
    if (tid == 0)
    {
        store_agent(&a.segment_counts[segment_slot], overflow ? 0u : handed);
        uint32_t flags = shared.block_flags;
        if (overflow)
            flags |= kScanOverflow;
        if (flags != 0)
            atomicOr(&a.row_flags[row], flags);
    }
    // The barrier waits for this workgroup's agent-scope stores; the counter is bumped only after that.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0)
    {
        const uint32_t xcd = __builtin_amdgcn_s_getreg(kXccIdRegister) & 7u;
        const int field = 8 + 6 * static_cast<int>(xcd);
        const unsigned long long previous =
            __hip_atomic_fetch_add(&a.row_counter[row], 1ull + (1ull << field), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        shared.block_is_last = (previous & 0xffull) == a.segments - 1 ? 1 : 0;
        // every other segment of the row ran on this XCD: their records are in this XCD's L2
        shared.block_all_local = ((previous >> field) & 63ull) == a.segments - 1 ? 1 : 0;
        shared.list_count = 0;
    }
    __syncthreads();
    if (!shared.block_is_last)
        return;

    // ---- last workgroup of the row: every load of the merge is issued before any is used (one trip)
    // Thread slot q stands for entry q / 16 of segment q % 16: no division by the record length, and
    // every row of 16 lanes sees one entry of each segment, so the candidates are spread evenly over
    // the lanes (which is what the prune's bound from the quad maxima needs).
    static_assert(kMaxSegments == 16, "the merge maps a thread slot to (entry, segment) with a shift by 4");
    const size_t row_slot = static_cast<size_t>(row) * a.segments;
    const uint32_t row_entries = record_entries * static_cast<uint32_t>(kMaxSegments);
    constexpr int kPerThread = kMergeStageSlots / kScanThreads;
    uint32_t loaded_keys[kPerThread];
    uint32_t loaded_indices[kPerThread];
    const bool all_local = shared.block_all_local != 0;
    // agent-scope loads go around the L2 to the memory side; records written on this XCD are read from its L2
    const auto load_record = [all_local](const uint32_t* address) { return all_local ? *address : load_agent(address); };
    const uint32_t row_flags = load_agent(&a.row_flags[row]);
    const bool stageable = row_entries <= static_cast<uint32_t>(kMergeStageSlots) && a.segments <= static_cast<uint32_t>(kMaxSegments);
    // all of a thread's slots belong to one segment (the workgroup's size is a multiple of 16)
    const uint32_t s = static_cast<uint32_t>(tid) & static_cast<uint32_t>(kMaxSegments - 1);
    const bool segment_exists = stageable && s < a.segments;
    // The counts of several rows share a 128-byte line, which this compute unit's vector cache may hold
    // from the merge of another row, taken before this row's segments stored theirs: always read around it.
    // (A record is 1 KB, aligned, and read by this workgroup only: a plain load cannot find it stale.)
    const uint32_t segment_count = segment_exists ? load_agent(&a.segment_counts[row_slot + s]) : 0u;
#pragma unroll
    for (int j = 0; j < kPerThread; ++j)
    {
        const uint32_t q = static_cast<uint32_t>(j * kScanThreads + tid);
        const uint32_t r = q >> 4;
        loaded_keys[j] = 0;
        loaded_indices[j] = 0;
        if (segment_exists && q < row_entries)
        {
            loaded_keys[j] = load_record(&out_values[(row_slot + s) * kSegmentRecordSlots + r]);
            loaded_indices[j] = load_record(&out_indices[(row_slot + s) * kSegmentRecordSlots + r]);
        }
    }
    const uint8_t result_flags = (row_flags & kScanSawNan) ? NCNN_MOE_ROW_FLAG_HAS_NAN : 0;
    __syncthreads();
    if (tid == 0)
    {
        a.row_counter[row] = 0;
        a.row_flags[row] = 0;
    }
    bool too_many = (row_flags & kScanOverflow) || !stageable;
    uint32_t thread_key[1] = {0u};
#pragma unroll
    for (int j = 0; j < kPerThread; ++j)
    {
        const uint32_t r = static_cast<uint32_t>(j * kScanThreads + tid) >> 4;
        loaded_keys[j] = r < segment_count ? loaded_keys[j] : 0u; // a segment that does not exist has count 0
        thread_key[0] = max(thread_key[0], loaded_keys[j]);
    }
    if (too_many) // the same in every thread: the row's flags and the segment count
    {
        // ties (or a very long row) left more candidates than the merge holds: the full-order kernels take the row
        if (tid == 0)
        {
            write_pending(a, row);
            a.row_state[row] = kRowNeedsGeneral;
        }
        return;
    }
    if (!greedy && (row_flags & kScanSawPositiveInfinity))
    {
        if (tid == 0)
        {
            write_error(a, row, NCNN_MOE_ROW_NO_FINITE_LOGIT, result_flags);
            a.row_state[row] = kRowDone;
        }
        return;
    }
    // prune: at least K candidates reach this lower bound of the K-th largest per-thread best
    uint32_t prune_key = workgroup_kth_of_quad_maxima(thread_key[0], top_k, tid, shared.bound);
    if (prune_key == 0u)
        prune_key = workgroup_kth_largest_key(thread_key, top_k, tid, shared.bound, true);
#pragma unroll
    for (int j = 0; j < kPerThread; ++j)
    {
        if (static_cast<uint32_t>(j * kScanThreads) >= row_entries)
            break; // no slot of this or a later round exists (a scalar test: nothing waits for a ballot)
        append_candidate(shared, loaded_keys[j] != 0u && loaded_keys[j] >= prune_key, loaded_keys[j],
                         static_cast<int32_t>(loaded_indices[j]), lane);
    }
    __syncthreads();
    if (shared.list_count > static_cast<uint32_t>(Shared::kListCap))
    {
        if (tid == 0)
        {
            write_pending(a, row);
            a.row_state[row] = kRowNeedsGeneral;
        }
        return;
    }
    finish_from_list(a, row, p, greedy, top_k, shared, result_flags, tid, uniform);
}

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_SAMPLER_SELECT_H
