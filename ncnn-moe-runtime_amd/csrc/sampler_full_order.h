// Full-order path: rows with no Top-K window (or one too wide for the select path) need the complete
// stable order, because the CPU sampler's sums run over it sequentially.
//   general_sort_kernel    stable LSD radix sort of one row by descending key, one workgroup per row
//   bf16_counting_sort_kernel  the same order for bf16 rows without indices, by counting the 65536 keys
//   general_replay_kernel  the sampler's walk over the sorted row
#ifndef NCNN_MOE_HIP_SAMPLER_FULL_ORDER_H
#define NCNN_MOE_HIP_SAMPLER_FULL_ORDER_H

#include "sampler_exact_sum.h"

namespace ncnn_moe_hip {

// A call that holds rows for the wide select and rows for these kernels runs the two passes side by
// side on two streams: the rows of the wide select are pending as well and are skipped here (a later
// launch without the flag takes those that the wide select could not finish).
__device__ __forceinline__ bool left_to_the_wide_select(const SamplerArgs& a, uint32_t row)
{
    if (a.leave_wide_rows == 0)
        return false;
    uint32_t effective_k = 0;
    int status = NCNN_MOE_ROW_OK;
    return resolve_row_mode(a.params[row], a.vocab, static_cast<uint32_t>(kSelectTopK), a.force_general, effective_k, status) != kModeGeneral;
}

// The row of a workgroup of a (parts, rows) grid, and whether the full-order kernels serve it.  Most rows
// of a mixed batch are not theirs, and a workgroup that finds that out from row_state has waited for a
// trip to memory: with sixteen parts a row those workgroups alone would keep a kernel going for 15 us.
// With the list, workgroup (part, j) takes the j-th listed row, and the others leave after one load of
// the list's length, which the scalar cache holds.
__device__ __forceinline__ bool spread_grid_row(const SamplerArgs& a, uint32_t& row)
{
    if (a.row_list != nullptr)
    {
        if (blockIdx.y >= a.row_list[0])
            return false;
        row = a.row_list[1u + blockIdx.y];
        return true;
    }
    row = blockIdx.y;
    return a.row_state[row] == kRowNeedsGeneral && !left_to_the_wide_select(a, row);
}

// The largest key that pass `pass` of a row's spread sort keeps: the first pass of a row that is sorted in part
// leaves out the elements behind the row's cut; every other pass keeps what it reads.
__device__ __forceinline__ uint32_t sort_last_key(const SamplerArgs& a, uint32_t row, int pass)
{
    if (pass != 0 || a.sort_lengths == nullptr)
        return 0xffffffffu;
    return a.sort_last_keys[row];
}

// Lists the rows that the full-order kernels serve (see SamplerArgs::row_list).  One workgroup.
__device__ __forceinline__ void list_full_order_rows(const SamplerArgs& a, uint32_t rows, uint32_t* list)
{
    __shared__ uint32_t wave_totals[kSortWaves];
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    uint32_t listed = 0;
    for (uint32_t first = 0; first < rows; first += kSortThreads)
    {
        const uint32_t row = first + static_cast<uint32_t>(tid);
        bool mine = false;
        if (row < rows && a.cut_by_options != 0u)
        {
            uint32_t effective_k = 0;
            int status = NCNN_MOE_ROW_OK;
            mine = resolve_row_mode(a.params[row], a.vocab, a.max_select_top_k, a.force_general, effective_k, status) == kModeGeneral;
        }
        else if (row < rows)
            mine = a.row_state[row] == kRowNeedsGeneral && !left_to_the_wide_select(a, row);
        const uint64_t mask = __builtin_amdgcn_ballot_w64(mine);
        if (lane == 0)
            wave_totals[wave] = static_cast<uint32_t>(__popcll(mask));
        __syncthreads();
        uint32_t before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w)
        {
            const uint32_t t = wave_totals[w];
            before += w < wave ? t : 0u;
            total += t;
        }
        if (mine)
            list[1u + listed + before + static_cast<uint32_t>(lanes_below(mask))] = row;
        listed += total;
        __syncthreads();
    }
    if (tid == 0)
        list[0] = listed;
}

__global__ __launch_bounds__(kSortThreads) void full_order_row_list_kernel(SamplerArgs a, uint32_t rows, uint32_t* list)
{
    list_full_order_rows(a, rows, list);
}

// How much of a full-order fp32 row needs sorting.  The sampler's sums add the row's terms exp(logit/T - max)
// in descending order, and a term below half an ulp of the sum it meets leaves that sum as it is: behind some
// point of the sorted row nothing moves any sum, and what lies there need not be in order (nor be sorted at
// all) - only counted.  For a temperature of 1 and logits spread like N(0, 4) that point lies past most of the
// row; at 0.5 it lies behind the first tenth.
// One workgroup per row looks at a sample of the row (16,384 logits, 256 evenly spaced runs of 64): counts of
// the keys' upper twelve bits (4,096 buckets: sign, exponent and three bits of the mantissa).  With the terms of
// the buckets' lower and upper ends it looks for the first bucket whose largest possible term is below 2^-26 of
// the least the buckets in front of it add up to (the sums' half ulp is 2^-25 to 2^-24 of them) - or, under a Top-K
// window, the first bucket behind twice the window by the sample's count - and has the sort
// keep the buckets in front of it: sort_last_keys.  This is a guess that costs or saves time, never exactness:
// the replay checks against its exact sums that the largest term left out moves none of them, and otherwise has
// the row sorted whole.  The exact counts that go with a cut (elements kept, finite logits, NaN seen) are taken
// by the sort's first counting pass, which reads the whole row; this kernel clears them.  Rows it does not cut
// get a last key of 0xffffffff and the row's length.
constexpr int kCutBuckets = 4096;
constexpr int kCutCopies = 4;                   // of the counters: a lane uses copy lane % 4 (few buckets hold most of a row)
constexpr int kCutStride = kCutBuckets + 1;     // (the copies of a counter lie in different banks)
constexpr uint32_t kCutSample = 4096;           // 16-byte groups of the row that are looked at
constexpr float kCutMinimum = 4096.0f;          // rows are not cut shorter than about this

__global__ __launch_bounds__(kSortThreads) void full_order_cut_kernel(SamplerArgs a)
{
    static_assert(kCutSample == 4u * kSortThreads && kCutBuckets == 4 * kSortThreads, "four loads and four buckets a thread");
    const uint32_t row = blockIdx.x;
    if (row == a.rows)
        return list_full_order_rows(a, a.rows, a.row_list_out); // (the workgroup behind the rows', where the host asks for one)
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    bool served;
    if (a.cut_by_options != 0u)
    {
        uint32_t effective_k = 0;
        int status = NCNN_MOE_ROW_OK;
        served = resolve_row_mode(a.params[row], a.vocab, a.max_select_top_k, a.force_general, effective_k, status) == kModeGeneral;
    }
    else
        served = a.row_state[row] == kRowNeedsGeneral && !left_to_the_wide_select(a, row);
    const float temperature = a.params[row].temperature;
    const uint32_t top_k = a.params[row].top_k;
    const float window = top_k > 0u && top_k < a.vocab ? static_cast<float>(top_k) : 0.0f;
    const auto sort_whole_row = [&]() {
        if (tid == 0)
        {
            a.sort_last_keys[row] = 0xffffffffu;
            a.sort_lengths[row] = a.vocab;
            a.disordered_rows[row] = (a.cut_by_options != 0u && !served) ? 2u : 0u; // (2: in no list of this call)
        }
    };
    if (!served || !(temperature > 0.0f))
        return sort_whole_row();
    __shared__ uint32_t counts[kCutCopies * kCutStride];
    __shared__ uint32_t wave_keys[kSortWaves];
    __shared__ float wave_counts[kSortWaves];
    __shared__ float wave_masses[kSortWaves];
    __shared__ uint32_t cut_bucket;

    // ---- the sample: group g of kCutSample lies at 16-byte group g * groups / kCutSample of the row
    const float* logits = static_cast<const float*>(a.logits) + static_cast<size_t>(row) * a.row_stride;
    const uint32_t misalignment = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(logits) & 15u) / 4u;
    const float* aligned_logits = logits - misalignment;
    const uint32_t aligned_end = misalignment + a.vocab; // positions [misalignment, aligned_end) hold the row
    const uint32_t groups = (aligned_end + 3u) / 4u;
    uint4 raw[4];
    uint32_t positions[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
    {
        // (runs of sixteen groups, 256 bytes: device memory is fetched by the line, and single groups spread over
        // the row would fetch all of it)
        const uint32_t g = static_cast<uint32_t>(k * kSortThreads + tid);
        const uint32_t run_first = static_cast<uint32_t>(static_cast<uint64_t>(g >> 4) * groups / (kCutSample >> 4));
        positions[k] = min((run_first + (g & 15u)) * 4u, aligned_end);
        if (groups < kCutSample)
            positions[k] = g < groups ? g * 4u : aligned_end; // a short row is looked at whole
        raw[k] = *reinterpret_cast<const uint4*>(aligned_logits + (positions[k] < aligned_end ? positions[k] : 0u));
    }
    for (int i = tid; i < kCutCopies * kCutStride; i += kSortThreads)
        counts[i] = 0u;
    if (tid == 0)
        cut_bucket = kCutBuckets;
    __syncthreads();
    uint32_t* const my_counts = counts + (lane & (kCutCopies - 1)) * kCutStride;
    uint32_t smallest_key = 0xffffffffu;
#pragma unroll
    for (int k = 0; k < 4; ++k)
    {
        const uint32_t words[4] = {raw[k].x, raw[k].y, raw[k].z, raw[k].w};
#pragma unroll
        for (uint32_t c = 0; c < 4u; ++c)
        {
            const uint32_t key = descending_key(__uint_as_float(words[c]));
            if (positions[k] + c >= misalignment && positions[k] + c < aligned_end)
            {
                atomicAdd(&my_counts[key >> 20], 1u);
                smallest_key = key > kPositiveInfinityKey ? min(smallest_key, key) : smallest_key;
            }
        }
    }
    smallest_key = ~wave_max_u32(~smallest_key);
    if (lane == 0)
        wave_keys[wave] = smallest_key;
    __syncthreads();
    uint32_t first_key = 0xffffffffu; // of the sample in sorted order, +inf aside: the largest logit's
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w)
        first_key = min(first_key, wave_keys[w]);
    if (first_key > kLastFiniteKey)
        return sort_whole_row(); // (no finite logit in the sample)
    // every sampled element stands for this many of the row
    const float weight = static_cast<float>(groups) / static_cast<float>(min(groups, kCutSample));

    // ---- thread t: buckets 4 t .. 4 t + 3; the terms are taken relative to the sample's largest logit (the
    // comparison below is one of ratios: any reference would do)
    constexpr uint32_t kFirstFiniteBucket = 0x008u, kLastFiniteBucket = 0xff7u; // keys 0x00800000 .. 0xff7fffff
    float bucket_counts[4];
    float bucket_least[4]; // the least that the bucket's elements add up to
    float lane_count = 0.0f, lane_mass = 0.0f;
    const float maximum = value_from_descending_key(first_key);
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        const uint32_t bucket = static_cast<uint32_t>(4 * tid + j);
        uint32_t count = 0;
#pragma unroll
        for (int copy = 0; copy < kCutCopies; ++copy)
            count += counts[copy * kCutStride + bucket];
        const bool finite = bucket >= kFirstFiniteBucket && bucket <= kLastFiniteBucket;
        bucket_counts[j] = static_cast<float>(count) * weight;
        const float lowest = value_from_descending_key((bucket << 20) | 0xfffffu);
        bucket_least[j] = finite && count != 0u ? bucket_counts[j] * __expf(fminf((lowest - maximum) / temperature, 0.0f)) : 0.0f;
        lane_count += bucket_counts[j];
        lane_mass += bucket_least[j];
    }
    // sums over the buckets in front of this thread's
    float count_through = lane_count, mass_through = lane_mass;
#pragma unroll
    for (int step = 1; step < kWaveSize; step <<= 1)
    {
        const float count_up = __shfl_up(count_through, step, kWaveSize);
        const float mass_up = __shfl_up(mass_through, step, kWaveSize);
        if (lane >= step)
        {
            count_through += count_up;
            mass_through += mass_up;
        }
    }
    if (lane == kWaveSize - 1)
    {
        wave_counts[wave] = count_through;
        wave_masses[wave] = mass_through;
    }
    __syncthreads();
    float count_before = count_through - lane_count;
    float mass_before = mass_through - lane_mass;
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w)
    {
        count_before += w < wave ? wave_counts[w] : 0.0f;
        mass_before += w < wave ? wave_masses[w] : 0.0f;
    }
    // the first bucket that can be left out, with all behind it
    uint32_t candidate = kCutBuckets;
#pragma unroll
    for (int j = 3; j >= 0; --j)
    {
        const uint32_t bucket = static_cast<uint32_t>(4 * tid + j);
        float count_here = count_before, mass_here = mass_before;
#pragma unroll
        for (int i = 0; i < j; ++i)
        {
            count_here += bucket_counts[i];
            mass_here += bucket_least[i];
        }
        const float highest = value_from_descending_key(bucket << 20);
        const float largest_term = __expf(fminf((highest - maximum) / temperature, 0.0f));
        // (a Top-K window ends the row's sums at K elements: a few times K, by the sample's count, are kept)
        const bool behind_the_window = window != 0.0f && count_here >= 2.0f * window + kCutMinimum;
        if (bucket > kFirstFiniteBucket && bucket <= kLastFiniteBucket && count_here >= kCutMinimum &&
            (largest_term < mass_here * 1.4901161193847656e-08f || behind_the_window)) // 2^-26
            candidate = bucket;
    }
    if (candidate < static_cast<uint32_t>(kCutBuckets))
        atomicMin(&cut_bucket, candidate);
    __syncthreads();
    const uint32_t cut = cut_bucket;
    if (cut >= static_cast<uint32_t>(kCutBuckets))
        return sort_whole_row();
    if (tid == 0)
    {
        a.sort_last_keys[row] = (cut << 20) - 1u;
        a.sort_lengths[row] = 0u;   // counted by sort_part_histogram_kernel's first pass
        a.finite_counts[row] = 0u;  // ... with the row's finite logits and whether it holds a NaN
        a.disordered_rows[row] = 0u;
    }
}

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
    if (a.row_state[row] != kRowNeedsGeneral || left_to_the_wide_select(a, row))
        return;
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    const uint32_t n = a.vocab;

    __shared__ uint32_t histogram[kPasses][256];
    __shared__ uint32_t digit_base[256];          // output position of the next key of each digit
    __shared__ uint32_t wave_counts[kSortWaves][256];
    __shared__ uint32_t tile_start[256];          // first slot of each digit in the staged tile
    __shared__ uint32_t global_offset[256];       // output position minus staged slot, per digit
    __shared__ uint32_t scan_partial[4];
    __shared__ uint32_t staged_keys[kSortTile];   // the tile ordered by digit, written out in runs
    __shared__ uint32_t staged_indices[PAIRS ? kSortTile : 1];

    const char* row_pointer = static_cast<const char*>(a.logits) +
        static_cast<size_t>(row) * a.row_stride * LogitsVector<DTYPE>::kElementBytes;
    uint32_t* keys[2] = {a.sort_keys[0] + row * a.sort_stride, a.sort_keys[1] + row * a.sort_stride};
    uint32_t* indices[2] = {a.sort_indices[0] + row * a.sort_stride, a.sort_indices[1] + row * a.sort_stride};

    for (int i = tid; i < kPasses * 256; i += kSortThreads)
        (&histogram[0][0])[i] = 0;
    __syncthreads();
    // Digit histograms of every pass (plain LDS atomics: matching equal digits with ballots first, to
    // spare the same-address conflicts of the upper digits, was measured and costs more than it saves).
    for (uint32_t first = 0; first < n; first += 8u * kSortThreads)
    {
        float batch[8]; // eight independent loads in flight per thread
#pragma unroll
        for (int k = 0; k < 8; ++k)
        {
            const uint32_t i = first + static_cast<uint32_t>(k * kSortThreads + tid);
            batch[k] = load_logit<DTYPE>(row_pointer, i < n ? i : n - 1u);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
        {
            const uint32_t i = first + static_cast<uint32_t>(k * kSortThreads + tid);
            const uint32_t key = descending_key(batch[k]);
            if (i < n)
            {
#pragma unroll
                for (int pass = 0; pass < kPasses; ++pass)
                    atomicAdd(&histogram[pass][(key >> (8 * (pass + kFirstDigit))) & 255u], 1u);
            }
        }
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
        // The next tile's keys are loaded while this tile is ranked, and the barriers inside the loop
        // order LDS traffic only: a tile reads one global buffer and writes the other, so nothing in the
        // loop has to wait for its scattered stores.
        auto load_tile = [&](uint32_t tile, uint32_t (&out_keys)[kSortPerThread], uint32_t (&out_indices)[kSortPerThread]) {
            const uint32_t wave_first = tile + static_cast<uint32_t>(wave) * (kWaveSize * kSortPerThread);
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                const uint32_t i = wave_first + static_cast<uint32_t>(e * kWaveSize + lane);
                const uint32_t source = i < n ? i : n - 1u; // always a valid address; masked below
                uint32_t key;
                uint32_t index = i;
                if (pass == 0)
                    key = descending_key(load_logit<DTYPE>(row_pointer, source));
                else
                {
                    key = source_keys[source];
                    if (PAIRS)
                        index = source_indices[source];
                }
                out_keys[e] = i < n ? key : 0xffffffffu;
                out_indices[e] = i < n ? index : i;
            }
        };
        uint32_t tile_keys[kSortPerThread];
        uint32_t tile_indices[kSortPerThread];
        load_tile(0, tile_keys, tile_indices);
        for (uint32_t tile = 0; tile < n; tile += kSortTile)
        {
            uint32_t next_keys[kSortPerThread];
            uint32_t next_indices[kSortPerThread];
            load_tile(tile + kSortTile < n ? tile + kSortTile : tile, next_keys, next_indices);
            for (int i = tid; i < kSortWaves * 256; i += kSortThreads)
                (&wave_counts[0][0])[i] = 0;
            uint32_t tile_ranks[kSortPerThread];
            const uint32_t wave_first = tile + static_cast<uint32_t>(wave) * (kWaveSize * kSortPerThread);
            lds_barrier();
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                const uint32_t i = wave_first + static_cast<uint32_t>(e * kWaveSize + lane);
                const bool valid = i < n;
                const uint32_t digit = (tile_keys[e] >> shift) & 255u;
                uint32_t peers_low, peers_high;
                wave_digit_peers(digit, valid, peers_low, peers_high);
                const uint32_t rank_in_round = __builtin_amdgcn_mbcnt_hi(peers_high, __builtin_amdgcn_mbcnt_lo(peers_low, 0u));
                uint32_t seen = 0;
                if (valid)
                    seen = wave_counts[wave][digit];
                tile_ranks[e] = seen + rank_in_round;
                if (valid && rank_in_round == 0)
                    wave_counts[wave][digit] = seen + static_cast<uint32_t>(__popc(peers_low) + __popc(peers_high));
            }
            lds_barrier();
            // per digit: slots of the waves inside the digit's run, the run's length, then the runs' starts
            uint32_t digit_total = 0;
            uint32_t inclusive = 0;
            if (tid < 256)
            {
                uint32_t counts[kSortWaves]; // read at once: sixteen dependent LDS round trips otherwise
#pragma unroll
                for (int w = 0; w < kSortWaves; ++w)
                    counts[w] = wave_counts[w][tid];
#pragma unroll
                for (int w = 0; w < kSortWaves; ++w)
                {
                    wave_counts[w][tid] = digit_total;
                    digit_total += counts[w];
                }
                inclusive = digit_total;
#pragma unroll
                for (int step = 1; step < kWaveSize; step <<= 1)
                {
                    const uint32_t up = __shfl_up(inclusive, step, kWaveSize);
                    if (lane >= step)
                        inclusive += up;
                }
                if (lane == kWaveSize - 1)
                    scan_partial[wave] = inclusive;
            }
            lds_barrier();
            if (tid < 256)
            {
                uint32_t start = inclusive - digit_total;
#pragma unroll
                for (int w = 0; w < 3; ++w) // tid < 256: waves 0 to 3
                    start += w < wave ? scan_partial[w] : 0u;
                tile_start[tid] = start;
                global_offset[tid] = digit_base[tid] - start;
                digit_base[tid] += digit_total;
            }
            lds_barrier();
            // stage the tile in digit order (stable: waves in order, ranks in order) ...
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                const uint32_t i = wave_first + static_cast<uint32_t>(e * kWaveSize + lane);
                if (i < n)
                {
                    const uint32_t digit = (tile_keys[e] >> shift) & 255u;
                    const uint32_t slot = tile_start[digit] + wave_counts[wave][digit] + tile_ranks[e];
                    staged_keys[slot] = tile_keys[e];
                    if (PAIRS)
                        staged_indices[slot] = tile_indices[e];
                }
            }
            lds_barrier();
            // ... and write it out: consecutive threads hold consecutive slots, so a digit's run goes to
            // consecutive addresses
            const uint32_t tile_count = min(static_cast<uint32_t>(kSortTile), n - tile);
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                const uint32_t slot = static_cast<uint32_t>(e * kSortThreads + tid);
                if (slot < tile_count)
                {
                    const uint32_t key = staged_keys[slot];
                    const uint32_t position = global_offset[(key >> shift) & 255u] + slot;
                    target_keys[position] = key;
                    if (PAIRS)
                        target_indices[position] = staged_indices[slot];
                }
            }
            lds_barrier();
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                tile_keys[e] = next_keys[e];
                tile_indices[e] = next_indices[e];
            }
        }
        __threadfence_block();
        __syncthreads();
    }
}

// ---- the same sort with a row spread over several workgroups.  A batch rarely holds more full-order
// rows than the GPU has compute units (a service batch of 512 rows: about a hundred), and one workgroup
// per row leaves the rest idle while each row takes the whole latency of four passes.  Here part g of a
// row owns a fixed range of tiles; every pass is two launches over a (parts, rows) grid:
//   sort_part_histogram_kernel  counts the pass's digits in each part, in the order the keys have NOW
//   sort_part_scatter_kernel    gives part g, for digit d, the positions behind all smaller digits of
//       the row and behind digit d's keys of the parts before it, and moves its tiles as the one-workgroup
//       kernel does (stable inside the part, parts in order: stable over the row).
// Pass p reads the logits (p = 0) or keys[(p + 1) & 1] and writes keys[p & 1]; four passes for fp32,
// two for bf16 rows that carry indices.
template <int DTYPE, bool PAIRS>
__device__ __forceinline__ void load_sort_keys(
    const SamplerArgs& a, uint32_t row, int pass, uint32_t first, uint32_t n, int tid_in_group, int group_stride,
    uint32_t (&out_keys)[kSortPerThread], uint32_t (&out_indices)[kSortPerThread])
{
    const char* row_pointer = static_cast<const char*>(a.logits) +
        static_cast<size_t>(row) * a.row_stride * LogitsVector<DTYPE>::kElementBytes;
    const uint32_t* source_keys = a.sort_keys[(pass + 1) & 1] + row * a.sort_stride;
    const uint32_t* source_indices = a.sort_indices[(pass + 1) & 1] + row * a.sort_stride;
    // (one loop per source, so that a thread's loads are in flight together)
    if (pass == 0)
    {
        float values[kSortPerThread];
#pragma unroll
        for (int e = 0; e < kSortPerThread; ++e)
        {
            const uint32_t i = first + static_cast<uint32_t>(e * group_stride + tid_in_group);
            values[e] = load_logit<DTYPE>(row_pointer, i < n ? i : n - 1u); // always a valid address; masked below
        }
#pragma unroll
        for (int e = 0; e < kSortPerThread; ++e)
        {
            const uint32_t i = first + static_cast<uint32_t>(e * group_stride + tid_in_group);
            out_keys[e] = i < n ? descending_key(values[e]) : 0xffffffffu;
            out_indices[e] = i;
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < kSortPerThread; ++e)
    {
        const uint32_t i = first + static_cast<uint32_t>(e * group_stride + tid_in_group);
        const uint32_t source = i < n ? i : n - 1u;
        out_keys[e] = source_keys[source];
        out_indices[e] = PAIRS ? source_indices[source] : i;
    }
#pragma unroll
    for (int e = 0; e < kSortPerThread; ++e)
    {
        const uint32_t i = first + static_cast<uint32_t>(e * group_stride + tid_in_group);
        if (i >= n)
        {
            out_keys[e] = 0xffffffffu;
            out_indices[e] = i;
        }
    }
}

// One workgroup counts kHistogramParts consecutive parts of a row, with the loads of all of them in flight
// together: a workgroup's time is one trip to memory and the hand-over of its counts, whatever it counts,
// so a part per workgroup only adds rounds of workgroups (configuration 4: 384 us a step with one part a
// workgroup, 374 with two, 379 with four, which leave half of the GPU's workgroup slots empty in the passes
// that read the kept keys).  grid (parts / kHistogramParts rounded up, rows).
constexpr int kHistogramParts = 2;

template <int DTYPE>
__global__ __launch_bounds__(kSortThreads) void sort_part_histogram_kernel(SamplerArgs a)
{
    constexpr int kFirstDigit = DTYPE == NCNN_MOE_LOGITS_F32 ? 0 : 2;
    const uint32_t first_part = blockIdx.x * kHistogramParts;
    uint32_t row;
    if (!spread_grid_row(a, row))
        return;
    const int tid = threadIdx.x;
    const int pass = static_cast<int>(a.sort_pass);
    // the first pass reads the whole row and keeps the elements that are sorted; the others read those
    const uint32_t n = pass == 0 ? a.vocab : sorted_length(a, row);
    const uint32_t last_key = sort_last_key(a, row, pass);
    const int shift = 8 * (pass + kFirstDigit + static_cast<int>(a.sort_low_digit_skipped));
    __shared__ uint32_t counts[kHistogramParts][8][257]; // (257: the copies of a digit's counter lie in eight different banks)
    for (int i = tid; i < kHistogramParts * 8 * 257; i += kSortThreads)
        (&counts[0][0][0])[i] = 0;
    __syncthreads();
    // The first pass of a row that is sorted in part also takes the row's exact counts: the elements that are
    // kept (the sum of the digits' counts), the finite logits and whether there is a NaN among all of them.
    const bool counting = pass == 0 && last_key != 0xffffffffu;
    uint32_t finite_seen = 0, nan_seen = 0;
    const uint32_t part_span = a.sort_tiles_per_part * kSortTile;
    for (uint32_t offset = 0; offset < part_span; offset += kSortTile)
    {
        uint32_t keys[kHistogramParts][kSortPerThread];
#pragma unroll
        for (int q = 0; q < kHistogramParts; ++q)
        {
            uint32_t unused[kSortPerThread];
            const uint32_t tile = min((first_part + q) * part_span + offset, n - 1u); // (a tile behind the row: its keys are not counted)
            load_sort_keys<DTYPE, false>(a, row, pass, tile, n, tid, kSortThreads, keys[q], unused);
        }
#pragma unroll
        for (int q = 0; q < kHistogramParts; ++q)
        {
            const uint32_t tile = (first_part + q) * part_span + offset;
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                // (eight copies of the counters, a lane using copy lane % 8: the uppermost digit of a row's keys
                // takes few values, and 64 atomics on one address take as many turns)
                const bool inside = tile + static_cast<uint32_t>(e * kSortThreads + tid) < n;
                if (inside && keys[q][e] <= last_key)
                    atomicAdd(&counts[q][tid & 7][(keys[q][e] >> shift) & 255u], 1u);
                if (counting)
                {
                    finite_seen += inside && keys[q][e] > kPositiveInfinityKey && keys[q][e] <= kLastFiniteKey ? 1u : 0u;
                    nan_seen |= inside && keys[q][e] == 0xffffffffu ? 1u : 0u;
                }
            }
        }
    }
    __syncthreads();
    if (counting)
    {
        __shared__ uint32_t wave_finite[kSortWaves], wave_kept[kSortWaves], wave_nan[kSortWaves];
        uint32_t kept = 0;
        if (tid < 256 * kHistogramParts)
        {
#pragma unroll
            for (int copy = 0; copy < 8; ++copy)
                kept += counts[tid >> 8][copy][tid & 255];
        }
        const uint32_t wave_index = static_cast<uint32_t>(tid) >> 6;
        const uint32_t finite_total = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(wave_prefix_sum_u32(finite_seen)), 63));
        const uint32_t kept_total = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(wave_prefix_sum_u32(kept)), 63));
        const uint32_t nan_total = wave_or_u32(nan_seen);
        if ((tid & 63) == 0)
        {
            wave_finite[wave_index] = finite_total;
            wave_kept[wave_index] = kept_total;
            wave_nan[wave_index] = nan_total;
        }
        __syncthreads();
        if (tid == 0)
        {
            uint32_t finite_all = 0, kept_all = 0, nan_all = 0;
            for (int w = 0; w < kSortWaves; ++w)
            {
                finite_all += wave_finite[w];
                kept_all += wave_kept[w];
                nan_all |= wave_nan[w];
            }
            atomicAdd(&a.sort_lengths[row], kept_all);
            atomicAdd(&a.finite_counts[row], finite_all);
            if (nan_all != 0u)
                atomicOr(&a.finite_counts[row], kRowHoldsNan);
        }
    }
    {
        const int q = tid >> 8; // (the first 256 * kHistogramParts threads)
        const int digit = tid & 255;
        static_assert(kSortThreads >= 256 * kHistogramParts, "a thread per part and digit");
        if (q < kHistogramParts && first_part + q < a.sort_parts)
        {
            uint32_t total = 0;
#pragma unroll
            for (int copy = 0; copy < 8; ++copy)
                total += counts[q][copy][digit];
            a.sort_part_counts[(static_cast<size_t>(row) * a.sort_parts + first_part + q) * 256 + digit] = total;
        }
    }
}

// (at most 64 registers a thread: two workgroups of 1,024 threads share a compute unit)
// ANY_ORDER: the keys of one digit value may leave in any order.  That holds for the first pass of a sort
// of keys alone (equal keys cannot be told apart, and there is no earlier pass whose order must survive);
// a key's rank among its wave's keys of the same digit is then what an LDS atomic returns.
template <int DTYPE, bool PAIRS, bool ANY_ORDER = false>
__global__ __launch_bounds__(kSortThreads) __attribute__((amdgpu_waves_per_eu(8, 8))) void sort_part_scatter_kernel(SamplerArgs a)
{
    constexpr int kFirstDigit = DTYPE == NCNN_MOE_LOGITS_F32 ? 0 : 2;
    const uint32_t part = blockIdx.x;
    uint32_t row;
    if (!spread_grid_row(a, row))
        return;
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    const int pass = static_cast<int>(a.sort_pass);
    // the first pass reads the whole row and keeps the elements that are sorted; the others read those
    const uint32_t n = pass == 0 ? a.vocab : sorted_length(a, row);
    const uint32_t last_key = sort_last_key(a, row, pass);
    const int shift = 8 * (pass + kFirstDigit + static_cast<int>(a.sort_low_digit_skipped));

    __shared__ uint32_t digit_base[256];          // output position of the next key of each digit
    __shared__ uint32_t wave_counts[kSortWaves][256];
    __shared__ uint32_t tile_start[256];          // first slot of each digit in the staged tile
    __shared__ uint32_t global_offset[256];       // output position minus staged slot, per digit
    __shared__ uint32_t scan_partial[4];
    __shared__ uint32_t staged_keys[kSortTile];   // the tile ordered by digit, written out in runs
    __shared__ uint32_t staged_indices[PAIRS ? kSortTile : 1];

    uint32_t* target_keys = a.sort_keys[pass & 1] + row * a.sort_stride;
    uint32_t* target_indices = a.sort_indices[pass & 1] + row * a.sort_stride;

    // the first tile is asked for before the parts' counts: the two trips to memory overlap
    const uint32_t first_tile = part * a.sort_tiles_per_part * kSortTile;
    const uint32_t end = min(n, first_tile + a.sort_tiles_per_part * kSortTile);
    if (first_tile >= end)
        return;
    uint32_t tile_keys[kSortPerThread];
    uint32_t tile_indices[kSortPerThread];
    load_sort_keys<DTYPE, PAIRS>(a, row, pass, first_tile + static_cast<uint32_t>(wave) * (kWaveSize * kSortPerThread), n, lane, kWaveSize,
                                 tile_keys, tile_indices);

    // where this part's keys of every digit go: behind the row's smaller digits and behind the same
    // digit's keys of the parts before this one
    {
        uint32_t row_total = 0, before = 0, inclusive = 0;
        if (tid < 256)
        {
            // (every part's count is asked for before the first is used: a loop of the parts' real number would
            // wait for each load in turn, sixteen trips to memory one behind the other)
            const uint32_t* counts = a.sort_part_counts + static_cast<size_t>(row) * a.sort_parts * 256 + tid;
            uint32_t part_counts[kMaxSortParts];
#pragma unroll
            for (uint32_t g = 0; g < static_cast<uint32_t>(kMaxSortParts); ++g)
                part_counts[g] = g < a.sort_parts ? counts[static_cast<size_t>(g) * 256] : 0u;
#pragma unroll
            for (uint32_t g = 0; g < static_cast<uint32_t>(kMaxSortParts); ++g)
            {
                row_total += part_counts[g];
                before += g < part ? part_counts[g] : 0u;
            }
            inclusive = row_total;
#pragma unroll
            for (int step = 1; step < kWaveSize; step <<= 1)
            {
                const uint32_t up = __shfl_up(inclusive, step, kWaveSize);
                if (lane >= step)
                    inclusive += up;
            }
            if (lane == kWaveSize - 1)
                scan_partial[wave] = inclusive;
        }
        __syncthreads();
        if (tid < 256)
        {
            uint32_t start = inclusive - row_total;
#pragma unroll
            for (int w = 0; w < 3; ++w) // tid < 256: waves 0 to 3
                start += w < wave ? scan_partial[w] : 0u;
            digit_base[tid] = start + before;
        }
        __syncthreads();
    }

    // A wave owns 512 consecutive keys of a tile and ranks them in 8 rounds of 64, so that the order
    // inside the wave is the input order (see general_sort_kernel).
    // (no later tile is fetched ahead: a workgroup has one tile or few, and two workgroups share a compute unit)
    for (uint32_t tile = first_tile; tile < end; tile += kSortTile)
    {
        if (tile != first_tile)
            load_sort_keys<DTYPE, PAIRS>(a, row, pass, tile + static_cast<uint32_t>(wave) * (kWaveSize * kSortPerThread), n, lane, kWaveSize,
                                         tile_keys, tile_indices);
        for (int i = tid; i < kSortWaves * 256; i += kSortThreads)
            (&wave_counts[0][0])[i] = 0;
        uint32_t tile_ranks[kSortPerThread];
        const uint32_t wave_first = tile + static_cast<uint32_t>(wave) * (kWaveSize * kSortPerThread);
        lds_barrier();
        // (a tile that lies inside the row and keeps every key - all tiles but a row's last in the passes behind
        // the first - is ranked and staged by code without the tests of each key: the pass's time is the
        // instructions it issues)
        const bool whole_tile = tile + kSortTile <= n && last_key == 0xffffffffu;
        const auto rank_tile = [&](auto whole_tag) {
            constexpr bool kWhole = decltype(whole_tag)::value;
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                const uint32_t i = wave_first + static_cast<uint32_t>(e * kWaveSize + lane);
                const bool valid = kWhole || (i < n && tile_keys[e] <= last_key);
                const uint32_t digit = (tile_keys[e] >> shift) & 255u;
                if (ANY_ORDER)
                {
                    tile_ranks[e] = valid ? atomicAdd(&wave_counts[wave][digit], 1u) : 0u;
                    continue;
                }
                uint32_t peers_low, peers_high;
                if constexpr (kWhole)
                    wave_digit_peers(digit, peers_low, peers_high);
                else
                    wave_digit_peers(digit, valid, peers_low, peers_high);
                const uint32_t rank_in_round = __builtin_amdgcn_mbcnt_hi(peers_high, __builtin_amdgcn_mbcnt_lo(peers_low, 0u));
                uint32_t seen = 0;
                if (valid)
                    seen = wave_counts[wave][digit];
                tile_ranks[e] = seen + rank_in_round;
                if (valid && rank_in_round == 0)
                    wave_counts[wave][digit] = seen + static_cast<uint32_t>(__popc(peers_low) + __popc(peers_high));
            }
        };
        if (whole_tile)
            rank_tile(std::true_type{});
        else
            rank_tile(std::false_type{});
        lds_barrier();
        uint32_t digit_total = 0;
        uint32_t inclusive = 0;
        if (tid < 256)
        {
            uint32_t counts[kSortWaves];
#pragma unroll
            for (int w = 0; w < kSortWaves; ++w)
                counts[w] = wave_counts[w][tid];
#pragma unroll
            for (int w = 0; w < kSortWaves; ++w)
            {
                wave_counts[w][tid] = digit_total;
                digit_total += counts[w];
            }
            inclusive = digit_total;
#pragma unroll
            for (int step = 1; step < kWaveSize; step <<= 1)
            {
                const uint32_t up = __shfl_up(inclusive, step, kWaveSize);
                if (lane >= step)
                    inclusive += up;
            }
            if (lane == kWaveSize - 1)
                scan_partial[wave] = inclusive;
        }
        lds_barrier();
        if (tid < 256)
        {
            uint32_t start = inclusive - digit_total;
#pragma unroll
            for (int w = 0; w < 3; ++w)
                start += w < wave ? scan_partial[w] : 0u;
            tile_start[tid] = start;
            global_offset[tid] = digit_base[tid] - start;
            digit_base[tid] += digit_total;
            if (tid == 255)
                scan_partial[3] = start + digit_total; // the tile's keys that are kept (read behind the next barrier;
                                                       // its readers as a wave's total are in front of this one)
        }
        lds_barrier();
        const auto stage_tile = [&](auto whole_tag) {
            constexpr bool kWhole = decltype(whole_tag)::value;
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                const uint32_t i = wave_first + static_cast<uint32_t>(e * kWaveSize + lane);
                if (kWhole || (i < n && tile_keys[e] <= last_key))
                {
                    const uint32_t digit = (tile_keys[e] >> shift) & 255u;
                    const uint32_t slot = tile_start[digit] + wave_counts[wave][digit] + tile_ranks[e];
                    staged_keys[slot] = tile_keys[e];
                    if (PAIRS)
                        staged_indices[slot] = tile_indices[e];
                }
            }
        };
        if (whole_tile)
            stage_tile(std::true_type{});
        else
            stage_tile(std::false_type{});
        lds_barrier();
        const uint32_t tile_count = scan_partial[3];
        const auto write_tile = [&](auto whole_tag) {
            constexpr bool kWhole = decltype(whole_tag)::value;
#pragma unroll
            for (int e = 0; e < kSortPerThread; ++e)
            {
                const uint32_t slot = static_cast<uint32_t>(e * kSortThreads + tid);
                if (kWhole || slot < tile_count)
                {
                    const uint32_t key = staged_keys[slot];
                    const uint32_t position = global_offset[(key >> shift) & 255u] + slot;
                    target_keys[position] = key;
                    if (PAIRS)
                        target_indices[position] = staged_indices[slot];
                }
            }
        };
        if (whole_tile)
            write_tile(std::true_type{});
        else
            write_tile(std::false_type{});
        lds_barrier();
    }
}

// bf16 rows without token indices: the 65536 possible keys are counted instead of sorted.  The keys of
// a bf16 row differ only in their upper 16 bits, and sampling needs the sorted keys alone, so the
// sorted row is its histogram: it is written as RUNS, one (key, end position) pair per key that occurs,
// in descending order of the logits, and the replay adds a run of equal terms in one step.  One
// workgroup per row.  Run keys go to sort_keys[1], run ends to sort_keys[0], the number of runs to the
// row's first word of sort_indices[0].
//
// The row is read once: 65536 counters of 16 bits, two to an LDS word (key16 2w in the lower half, 2w + 1
// in the upper), counted with one LDS atomic per logit.  A counter that passes 65535 carries into its
// neighbour or out of the word; every such carry makes the sum of the decoded counters smaller than the
// number of logits (by 65535 or 65536 per carry, never larger), so the sum is the test: a row that fails it
// (some value occurs 65536 times or more) is counted again in two rounds of 32768 counters of 32 bits.
constexpr int kCountWords = 32768;
constexpr int kCachedRuns = 6144; // runs of a row the replay keeps in LDS (48 KB)

// Counts the row's keys into `bins`.  PACKED: every key, 16-bit counters; else the keys whose top bit is
// `round`, 32-bit counters indexed by the lower 15 bits.  16-byte loads of eight logits, four per thread
// and batch, the next batch in flight while this one is counted; the row is read from the 16-byte
// boundary below its first element.
template <bool PACKED>
__device__ __forceinline__ void count_bf16_keys(
    const uint16_t* aligned_logits, uint32_t misalignment, uint32_t aligned_end, uint32_t round, uint32_t* bins, int tid)
{
    constexpr uint32_t kBatch = 4u * 8u * kSortThreads;
    const auto load_batch = [&](uint32_t first, uint4 (&raw)[4]) {
#pragma unroll
        for (int k = 0; k < 4; ++k)
        {
            const uint32_t position = first + static_cast<uint32_t>(k * kSortThreads + tid) * 8u;
            raw[k] = *reinterpret_cast<const uint4*>(aligned_logits + (position < aligned_end ? position : 0u));
        }
    };
    uint4 raw[4];
    load_batch(0, raw);
    for (uint32_t first = 0; first < aligned_end; first += kBatch)
    {
        uint4 next[4];
        load_batch(first + kBatch < aligned_end ? first + kBatch : first, next);
        // A batch that lies wholly inside the row (all but the first, if the row does not start on a 16-byte
        // boundary, and the last) is counted without a test per logit and without a branch: the kernel is bound
        // by the instructions it issues per logit, not by HBM.
        if (PACKED && first >= misalignment && first + kBatch <= aligned_end)
        {
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                const uint32_t words[4] = {raw[k].x, raw[k].y, raw[k].z, raw[k].w};
#pragma unroll
                for (int c = 0; c < 8; ++c)
                {
                    // descending_key of the logit's fp32 value, upper half, but for NaN and -0: those are counted
                    // under the keys that the plain mapping gives them (which no other value has) and moved to
                    // their places by fold_special_bf16_counts
                    const uint32_t bits = (c & 1) ? (words[c >> 1] & 0xffff0000u) : (words[c >> 1] << 16);
                    const uint32_t sign = static_cast<uint32_t>(static_cast<int32_t>(bits) >> 31);
                    const uint32_t key16 = (bits ^ (~sign & 0x7fffffffu)) >> 16;
                    atomicAdd(&bins[key16 >> 1], 1u << ((key16 & 1u) << 4));
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k)
                raw[k] = next[k];
            continue;
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
        {
            const uint32_t position = first + static_cast<uint32_t>(k * kSortThreads + tid) * 8u;
            const uint32_t words[4] = {raw[k].x, raw[k].y, raw[k].z, raw[k].w};
#pragma unroll
            for (int c = 0; c < 8; ++c)
            {
                const uint32_t bits = (c & 1) ? (words[c >> 1] >> 16) : (words[c >> 1] & 0xffffu);
                const uint32_t element = position + c;
                const uint32_t key16 = descending_key(__uint_as_float(bits << 16)) >> 16;
                const bool inside = element >= misalignment && element < aligned_end;
                if (PACKED)
                {
                    if (inside)
                        atomicAdd(&bins[key16 >> 1], (key16 & 1u) ? 0x10000u : 1u);
                }
                else if (inside && (key16 >> 15) == round)
                    atomicAdd(&bins[key16 & 0x7fffu], 1u);
            }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
            raw[k] = next[k];
    }
}

// count_bf16_keys<true> counts the logits of whole batches under descending_key's plain mapping (the bits of a
// negative value; the complement of a positive value's lower 15 bits), which gives NaN and -0 keys of their
// own: 0x0000-0x007e (positive NaN, in front of +inf at 0x007f), 0xff81-0xffff (negative NaN, behind -inf at
// 0xff80) and 0x8000 (-0, next to +0 at 0x7fff).  The first wave moves those counts to where descending_key
// puts the values: all NaN at 0xffff, -0 with +0.  Returns false if a sum does not fit its 16-bit counter (the
// caller then counts the row again in 32-bit counters, with descending_key itself).  Call between barriers.
__device__ __forceinline__ bool fold_special_bf16_counts(uint32_t* bins, int tid)
{
    bool fits = true;
    if (tid < kWaveSize)
    {
        const uint32_t lane = static_cast<uint32_t>(tid);
        // positive NaN: words 0 .. 63 but for the upper half of word 63 (+inf)
        const uint32_t front = bins[lane];
        const uint32_t front_nan = (front & 0xffffu) + (lane < 63u ? front >> 16 : 0u);
        bins[lane] = lane < 63u ? 0u : front & 0xffff0000u;
        // negative NaN: words 0x7fc0 .. 0x7fff but for the lower half of word 0x7fc0 (-inf); the upper half of
        // word 0x7fff is where they all go
        const uint32_t back = bins[0x7fc0u + lane];
        const uint32_t back_nan = (back >> 16) + (lane > 0u ? back & 0xffffu : 0u);
        const uint32_t all_nan = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(wave_prefix_sum_u32(front_nan + back_nan)), kWaveSize - 1));
        fits = all_nan <= 0xffffu;
        if (fits)
            bins[0x7fc0u + lane] = lane == 0u ? back & 0xffffu : (lane == 63u ? all_nan << 16 : 0u);
        else
            bins[lane] = front; // (nothing is moved: the counters are abandoned)
        if (lane == 0u)
        {
            // -0 (key 0x8000: lower half of word 0x4000) joins +0 (key 0x7fff: upper half of word 0x3fff)
            const uint32_t negative_zero = bins[0x4000u] & 0xffffu;
            const uint32_t positive_zero = bins[0x3fffu] >> 16;
            if (negative_zero + positive_zero <= 0xffffu)
            {
                bins[0x4000u] &= 0xffff0000u;
                bins[0x3fffu] = (bins[0x3fffu] & 0xffffu) | ((negative_zero + positive_zero) << 16);
            }
            else
                fits = false;
        }
        fits = __builtin_amdgcn_ballot_w64(!fits) == 0ull;
    }
    return fits;
}

constexpr int kCountBlocks = kCountWords / kWaveSize; // blocks of 64 consecutive counter words

struct CountScratch
{
    alignas(16) uint32_t block_totals[kCountBlocks]; // elements counted in each block
    alignas(16) uint32_t block_runs[kCountBlocks];   // counters above zero in each block
};

// Turns the counters into runs.  The words are taken 64 consecutive ones at a time (a block: lane l reads word
// 64 b + l, no bank conflicts), and block b belongs to wave b % 16: the keys in use lie close together (a row of
// logits between -8 and 16 touches four of sixteen equal stretches of the key space), and dealt out this way every
// wave gets its share of them.  The order of the keys is (block, lane, half).  Returns false (and writes nothing)
// when PACKED counters have overflowed.  key_base: key16 of word 0's first counter; written / runs_written: totals
// of an earlier round.
// in_place != nullptr (PACKED only, first round): when the row's runs fit `in_place_capacity`, they are written over
// the counters themselves (every counter is in a register by then), keys from bins[0] on and ends from
// bins[in_place_capacity] on, instead of to run_keys / run_ends; *in_place tells which.
template <bool PACKED>
__device__ __forceinline__ bool write_runs_of_counts(
    uint32_t* bins, uint32_t expected, uint32_t key_base, uint32_t& written, uint32_t& runs_written,
    uint32_t* run_keys, uint32_t* run_ends, CountScratch& scratch, int tid, bool* in_place = nullptr, uint32_t in_place_capacity = 0)
{
    constexpr int kTrips = kCountBlocks / kSortWaves; // 32
    static_assert(kTrips == 32 && kSortWaves == 16, "a wave's block totals fill lanes 0..31; eight blocks a lane in the scan");
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    uint32_t words[kTrips];
    uint32_t my_total = 0, my_runs = 0; // lane j: the totals of the wave's trip j
#pragma unroll
    for (int j = 0; j < kTrips; ++j)
        words[j] = bins[static_cast<uint32_t>((j * kSortWaves + wave) * kWaveSize + lane)];
#pragma unroll
    for (int j = 0; j < kTrips; ++j)
    {
        if (__ballot(words[j] != 0u) == 0ull)
            continue; // most blocks are empty
        const uint32_t low = PACKED ? (words[j] & 0xffffu) : words[j];
        const uint32_t high = PACKED ? (words[j] >> 16) : 0u;
        const uint32_t lane_runs = (low != 0u ? 1u : 0u) + (high != 0u ? 1u : 0u);
        uint32_t block_total, block_runs;
        if (PACKED)
        {
            // one sum for both: a block's 16-bit counters sum to less than 2^23, its runs to at most 128
            const uint32_t both = static_cast<uint32_t>(
                __builtin_amdgcn_readlane(static_cast<int>(wave_prefix_sum_u32(((low + high) << 8) | lane_runs)), 63));
            block_total = both >> 8;
            block_runs = both & 0xffu;
        }
        else
        {
            block_total = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(wave_prefix_sum_u32(low)), 63));
            block_runs = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(wave_prefix_sum_u32(lane_runs)), 63));
        }
        my_total = lane == j ? block_total : my_total;
        my_runs = lane == j ? block_runs : my_runs;
    }
    if (lane < kTrips)
    {
        scratch.block_totals[lane * kSortWaves + wave] = my_total;
        scratch.block_runs[lane * kSortWaves + wave] = my_runs;
    }
    __syncthreads(); // every counter is in a register now, every block total in the scratch
    // Every wave scans the 512 block totals: lane l takes blocks 8 l .. 8 l + 7.  The wave's trip j is block
    // 16 j + wave: lane 2 j + wave / 8, slot wave % 8.
    uint32_t first_element, first_run; // of this lane's block of slot wave % 8, before `written` / `runs_written`
    uint32_t all, all_runs;
    {
        const uint4 t0 = *reinterpret_cast<const uint4*>(&scratch.block_totals[8 * lane]);
        const uint4 t1 = *reinterpret_cast<const uint4*>(&scratch.block_totals[8 * lane + 4]);
        const uint4 r0 = *reinterpret_cast<const uint4*>(&scratch.block_runs[8 * lane]);
        const uint4 r1 = *reinterpret_cast<const uint4*>(&scratch.block_runs[8 * lane + 4]);
        const uint32_t totals[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
        const uint32_t runs[8] = {r0.x, r0.y, r0.z, r0.w, r1.x, r1.y, r1.z, r1.w};
        uint32_t lane_total = 0, lane_runs = 0;
        uint32_t slot_total = 0, slot_runs = 0; // of the slots in front of slot wave % 8
#pragma unroll
        for (int i = 0; i < 8; ++i)
        {
            slot_total = i == (wave & 7) ? lane_total : slot_total;
            slot_runs = i == (wave & 7) ? lane_runs : slot_runs;
            lane_total += totals[i];
            lane_runs += runs[i];
        }
        const uint32_t inclusive_total = wave_prefix_sum_u32(lane_total);
        const uint32_t inclusive_runs = wave_prefix_sum_u32(lane_runs);
        first_element = inclusive_total - lane_total + slot_total;
        first_run = inclusive_runs - lane_runs + slot_runs;
        all = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(inclusive_total), 63));
        all_runs = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(inclusive_runs), 63));
    }
    __syncthreads(); // the scratch is written again by a later call
    if (PACKED && all != expected)
        return false;
    if (in_place != nullptr)
    {
        *in_place = runs_written == 0u && all_runs <= in_place_capacity;
        if (*in_place)
        {
            run_keys = bins;
            run_ends = bins + in_place_capacity;
        }
    }
#pragma unroll
    for (int j = 0; j < kTrips; ++j)
    {
        const uint32_t low = PACKED ? (words[j] & 0xffffu) : words[j];
        const uint32_t high = PACKED ? (words[j] >> 16) : 0u;
        const uint64_t has_low = __ballot(low != 0u);
        const uint64_t has_high = PACKED ? __ballot(high != 0u) : 0ull;
        if ((has_low | has_high) == 0ull)
            continue;
        const uint32_t source = static_cast<uint32_t>(2 * j + (wave >> 3));
        const uint32_t position = written + static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(first_element), source));
        const uint32_t run = runs_written + static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(first_run), source));
        const uint32_t inclusive = wave_prefix_sum_u32(low + high);
        const uint32_t before = position + inclusive - (low + high);
        uint32_t slot = run + static_cast<uint32_t>(lanes_below(has_low) + lanes_below(has_high));
        const uint32_t word = static_cast<uint32_t>((j * kSortWaves + wave) * kWaveSize + lane);
        const uint32_t first_key16 = key_base + (PACKED ? 2u * word : word);
        // the lower half of a key is all ones for a non-negative logit and for NaN, else zero
        const auto full_key = [](uint32_t key16) {
            return key16 == 0xffffu ? 0xffffffffu : (key16 << 16) | ((key16 >> 15) == 0u ? 0xffffu : 0u);
        };
        if (low != 0u)
        {
            run_keys[slot] = full_key(first_key16);
            run_ends[slot] = before + low;
            ++slot;
        }
        if (PACKED && high != 0u)
        {
            run_keys[slot] = full_key(first_key16 + 1u);
            run_ends[slot] = before + low + high;
        }
    }
    written += all;
    runs_written += all_runs;
    return true;
}

__global__ __launch_bounds__(kSortThreads) void bf16_counting_sort_kernel(SamplerArgs a)
{
    const uint32_t row = blockIdx.x;
    if (a.row_state[row] != kRowNeedsGeneral || left_to_the_wide_select(a, row))
        return;
    const int tid = threadIdx.x;
    const uint32_t n = a.vocab;

    __shared__ uint32_t bins[kCountWords];
    __shared__ CountScratch scratch;

    const uint16_t* logits = reinterpret_cast<const uint16_t*>(
        static_cast<const char*>(a.logits) + static_cast<size_t>(row) * a.row_stride * 2u);
    uint32_t* run_keys = a.sort_keys[1] + row * a.sort_stride;
    uint32_t* run_ends = a.sort_keys[0] + row * a.sort_stride;
    const uint32_t misalignment = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(logits) & 15u) / 2u;
    const uint16_t* aligned_logits = logits - misalignment;
    const uint32_t aligned_end = misalignment + n; // positions [misalignment, aligned_end) hold the row

    const auto clear_bins = [&]() {
        uint4* wide = reinterpret_cast<uint4*>(bins);
#pragma unroll
        for (int j = 0; j < kCountWords / 4 / kSortThreads; ++j)
            wide[j * kSortThreads + tid] = uint4{0u, 0u, 0u, 0u};
        __syncthreads();
    };
    uint32_t runs_written = 0;
    uint32_t written = 0;
    NCNN_MOE_STAMP(blockIdx.x, 14, 0);
    clear_bins();
    count_bf16_keys<true>(aligned_logits, misalignment, aligned_end, 0u, bins, tid);
    __syncthreads();
    __shared__ uint32_t specials_fit;
    {
        const bool fits = fold_special_bf16_counts(bins, tid);
        if (tid == 0)
            specials_fit = fits ? 1u : 0u;
    }
    __syncthreads();
    NCNN_MOE_STAMP(blockIdx.x, 14, 1);
    // (counts of NaN or of zeros that do not fit 16 bits: a number of logits that no sum of counters reaches)
    const bool packed_sound =
        write_runs_of_counts<true>(bins, specials_fit != 0u ? n : 0xffffffffu, 0u, written, runs_written, run_keys, run_ends, scratch, tid);
    NCNN_MOE_STAMP(blockIdx.x, 14, 2);
    if (!packed_sound)
    {
        for (uint32_t round = 0; round < 2; ++round)
        {
            __syncthreads();
            clear_bins();
            count_bf16_keys<false>(aligned_logits, misalignment, aligned_end, round, bins, tid);
            __syncthreads();
            write_runs_of_counts<false>(bins, 0u, round << 15, written, runs_written, run_keys, run_ends, scratch, tid);
        }
    }
    if (tid == 0)
        a.sort_indices[0][row * a.sort_stride] = runs_written;
}

struct RecoverScratch
{
    uint32_t wave_counts[2][kReplayWaves]; // of alternate trips
    int32_t found;
};

// Token index of position `rank` of the sorted row, from the logits: the sort is stable, so it is
// the (rank - first position of that key)-th element, in index order, whose key equals keys[rank].
// Every thread of the workgroup must call it.
template <int DTYPE>
__device__ __noinline__ int32_t recover_token_of_key(
    const void* row_pointer, uint32_t vocab, uint32_t key, uint32_t ordinal, uint32_t occurrences, RecoverScratch& scratch, int tid);

template <int DTYPE>
__device__ __forceinline__ int32_t recover_token_index(
    const void* row_pointer, uint32_t vocab, const uint32_t* keys, uint32_t sorted, uint32_t rank, RecoverScratch& scratch, int tid)
{
    const uint32_t key = keys[rank];
    // first position holding this key, and the first behind it (`sorted` keys are there; a row sorted in part ends
    // between two different keys)
    const uint32_t low = wave_partition_point(rank, [keys, key](uint32_t position) { return keys[position] < key; });
    const uint32_t high = rank + 1u +
        wave_partition_point(sorted - rank - 1u, [keys, key, rank](uint32_t position) { return keys[rank + 1u + position] <= key; });
    return recover_token_of_key<DTYPE>(row_pointer, vocab, key, rank - low, high - low, scratch, tid);
}

// The ordinal-th of the `occurrences` elements of the row, in index order, whose key equals `key`.  The workgroup
// reads the row from the end that is nearer in occurrences (front to back for the first half of them, back to front
// for the rest: a quarter of the row on average instead of half, half of it at most), in trips of sixteen
// consecutive slices, one per wave; the 16-byte loads of the next trip are in flight while this one's matches are
// counted (the barrier between trips does not wait for them).  After each trip the waves' match counts tell whether
// the wanted match lies in it, and the wave whose slice holds it locates the element from the masks it still has in
// registers.  Every thread of the workgroup must call it.
template <int DTYPE>
__device__ __noinline__ int32_t recover_token_of_key(
    const void* row_pointer, uint32_t vocab, uint32_t key, uint32_t ordinal, uint32_t occurrences, RecoverScratch& scratch, int tid)
{
    using Vector = LogitsVector<DTYPE>;
    constexpr uint32_t kWidth = Vector::kWidth;
    constexpr int kLoads = 4;
    constexpr uint32_t kSlice = kLoads * kWaveSize * kWidth; // positions a wave looks at per trip
    constexpr uint32_t kTrip = kSlice * kReplayWaves;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    // positions count from the 16-byte boundary below the row: [misalignment, end) hold the row
    const uint32_t misalignment =
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row_pointer) & 15u) / Vector::kElementBytes;
    const char* aligned_base = static_cast<const char*>(row_pointer) - static_cast<size_t>(misalignment) * Vector::kElementBytes;
    const uint32_t end = misalignment + vocab;
    const uint32_t trips = (end + kTrip - 1u) / kTrip;

    // An element matches when its key equals `key`.  Keys are one-to-one with the logits' bit patterns except
    // that the two zeros share a key, and all NaNs another: the raw bits are compared (with the sign masked for
    // zero), which takes a third of the instructions of building every element's key.  One test without a branch
    // serves all three cases, with constants that are the same in every lane:
    //   ((bits & kept) ^ flipped) - floor <= room     (unsigned; a difference below zero wraps far above `room`)
    // a value: kept = every bit (no sign for zero), flipped = its pattern, floor = room = 0: equality;
    // NaN: kept = the bits without the sign, flipped = 0, floor = infinity + 1, room = the patterns above that.
    // A bf16 logit is tested where it lies in its 32-bit word, the constants shifted to the upper half for the odd ones.
    constexpr uint32_t kAbsoluteBits = DTYPE == NCNN_MOE_LOGITS_F32 ? 0x7fffffffu : 0x7fffu;
    constexpr uint32_t kEveryBit = DTYPE == NCNN_MOE_LOGITS_F32 ? 0xffffffffu : 0xffffu;
    constexpr uint32_t kInfinityBits = DTYPE == NCNN_MOE_LOGITS_F32 ? 0x7f800000u : 0x7f80u;
    const bool wants_nan = key == 0xffffffffu;
    const uint32_t value_bits = __float_as_uint(value_from_descending_key(key));
    const uint32_t pattern = DTYPE == NCNN_MOE_LOGITS_F32 ? value_bits : value_bits >> 16;
    const uint32_t kept = wants_nan || (pattern & kAbsoluteBits) == 0u ? kAbsoluteBits : kEveryBit;
    const uint32_t flipped = wants_nan ? 0u : pattern & kept;
    const uint32_t floor = wants_nan ? kInfinityBits + 1u : 0u;
    const uint32_t room = wants_nan ? kAbsoluteBits - (kInfinityBits + 1u) : 0u;
    const uint32_t kept_high = kept << 16, flipped_high = flipped << 16, floor_high = floor << 16, room_high = room << 16;
    // the matches among the kWidth logits of one 16-byte load, bit c for the c-th
    const auto matches_of = [&](const uint4& loaded) {
        const uint32_t words[4] = {loaded.x, loaded.y, loaded.z, loaded.w};
        uint32_t mask = 0;
#pragma unroll
        for (uint32_t c = 0; c < kWidth; ++c)
        {
            bool match;
            if (DTYPE == NCNN_MOE_LOGITS_F32)
                match = ((words[c] & kept) ^ flipped) - floor <= room;
            else if ((c & 1u) == 0u)
                match = ((words[c >> 1] & kept) ^ flipped) - floor <= room;
            else
                match = ((words[c >> 1] & kept_high) ^ flipped_high) - floor_high <= room_high;
            mask |= match ? 1u << c : 0u;
        }
        return mask;
    };

    // backward: the wanted match is the target-th counted from the row's end, and everything below counts from there
    const bool backward = ordinal < occurrences && ordinal >= occurrences - ordinal;
    const uint32_t target = backward ? occurrences - 1u - ordinal : ordinal;

    if (tid == 0)
        scratch.found = -1;
    const auto load_trip = [&](uint32_t trip, uint4 (&raw)[kLoads]) {
        const uint32_t first = trip * kTrip + static_cast<uint32_t>(wave) * kSlice;
#pragma unroll
        for (int k = 0; k < kLoads; ++k)
        {
            const uint32_t position = first + static_cast<uint32_t>(k * kWaveSize + lane) * kWidth;
            raw[k] = load_global_uint4(aligned_base + static_cast<size_t>(position < end ? position : 0u) * Vector::kElementBytes);
        }
    };
    uint32_t seen = 0; // matches in the trips before this one
    // One trip: starts the loads of the next into `next`, counts the matches of `raw`.  True when the search is over.
    const auto search_trip = [&](uint32_t step, uint4 (&raw)[kLoads], uint4 (&next)[kLoads]) -> bool {
        const uint32_t trip = backward ? trips - 1u - step : step;
        // (the last step loads its own trip again: a load under a condition would make the wait below one for every
        // load in flight, the new ones included)
        load_trip(step + 1u < trips ? (backward ? trip - 1u : trip + 1u) : trip, next);
        const uint32_t parity = step & 1u;
        const uint32_t first = trip * kTrip + static_cast<uint32_t>(wave) * kSlice;
        // per load k: the lane's matches among the kWidth positions from first + (k * 64 + lane) * kWidth
        uint32_t masks[kLoads];
        uint32_t lane_matches = 0;
#pragma unroll
        for (int k = 0; k < kLoads; ++k)
        {
            const uint32_t position = first + static_cast<uint32_t>(k * kWaveSize + lane) * kWidth;
            const uint32_t mask = matches_of(raw[k]);
            // positions in front of the row's first element and behind its last are no elements of it
            const uint32_t below = position < misalignment ? min(misalignment - position, kWidth) : 0u;
            const uint32_t inside = position < end ? min(end - position, kWidth) : 0u;
            masks[k] = mask & ((1u << inside) - 1u) & ~((1u << below) - 1u);
            lane_matches += static_cast<uint32_t>(__popc(masks[k]));
        }
        const uint32_t wave_matches =
            static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(wave_prefix_sum_u32(lane_matches)), kWaveSize - 1));
        if (lane == 0)
            scratch.wave_counts[parity][wave] = wave_matches;
        lds_barrier();
        // lane w holds wave w's count; a prefix sum over the lanes gives every wave the matches on either side of it
        const uint32_t count_of_lane = lane < kReplayWaves ? scratch.wave_counts[parity][lane] : 0u;
        const uint32_t through_lane = wave_prefix_sum_u32(count_of_lane);
        const uint32_t trip_matches = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(through_lane), kReplayWaves - 1));
        const uint32_t through_wave = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(through_lane), wave));
        // matches between the end the search started from and this wave's slice
        const uint32_t skipped = seen + (backward ? trip_matches - through_wave : through_wave - wave_matches);
        if (target >= seen + trip_matches)
        {
            seen += trip_matches;
            return step + 1u >= trips;
        }
        if (target >= skipped && target < skipped + wave_matches)
        {
            uint32_t remaining = target - skipped; // matches of this slice still to skip
            bool done = false;
#pragma unroll
            for (int i = 0; i < kLoads; ++i)
            {
                // (static indices either way: the loads are looked at in the search's direction)
                const uint32_t load_mask = backward ? masks[kLoads - 1 - i] : masks[i];
                const uint32_t k = backward ? static_cast<uint32_t>(kLoads - 1 - i) : static_cast<uint32_t>(i);
                if (done || __ballot(load_mask != 0u) == 0)
                    continue; // most loads hold no match at all: no scan for them
                const uint32_t count = static_cast<uint32_t>(__popc(load_mask));
                const uint32_t inclusive = wave_prefix_sum_u32(count); // matches in lanes 0..lane of this load
                const uint32_t total = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(inclusive), kWaveSize - 1));
                if (remaining < total)
                {
                    // matches of this load that the search passes before it reaches this lane's
                    const uint32_t passed = backward ? total - inclusive : inclusive - count;
                    if (remaining >= passed && remaining < passed + count)
                    {
                        uint32_t mask = load_mask;
                        for (uint32_t dropped = passed; dropped < remaining; ++dropped)
                            mask = backward ? mask & ~(0x80000000u >> __builtin_clz(mask)) : mask & (mask - 1u);
                        const uint32_t bit = backward ? 31u - static_cast<uint32_t>(__builtin_clz(mask))
                                                      : static_cast<uint32_t>(__builtin_ctz(mask));
                        const uint32_t position = first + (k * kWaveSize + static_cast<uint32_t>(lane)) * kWidth + bit;
                        scratch.found = static_cast<int32_t>(position - misalignment);
                    }
                    done = true;
                }
                else
                    remaining -= total;
            }
        }
        return true;
    };
    // two sets of registers take turns, so that no set is copied (a copy would wait for the loads it copies)
    uint4 even[kLoads], odd[kLoads];
    load_trip(backward ? trips - 1u : 0u, even);
    for (uint32_t step = 0;; step += 2u)
    {
        if (search_trip(step, even, odd))
            break;
        if (search_trip(step + 1u, odd, even))
            break;
    }
    __syncthreads();
    const int32_t found = scratch.found;
    __syncthreads();
    return found;
}

// Full-order rows: walks the sorted row as the CPU sampler does (src/engine/session.cpp:84-134,
// :429-442).  One workgroup per row.  With RUNS the row comes from bf16_counting_sort_kernel as runs
// of equal keys; otherwise sort_keys[1] holds one key per element.
// The walk over one sorted row, from the sorted keys (or runs) and their terms to the row's result.  Every thread
// of the workgroup (kReplayThreads) calls it.
template <int DTYPE, bool RUNS>
__device__ __forceinline__ void replay_row(
    const SamplerArgs& a, uint32_t row, const ncnn_moe_sample_params& p, const uint32_t* keys, const uint32_t* run_ends,
    uint32_t run_total, const float* terms0, int tid)
{
    NCNN_MOE_STAMP(blockIdx.x, 15, 1);
    const bool have_indices = !RUNS && a.distribution_count != nullptr; // the pair sort ran: indices are valid
    const uint32_t* indices = have_indices ? a.sort_indices[1] + row * a.sort_stride : nullptr;
    const uint32_t vocab = a.vocab;
    // a row of elements may be sorted in part: its first elements in sorted order, all finite, and counts of the rest
    const bool sorted_in_part = !RUNS && a.sort_lengths != nullptr && a.sort_last_keys[row] != 0xffffffffu;
    // items: what `keys` holds one entry of (an element, or a run of equal keys)
    const uint32_t items = RUNS ? run_total : sorted_length(a, row);
    const char* row_pointer = static_cast<const char*>(a.logits) +
        static_cast<size_t>(row) * a.row_stride * LogitsVector<DTYPE>::kElementBytes;

    __shared__ ReplayScratch scratch;
    __shared__ RecoverScratch recover_scratch;

    uint8_t flags = NCNN_MOE_ROW_FLAG_GENERAL_PATH;
    {
        uint32_t effective_k = 0;
        int status = 0;
        if (resolve_row_mode(p, vocab, a.max_select_top_k, 0, effective_k, status) != kModeGeneral)
            flags |= NCNN_MOE_ROW_FLAG_FALLBACK;
    }
    if (sorted_in_part ? (a.finite_counts[row] & kRowHoldsNan) != 0u : keys[items - 1] == 0xffffffffu)
        flags |= NCNN_MOE_ROW_FLAG_HAS_NAN;
    if (tid == 0)
        a.row_state[row] = kRowDone;

    SortedRow layout; // only the run fields are used here
    layout.keys = keys;
    layout.run_ends = run_ends;
    layout.run_count = items;
    // first element of an item
    auto first_element = [&](uint32_t item) -> uint32_t {
        if constexpr (RUNS)
            return item < items ? run_first_element(layout, item) : vocab;
        else
            return item;
    };
    auto token_at = [&](uint32_t rank) -> int32_t {
        if (have_indices)
            return static_cast<int32_t>(indices[rank]);
        if constexpr (RUNS)
        {
            const uint32_t run = run_of_element(layout, rank);
            const uint32_t run_first = run_first_element(layout, run);
            return recover_token_of_key<DTYPE>(row_pointer, vocab, keys[run], rank - run_first, run_ends[run] - run_first, recover_scratch, tid);
        }
        else
            return recover_token_index<DTYPE>(row_pointer, vocab, keys, items, rank, recover_scratch, tid);
    };

    if (p.temperature == 0.0f)
    {
        // a greedy row whose select overflowed (every logit tied): first finite logit in sorted order,
        // non-finite logits skipped (src/engine/session.cpp:404-424)
        const uint32_t low = wave_partition_point(items, [keys](uint32_t item) { return keys[item] <= kPositiveInfinityKey; });
        const bool any_finite = low < items && keys[low] <= kLastFiniteKey;
        int32_t token = -1;
        if (any_finite)
            token = token_at(first_element(low));
        if (tid == 0)
        {
            if (any_finite)
            {
                write_token(a, row, p, token, 1.0f, 1u, 0, flags);
                if (a.distribution_count != nullptr)
                {
                    a.distribution_count[row] = 1;
                    if (a.distribution_cap > 0)
                    {
                        a.distribution_ids[static_cast<size_t>(row) * a.distribution_cap] = token;
                        a.distribution_probabilities[static_cast<size_t>(row) * a.distribution_cap] = 1.0f;
                    }
                }
            }
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
    // first item whose key is not finite
    const uint32_t low = wave_partition_point(items, [keys](uint32_t item) { return keys[item] <= kLastFiniteKey; });
    const uint32_t finite_elements = sorted_in_part ? a.finite_counts[row] & ~kRowHoldsNan : first_element(low);
    uint32_t n = finite_elements;
    if (p.top_k > 0 && p.top_k < vocab && n > p.top_k)
        n = p.top_k;
    NCNN_MOE_STAMP(blockIdx.x, 15, 2);
    const uint4* chunk_steps = nullptr;
    if constexpr (!RUNS)
    {
        if (a.chunk_steps_ready != 0)
            chunk_steps = a.chunk_steps + static_cast<size_t>(row) * a.chunk_capacity;
    }
    // (the finite runs and the elements they hold: a sum over all of them need not look for its last run)
    bool tail_matters = false;
    replay_sorted_window<RUNS>(
        a, row, p, keys, run_ends, items, n, indices, flags, scratch, tid, token_at, terms0, chunk_steps, RUNS ? vocab : items,
        RUNS ? low : 0u, finite_elements, sorted_in_part ? items : 0xffffffffu, sorted_in_part ? a.sort_last_keys[row] + 1u : 0u, &tail_matters);
    // An element that was left out of the sort could have moved a sum, or been the one drawn: the row stays
    // pending, and the launch behind this one sorts it whole.
    if (tail_matters && tid == 0)
    {
        a.sort_last_keys[row] = 0xffffffffu;
        a.sort_lengths[row] = vocab;
        a.row_state[row] = kRowNeedsGeneral;
    }
}

template <int DTYPE, bool RUNS>
__global__ __launch_bounds__(kReplayThreads) void general_replay_kernel(SamplerArgs a)
{
    const uint32_t row = blockIdx.x;
    if (a.row_state[row] != kRowNeedsGeneral || left_to_the_wide_select(a, row))
        return;
    const int tid = threadIdx.x;
    NCNN_MOE_STAMP(blockIdx.x, 15, 0);
    const ncnn_moe_sample_params p = a.params[row];
    const uint32_t* keys = a.sort_keys[1] + row * a.sort_stride;
    uint32_t run_total_of_row = 0;
    const uint32_t* run_ends = RUNS ? a.sort_keys[0] + row * a.sort_stride : nullptr;
    // exp(logit/T - maximum) of every item, computed once for the three sums that use it (greedy rows add nothing)
    const float* terms0 = nullptr;
    const auto term_of_key = [&p](uint32_t key, float maximum) {
        return expf_libm(value_from_descending_key(key) / p.temperature - maximum);
    };
    if constexpr (RUNS)
    {
        // a row of few runs is walked from LDS; the terms of a longer one go to the sort's spare index buffer
        __shared__ uint32_t cached_keys[kCachedRuns];
        __shared__ __align__(16) uint32_t cached_ends[kCachedRuns];
        __shared__ __align__(16) float cached_terms[kCachedRuns];
        const uint32_t run_total = a.sort_indices[0][row * a.sort_stride];
        run_total_of_row = run_total;
        const float maximum = value_from_descending_key(keys[0]) / p.temperature;
        if (run_total <= static_cast<uint32_t>(kCachedRuns))
        {
            for (uint32_t i = threadIdx.x; i < run_total; i += kReplayThreads)
            {
                const uint32_t key = keys[i];
                cached_keys[i] = key;
                cached_ends[i] = run_ends[i];
                cached_terms[i] = term_of_key(key, maximum);
            }
            __syncthreads();
            keys = cached_keys;
            run_ends = cached_ends;
            terms0 = cached_terms;
        }
        else
        {
            float* terms = reinterpret_cast<float*>(a.sort_indices[1] + row * a.sort_stride);
            if (p.temperature != 0.0f)
            {
                for (uint32_t i = threadIdx.x; i < run_total; i += kReplayThreads)
                    terms[i] = term_of_key(keys[i], maximum);
            }
            __syncthreads();
            terms0 = terms;
        }
    }
    else
    {
        // (a row whose keys the terms kernel could not put in order, or one that a select kernel handed on after the
        // rows were listed by their options: the launch behind this one sorts it whole)
        const uint32_t unordered = (a.sort_low_digit_skipped != 0u || a.rows_listed_by_options != 0u) ? a.disordered_rows[row] : 0u;
        if ((a.sort_low_digit_skipped != 0u && (unordered & 1u) != 0u) || (a.rows_listed_by_options != 0u && (unordered & 2u) != 0u))
        {
            if (tid == 0)
            {
                a.sort_last_keys[row] = 0xffffffffu;
                a.sort_lengths[row] = a.vocab;
            }
            return;
        }
        float* terms = sorted_terms(a, row);
        if (a.terms_precomputed == 0 && p.temperature != 0.0f)
        {
            const float maximum = value_from_descending_key(keys[0]) / p.temperature;
            const uint32_t sorted = sorted_length(a, row);
            for (uint32_t i = threadIdx.x; i < sorted; i += kReplayThreads)
                terms[i] = term_of_key(keys[i], maximum);
            __syncthreads();
        }
        terms0 = terms;
    }
    replay_row<DTYPE, RUNS>(a, row, p, keys, run_ends, run_total_of_row, terms0, tid);
}

// bf16 full-order rows in ONE kernel: bf16_counting_sort_kernel and general_replay_kernel<BF16, runs> back to
// back in one workgroup per row, which both are.  The runs never leave the compute unit: once every counter
// sits in a register they are written over the counters themselves (keys, ends and, behind them, the terms: a
// third of the 128 KB each), which saves the runs' trip through device memory and a launch.  A row with more
// runs than that, or one whose counters overflowed 16 bits, writes its runs to device memory as the two
// kernels do, and walks them from there.
constexpr uint32_t kRunsInPlace = (kCountWords / 3) & ~3u; // 10,920 runs with their ends and terms in the counters' LDS (each array on a 16-byte boundary)

__global__ __launch_bounds__(kSortThreads) void bf16_counting_replay_kernel(SamplerArgs a)
{
    static_assert(kSortThreads == kReplayThreads, "the count and the walk share a workgroup");
    const uint32_t row = blockIdx.x;
    if (a.row_state[row] != kRowNeedsGeneral || left_to_the_wide_select(a, row))
        return;
    const int tid = threadIdx.x;
    const uint32_t n = a.vocab;

    __shared__ uint32_t arena[kCountWords];
    __shared__ CountScratch scratch;
    __shared__ uint32_t specials_fit;

    const uint16_t* logits = reinterpret_cast<const uint16_t*>(
        static_cast<const char*>(a.logits) + static_cast<size_t>(row) * a.row_stride * 2u);
    uint32_t* global_keys = a.sort_keys[1] + row * a.sort_stride;
    uint32_t* global_ends = a.sort_keys[0] + row * a.sort_stride;
    const uint32_t misalignment = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(logits) & 15u) / 2u;
    const uint16_t* aligned_logits = logits - misalignment;
    const uint32_t aligned_end = misalignment + n;

    const auto clear_bins = [&]() {
        uint4* wide = reinterpret_cast<uint4*>(arena);
#pragma unroll
        for (int j = 0; j < kCountWords / 4 / kSortThreads; ++j)
            wide[j * kSortThreads + tid] = uint4{0u, 0u, 0u, 0u};
        __syncthreads();
    };
    uint32_t runs_written = 0;
    uint32_t written = 0;
    NCNN_MOE_STAMP(blockIdx.x, 14, 0);
    clear_bins();
    count_bf16_keys<true>(aligned_logits, misalignment, aligned_end, 0u, arena, tid);
    __syncthreads();
    {
        const bool fits = fold_special_bf16_counts(arena, tid);
        if (tid == 0)
            specials_fit = fits ? 1u : 0u;
    }
    __syncthreads();
    NCNN_MOE_STAMP(blockIdx.x, 14, 1);
    bool in_place = false;
    const bool packed_sound = write_runs_of_counts<true>(
        arena, specials_fit != 0u ? n : 0xffffffffu, 0u, written, runs_written, global_keys, global_ends, scratch, tid, &in_place, kRunsInPlace);
    NCNN_MOE_STAMP(blockIdx.x, 14, 2);
    if (!packed_sound)
    {
        in_place = false;
        for (uint32_t round = 0; round < 2; ++round)
        {
            __syncthreads();
            clear_bins();
            count_bf16_keys<false>(aligned_logits, misalignment, aligned_end, round, arena, tid);
            __syncthreads();
            write_runs_of_counts<false>(arena, 0u, round << 15, written, runs_written, global_keys, global_ends, scratch, tid);
        }
    }
    __syncthreads(); // the runs are where the walk reads them (LDS, or device memory written by this workgroup)
    NCNN_MOE_STAMP(blockIdx.x, 15, 0);

    const ncnn_moe_sample_params p = a.params[row];
    const uint32_t run_total = runs_written;
    uint32_t* const cached_keys = arena;
    uint32_t* const cached_ends = arena + kRunsInPlace;
    float* const cached_terms = reinterpret_cast<float*>(arena + 2 * kRunsInPlace);
    const uint32_t* keys = global_keys;
    const uint32_t* run_ends = global_ends;
    const float* terms0 = nullptr;
    const auto term_of_key = [&p](uint32_t key, float maximum) {
        return expf_libm(value_from_descending_key(key) / p.temperature - maximum);
    };
    if (in_place || run_total <= kRunsInPlace)
    {
        if (!in_place)
        {
            // (a row that was counted in two rounds: its runs come back from device memory, the counters are dead)
            for (uint32_t i = threadIdx.x; i < run_total; i += kReplayThreads)
            {
                cached_keys[i] = global_keys[i];
                cached_ends[i] = global_ends[i];
            }
            __syncthreads();
        }
        const float maximum = value_from_descending_key(cached_keys[0]) / p.temperature;
        for (uint32_t i = threadIdx.x; i < run_total; i += kReplayThreads)
            cached_terms[i] = term_of_key(cached_keys[i], maximum);
        __syncthreads();
        keys = cached_keys;
        run_ends = cached_ends;
        terms0 = cached_terms;
    }
    else
    {
        float* terms = reinterpret_cast<float*>(a.sort_indices[1] + row * a.sort_stride);
        if (p.temperature != 0.0f)
        {
            const float maximum = value_from_descending_key(global_keys[0]) / p.temperature;
            for (uint32_t i = threadIdx.x; i < run_total; i += kReplayThreads)
                terms[i] = term_of_key(global_keys[i], maximum);
        }
        __syncthreads();
        terms0 = terms;
    }
    replay_row<NCNN_MOE_LOGITS_BF16, true>(a, row, p, keys, run_ends, run_total, terms0, tid);
}

// exp(logit/T - maximum) of every element of the sorted full-order rows, written over the sort's other key
// buffer: the replay that follows adds these terms one workgroup per row, and computing them there would
// put a few dozen instructions per element on that workgroup's path; here the whole GPU shares them.
// grid (parts, rows).
//
// After a sort that left out the keys' lowest byte (SamplerArgs::sort_low_digit_skipped) the keys arrive ordered
// by their upper 24 bits, and the keys that agree in those - neighbours, one to three of them where a row's
// logits are spread over the floats, because 256 consecutive floats rarely hold two - are put in order here: an
// element looks at up to kTouchUpReach neighbours on either side as far as they share its upper 24 bits, counts
// those in front of it that belong behind it and those behind it that belong in front, and moves by the
// difference (equal keys keep their places).  That is the element's place in the sorted row whenever it has seen
// all of its group.  A group that reaches further is harmless if it is in order already (a run of equal keys: a
// row of rounded logits, a padded vocabulary), and whether it is shows between neighbours: a group longer than
// the reach that holds two adjacent keys out of order has an element that sees them without seeing the group's
// end (the group's first or last element if they lie within reach of it, else the first of the two), and that
// element marks the row in disordered_rows: the replay leaves such a row to the launch that sorts it whole.
constexpr int kTermsThreads = 256;
constexpr int kTermsPerThread = 8;
constexpr int kTermsTile = kTermsThreads * kTermsPerThread;
constexpr int kTouchUpReach = 16;
constexpr int kTouchUpNear = 6; // neighbours on either side that every element looks at, without a branch

// The place in the sorted row of the element at position i, whose key is `key` and lies at mine[0] among its
// neighbours' keys (positions in front of the row hold 0, positions behind it 0xffffffff: neither is ever counted,
// and neither is out of order where it stands).  A group of up to kTouchUpNear keys is seen whole within
// kTouchUpNear steps, by straight-line code: an instruction costs this kernel as much as a byte (its time is the
// instructions its waves issue), and a loop that ends where the group does is some fifty of them a step.  A key
// in front belongs behind this one if it lies in (key, key | 255], one behind belongs in front if it lies in
// [key & ~255, key): a subtraction and a compare each.  `further`: the group may reach beyond what was looked at.
__device__ __forceinline__ uint32_t touched_up_place(const uint32_t* mine, uint32_t key, uint32_t i, bool& further)
{
    const uint32_t low = key & 255u;
    const uint32_t room_above = 255u - low;
    uint32_t place = i;
#pragma unroll
    for (int d = 1; d <= kTouchUpNear; ++d)
    {
        place -= mine[-d] - key - 1u < room_above ? 1u : 0u;
        place += key - mine[d] - 1u < low ? 1u : 0u;
    }
    further = ((mine[-kTouchUpNear] ^ key) < 256u) | ((mine[kTouchUpNear] ^ key) < 256u);
    return place;
}

// The same for an element of a longer group (rare among spread logits; every element of a row of rounded ones),
// one step at a time up to kTouchUpReach on either side.
__device__ __forceinline__ uint32_t touched_up_place_of_long_group(const uint32_t* mine, uint32_t i, uint32_t& lost)
{
    const uint32_t key = mine[0];
    uint32_t belong_behind = 0, belong_in_front = 0;
    uint32_t previous = key;
    bool out_of_order = false, end_seen = false;
#pragma nounroll
    for (int d = 1; d <= kTouchUpReach; ++d)
    {
        const uint32_t other = mine[-d];
        if ((other ^ key) >= 256u)
        {
            end_seen = true;
            break;
        }
        belong_behind += other > key ? 1u : 0u;
        out_of_order |= other > previous;
        previous = other;
    }
    bool all_seen = end_seen;
    end_seen = false;
    previous = key;
#pragma nounroll
    for (int d = 1; d <= kTouchUpReach; ++d)
    {
        const uint32_t other = mine[d];
        if ((other ^ key) >= 256u)
        {
            end_seen = true;
            break;
        }
        belong_in_front += other < key ? 1u : 0u;
        out_of_order |= previous > other;
        previous = other;
    }
    all_seen = all_seen && end_seen;
    lost |= !all_seen && out_of_order ? 1u : 0u;
    return i - belong_behind + belong_in_front;
}

__global__ __launch_bounds__(kTermsThreads) void full_order_terms_kernel(SamplerArgs a)
{
    uint32_t row;
    if (!spread_grid_row(a, row))
        return;
    __shared__ uint64_t exp2_table[32]; // a copy in LDS: the lookups of a wave are 64 different addresses
    __shared__ uint32_t tile_keys[kTermsTile + 2 * kTouchUpReach];
    if (threadIdx.x < 32)
        exp2_table[threadIdx.x] = kExp2Table[threadIdx.x];
    const uint32_t n = sorted_length(a, row);
    const uint32_t tile_first = blockIdx.x * kTermsTile;
    if (tile_first >= n)
        return; // (behind the row's sorted elements: no chunk reads this block's sum)
    const bool touch_up = a.sort_low_digit_skipped != 0u;
    const float temperature = a.params[row].temperature;
    const uint32_t* keys = a.sort_keys[touch_up ? 0 : 1] + row * a.sort_stride;
    uint32_t* const ordered_keys = a.sort_keys[1] + row * a.sort_stride;
    float* terms = sorted_terms(a, row);
    const uint32_t first = tile_first + threadIdx.x;
    const uint32_t behind_the_row = 0xffffffffu; // (in place of the keys behind the row's end; see touched_up_place)
    uint32_t loaded[kTermsPerThread];
#pragma unroll
    for (int j = 0; j < kTermsPerThread; ++j)
    {
        const uint32_t i = first + static_cast<uint32_t>(j * kTermsThreads);
        loaded[j] = i < n ? keys[i] : behind_the_row;
    }
    uint32_t smallest_key;
    uint32_t places[kTermsPerThread];
    if (!touch_up)
    {
        smallest_key = keys[0];
#pragma unroll
        for (int j = 0; j < kTermsPerThread; ++j)
            places[j] = first + static_cast<uint32_t>(j * kTermsThreads);
        __syncthreads();
    }
    else
    {
        // the row's smallest key is in the first group: the first of the row if that group is in order, and
        // within reach of the row's first element if it is not (or the row is marked)
        const uint32_t lane = threadIdx.x & (kWaveSize - 1);
        const uint32_t front = lane <= static_cast<uint32_t>(kTouchUpReach) && lane < n ? keys[lane] : 0xffffffffu;
        smallest_key = ~wave_max_u32(~front);
        // the tile's keys, with kTouchUpReach of the tiles on either side, at tile_keys[position - tile_first + reach]
#pragma unroll
        for (int j = 0; j < kTermsPerThread; ++j)
            tile_keys[kTouchUpReach + j * kTermsThreads + static_cast<int>(threadIdx.x)] = loaded[j];
        if (threadIdx.x < 2 * kTouchUpReach)
        {
            const bool left = threadIdx.x < static_cast<uint32_t>(kTouchUpReach);
            const int64_t position = left ? static_cast<int64_t>(tile_first) - kTouchUpReach + threadIdx.x
                                          : static_cast<int64_t>(tile_first) + kTermsTile + (threadIdx.x - kTouchUpReach);
            const uint32_t slot = left ? threadIdx.x : static_cast<uint32_t>(kTermsTile) + threadIdx.x;
            uint32_t key = position < 0 ? 0u : behind_the_row;
            if (position >= 0 && position < static_cast<int64_t>(n))
                key = keys[position];
            tile_keys[slot] = key;
        }
        __syncthreads();
        // A tile that is in order as it stands, with the neighbours its elements would look at, needs nothing
        // (every tile of a row whose keys end in the same byte: logits that were rounded to bf16 or fp16, whose
        // groups are long runs of equal keys): no pair of keys within reach of an element is out of order unless
        // two adjacent keys between them are.
        bool out_of_order = false;
#pragma unroll
        for (int j = 0; j < kTermsPerThread; ++j)
        {
            places[j] = first + static_cast<uint32_t>(j * kTermsThreads);
            out_of_order |= tile_keys[kTouchUpReach + j * kTermsThreads + static_cast<int>(threadIdx.x) + 1] < loaded[j];
        }
        if (threadIdx.x < static_cast<uint32_t>(kTouchUpReach))
            out_of_order |= tile_keys[threadIdx.x + 1u] < tile_keys[threadIdx.x];
        else if (threadIdx.x < 2u * kTouchUpReach - 1u)
            out_of_order |= tile_keys[kTermsTile + threadIdx.x + 1u] < tile_keys[kTermsTile + threadIdx.x];
        const bool touch_tile = __syncthreads_or(out_of_order ? 1 : 0) != 0;
        uint32_t long_groups = 0;
        if (touch_tile)
        {
#pragma unroll
            for (int j = 0; j < kTermsPerThread; ++j)
            {
                const uint32_t i = first + static_cast<uint32_t>(j * kTermsThreads);
                bool further = false;
                places[j] = touched_up_place(tile_keys + kTouchUpReach + j * kTermsThreads + static_cast<int>(threadIdx.x), loaded[j], i, further);
                long_groups |= further && i < n ? 1u << j : 0u;
            }
        }
        if (long_groups != 0u)
        {
            uint32_t lost = 0;
#pragma nounroll
            for (int j = 0; j < kTermsPerThread; ++j)
            {
                if ((long_groups >> j & 1u) == 0u)
                    continue;
                const uint32_t i = first + static_cast<uint32_t>(j * kTermsThreads);
                const uint32_t place = touched_up_place_of_long_group(tile_keys + kTouchUpReach + j * kTermsThreads + static_cast<int>(threadIdx.x), i, lost);
#pragma unroll
                for (int at = 0; at < kTermsPerThread; ++at)
                    places[at] = at == j ? place : places[at];
            }
            if (lost != 0u)
                atomicOr(&a.disordered_rows[row], 1u);
        }
    }
    const float maximum = value_from_descending_key(smallest_key) / temperature;
    double sum = 0.0;
#pragma unroll
    for (int j = 0; j < kTermsPerThread; ++j)
    {
        const uint32_t i = first + static_cast<uint32_t>(j * kTermsThreads);
        if (i < n)
        {
            const float term = expf_libm(value_from_descending_key(loaded[j]) / temperature - maximum, exp2_table);
            terms[places[j]] = term;
            if (touch_up)
                ordered_keys[places[j]] = loaded[j];
            sum += static_cast<double>(term);
        }
    }
    // the block's sum (fp64: an estimate of where the sequential fp32 sum stands, for full_order_chunk_steps_kernel)
    __shared__ double wave_sums[kTermsThreads / kWaveSize];
#pragma unroll
    for (int step = kWaveSize / 2; step > 0; step >>= 1)
        sum += __shfl_down(sum, step, kWaveSize);
    if ((threadIdx.x & (kWaveSize - 1)) == 0)
        wave_sums[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0)
    {
        double total = 0.0;
#pragma unroll
        for (int w = 0; w < kTermsThreads / kWaveSize; ++w)
            total += wave_sums[w];
        a.term_sums[static_cast<size_t>(row) * a.term_sum_parts + blockIdx.x] = total;
    }
}

// What every whole chunk of kReplayChunk terms does to the normaliser's running sum, computed by the whole GPU
// before the replay walks the row one workgroup per row: the composition of the chunk's steps (see
// sampler_exact_sum.h) for the exponent that the sum most likely has when it reaches the chunk, guessed from
// the fp64 sum of the terms in front of it.  The replay checks the guess against its exact sum: where the
// exponent is the one assumed here and the composed step leaves the mantissa inside its binade (the mantissa
// never decreases, so nothing inside the chunk left it either), the chunk costs it one addition instead of a
// round; everywhere else it runs the round as before.  A wrong guess costs time, never exactness.
// grid (chunks, rows); thread t composes the chunk's terms 16 t .. 16 t + 15.
constexpr int kChunkStepThreads = 256;
constexpr int kChunkStepPerThread = kReplayChunk / kChunkStepThreads;

__global__ __launch_bounds__(kChunkStepThreads) void full_order_chunk_steps_kernel(SamplerArgs a)
{
    static_assert(kChunkStepPerThread * kChunkStepThreads == kReplayChunk && kChunkStepPerThread % 4 == 0, "float4 loads over a whole chunk");
    static_assert(kReplayChunk % (kTermsThreads * kTermsPerThread) == 0, "a chunk is a whole number of the terms kernel's blocks");
    const uint32_t chunk = blockIdx.x;
    uint32_t row;
    if (!spread_grid_row(a, row))
        return;
    const int tid = threadIdx.x;
    const int lane = tid & (kWaveSize - 1);
    const int wave = tid >> 6;
    constexpr int kWaves = kChunkStepThreads / kWaveSize;
    __shared__ double wave_sums[kWaves];
    __shared__ ParityStep wave_totals[kWaves];
    const float* terms = sorted_terms(a, row);
    uint4* const out = a.chunk_steps + static_cast<size_t>(row) * a.chunk_capacity + chunk;
    const uint32_t base = chunk * kReplayChunk;
    const uint32_t n = sorted_length(a, row);
    if (base >= n)
        return; // (behind the row's sorted elements: the replay does not look at this chunk)
    // the chunk's terms are asked for first: the estimate below is a chain of loads, a reduction and a barrier
    // (the row's last chunk may be a partial one: the terms behind the row count as zero)
    const uint32_t first = base + static_cast<uint32_t>(tid) * kChunkStepPerThread;
    float4 loaded[kChunkStepPerThread / 4];
#pragma unroll
    for (int j = 0; j < kChunkStepPerThread / 4; ++j)
    {
        const uint32_t at = first + 4u * static_cast<uint32_t>(j);
        if (at + 4u <= n)
            loaded[j] = *reinterpret_cast<const float4*>(terms + at);
        else
            loaded[j] = float4{at < n ? terms[at] : 0.0f, at + 1u < n ? terms[at + 1u] : 0.0f,
                               at + 2u < n ? terms[at + 2u] : 0.0f, 0.0f};
    }
    // the sum in front of the chunk: the blocks of the terms kernel before it, or (first chunk) the head of
    // terms that every running sum adds one by one
    double before = 0.0;
    if (chunk == 0)
    {
        for (int i = tid; i < kSequentialHead; i += kChunkStepThreads)
            before += static_cast<double>(terms[i]);
    }
    else
    {
        const uint32_t blocks = chunk * (kReplayChunk / (kTermsThreads * kTermsPerThread));
        for (uint32_t block = tid; block < blocks; block += kChunkStepThreads)
            before += a.term_sums[static_cast<size_t>(row) * a.term_sum_parts + block];
    }
#pragma unroll
    for (int step = kWaveSize / 2; step > 0; step >>= 1)
        before += __shfl_down(before, step, kWaveSize);
    if (lane == 0)
        wave_sums[wave] = before;
    __syncthreads();
    double estimate = 0.0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w)
        estimate += wave_sums[w];
    const float estimate_f32 = static_cast<float>(estimate);
    if (!(estimate_f32 > 0.0f) || !is_finite_f32(estimate_f32))
    {
        if (tid == 0)
            *out = uint4{0u, 0u, 0u, 0u};
        return;
    }
    int exponent;
    uint32_t unused_mantissa;
    decode_sum(estimate_f32, exponent, unused_mantissa);
    ParityStep total{0u, 0u};
#pragma unroll
    for (int j = 0; j < kChunkStepPerThread; j += 4)
    {
        const float4 four = loaded[j / 4];
        const float values[4] = {four.x, four.y, four.z, four.w};
#pragma unroll
        for (int c = 0; c < 4; ++c)
        {
            const ParityStep step = step_of_term(values[c], exponent);
            const bool counted = first + j + c >= static_cast<uint32_t>(kSequentialHead); // the head is added before the chunks
            total = compose_steps(total, ParityStep{counted ? step.even : 0u, counted ? step.odd : 0u});
        }
    }
    const ParityStep inclusive = wave_scan_steps(total);
    if (lane == kWaveSize - 1)
        wave_totals[wave] = inclusive;
    __syncthreads();
    if (tid == 0)
    {
        ParityStep all{0u, 0u};
#pragma unroll
        for (int w = 0; w < kWaves; ++w)
            all = compose_steps(all, wave_totals[w]);
        *out = uint4{static_cast<uint32_t>(exponent), all.even, all.odd, 1u};
    }
}

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_SAMPLER_FULL_ORDER_H
