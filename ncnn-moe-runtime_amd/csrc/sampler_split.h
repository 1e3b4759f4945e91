// Split rows: the HBM pass for small batches, where a row is covered by several workgroups of one chunk
// each so that every compute unit streams (greedy rows and Top-K windows up to kFastTopK).
//
// Every workgroup of a row keeps the logits of its chunk that can belong to the row's Top-K window (the
// values at or above a bound that at least K values of the chunk reach) and hands them over through a
// record in device memory; the workgroup of the row that arrives last merges the records and finishes
// the row.  Between the last logit and the row's result lies a chain of dependent steps, and at these
// batch sizes that chain, not the streaming, sets the time of the launch.  The hand-over is therefore
// built so that nothing on it waits for a store to be acknowledged:
//   * a record entry is 8 bytes, (key, epoch | token index), written with one store; the epoch is a
//     per-row launch number kept in device memory, so a reader tells an entry of this launch from what an
//     earlier launch left behind without any clearing;
//   * a workgroup issues its entries and, without waiting for them, counts itself on the row's counter;
//   * the last workgroup reads every record (first through this XCD's L2, which holds what the row's
//     other workgroups wrote if they ran on this XCD) and checks the epochs: an entry that has not landed
//     yet, or a stale line, fails the check and the records are read again around the L2.  Such a retry
//     waits only for stores that were issued before their workgroup counted itself, never for another
//     workgroup to run;
//   * the merge cuts the row's candidates with one histogram over the key range [largest segment bound,
//     row maximum] in LDS, scanned by every wave for itself, and ranks what is left.
#ifndef NCNN_MOE_HIP_SAMPLER_SPLIT_H
#define NCNN_MOE_HIP_SAMPLER_SPLIT_H

#include "sampler_select.h"

namespace ncnn_moe_hip {

constexpr int kSplitHeaderEntries = 2;  // (segment bound, count | flags) and (segment maximum, 0)
// The kernel comes in two shapes: rows of up to 16 one-chunk workgroups, whose merge reads a segment's record with
// 32 lanes, and rows of 17 to kSplitMaxSegments (fp32 rows beyond 163,840 logits, bf16 rows beyond 196,608), read
// with 16 lanes a segment.  A record's place in memory is the same for both: a row's records lie kSplitMaxSegments apart.
constexpr uint32_t kSplitIndexBits = 19; // a split row holds at most 32 chunks of 12,288 logits
constexpr uint32_t kSplitIndexMask = (1u << kSplitIndexBits) - 1u;
constexpr uint32_t kSplitLastEpoch = (1u << (32 - kSplitIndexBits)) - 1u; // epochs run 1 .. 8191; 0 never tags an entry
constexpr int kSplitBins = kWaveSize;    // one histogram bin per lane of the scanning wave
constexpr int kSplitBinCapacity = 16;    // candidates of one bin that the merge orders in place (more: the list and its rankings)
constexpr uint32_t kSplitRetryLimit = 1u << 16;
static_assert(kSplitMaxSegments * kSegmentValuesBF16 + 8 <= (1 << kSplitIndexBits), "token indices of a split row fit the entry");
static_assert(kSplitHeaderEntries + 2 * kFastTopK + 16 <= kSplitRecordSlots, "a record holds the widest hand-over");

struct SplitSegmentInfo
{
    uint32_t bound;
    uint32_t maximum;
    uint32_t count_and_flags; // bits 0-7 entries handed over, bits 8-10 ScanFlags, bit 31 the header was valid
};

struct SplitShared
{
    SelectShared<false> select;
    uint32_t histogram[kSplitBins];
    alignas(16) uint32_t bin_keys[kSplitBins * kSplitBinCapacity];   // the candidates of a bin, in the order the histogram's atomics placed them
    alignas(16) uint32_t bin_indices[kSplitBins * kSplitBinCapacity];
    uint32_t retry;
    uint32_t segment_maximum;
    uint64_t exp2_table[32];
    int is_last;
};

// A scalar load through the scalar cache, for a word that nobody writes before the caller's last use
// of it in this launch (the cache starts a launch empty).  Every wave of a workgroup, and every workgroup
// of a row, asks for the same word: through the cache that costs next to nothing, around it (glc) seven
// thousand loads of 64 words took 100 us.
__device__ __forceinline__ uint32_t scalar_load_u32(const uint32_t* address)
{
    uint32_t value;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(value) : "s"(address) : "memory");
    return value;
}

// One record entry.  Stores go through to device memory (any workgroup of the row may merge); the first
// read of the merge stops at this XCD's L2 (and goes around the compute unit's vector cache), a repeated
// one goes around the L2 as well.
__device__ __forceinline__ void store_entry(unsigned long long* address, uint32_t key, uint32_t tagged)
{
    __hip_atomic_store(address, static_cast<unsigned long long>(key) | (static_cast<unsigned long long>(tagged) << 32),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ unsigned long long load_entry(const unsigned long long* address, bool around_l2)
{
    return around_l2 ? __hip_atomic_load(address, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                     : __hip_atomic_load(address, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

template <int DTYPE, int SEGMENTS = 16>
__global__ __launch_bounds__(kScanThreads, DTYPE == NCNN_MOE_LOGITS_F32 ? 8 : 4) void split_select_kernel(SamplerArgs a)
{
    static_assert(SEGMENTS == 16 || SEGMENTS == kSplitMaxSegments, "a wave reads the headers of all segments: 2 x 16 or 2 x 32 lanes");
    constexpr int kSplitLanesPerSegment = kScanThreads / SEGMENTS; // lanes that read one segment's record: 32 or 16
    // entries of a record that a lane reads: all 160 of it with 32 lanes a segment; with 16 lanes six each, and a
    // segment hands over at most 94 candidates (a longer list is cut to its exact window first): ten entries a lane
    // would take the merge past the registers that eight waves a SIMD leave it
    constexpr int kSplitSlotsPerLane = SEGMENTS == 16 ? (kSplitRecordSlots + kSplitLanesPerSegment - 1) / kSplitLanesPerSegment : 6;
    constexpr uint32_t kRecordCap = static_cast<uint32_t>(kSplitLanesPerSegment * kSplitSlotsPerLane - kSplitHeaderEntries);
    static_assert(kRecordCap + kSplitHeaderEntries <= kSplitRecordSlots && kRecordCap >= static_cast<uint32_t>(kFastTopK) + 16u, "a record holds a window and its ties");
    constexpr int kSegmentsPerWave = kWaveSize / kSplitLanesPerSegment; // 2 or 4
    using Vector = LogitsVector<DTYPE>;
    constexpr int kWidth = Vector::kWidth;
    constexpr int kVectors = Vector::kVectorsPerLane;
    constexpr int kLaneValues = kVectors * kWidth;
    constexpr uint32_t kChunk = static_cast<uint32_t>(kScanThreads) * kLaneValues;
    constexpr uint32_t kNegativeInfinity = 0xff800000u;
    constexpr uint32_t kPositiveInfinity = 0x7f800000u;

    // Workgroups are handed to the eight XCDs in turn: a grouped grid numbers them so that the segments
    // of a row land on one XCD and the merge finds their records in that XCD's L2.  (Nothing relies on
    // it: a record that is not there fails the epoch check and is read again from device memory.)
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
    const int wave = tid >> 6;

    __shared__ SplitShared shared;
    SelectShared<false>& select = shared.select;

    NCNN_MOE_LSTAMP_DECLARE;
    NCNN_MOE_LSTAMP(0);
    NCNN_MOE_LSTAMP_VALUE(10, static_cast<unsigned long long>(__builtin_amdgcn_s_getreg((31 << 11) | 4)) |
                         (static_cast<unsigned long long>(__builtin_amdgcn_s_getreg(kXccIdRegister)) << 32));
    // The chunk's loads go out before anything that waits for the row's options.
    const char* row_pointer = static_cast<const char*>(a.logits) +
        static_cast<size_t>(row) * a.row_stride * Vector::kElementBytes;
    const uint32_t misalignment =
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row_pointer) & 15u) / Vector::kElementBytes;
    const char* aligned_base = row_pointer - static_cast<size_t>(misalignment) * Vector::kElementBytes;
    const uint32_t valid_begin = misalignment;
    const uint32_t valid_end = misalignment + a.vocab;
    const uint32_t chunk_base = segment * kChunk;
    const uint32_t segment_end = min(valid_end, chunk_base + kChunk);

    // The first workgroup on every XCD touches the small operands of that XCD's rows (options, draw,
    // epoch) before the memory system fills up with the logits: a first access to them
    // by a workgroup that starts a microsecond later queues behind tens of megabytes and takes several
    // microseconds; once they sit in the XCD's L2 it takes a few hundred nanoseconds.
    uint32_t touched = 0;
    if (a.xcd_grouped != 0u && blockIdx.x < 8u)
    {
        const uint32_t other_row = blockIdx.x + 8u * static_cast<uint32_t>(tid);
        if (other_row < a.rows)
        {
            touched = reinterpret_cast<const uint32_t*>(a.params + other_row)[0] ^ reinterpret_cast<const uint32_t*>(a.params + other_row)[5] ^
                __float_as_uint(a.uniforms[other_row]) ^ a.row_epoch[other_row];
        }
    }
    uint4 raw[kVectors];
    load_chunk<DTYPE, kVectors>(raw, aligned_base, chunk_base, valid_begin, segment_end, valid_end, tid);
    NCNN_MOE_LSTAMP(9); // (the loads are on their way)
    const ncnn_moe_sample_params p = a.params[row];
    const float uniform = a.uniforms[row];
    const uint64_t exp2_entry = kExp2Table[tid & 31]; // staged in LDS below: the merge's exponentials find it there
    const uint32_t epoch = scalar_load_u32(&a.row_epoch[row]);
    uint32_t effective_k = 0;
    int status = NCNN_MOE_ROW_OK;
    const int mode = resolve_row_mode(p, a.vocab, kFastTopK, a.force_general, effective_k, status);
    if (mode == kModeInvalid || mode == kModeGeneral)
    {
        // (a row with a window of 65 to 1024 is left alone when a wide select runs beside this kernel)
        const bool not_mine = a.leave_wide_rows != 0 && mode == kModeGeneral && a.force_general == 0 &&
            effective_k <= static_cast<uint32_t>(kSelectTopK);
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
    const uint32_t record_entries = min(segment_record_entries(effective_k), kRecordCap);
    if (tid == 0)
    {
        select.block_flags = 0;
        select.list_count = 0;
        shared.segment_maximum = 0xffffffffu; // unknown unless the bound routine below reports it
        shared.retry = 0;
    }
    if (tid < 32)
        shared.exp2_table[tid] = exp2_entry;
    if (tid >= kScanThreads - kSplitBins)
        shared.histogram[tid - (kScanThreads - kSplitBins)] = 0; // (of the merge, should this workgroup be the row's last)
    if (touched == 0x9e3779b9u)
        select.block_flags = 0; // keeps the touching loads alive; the value is never that
    __syncthreads(); // also waits for the chunk
    NCNN_MOE_LSTAMP(1);
    // The launch ends with its last rows: once their logits are there, their workgroups go first where they
    // share a compute unit's vector units with workgroups of earlier rows (the workgroups of a compute unit
    // come from the four quarters of the grid, one each).  Not before: a wave of lower priority would also
    // issue its loads later.
    {
        const uint32_t quarter = row * 4u / max(a.rows, 1u);
        if (quarter >= 3u)
            __builtin_amdgcn_s_setprio(3);
        else if (quarter == 2u)
            __builtin_amdgcn_s_setprio(2);
        else if (quarter == 1u)
            __builtin_amdgcn_s_setprio(1);
    }

    // ---- the chunk: maxima, flags.  Nearly every chunk lies inside the row (only a row's last chunk, or
    // the first one of a row that does not start on a 16-byte boundary, holds foreign elements): those skip
    // the masking, a few hundred instructions per wave that four workgroups per compute unit would
    // otherwise all issue at the moment their logits arrive.
    float values[kLaneValues];
    float lane_max = __uint_as_float(kNegativeInfinity);
    bool saw_nan = false;
    const bool interior = chunk_base >= valid_begin && chunk_base + kChunk <= segment_end; // the same in every thread
    if (interior)
    {
#pragma unroll
        for (int v = 0; v < kVectors; ++v)
            Vector::unpack(raw[v], &values[v * kWidth]);
#pragma unroll
        for (int i = 0; i < kLaneValues; i += 2)
        {
            saw_nan = saw_nan || __builtin_isunordered(values[i], values[i + 1]);
            lane_max = fmaxf(lane_max, fmaxf(values[i], values[i + 1]));
        }
    }
    else
    {
#pragma unroll
        for (int v = 0; v < kVectors; ++v)
        {
            const uint32_t first = chunk_base + static_cast<uint32_t>(v * kScanThreads + tid) * kWidth;
            const bool any_valid = first < segment_end && first + kWidth > valid_begin;
            if (any_valid)
                Vector::unpack(raw[v], &values[v * kWidth]);
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
#pragma unroll
            for (int c = 0; c < kWidth; ++c)
            {
                const float x = values[v * kWidth + c];
                saw_nan = saw_nan || (x != x);
                lane_max = fmaxf(lane_max, x);
            }
        }
    }
    uint32_t local_flags = saw_nan ? kScanSawNan : 0u;
    if (__ballot(lane_max == __uint_as_float(kPositiveInfinity)) != 0)
    {
        local_flags |= lane_max == __uint_as_float(kPositiveInfinity) ? kScanSawPositiveInfinity : 0u;
        if (greedy)
        {
            // greedy skips every non-finite logit (session.cpp:411-412): rare, so redone out of line
            lane_max = __uint_as_float(kNegativeInfinity);
#pragma unroll
            for (int i = 0; i < kLaneValues; ++i)
            {
                if (values[i] == __uint_as_float(kPositiveInfinity))
                    values[i] = __uint_as_float(kNegativeInfinity);
                lane_max = fmaxf(lane_max, values[i]);
            }
        }
    }

    // ---- bound: at least K logits of the chunk reach it, so the row's K-th best is no smaller
    const uint32_t lane_keys[1] = {lane_max == __uint_as_float(kNegativeInfinity) ? 0u : ascending_key(lane_max)};
    uint32_t bound_key = workgroup_kth_of_quad_maxima(lane_keys[0], top_k, tid, select.bound, &shared.segment_maximum);
    if (bound_key == 0u) // a chunk with few values: the exact K-th largest lane maximum
        bound_key = workgroup_kth_largest_key(lane_keys, top_k, tid, select.bound, true);
    NCNN_MOE_LSTAMP(2);
    // no bound (fewer than K lanes hold a finite logit): every finite logit is a candidate
    const float threshold = bound_key == 0u ? -3.402823466e+38f : fmaxf(value_from_ascending_key(bound_key), -3.402823466e+38f);

    // ---- collect the values at or above the bound.  Nearly every lane that holds a candidate holds
    // exactly one, its maximum: each lane counts its candidates and locates its maximum without a branch,
    // one append per wave takes the maxima, and the lanes that hold more hand the others over one per
    // round.  (A compare, a ballot and a branch per slot costs a wave twice as much: each is a trip from
    // the vector to the scalar unit.)
    int lane_hits = 0;
    int best_at = 0;
#pragma unroll
    for (int i = 0; i < kLaneValues; ++i)
    {
        lane_hits += values[i] >= threshold ? 1 : 0;
        best_at = values[i] == lane_max ? i : best_at;
    }
    const auto element_of = [&](int i) {
        return static_cast<int32_t>(chunk_base + static_cast<uint32_t>((i / kWidth) * kScanThreads + tid) * kWidth +
                                    static_cast<uint32_t>(i % kWidth) - misalignment);
    };
    append_candidate(select, lane_hits >= 1, ascending_key(lane_max), element_of(best_at), lane);
    if (__ballot(lane_hits > 1) != 0)
    {
        uint32_t rest = 0; // bit i: value i is a candidate that has not been appended
#pragma unroll
        for (int i = 0; i < kLaneValues; ++i)
            rest |= (lane_hits > 1 && values[i] >= threshold && i != best_at) ? (1u << i) : 0u;
        while (__ballot(rest != 0u) != 0)
        {
            // the value is read back from the row (its register is not known until run time; picking it out of
            // the registers, by selects or by handing the lane's values to the wave's other lanes, was no faster)
            const int i = rest != 0u ? __builtin_ctz(rest) : 0;
            const int32_t element = element_of(i);
            float x = 0.0f;
            if (rest != 0u)
            {
                if constexpr (DTYPE == NCNN_MOE_LOGITS_F32)
                    x = reinterpret_cast<const float*>(row_pointer)[element];
                else
                    x = __uint_as_float(static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(row_pointer)[element]) << 16);
            }
            append_candidate(select, rest != 0u, ascending_key(x), element, lane);
            rest &= rest - 1u;
        }
    }
    if (local_flags != 0)
        atomicOr(&select.block_flags, local_flags);
    __syncthreads();
    NCNN_MOE_LSTAMP(3);
    bool overflow = select.list_count > static_cast<uint32_t>(kNarrowListCap);
    // the record holds 2K + 16 candidates: a longer list (a loose bound, ties) is cut to the exact window first
    if (!overflow && select.list_count > record_entries)
        bound_key = tighten_list(select, bound_key, top_k, tid);
    const uint32_t handed = select.list_count;
    overflow = overflow || handed > record_entries;
    const uint32_t segment_flags = select.block_flags | (overflow ? static_cast<uint32_t>(kScanOverflow) : 0u);
    const uint32_t own_count = overflow ? 0u : handed;

    // ---- hand-over: the entries go out, nothing waits for them
    unsigned long long* const row_records = a.split_records + static_cast<size_t>(row) * kSplitMaxSegments * kSplitRecordSlots;
    unsigned long long* const own_record = row_records + static_cast<size_t>(segment) * kSplitRecordSlots;
    const uint32_t tag = epoch << kSplitIndexBits;
    for (uint32_t j = tid; j < own_count; j += kScanThreads)
        store_entry(&own_record[kSplitHeaderEntries + j], select.list_keys[j], tag | static_cast<uint32_t>(select.list_indices[j]));
    if (tid == 0)
    {
        store_entry(&own_record[0], bound_key, tag | own_count | (segment_flags << 8));
        store_entry(&own_record[1], shared.segment_maximum, tag);
    }
    // How the row's last workgroup reads the records: lanes 32 h .. 32 h + 31 of wave w read the record of
    // segment 2 w + h, entry by entry (consecutive lanes, consecutive entries); the workgroup's own list
    // stays in LDS.  (Issuing these loads before the counter's atomic, so that they travel beside it, does
    // not pay: two times out of three an entry of a workgroup that counted itself a moment earlier has
    // not landed yet, and the second trip costs more than the first saved.)
    const uint32_t read_segment = static_cast<uint32_t>(kSegmentsPerWave * wave + lane / kSplitLanesPerSegment);
    const int read_lane = lane & (kSplitLanesPerSegment - 1);
    const uint32_t entries_to_read = static_cast<uint32_t>(kSplitHeaderEntries) + record_entries;
    const unsigned long long* const read_record = row_records + static_cast<size_t>(read_segment) * kSplitRecordSlots;
    const bool reads_own = read_segment == segment;
    const bool reads_any = read_segment < a.segments && !reads_own;
    unsigned long long loaded[kSplitSlotsPerLane];
    const auto load_records = [&](bool around_l2) {
#pragma unroll
        for (int j = 0; j < kSplitSlotsPerLane; ++j)
        {
            const uint32_t entry = static_cast<uint32_t>(j * kSplitLanesPerSegment + read_lane);
            if (!reads_own) // the lanes that stand for this workgroup's own segment keep what they took from its list
                loaded[j] = 0ull;
            if (reads_any && entry < entries_to_read)
                loaded[j] = load_entry(&read_record[entry], around_l2);
        }
    };
    // The last wave counts the workgroup in (its lanes stored nothing unless the list is very long, so
    // the atomic's return does not queue behind a store's acknowledgement).
    if (tid == kScanThreads - kWaveSize)
    {
        const unsigned long long previous = __hip_atomic_fetch_add(&a.row_counter[row], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        shared.is_last = previous == a.segments - 1 ? 1 : 0;
    }
    lds_barrier();
    NCNN_MOE_LSTAMP(4);
    if (!shared.is_last)
    {
        NCNN_MOE_LSTAMP_FLUSH(row, segment, 0, 4);
        NCNN_MOE_LSTAMP_FLUSH(row, segment, 9, 14);
        return;
    }

    // ---- last workgroup of the row.  The row's next launch gets a new epoch whatever happens below.
    if (tid == 0)
    {
        a.row_counter[row] = 0;
        store_agent(&a.row_epoch[row], epoch == kSplitLastEpoch ? 1u : epoch + 1u);
    }
    // this workgroup's own candidates, from its list (entry numbering as in a record)
    if (reads_own)
    {
#pragma unroll
        for (int j = 0; j < kSplitSlotsPerLane; ++j)
        {
            const uint32_t entry = static_cast<uint32_t>(j * kSplitLanesPerSegment + read_lane);
            loaded[j] = 0ull;
            if (entry >= static_cast<uint32_t>(kSplitHeaderEntries) && entry - kSplitHeaderEntries < own_count)
            {
                const uint32_t q = entry - kSplitHeaderEntries;
                loaded[j] = static_cast<unsigned long long>(select.list_keys[q]) |
                    (static_cast<unsigned long long>(tag | static_cast<uint32_t>(select.list_indices[q])) << 32);
            }
        }
    }
    // Every wave reads the headers of all the row's segments for itself (lane s the first entry of segment s,
    // lane 16 + s the second): the row's bound, maximum and flags then come from exchanges inside the wave,
    // without a trip through LDS and a barrier behind the records' arrival.
    const uint32_t header_segment = static_cast<uint32_t>(lane & (SEGMENTS - 1));
    const bool header_lane = lane < 2 * SEGMENTS && header_segment < a.segments;
    const bool own_header = header_segment == segment;
    const unsigned long long* const header_address =
        row_records + static_cast<size_t>(header_segment) * kSplitRecordSlots + (lane >= SEGMENTS ? 1 : 0);
    unsigned long long header = 0ull;
    const auto load_headers = [&](bool around_l2) {
        if (header_lane && !own_header)
            header = load_entry(header_address, around_l2);
    };
    load_headers(false);
    load_records(false);
    uint32_t lower = 0, upper = 0, row_flags = 0;
    uint32_t my_count = 0;
    uint32_t attempts = 0;
    int bins[kSplitSlotsPerLane];
    uint32_t bin_counts = 0;
    for (uint32_t attempt = 0;; ++attempt)
    {
        attempts = attempt + 1u;
        uint32_t word = static_cast<uint32_t>(header);
        uint32_t tag_word = static_cast<uint32_t>(header >> 32);
        if (lane < 2 * SEGMENTS && own_header)
        {
            word = lane < SEGMENTS ? bound_key : shared.segment_maximum;
            tag_word = lane < SEGMENTS ? (tag | own_count | (segment_flags << 8)) : tag;
        }
        bool valid = !header_lane || (tag_word >> kSplitIndexBits) == epoch;
        // rows of 16 lanes: the first (two, of 32 segments) hold the segments' bounds, counts and flags, the next their maxima
        const auto larger = [](uint32_t x, uint32_t y) { return max(x, y); };
        const uint32_t extremes = row16_reduce_u32(header_lane ? word : 0u, larger);
        const uint32_t flag_bits = row16_reduce_u32((header_lane && lane < SEGMENTS) ? ((tag_word >> 8) & 7u) : 0u,
                                                    [](uint32_t x, uint32_t y) { return x | y; });
        lower = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(extremes), 0));
        upper = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(extremes), SEGMENTS));
        row_flags = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(flag_bits), 0));
        if (SEGMENTS == 32)
        {
            lower = max(lower, static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(extremes), 16)));
            upper = max(upper, static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(extremes), 48)));
            row_flags |= static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(flag_bits), 16));
        }
        // the count of the segment whose record this lane reads: lane s of the first rows holds segment s's
        const uint32_t count_word = (header_lane && lane < SEGMENTS) ? (tag_word & 0xffu) : 0u;
        my_count = 0;
#pragma unroll
        for (int g = 0; g < kSegmentsPerWave; ++g)
        {
            const uint32_t count_there = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(count_word), kSegmentsPerWave * wave + g));
            my_count = lane / kSplitLanesPerSegment == g ? count_there : my_count;
        }
        if (reads_any)
        {
#pragma unroll
            for (int j = 0; j < kSplitSlotsPerLane; ++j)
            {
                const uint32_t entry = static_cast<uint32_t>(j * kSplitLanesPerSegment + read_lane);
                if (entry >= static_cast<uint32_t>(kSplitHeaderEntries) && entry - kSplitHeaderEntries < my_count)
                    valid = valid && (static_cast<uint32_t>(loaded[j] >> 32) >> kSplitIndexBits) == epoch;
            }
        }
        if (__ballot(!valid) != 0ull && lane == 0)
            shared.retry = 1; // something of this launch has not landed yet (or the L2 held a stale line)

        // ---- cut and order in one pass: a histogram of the candidates at or above the largest segment
        // bound (at least K logits of that segment reach it, so nothing below it is in the window) over
        // [that bound, row maximum], bin 0 at the top.  The atomic that counts a candidate also gives it a
        // place in its bin's short list; behind the barrier a scan over the bins tells every candidate how
        // many lie in the bins above its own, its bin's list how many of its own bin go before it: that is its
        // place in the window.
        const uint32_t span = upper >= lower ? upper - lower : 0u;
        const float scale = static_cast<float>(kSplitBins) / (static_cast<float>(span) + 1.0f);
#pragma unroll
        for (int j = 0; j < kSplitSlotsPerLane; ++j)
        {
            bins[j] = -1;
            if (static_cast<uint32_t>(j * kSplitLanesPerSegment) >= entries_to_read)
                continue; // no entry of this or a later round exists (a scalar test)
            const uint32_t entry = static_cast<uint32_t>(j * kSplitLanesPerSegment + read_lane);
            const uint32_t key = static_cast<uint32_t>(loaded[j]);
            const bool candidate = entry >= static_cast<uint32_t>(kSplitHeaderEntries) && entry - kSplitHeaderEntries < my_count && key >= lower;
            if (candidate)
            {
                const uint32_t distance = min(key, upper) - lower;
                const int from_bottom = min(kSplitBins - 1, static_cast<int>(static_cast<float>(distance) * scale));
                bins[j] = kSplitBins - 1 - from_bottom;
                const uint32_t place = atomicAdd(&shared.histogram[bins[j]], 1u);
                if (place < static_cast<uint32_t>(kSplitBinCapacity))
                {
                    shared.bin_keys[bins[j] * kSplitBinCapacity + place] = key;
                    shared.bin_indices[bins[j] * kSplitBinCapacity + place] = static_cast<uint32_t>(loaded[j] >> 32) & kSplitIndexMask;
                }
            }
        }
        lds_barrier();
        bin_counts = shared.histogram[lane];
        if (shared.retry == 0)
            break;
        // An entry of this launch has not landed yet: read the records again from device memory.  The
        // stores in question were issued before their workgroup counted itself, so they land without
        // anyone else having to run.
        lds_barrier(); // every wave has read the flag and its bins before they are cleared
        if (tid < kSplitBins)
            shared.histogram[tid] = 0;
        if (tid == 0)
            shared.retry = 0;
        if (attempt >= kSplitRetryLimit)
            break;
        load_headers(true);
        load_records(true);
        lds_barrier();
    }
    if (epoch == kSplitLastEpoch)
    {
        // the epochs start over: nothing that the old ones tagged may be left (the records are read)
        for (uint32_t j = tid; j < static_cast<uint32_t>(kSplitMaxSegments * kSplitRecordSlots); j += kScanThreads)
            store_entry(&row_records[j], 0u, 0u);
    }
    NCNN_MOE_LSTAMP(5);
    NCNN_MOE_LSTAMP_VALUE(8, attempts);
    const uint8_t result_flags = (row_flags & kScanSawNan) ? NCNN_MOE_ROW_FLAG_HAS_NAN : 0;
    if (attempts > kSplitRetryLimit || (row_flags & kScanOverflow))
    {
        // entries that never landed, or ties (or values that defeat the bound) that left more candidates than a
        // record holds: the full-order kernels take the row
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

    // The first bin at which the count from the top reaches K ends the selection.
    const uint32_t from_top = wave_prefix_sum_u32(bin_counts);
    const uint64_t reached = __ballot(from_top >= static_cast<uint32_t>(top_k));
    const int cut = reached != 0 ? __builtin_ctzll(reached) : kSplitBins - 1;
    const uint32_t selected = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(from_top), cut));
    const uint32_t fullest = wave_max_u32(lane <= cut ? bin_counts : 0u); // of the bins that hold the window
    if (fullest <= static_cast<uint32_t>(kSplitBinCapacity))
    {
        // (above, bin count) of every bin in one word, fetched by the candidates of that bin
        const uint32_t packed = ((from_top - bin_counts) << 16) | bin_counts;
#pragma unroll
        for (int j = 0; j < kSplitSlotsPerLane; ++j)
        {
            if (static_cast<uint32_t>(j * kSplitLanesPerSegment) >= entries_to_read)
                break;
            const int bin = bins[j] >= 0 ? bins[j] : 0;
            const uint32_t of_bin = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(bin << 2, static_cast<int>(packed)));
            if (bins[j] >= 0 && bins[j] <= cut)
            {
                const uint32_t key = static_cast<uint32_t>(loaded[j]);
                const uint32_t index = static_cast<uint32_t>(loaded[j] >> 32) & kSplitIndexMask;
                const uint32_t in_bin = of_bin & 0xffffu;
                uint32_t before = of_bin >> 16;
                for (uint32_t first = 0; first < fullest; first += 4u) // (fullest is the same in every lane)
                {
                    const uint4 other_keys = *reinterpret_cast<const uint4*>(&shared.bin_keys[bin * kSplitBinCapacity + first]);
                    const uint4 other_indices = *reinterpret_cast<const uint4*>(&shared.bin_indices[bin * kSplitBinCapacity + first]);
                    before += (first + 0u < in_bin && (other_keys.x > key || (other_keys.x == key && other_indices.x < index))) ? 1u : 0u;
                    before += (first + 1u < in_bin && (other_keys.y > key || (other_keys.y == key && other_indices.y < index))) ? 1u : 0u;
                    before += (first + 2u < in_bin && (other_keys.z > key || (other_keys.z == key && other_indices.z < index))) ? 1u : 0u;
                    before += (first + 3u < in_bin && (other_keys.w > key || (other_keys.w == key && other_indices.w < index))) ? 1u : 0u;
                }
                if (before < static_cast<uint32_t>(top_k))
                {
                    select.final_values[before] = value_from_ascending_key(key);
                    select.final_indices[before] = static_cast<int32_t>(index);
                }
            }
        }
        lds_barrier();
        NCNN_MOE_LSTAMP(6);
        if (wave == 0)
        {
            const int n = static_cast<int>(min(selected, static_cast<uint32_t>(top_k)));
            if (lane == 0)
                a.row_state[row] = kRowDone;
            if (n == 0)
            {
                if (lane == 0)
                    write_error(a, row, NCNN_MOE_ROW_NO_FINITE_LOGIT, result_flags);
            }
            else
            {
                const float value = lane < n ? select.final_values[lane] : 0.0f;
                const int32_t index = lane < n ? select.final_indices[lane] : -1;
                finish_ordered_wave(a, row, p, greedy, value, index, n, lane, result_flags, uniform, shared.exp2_table);
            }
        }
        NCNN_MOE_LSTAMP(7);
        NCNN_MOE_LSTAMP_FLUSH(row, segment, 0, 14);
        return;
    }
    // A bin of the window holds more candidates than its list (ties, or a window that is most of its range's
    // lower end): the candidates above the cut go to the list and are ranked from there.
    if (selected > static_cast<uint32_t>(kNarrowListCap))
    {
        if (tid == 0)
        {
            write_pending(a, row);
            a.row_state[row] = kRowNeedsGeneral;
        }
        return;
    }
    if (tid == 0)
        select.list_count = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kSplitSlotsPerLane; ++j)
    {
        if (static_cast<uint32_t>(j * kSplitLanesPerSegment) >= entries_to_read)
            break; // no entry of this or a later round exists (a scalar test)
        append_candidate(select, bins[j] >= 0 && bins[j] <= cut, static_cast<uint32_t>(loaded[j]),
                         static_cast<int32_t>(static_cast<uint32_t>(loaded[j] >> 32) & kSplitIndexMask), lane);
    }
    __syncthreads();
    NCNN_MOE_LSTAMP(6);
    finish_from_list(a, row, p, greedy, top_k, select, result_flags, tid, uniform, shared.exp2_table);
    NCNN_MOE_LSTAMP(7);
    NCNN_MOE_LSTAMP_FLUSH(row, segment, 0, 14);
}

#ifdef NCNN_MOE_TESTING
// The split kernel's grid and loads with nothing behind them: every workgroup reads its chunk and one lane
// per wave stores a word that depends on all of it.  What a launch of this shape costs for streaming the
// logits alone (a probe for the benchmark's detail, not part of the sampling path; in the testing build only).
template <int DTYPE>
__global__ __launch_bounds__(kScanThreads, DTYPE == NCNN_MOE_LOGITS_F32 ? 8 : 4) void split_stream_only_kernel(SamplerArgs a, uint32_t* sink)
{
    using Vector = LogitsVector<DTYPE>;
    constexpr int kVectors = Vector::kVectorsPerLane;
    constexpr uint32_t kChunk = static_cast<uint32_t>(kScanThreads) * kVectors * Vector::kWidth;
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
    const char* row_pointer = static_cast<const char*>(a.logits) +
        static_cast<size_t>(row) * a.row_stride * Vector::kElementBytes;
    const uint32_t misalignment =
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row_pointer) & 15u) / Vector::kElementBytes;
    const char* aligned_base = row_pointer - static_cast<size_t>(misalignment) * Vector::kElementBytes;
    const uint32_t valid_end = misalignment + a.vocab;
    const uint32_t chunk_base = segment * kChunk;
    uint4 raw[kVectors];
    load_chunk<DTYPE, kVectors>(raw, aligned_base, chunk_base, misalignment, min(valid_end, chunk_base + kChunk), valid_end, tid);
    uint32_t folded = 0;
#pragma unroll
    for (int v = 0; v < kVectors; ++v)
        folded ^= raw[v].x ^ raw[v].y ^ raw[v].z ^ raw[v].w;
    folded = wave_max_u32(folded);
    if ((tid & (kWaveSize - 1)) == 0)
        sink[(static_cast<size_t>(row) * a.segments + segment) * kScanWaves + (tid >> 6)] = folded;
}
#endif // NCNN_MOE_TESTING

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_SAMPLER_SPLIT_H
