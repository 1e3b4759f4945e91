// Device-side building blocks of the gfx950 generation sampler: row-mode resolution, the
// exponential that reproduces libm expf bit for bit, order-preserving sort keys and wave64 helpers.
#ifndef NCNN_MOE_HIP_SAMPLER_DEVICE_H
#define NCNN_MOE_HIP_SAMPLER_DEVICE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ncnn_moe_hip_sampler.h"

namespace ncnn_moe_hip {

constexpr int kWaveSize = 64;

// Top-K select ("fast") path geometry: a workgroup of 512 threads (8 waves) owns a segment of
// consecutive logits, a few 16-byte vectors per lane (5 fp32 vectors = 20 logits, 3 bf16 vectors =
// 24 logits) times the chunk count.  Few loads per lane and many waves per CU stream fastest.
constexpr int kScanThreads = 512;
constexpr int kScanWaves = kScanThreads / kWaveSize;
constexpr int kVectorsPerLaneF32 = 5;
constexpr int kVectorsPerLaneBF16 = 3;
constexpr int kSegmentValuesF32 = kScanThreads * kVectorsPerLaneF32 * 4;   // 10240 logits per chunk
constexpr int kSegmentValuesBF16 = kScanThreads * kVectorsPerLaneBF16 * 8; // 12288 logits per chunk
constexpr int kFastTopK = 64;            // widest Top-K window finished by one wave
constexpr int kSelectTopK = 1024;
constexpr int kTwoKeyBoundTopK = 512; // wider windows bound their first chunk by a select over all its values         // widest Top-K window of the select path (rows of one segment)
// s_getreg operand of the XCC_ID hardware register (id 20, offset 0, 4 bits): the XCD a wave runs on
constexpr int kXccIdRegister = ((4 - 1) << 11) | (0 << 6) | 20;
constexpr int kNarrowListCap = 512;      // candidate list for Top-K windows up to kFastTopK
constexpr int kWideListCap = 4096;       // candidate list for Top-K windows up to kSelectTopK
constexpr int kSegmentRecordSlots = 256; // candidate slots of a segment's record in HBM
constexpr int kMaxSegments = 16;
constexpr int kSplitMaxSegments = 32;   // ... of one chunk each, on the split path
constexpr int kSplitRecordSlots = 160;   // 8-byte entries of a segment's record on the split path: 2 header entries + up to 2 * 64 + 16 candidates
constexpr int kWholeRowBatch = 256;          // from this many rows on, one workgroup streams a whole row
constexpr int kSingleChunkWorkgroups = 8192;  // a smaller batch is split into one-chunk workgroups up to this many (several rounds of 4 per CU beat fewer, looped ones)
constexpr int kLoopedWorkgroups = 512;        // ... and when each streams several chunks (2 per CU)
         // segments per row the row merge can stage in one trip
constexpr int kMergeStageSlots = 4096;   // record slots of a row loaded in one trip (8 per thread)

// Full-order ("general") path geometry.
constexpr int kSortThreads = 1024;
constexpr int kSortWaves = kSortThreads / kWaveSize;
constexpr int kSortPerThread = 8;
constexpr int kSortTile = kSortThreads * kSortPerThread;
constexpr int kMaxSortParts = 16;             // workgroups one row's radix sort is spread over
constexpr int kReplayThreads = 1024;
// The exact running sums are the work of the workgroup's first eight waves (two per SIMD), each thread
// composing a few consecutive terms: every wave that takes part pays the scan across its lanes and the
// composition of the waves' totals again, and a thread's terms are a chain of dependent instructions.
// Measured on full-order batches.  Rows of single elements (configuration 4): sixteen waves x 4 terms 964 us,
// eight x 8 931, eight x 4 967, four x 16 976, sixteen x 8 939.  Rows of runs (configuration 3): eight waves
// x 2 runs 120.4 us, eight x 3 120.5, eight x 1 122, four x 2 121.7, four x 4 123, eight x 4 123.9,
// sixteen x 2 126, sixteen x 4 129, four x 8 137: short chunks lose nothing, because a sum that stops
// early (Top-P, the draw) stops a chunk sooner.
constexpr int kSumWaves = 8;
constexpr int kSumThreads = kSumWaves * 64;
constexpr int kReplayPerThread = 8;
constexpr int kRunsWaves = 8;
constexpr int kRunsPerThread = 2;
constexpr int kRunsChunk = kRunsWaves * 64 * kRunsPerThread;
constexpr int kReplayChunk = kSumThreads * kReplayPerThread;

// Wall-clock stamps for a timeline of the split path, compiled in only with -DNCNN_MOE_TIMELINE (a
// separate library, built by `make timeline`; the shipped one carries none).
#ifdef NCNN_MOE_TIMELINE
constexpr int kTimelineRows = 64;
constexpr int kTimelineSlots = 16;
__device__ unsigned long long g_timeline[kTimelineRows * kMaxSegments * kTimelineSlots];
#define NCNN_MOE_STAMP(row, segment, slot)                                                                   \
    do                                                                                                       \
    {                                                                                                        \
        if (threadIdx.x == 0 && (row) < static_cast<uint32_t>(kTimelineRows))                                \
            g_timeline[((row) * kMaxSegments + (segment)) * kTimelineSlots + (slot)] = wall_clock64();       \
    } while (0)
#define NCNN_MOE_STAMP_VALUE(row, segment, slot, value)                                                     \
    do                                                                                                       \
    {                                                                                                        \
        if (threadIdx.x == 0 && (row) < static_cast<uint32_t>(kTimelineRows))                                \
            g_timeline[((row) * kMaxSegments + (segment)) * kTimelineSlots + (slot)] = (value);              \
    } while (0)
// stamps of the row's last workgroup, from code that does not know its segment; the calling lane is that wave's first
__device__ unsigned long long g_timeline_rows[kTimelineRows * kTimelineSlots];
#define NCNN_MOE_STAMP_ROW(row, slot)                                                                        \
    do                                                                                                       \
    {                                                                                                        \
        if ((threadIdx.x & 63) == 0 && (row) < static_cast<uint32_t>(kTimelineRows))                         \
            g_timeline_rows[(row) * kTimelineSlots + (slot)] = wall_clock64();                               \
    } while (0)
// successive stamps of one code path: slot numbers from a counter kept in g_timeline[..][15]
#define NCNN_MOE_STAMP_NEXT(row, segment)                                                                    \
    do                                                                                                       \
    {                                                                                                        \
        if (threadIdx.x == 0 && (row) < static_cast<uint32_t>(kTimelineRows))                                \
        {                                                                                                    \
            unsigned long long* base_ = g_timeline + ((row) * kMaxSegments + (segment)) * kTimelineSlots;    \
            const unsigned long long slot_ = base_[15];                                                      \
            if (slot_ < 15)                                                                                  \
            {                                                                                                \
                base_[slot_] = wall_clock64();                                                               \
                base_[15] = slot_ + 1;                                                                       \
            }                                                                                                \
        }                                                                                                    \
    } while (0)
#define NCNN_MOE_STAMP_RESET(row, segment) NCNN_MOE_STAMP_VALUE(row, segment, 15, 0ull)
// events counted rather than timed (the reader takes differences between launches)
#define NCNN_MOE_COUNT(row, segment, slot)                                                                   \
    do                                                                                                       \
    {                                                                                                        \
        if (threadIdx.x == 0 && (row) < static_cast<uint32_t>(kTimelineRows))                                \
            g_timeline[((row) * kMaxSegments + (segment)) * kTimelineSlots + (slot)] += 1;                   \
    } while (0)
#define NCNN_MOE_STAMP_VALUE_FROM(leader, row, segment, slot, value)                                        \
    do                                                                                                       \
    {                                                                                                        \
        if ((leader) && (row) < static_cast<uint32_t>(kTimelineRows))                                        \
            g_timeline[((row) * kMaxSegments + (segment)) * kTimelineSlots + (slot)] = (value);              \
    } while (0)
// Stamps of the split kernel are kept in LDS while the workgroup runs and written out when it leaves: a
// store to device memory in the middle of the kernel would be waited for by the next full barrier.
#define NCNN_MOE_LSTAMP_DECLARE __shared__ unsigned long long timeline_staging[kTimelineSlots]
#define NCNN_MOE_LSTAMP(slot)                                                                                \
    do                                                                                                       \
    {                                                                                                        \
        if (threadIdx.x == 0)                                                                                \
            timeline_staging[slot] = wall_clock64();                                                         \
    } while (0)
#define NCNN_MOE_LSTAMP_VALUE(slot, value)                                                                   \
    do                                                                                                       \
    {                                                                                                        \
        if (threadIdx.x == 0)                                                                                \
            timeline_staging[slot] = (value);                                                                \
    } while (0)
#define NCNN_MOE_LSTAMP_FLUSH(row, segment, first, last)                                                     \
    do                                                                                                       \
    {                                                                                                        \
        if (threadIdx.x == 0 && (row) < static_cast<uint32_t>(kTimelineRows) && (segment) < static_cast<uint32_t>(kMaxSegments)) \
        {                                                                                                    \
            for (int slot_ = (first); slot_ <= (last); ++slot_)                                              \
                g_timeline[((row) * kMaxSegments + (segment)) * kTimelineSlots + slot_] = timeline_staging[slot_]; \
        }                                                                                                    \
    } while (0)
#else
#define NCNN_MOE_LSTAMP_DECLARE ((void)0)
#define NCNN_MOE_LSTAMP(slot) ((void)0)
#define NCNN_MOE_LSTAMP_VALUE(slot, value) ((void)0)
#define NCNN_MOE_LSTAMP_FLUSH(row, segment, first, last) ((void)0)
#define NCNN_MOE_STAMP_VALUE_FROM(leader, row, segment, slot, value) ((void)0)
#define NCNN_MOE_STAMP_ROW(row, slot) ((void)0)
#define NCNN_MOE_COUNT(row, segment, slot) ((void)0)
#define NCNN_MOE_STAMP_NEXT(row, segment) ((void)0)
#define NCNN_MOE_STAMP_RESET(row, segment) ((void)0)
#define NCNN_MOE_STAMP(row, segment, slot) ((void)0)
#define NCNN_MOE_STAMP_VALUE(row, segment, slot, value) ((void)0)
#endif

enum RowMode : int
{
    kModeInvalid = 0,
    kModeGreedy = 1,
    kModeTopK = 2,
    kModeGeneral = 3
};

enum RowState : uint32_t
{
    kRowDone = 0,
    kRowNeedsGeneral = 1
};

// Bits accumulated per row while its segments are scanned.
enum ScanFlags : uint32_t
{
    kScanSawNan = 1u,
    kScanSawPositiveInfinity = 2u,
    kScanOverflow = 4u
};

__host__ __device__ __forceinline__ bool is_finite_f32(float value)
{
    union
    {
        float f;
        uint32_t u;
    } bits;
    bits.f = value;
    return (bits.u & 0x7f800000u) != 0x7f800000u;
}

// validate_sampling_options, src/engine/session.cpp:65-74 of the reference.
__host__ __device__ __forceinline__ int validate_params(const ncnn_moe_sample_params& p)
{
    if (!is_finite_f32(p.temperature) || p.temperature < 0.0f)
        return NCNN_MOE_ROW_BAD_TEMPERATURE;
    if (!is_finite_f32(p.top_p) || p.top_p <= 0.0f || p.top_p > 1.0f)
        return NCNN_MOE_ROW_BAD_TOP_P;
    if (!is_finite_f32(p.min_p) || p.min_p < 0.0f || p.min_p > 1.0f)
        return NCNN_MOE_ROW_BAD_MIN_P;
    return NCNN_MOE_ROW_OK;
}

// Which path serves the row.  effective_k is the length of the Top-K window (vocab when Top-K is off,
// session.cpp:86-87), 1 for greedy.  max_select_top_k is the widest window the launch's select kernel
// handles: kFastTopK when rows are split into segments, kSelectTopK when a workgroup sees a whole row.
__host__ __device__ __forceinline__ int resolve_row_mode(
    const ncnn_moe_sample_params& p, uint32_t vocab, uint32_t max_select_top_k, int force_general,
    uint32_t& effective_k, int& status)
{
    status = validate_params(p);
    effective_k = 0;
    if (status != NCNN_MOE_ROW_OK)
        return kModeInvalid;
    if (p.temperature == 0.0f)
    {
        effective_k = 1;
        return kModeGreedy;
    }
    effective_k = (p.top_k == 0u || p.top_k >= vocab) ? vocab : p.top_k;
    if (!force_general && effective_k <= max_select_top_k)
        return kModeTopK;
    return kModeGeneral;
}

// Entries of a segment's record that the row merge reads: twice the Top-K window plus 16 (a segment
// hands over K candidates and a few more; ties beyond that overflow to the full-order path).
__host__ __device__ __forceinline__ uint32_t segment_record_entries(uint32_t effective_k)
{
    const uint32_t entries = effective_k * 2u + 16u;
    return entries > static_cast<uint32_t>(kSegmentRecordSlots) ? static_cast<uint32_t>(kSegmentRecordSlots) : entries;
}

// 2^(i/32) as double bits with i << 47 subtracted, i = 0..31 (correctly rounded).
#define NCNN_MOE_EXP2_TABLE_VALUES \
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull, \
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull, \
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull, \
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull, \
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull, \
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull, \
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull, \
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull,

__device__ __constant__ const uint64_t kExp2Table[32] = {NCNN_MOE_EXP2_TABLE_VALUES};

// expf with the results of glibc 2.35 expf on x86-64 with FMA (the CPU sampler's std::exp,
// src/engine/session.cpp:98): x * 32/ln2 = k + r, exp(x) = 2^(k/32) * (1 + c2 r + c1 r^2 + c0 r^3),
// all in double, one rounding to float at the end.  The reduction uses fma(32/ln2, x, -k), as the
// FMA build of that routine does; the polynomial rounds identically with or without fused steps.
// table: the 32 entries of kExp2Table, in constant memory or a copy of them in LDS (a caller on a
// latency-critical path stages it there while it waits for something else).
__device__ __forceinline__ float expf_libm(float x, const uint64_t* table = kExp2Table)
{
    const uint32_t bits = __float_as_uint(x);
    const uint32_t abstop = (bits >> 20) & 0x7ffu;
    if (abstop >= 0x42bu) // |x| >= 88 or not finite
    {
        if (bits == 0xff800000u)
            return 0.0f;
        if (abstop >= 0x7f8u)
            return x + x;
        if (x > 0x1.62e42ep6f)
            return __uint_as_float(0x7f800000u);
        if (x < -0x1.9fe368p6f)
            return 0.0f;
    }
    const double inverse_ln2_scaled = 0x1.71547652b82fep+0 * 32.0;
    const double shift = 0x1.8p+52;
    const double c0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
    const double c1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
    const double c2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    const double xd = static_cast<double>(x);
    const double z = inverse_ln2_scaled * xd;
    double kd = z + shift;
    const uint64_t ki = static_cast<uint64_t>(__double_as_longlong(kd));
    kd -= shift;
    const double r = fma(inverse_ln2_scaled, xd, -kd);
    const uint64_t scale_bits = table[ki & 31u] + (ki << 47);
    const double scale = __longlong_as_double(static_cast<long long>(scale_bits));
    const double p = fma(c0, r, c1);
    const double r2 = r * r;
    double y = fma(c2, r, 1.0);
    y = fma(p, r2, y);
    y = y * scale;
    return static_cast<float>(y);
}

// Ascending sort key for the order (logit descending, index ascending under a stable sort):
// the complement of the usual order-preserving float key, with -0 folded onto +0 so that the two
// tie (LogitOrder compares with ==, src/engine/session.cpp:30-35) and NaN mapped to the last key.
__device__ __forceinline__ uint32_t descending_key(float value)
{
    uint32_t bits = __float_as_uint(value);
    if (value != value)
        return 0xffffffffu;
    if (bits == 0x80000000u)
        bits = 0u;
    const uint32_t ordered = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    return ~ordered;
}

__device__ __forceinline__ float value_from_descending_key(uint32_t key)
{
    const uint32_t ordered = ~key;
    const uint32_t bits = (ordered & 0x80000000u) ? (ordered & 0x7fffffffu) : ~ordered;
    return __uint_as_float(bits);
}

constexpr uint32_t kLastFiniteKey = 0xff7fffffu;   // key of -FLT_MAX
constexpr uint32_t kPositiveInfinityKey = 0x007fffffu;

__device__ __forceinline__ int lane_id()
{
    return static_cast<int>(__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)));
}

// Number of set bits of mask below the calling lane.
__device__ __forceinline__ int lanes_below(uint64_t mask)
{
    return static_cast<int>(__builtin_amdgcn_mbcnt_hi(
        static_cast<uint32_t>(mask >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u)));
}

// The valid lanes of the wave that hold the same 8-bit digit as the calling lane, as the two halves of
// a lane mask (a lane that is not valid gets no peers and is nobody's peer).  Four instructions per bit of the
// digit: the bit spread over a register (one signed bit-field extract; written as `digit << (31 - b) >> 31` the
// compiler makes a shift for the compare and another for the mask), the compare that collects the wave's bits,
// and for each half of the mask one three-input operation, mask & ~(wave's bits ^ own bit).  (From the plain C
// expression the compiler made two exclusive-ors per bit and a three-input OR per two bits: 5.75 a bit.)
template <int BIT>
__device__ __forceinline__ void narrow_digit_peers(uint32_t digit, uint32_t& low, uint32_t& high)
{
    uint32_t mine; // all ones if the bit is set
    asm("v_bfe_i32 %0, %1, %2, 1" : "=v"(mine) : "v"(digit), "n"(BIT));
    const uint64_t set = __builtin_amdgcn_ballot_w64(mine != 0u);
    constexpr uint32_t kKeepWhereEqual = 0xf0u & ~(0xccu ^ 0xaau); // a & ~(b ^ c), inputs in the order of the operands
    low = __builtin_amdgcn_bitop3_b32(low, static_cast<uint32_t>(set), mine, kKeepWhereEqual);
    high = __builtin_amdgcn_bitop3_b32(high, static_cast<uint32_t>(set >> 32), mine, kKeepWhereEqual);
}

__device__ __forceinline__ void wave_digit_peers(uint32_t digit, bool valid, uint32_t& low, uint32_t& high);

// (every lane of the wave is valid)
__device__ __forceinline__ void wave_digit_peers(uint32_t digit, uint32_t& low, uint32_t& high)
{
    low = 0xffffffffu;
    high = 0xffffffffu;
    narrow_digit_peers<0>(digit, low, high);
    narrow_digit_peers<1>(digit, low, high);
    narrow_digit_peers<2>(digit, low, high);
    narrow_digit_peers<3>(digit, low, high);
    narrow_digit_peers<4>(digit, low, high);
    narrow_digit_peers<5>(digit, low, high);
    narrow_digit_peers<6>(digit, low, high);
    narrow_digit_peers<7>(digit, low, high);
}

__device__ __forceinline__ void wave_digit_peers(uint32_t digit, bool valid, uint32_t& low, uint32_t& high)
{
    const uint64_t all = __builtin_amdgcn_ballot_w64(valid);
    low = valid ? static_cast<uint32_t>(all) : 0u;
    high = valid ? static_cast<uint32_t>(all >> 32) : 0u;
    narrow_digit_peers<0>(digit, low, high);
    narrow_digit_peers<1>(digit, low, high);
    narrow_digit_peers<2>(digit, low, high);
    narrow_digit_peers<3>(digit, low, high);
    narrow_digit_peers<4>(digit, low, high);
    narrow_digit_peers<5>(digit, low, high);
    narrow_digit_peers<6>(digit, low, high);
    narrow_digit_peers<7>(digit, low, high);
}

// Workgroup barrier that orders LDS traffic only: waits for this wave's LDS operations, not for its
// outstanding global loads and stores (which __syncthreads() would also wait for).
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// A 16-byte load from device memory through a pointer whose address space the compiler cannot see (an argument
// of a function that is not inlined): as a global load it counts against the vector-memory counter only, where a
// flat load also counts as an LDS operation and is waited for by lds_barrier().
__device__ __forceinline__ uint4 load_global_uint4(const void* address)
{
    typedef uint32_t NativeVector __attribute__((ext_vector_type(4)));
    const NativeVector loaded = *(const __attribute__((address_space(1))) NativeVector*)(address);
    return make_uint4(loaded.x, loaded.y, loaded.z, loaded.w);
}

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

__device__ __forceinline__ float read_lane(float value, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(value), lane));
}

__device__ __forceinline__ int read_lane(int value, int lane)
{
    return __builtin_amdgcn_readlane(value, lane);
}

template <int CONTROL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_source(uint32_t value)
{
    // a lane whose source the control or the row mask leaves out reads 0
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(value), CONTROL, ROW_MASK, 0xf, false));
}

// The fp32 sums behind each of 64 non-negative terms, one term per lane, added in lane order as a
// sequential loop adds them: lane l returns ((t0 + t1) + ...) + tl.  Every lane adds the sum its lower
// neighbour holds (wave_shr:1) to its own term, 63 times over; after turn k the lanes up to k hold their
// final value, since lane l's depends on lane l - 1's alone.  63 dependent additions and no branch: a
// loop that broadcasts one term per turn and tests a stop condition costs several times that, in every
// wave of the workgroup at once.
__device__ __forceinline__ float wave_sequential_sums(float term)
{
    float sums = term;
#pragma unroll
    for (int turn = 1; turn < kWaveSize; ++turn)
    {
        // lane 0 has no lower neighbour and reads 0: 0 + t0 = t0 (the terms are not negative zero)
        const float below = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sums), 0x138, 0xf, 0xf, true));
        sums = below + term;
    }
    return sums;
}

// The same for the wave's first `count` lanes (count: the same in every lane): count - 1 turns, rounded up to
// whole trips of four (a turn too many changes nothing: a lane whose lower neighbour is final computes its own
// final value again).  The lanes from `count` on return no sum of anything.
__device__ __forceinline__ float wave_sequential_sums_of_first(float term, int count)
{
    float sums = term;
    for (int turn = 1; turn < count; turn += 4)
    {
#pragma unroll
        for (int k = 0; k < 4; ++k)
        {
            const float below = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sums), 0x138, 0xf, 0xf, true));
            sums = below + term;
        }
    }
    return sums;
}

// Reduction over each row of 16 lanes (every lane receives its row's result), by four DPP exchanges:
// inside pairs, quads, half rows, rows.
template <typename Op>
__device__ __forceinline__ uint32_t row16_reduce_u32(uint32_t value, Op op)
{
    value = op(value, dpp_source<0xB1, 0xf>(value));  // quad_perm [1,0,3,2]
    value = op(value, dpp_source<0x4E, 0xf>(value));  // quad_perm [2,3,0,1]
    value = op(value, dpp_source<0x141, 0xf>(value)); // row_half_mirror
    value = op(value, dpp_source<0x140, 0xf>(value)); // row_mirror
    return value;
}

// Maximum over the wave, returned to every lane.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t value)
{
    const auto larger = [](uint32_t x, uint32_t y) { return max(x, y); };
    value = row16_reduce_u32(value, larger);
    value = max(value, dpp_source<0x142, 0xa>(value)); // row_bcast15 into rows 1 and 3
    value = max(value, dpp_source<0x143, 0xc>(value)); // row_bcast31 into rows 2 and 3
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(value), 63));
}

// Bitwise OR over the wave, returned to every lane (the same value in all: a scalar).
__device__ __forceinline__ uint32_t wave_or_u32(uint32_t value)
{
    const auto either = [](uint32_t x, uint32_t y) { return x | y; };
    value = row16_reduce_u32(value, either);
    value |= dpp_source<0x142, 0xa>(value); // row_bcast15 into rows 1 and 3
    value |= dpp_source<0x143, 0xc>(value); // row_bcast31 into rows 2 and 3
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(value), 63));
}

// Inclusive prefix sum over the wave's lanes (lane i: sum of lanes 0 .. i), by DPP shifts inside rows of
// 16 lanes and two broadcasts across rows.  A lane that a shift leaves without a source adds zero.
__device__ __forceinline__ uint32_t wave_prefix_sum_u32(uint32_t value)
{
    value += dpp_source<0x111, 0xf>(value); // row_shr:1
    value += dpp_source<0x112, 0xf>(value); // row_shr:2
    value += dpp_source<0x114, 0xf>(value); // row_shr:4
    value += dpp_source<0x118, 0xf>(value); // row_shr:8
    value += dpp_source<0x142, 0xa>(value); // row_bcast15: rows 1 and 3 add the row before
    value += dpp_source<0x143, 0xc>(value); // row_bcast31: rows 2 and 3 add rows 0 + 1
    return value;
}

// One compare-exchange stage across lanes at distance j; keep_max selects which partner value stays.
__device__ __forceinline__ float exchange_stage(float value, int j, bool keep_max)
{
    const float other = __shfl_xor(value, j, kWaveSize);
    return keep_max ? fmaxf(value, other) : fminf(value, other);
}

// Sorts one value per lane into descending order across the wave (lane 0 holds the largest).
__device__ __forceinline__ float wave_sort_descending(float value, int lane)
{
#pragma unroll
    for (int k = 2; k <= kWaveSize; k <<= 1)
    {
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1)
        {
            const bool descending_block = (lane & k) == 0 || k == kWaveSize;
            const bool lower_lane = (lane & j) == 0;
            value = exchange_stage(value, j, lower_lane == descending_block);
        }
    }
    return value;
}

// value is bitonic across the wave; returns it sorted descending.
__device__ __forceinline__ float wave_bitonic_merge_descending(float value, int lane)
{
#pragma unroll
    for (int j = kWaveSize >> 1; j > 0; j >>= 1)
        value = exchange_stage(value, j, (lane & j) == 0);
    return value;
}

__device__ __forceinline__ bool candidate_before(float a_value, int a_index, float b_value, int b_index)
{
    return a_value > b_value || (a_value == b_value && a_index < b_index);
}

} // namespace ncnn_moe_hip

#endif // NCNN_MOE_HIP_SAMPLER_DEVICE_H
