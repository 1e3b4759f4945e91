// C ABI of the gfx950 generation sampler: handle, device buffers and kernel launches.
#include "ncnn_moe_hip_sampler.h"
#include "ncnn_moe_hip_sampler_testing.h"

#include "sampler_kernels.h"
#include "sampler_verify.h"

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

using namespace ncnn_moe_hip;

struct ncnn_moe_hip_sampler
{
    int device = 0;
    uint32_t max_rows = 0;
    uint32_t max_vocab = 0;
    uint32_t max_segments = 0;
    uint64_t logits_stride_f32 = 0; // elements per row of the handle's logits buffer, fp32 view
    int force_general = 0;
    int scatter_segments = 0;
    int spread_sort = 1; // a long row's radix sort runs on several workgroups
    int fused_bf16 = 1;  // bf16 full-order rows are counted and walked by one kernel
    // a call with rows for the wide select and rows for the full-order kernels runs the two side by side
    hipStream_t side_stream = nullptr;
    hipEvent_t side_fork = nullptr;
    hipEvent_t side_join = nullptr;
    hipEvent_t cut_done = nullptr;
    hipStream_t stream = nullptr;

    void* logits = nullptr;
    int logits_dtype = NCNN_MOE_LOGITS_F32;
    uint32_t logits_rows = 0;
    uint32_t logits_vocab = 0;
    uint64_t logits_stride = 0;

    ncnn_moe_sample_params* params = nullptr;
    float* uniforms = nullptr;
    ncnn_moe_sample_result* results = nullptr;
    // the host entry's small operands are staged as one block of pinned memory, params | uniforms | stop ids,
    // that the kernels read in place; its results are written by the kernels straight into pinned memory
    uint8_t* input_block_host = nullptr; // pinned
    uint8_t* input_block_mapped = nullptr; // the pinned block as the device addresses it
    size_t input_uniforms_offset = 0;
    size_t input_stops_offset = 0;
    uint32_t input_stop_capacity = 0;
    ncnn_moe_sample_result* results_host = nullptr;   // pinned
    ncnn_moe_sample_result* results_host_device = nullptr; // the same memory as the device addresses it

    float* segment_values = nullptr;
    int32_t* segment_indices = nullptr;
    uint32_t* segment_counts = nullptr;
    unsigned long long* row_counter = nullptr;
    uint32_t* row_flags = nullptr;
    uint32_t* row_state = nullptr;
    unsigned long long* split_records = nullptr;
    uint32_t* row_epoch = nullptr;

    uint32_t* sort_keys[2] = {nullptr, nullptr};
    uint32_t* sort_indices[2] = {nullptr, nullptr};
    uint64_t sort_stride = 0;
    uint32_t* row_list = nullptr;         // [1 + rows], see SamplerArgs::row_list
    uint32_t* sort_cuts = nullptr;        // [4][rows]: SamplerArgs::sort_lengths, sort_last_keys, finite_counts, disordered_rows
    int partial_sort = 1;                 // full-order fp32 rows are sorted only as far as their terms can move a sum
    int skip_low_digit = 1;               // ... by three passes over the keys' upper 24 bits, the lowest byte put in order by the terms kernel
    int wide_sampled_bound = 1;           // the wide select bounds its widest windows from a sample of the whole row
    uint32_t* sort_part_counts = nullptr; // [rows][kMaxSortParts][256]
    double* term_sums = nullptr;          // [rows][term_sum_parts]: fp64 sums of the terms kernel's blocks
    uint4* chunk_steps = nullptr;         // [rows][chunk_capacity]: composed step of every whole chunk of a sorted row's terms
    uint32_t term_sum_parts = 0;
    uint32_t chunk_capacity = 0;
    int chunk_steps_enabled = 1;

    int32_t* distribution_ids = nullptr;
    float* distribution_probabilities = nullptr;
    uint32_t* distribution_count = nullptr;
    // speculative verification: exported distributions of 2 * kMaxDrafts + 1 rows and the small operands
    int32_t* verify_ids = nullptr;
    float* verify_probabilities = nullptr;
    uint32_t* verify_counts = nullptr;
    // speculative verification of filtered distributions longer than kVerifyCap: rows x max_vocab lists and
    // two dense vectors over the vocabulary
    int32_t* verify_long_ids = nullptr;
    float* verify_long_probabilities = nullptr;
    float* verify_dense = nullptr;
    // the options of the last step that needed them: the next step with the same options goes there at once
    bool verify_dense_known = false;
    ncnn_moe_sample_params verify_dense_options{};
    // operands and outcome of a step travel as one block each, through pinned host memory
    struct VerifyInput
    {
        ncnn_moe_sample_params params[2 * NCNN_MOE_MAX_DRAFT_TOKENS + 1];
        float row_uniforms[2 * NCNN_MOE_MAX_DRAFT_TOKENS + 1];
        int32_t proposed[NCNN_MOE_MAX_DRAFT_TOKENS];
        float uniforms[NCNN_MOE_MAX_DRAFT_TOKENS + 1];
    };
    struct VerifyOutput
    {
        ncnn_moe_verify_result result;
        float accepted[NCNN_MOE_MAX_DRAFT_TOKENS];
    };
    VerifyInput* verify_input_host = nullptr;   // pinned
    VerifyOutput* verify_output_host = nullptr; // pinned
    VerifyInput* verify_input_mapped = nullptr;   // the pinned blocks as the device addresses them: the kernels
    VerifyOutput* verify_output_mapped = nullptr; // read the operands and write the outcome in place

    ncnn_moe_sample_params* single_params = nullptr;
    float* single_uniform = nullptr;
    ncnn_moe_sample_result* single_result = nullptr;

    std::string last_error;
};

namespace {

uint64_t round_up(uint64_t value, uint64_t multiple)
{
    return (value + multiple - 1) / multiple * multiple;
}

int fail(ncnn_moe_hip_sampler* s, int rc, const std::string& message)
{
    if (s != nullptr)
        s->last_error = message;
    return rc;
}

int hip_fail(ncnn_moe_hip_sampler* s, hipError_t error, const char* what)
{
    return fail(s, NCNN_MOE_SAMPLER_HIP_ERROR, std::string(what) + ": " + hipGetErrorString(error));
}

#define SAMPLER_HIP_CHECK(s, call)                   \
    do                                               \
    {                                                \
        const hipError_t error_ = (call);            \
        if (error_ != hipSuccess)                    \
            return hip_fail((s), error_, #call);     \
    } while (0)

uint64_t logits_span(uint32_t vocab, int dtype, const void* logits, uint64_t row_stride)
{
    const uint32_t width = dtype == NCNN_MOE_LOGITS_F32 ? 4u : 8u;
    const uint32_t element = dtype == NCNN_MOE_LOGITS_F32 ? 4u : 2u;
    const bool aligned = (reinterpret_cast<uintptr_t>(logits) & 15u) == 0 && (row_stride * element) % 16u == 0;
    return static_cast<uint64_t>(vocab) + (aligned ? 0u : width - 1u);
}

// How the select kernel covers a row: `segments` workgroups, each streaming `chunks_per_segment`
// chunks.  Small batches are split so that every CU streams; the last workgroup of a row to arrive
// merges the segments.  From kWholeRowBatch rows on a workgroup streams the whole row and finishes it.
// The wide variant (Top-K windows up to kSelectTopK) always takes whole rows.
struct SelectGeometry
{
    uint32_t segments = 1;
    uint32_t chunks_per_segment = 1;
    bool looped = true;
    bool wide = false;
};

uint64_t chunk_values(int dtype)
{
    return dtype == NCNN_MOE_LOGITS_F32 ? kSegmentValuesF32 : kSegmentValuesBF16;
}

SelectGeometry select_geometry(int dtype, uint64_t span, uint32_t rows, bool wide)
{
    SelectGeometry g;
    g.wide = wide;
    const uint64_t total_chunks = std::max<uint64_t>(1, (span + chunk_values(dtype) - 1) / chunk_values(dtype));
    auto split = [&](int workgroups, int most) {
        const uint64_t wanted = (static_cast<uint64_t>(workgroups) + rows - 1) / rows;
        uint64_t segments = std::min<uint64_t>(std::min<uint64_t>(wanted, total_chunks), static_cast<uint64_t>(most));
        const uint64_t chunks_per_segment = (total_chunks + segments - 1) / segments;
        segments = (total_chunks + chunks_per_segment - 1) / chunks_per_segment;
        g.segments = static_cast<uint32_t>(segments);
        g.chunks_per_segment = static_cast<uint32_t>(chunks_per_segment);
    };
    if (wide || rows >= static_cast<uint32_t>(kWholeRowBatch))
    {
        g.segments = 1;
        g.chunks_per_segment = static_cast<uint32_t>(total_chunks);
    }
    else
    {
        split(kSingleChunkWorkgroups, kSplitMaxSegments);
        // (bf16 rows of more than 16 chunks: from about 2,300 one-chunk workgroups on the looped kernel is as fast or
        // faster - 128 x 262,144: 27.6 us against 31.1; fp32 rows are faster in one-chunk workgroups at every batch size)
        const bool long_bf16_rows = dtype == NCNN_MOE_LOGITS_BF16 && g.segments > static_cast<uint32_t>(kMaxSegments) &&
            static_cast<uint64_t>(rows) * g.segments > 2304u;
        if (g.chunks_per_segment > 1 || long_bf16_rows)
            split(kLoopedWorkgroups, kMaxSegments); // the looped kernel keeps two workgroups per CU resident
    }
    g.looped = g.chunks_per_segment > 1 || g.segments == 1;
    return g;
}

// Device memory that the select kernels use beyond their operands: the segments' candidate records
// and per-row hand-over words.  A handle allocates them in create(); the entry that allocates nothing
// points them into its static array.
struct SelectScratch
{
    float* segment_values;
    int32_t* segment_indices;
    uint32_t* segment_counts;
    unsigned long long* row_counter;
    uint32_t* row_flags;
    uint32_t* row_state;
    unsigned long long* split_records;
    uint32_t* row_epoch;
};

void use_select_scratch(SamplerArgs& a, const SelectScratch& scratch)
{
    a.segment_values = scratch.segment_values;
    a.segment_indices = scratch.segment_indices;
    a.segment_counts = scratch.segment_counts;
    a.row_counter = scratch.row_counter;
    a.row_flags = scratch.row_flags;
    a.row_state = scratch.row_state;
    a.split_records = scratch.split_records;
    a.row_epoch = scratch.row_epoch;
}

template <int DTYPE>
void launch_select(const SelectGeometry& g, uint32_t rows, hipStream_t stream, SamplerArgs a, int only_pending, bool scatter_segments)
{
    a.segments = g.segments;
    a.chunks_per_segment = g.chunks_per_segment;
    a.max_select_top_k = g.wide ? kSelectTopK : kFastTopK;
    a.only_pending = only_pending;
    dim3 grid(g.segments, rows, 1);
    a.xcd_grouped = 0;
    if (g.segments > 1 && !scatter_segments)
    {
        // one-dimensional, rows padded to a multiple of eight: workgroup 8 t + x is segment t % segments of
        // row 8 (t / segments) + x, so that the XCDs' turns put the segments of a row on one XCD
        a.xcd_grouped = 1;
        grid = dim3(((rows + 7u) / 8u) * 8u * g.segments, 1, 1);
    }
    if (g.wide)
        hipLaunchKernelGGL((scan_select_kernel<DTYPE, true, true>), grid, dim3(kScanThreads), 0, stream, a);
    else if (g.looped)
        hipLaunchKernelGGL((scan_select_kernel<DTYPE, true, false>), grid, dim3(kScanThreads), 0, stream, a);
    else if (g.segments > static_cast<uint32_t>(kMaxSegments))
        hipLaunchKernelGGL((split_select_kernel<DTYPE, kSplitMaxSegments>), grid, dim3(kScanThreads), 0, stream, a);
    else if (g.segments > 1)
        hipLaunchKernelGGL((split_select_kernel<DTYPE, 16>), grid, dim3(kScanThreads), 0, stream, a);
    else
        hipLaunchKernelGGL((scan_select_kernel<DTYPE, false, false>), grid, dim3(kScanThreads), 0, stream, a);
}

// Where a launch writes the rows' filtered distributions (cap entries per row); count == nullptr: nowhere.
struct DistributionExport
{
    int32_t* ids = nullptr;
    float* probabilities = nullptr;
    uint32_t* count = nullptr;
    uint32_t cap = 0;
};

constexpr uint32_t kSideBySideRows = 32; // rows of each kind from which sample() runs the two later passes side by side

// Which kernels a call enqueues.  Rows a pass cannot serve are marked pending and taken by the next.
struct SamplerPasses
{
    bool select = true;      // the batch-shaped select kernel
    bool wide_select = false; // one workgroup per row still pending: Top-K windows up to kSelectTopK
    bool full_order = false; // sort + replay for every row still pending
    bool side_by_side = false; // the wide select on the handle's second stream, beside the full-order kernels
};

// Enqueues the sampling path for `rows` rows.
int launch_sampler(
    ncnn_moe_hip_sampler* s, const void* logits, int dtype, uint32_t rows, uint32_t vocab, uint64_t row_stride,
    const ncnn_moe_sample_params* params, const float* uniforms, const int32_t* stop_ids,
    ncnn_moe_sample_result* results, DistributionExport export_to, SamplerPasses passes, hipStream_t stream)
{
    const bool want_distribution = export_to.count != nullptr;
    SamplerArgs a;
    std::memset(&a, 0, sizeof(a));
    a.logits = logits;
    a.row_stride = row_stride;
    a.rows = rows;
    a.vocab = vocab;
    const uint64_t span = logits_span(vocab, dtype, logits, row_stride);
    a.force_general = s->force_general;
    a.wide_sampled_bound = s->wide_sampled_bound != 0 ? 1u : 0u;
    a.params = params;
    a.uniforms = uniforms;
    a.stop_ids = stop_ids;
    a.results = results;
    use_select_scratch(a, SelectScratch{s->segment_values, s->segment_indices, s->segment_counts, s->row_counter, s->row_flags, s->row_state,
                                        s->split_records, s->row_epoch});
    a.sort_keys[0] = s->sort_keys[0];
    a.sort_keys[1] = s->sort_keys[1];
    a.sort_indices[0] = s->sort_indices[0];
    a.sort_indices[1] = s->sort_indices[1];
    a.sort_stride = s->sort_stride;
    a.sort_part_counts = s->sort_part_counts;
    a.term_sums = s->term_sums;
    a.chunk_steps = s->chunk_steps;
    a.term_sum_parts = s->term_sum_parts;
    a.chunk_capacity = s->chunk_capacity;
    if (want_distribution)
    {
        a.distribution_ids = export_to.ids;
        a.distribution_probabilities = export_to.probabilities;
        a.distribution_cap = export_to.cap;
        a.distribution_count = export_to.count;
    }
    const SelectGeometry batch_geometry = select_geometry(dtype, span, rows, false);
    if (batch_geometry.looped && batch_geometry.segments > s->max_segments)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "vocab exceeds the handle's max_vocab");

    // only_pending: 1 = the rows an earlier launch left pending, 2 = the rows whose options ask for a wide window
    const auto launch_wide = [&](hipStream_t on, int only_pending) {
        const SelectGeometry row_geometry = select_geometry(dtype, span, rows, true);
        if (dtype == NCNN_MOE_LOGITS_F32)
            launch_select<NCNN_MOE_LOGITS_F32>(row_geometry, rows, on, a, only_pending, s->scatter_segments != 0);
        else
            launch_select<NCNN_MOE_LOGITS_BF16>(row_geometry, rows, on, a, only_pending, s->scatter_segments != 0);
    };
    // A long row's radix sort is spread over several workgroups (two tiles each, at most kMaxSortParts):
    // two launches per pass over a (parts, rows) grid.  Short rows keep the one-workgroup kernel.
    const uint32_t sort_tiles = static_cast<uint32_t>((static_cast<uint64_t>(vocab) + kSortTile - 1) / kSortTile);
    const uint32_t sort_tiles_per_part = std::max<uint32_t>(1, (sort_tiles + kMaxSortParts - 1) / kMaxSortParts);
    const uint32_t sort_parts = std::max<uint32_t>(1, (sort_tiles + sort_tiles_per_part - 1) / sort_tiles_per_part);
    // fp32 rows whose sort is spread over the GPU are sorted only as far as their terms can move a sum
    // (full_order_cut_kernel); a row whose replay finds that guess too short stays pending, and a second launch of
    // the full-order kernels, behind the first, sorts it whole.
    const bool partial_sort = passes.full_order && dtype == NCNN_MOE_LOGITS_F32 && !want_distribution && sort_tiles >= 4 &&
        s->spread_sort != 0 && s->partial_sort != 0;
    if (partial_sort)
    {
        a.sort_lengths = s->sort_cuts;
        a.sort_last_keys = s->sort_cuts + s->max_rows;
        a.finite_counts = s->sort_cuts + 2 * static_cast<size_t>(s->max_rows);
        a.disordered_rows = s->sort_cuts + 3 * static_cast<size_t>(s->max_rows);
    }
    // Side by side (see below) with the first select in the call: the wide select is forked off in front of it
    // and picks its rows by their options, and the first select leaves those rows alone.
    const bool side_by_side = passes.side_by_side && passes.wide_select && passes.full_order && s->side_stream != nullptr;
    const bool early_wide = side_by_side && passes.select;
    // The kernel that guesses the rows' cuts needs the logits and the options only: it runs on the second stream
    // beside the first select, for the rows whose options no select pass serves (a row that a select pass hands
    // on, its window overflowing with ties, is sorted whole).
    const bool early_cut = partial_sort && passes.select && s->side_stream != nullptr;
    if (early_wide || early_cut)
    {
        if (hipEventRecord(s->side_fork, stream) != hipSuccess || hipStreamWaitEvent(s->side_stream, s->side_fork, 0) != hipSuccess)
            return fail(s, NCNN_MOE_SAMPLER_HIP_ERROR, "fork to the second stream failed");
        if (early_cut)
        {
            // the rows' list, their cuts and the sort's first counting pass: all three need the logits and the options only
            SamplerArgs cut = a;
            cut.leave_wide_rows = 0;
            cut.cut_by_options = 1;
            cut.max_select_top_k = passes.wide_select || batch_geometry.wide ? kSelectTopK : kFastTopK;
            cut.row_list_out = s->row_list; // (one more workgroup, which lists the rows)
            hipLaunchKernelGGL(full_order_cut_kernel, dim3(rows + 1), dim3(kSortThreads), 0, s->side_stream, cut);
            cut.row_list = s->row_list;
            cut.sort_low_digit_skipped = s->skip_low_digit != 0 ? 1u : 0u;
            cut.sort_parts = sort_parts;
            cut.sort_tiles_per_part = sort_tiles_per_part;
            cut.sort_pass = 0;
            // (the event rides on the kernel's own completion signal where the stream is not being captured: a record
            // of its own is one more packet for the caller's stream to wait behind)
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            (void)hipStreamIsCapturing(stream, &capturing);
            if (capturing == hipStreamCaptureStatusNone)
                hipExtLaunchKernelGGL((sort_part_histogram_kernel<NCNN_MOE_LOGITS_F32>), dim3((sort_parts + kHistogramParts - 1) / kHistogramParts, rows),
                                      dim3(kSortThreads), 0, s->side_stream, nullptr, s->cut_done, 0, cut);
            else
            {
                hipLaunchKernelGGL((sort_part_histogram_kernel<NCNN_MOE_LOGITS_F32>), dim3((sort_parts + kHistogramParts - 1) / kHistogramParts, rows),
                                   dim3(kSortThreads), 0, s->side_stream, cut);
                if (hipEventRecord(s->cut_done, s->side_stream) != hipSuccess)
                    return fail(s, NCNN_MOE_SAMPLER_HIP_ERROR, "fork to the second stream failed");
            }
        }
        if (early_wide)
            launch_wide(s->side_stream, 2);
    }
    if (passes.select)
    {
        SamplerArgs first = a;
        first.leave_wide_rows = early_wide ? 1 : 0;
        if (dtype == NCNN_MOE_LOGITS_F32)
            launch_select<NCNN_MOE_LOGITS_F32>(batch_geometry, rows, stream, first, 0, s->scatter_segments != 0);
        else
            launch_select<NCNN_MOE_LOGITS_BF16>(batch_geometry, rows, stream, first, 0, s->scatter_segments != 0);
    }
    // first_counted: the first pass's counting kernel has run on the second stream (see early_cut)
    const auto launch_spread_sort = [&](SamplerArgs spread, auto dtype_tag, auto pairs_tag, bool first_counted) {
        constexpr int kType = decltype(dtype_tag)::value;
        constexpr bool kPairs = decltype(pairs_tag)::value;
        spread.sort_parts = sort_parts;
        spread.sort_tiles_per_part = sort_tiles_per_part;
        const int passes = kType == NCNN_MOE_LOGITS_F32 ? 4 - static_cast<int>(spread.sort_low_digit_skipped) : 2;
        for (int pass = 0; pass < passes; ++pass)
        {
            spread.sort_pass = static_cast<uint32_t>(pass);
            if (pass != 0 || !first_counted)
                hipLaunchKernelGGL((sort_part_histogram_kernel<kType>), dim3((sort_parts + kHistogramParts - 1) / kHistogramParts, rows), dim3(kSortThreads), 0, stream, spread);
            if (pass == 0 && !kPairs) // (keys alone: the first pass need not keep the order of equal digits)
                hipLaunchKernelGGL((sort_part_scatter_kernel<kType, kPairs, true>), dim3(sort_parts, rows), dim3(kSortThreads), 0, stream, spread);
            else
                hipLaunchKernelGGL((sort_part_scatter_kernel<kType, kPairs>), dim3(sort_parts, rows), dim3(kSortThreads), 0, stream, spread);
        }
    };
    // `leftovers`: the launch behind the wide select, for the few rows (usually none) that it could not
    // finish; it is kept to two kernels, because every launch costs its few microseconds even with no row to serve.
    const auto launch_full_order = [&](SamplerArgs a, bool leftovers) {
        const bool spread_sort = sort_tiles >= 4 && s->spread_sort != 0 && !leftovers;
        const bool runs = dtype == NCNN_MOE_LOGITS_BF16 && !want_distribution;
        // (keys alone, sorted in part or whole by the spread sort: its pass over the lowest byte is left out)
        a.sort_low_digit_skipped = !leftovers && partial_sort && s->skip_low_digit != 0 ? 1u : 0u;
        const bool listed_early = !leftovers && partial_sort && early_cut;
        if (listed_early)
        {
            // (listed, cut and counted for the first pass on the second stream)
            a.row_list = s->row_list;
            a.rows_listed_by_options = 1;
            (void)hipStreamWaitEvent(stream, s->cut_done, 0);
        }
        else if (!leftovers && !runs)
        {
            // (the kernels over a (parts, rows) grid find their rows in a list)
            hipLaunchKernelGGL(full_order_row_list_kernel, dim3(1), dim3(kSortThreads), 0, stream, a, rows, s->row_list);
            a.row_list = s->row_list;
        }
        if (!leftovers && partial_sort && !early_cut)
            hipLaunchKernelGGL(full_order_cut_kernel, dim3(rows), dim3(kSortThreads), 0, stream, a);
        // the token indices ride along with the keys only when the whole distribution is exported
        const auto sort_rows = [&](auto dtype_tag, auto pairs_tag) {
            constexpr int kType = decltype(dtype_tag)::value;
            constexpr bool kPairs = decltype(pairs_tag)::value;
            if (spread_sort)
                launch_spread_sort(a, dtype_tag, pairs_tag, listed_early);
            else
                hipLaunchKernelGGL((general_sort_kernel<kType, kPairs>), dim3(rows), dim3(kSortThreads), 0, stream, a);
        };
        using F32 = std::integral_constant<int, NCNN_MOE_LOGITS_F32>;
        using BF16 = std::integral_constant<int, NCNN_MOE_LOGITS_BF16>;
        // (bf16 rows that need no exported distribution: counted and walked by one kernel, unless a test asks for the two)
        const bool fused_runs = runs && s->fused_bf16 != 0;
        if (fused_runs)
            hipLaunchKernelGGL(bf16_counting_replay_kernel, dim3(rows), dim3(kSortThreads), 0, stream, a);
        else if (runs)
            hipLaunchKernelGGL(bf16_counting_sort_kernel, dim3(rows), dim3(kSortThreads), 0, stream, a);
        else if (dtype == NCNN_MOE_LOGITS_F32 && want_distribution)
            sort_rows(F32{}, std::true_type{});
        else if (dtype == NCNN_MOE_LOGITS_F32)
            sort_rows(F32{}, std::false_type{});
        else
            sort_rows(BF16{}, std::true_type{});
        if (!runs && !leftovers)
        {
            const uint32_t parts = (vocab + kTermsThreads * kTermsPerThread - 1) / (kTermsThreads * kTermsPerThread);
            hipLaunchKernelGGL(full_order_terms_kernel, dim3(parts, rows), dim3(kTermsThreads), 0, stream, a);
            a.terms_precomputed = 1;
            const uint32_t chunks = (vocab + kReplayChunk - 1) / kReplayChunk;
            if (vocab >= static_cast<uint32_t>(kReplayChunk) && s->chunk_steps_enabled != 0)
            {
                hipLaunchKernelGGL(full_order_chunk_steps_kernel, dim3(chunks, rows), dim3(kChunkStepThreads), 0, stream, a);
                a.chunk_steps_ready = 1;
            }
        }
        if (fused_runs)
            return;
        if (runs)
            hipLaunchKernelGGL((general_replay_kernel<NCNN_MOE_LOGITS_BF16, true>), dim3(rows), dim3(kReplayThreads), 0, stream, a);
        else if (dtype == NCNN_MOE_LOGITS_F32)
            hipLaunchKernelGGL((general_replay_kernel<NCNN_MOE_LOGITS_F32, false>), dim3(rows), dim3(kReplayThreads), 0, stream, a);
        else
            hipLaunchKernelGGL((general_replay_kernel<NCNN_MOE_LOGITS_BF16, false>), dim3(rows), dim3(kReplayThreads), 0, stream, a);
    };
    // Rows for the wide select and rows for the full-order kernels are disjoint and each pass keeps few
    // compute units busy (one workgroup per row): with both kinds in the call the two passes run side by
    // side, the wide select on the handle's second stream.  (Starting it only beside the replay, behind a
    // sort that is spread over every compute unit, was measured and is slower: the two one-workgroup-per-row
    // kernels then share compute units and the wide select takes 330 us instead of 210.)
    // The full-order kernels leave the wide select's rows alone, and are enqueued once more behind the
    // join for the rows that the wide select (or, when that one started beside it, the first select) could
    // not finish: ties beyond their lists; without such rows that launch exits at once.
    if (side_by_side)
    {
        if (!early_wide)
        {
            if (hipEventRecord(s->side_fork, stream) != hipSuccess || hipStreamWaitEvent(s->side_stream, s->side_fork, 0) != hipSuccess)
                return fail(s, NCNN_MOE_SAMPLER_HIP_ERROR, "fork to the second stream failed");
            launch_wide(s->side_stream, 1);
        }
        SamplerArgs own_rows = a;
        own_rows.leave_wide_rows = 1;
        launch_full_order(own_rows, false);
        if (hipEventRecord(s->side_join, s->side_stream) != hipSuccess || hipStreamWaitEvent(stream, s->side_join, 0) != hipSuccess)
            return fail(s, NCNN_MOE_SAMPLER_HIP_ERROR, "join of the second stream failed");
        launch_full_order(a, true);
    }
    else
    {
        if (passes.wide_select)
            launch_wide(stream, 1);
        if (passes.full_order)
            launch_full_order(a, false);
        if (partial_sort)
            launch_full_order(a, true);
    }
    SAMPLER_HIP_CHECK(s, hipGetLastError());
    return NCNN_MOE_SAMPLER_SUCCESS;
}

// Would a select kernel serving windows up to max_top_k leave the row to a later pass?
bool row_left_pending(const ncnn_moe_sample_params& p, uint32_t vocab, uint32_t max_top_k)
{
    uint32_t effective_k = 0;
    int status = NCNN_MOE_ROW_OK;
    return resolve_row_mode(p, vocab, max_top_k, 0, effective_k, status) == kModeGeneral;
}

int check_shape(ncnn_moe_hip_sampler* s, int dtype, uint32_t rows, uint32_t vocab)
{
    if (dtype != NCNN_MOE_LOGITS_F32 && dtype != NCNN_MOE_LOGITS_BF16)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "unknown logits dtype");
    if (rows == 0 || rows > s->max_rows)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "rows must be in [1, max_rows]");
    if (vocab > s->max_vocab)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "vocab exceeds the handle's max_vocab");
    return NCNN_MOE_SAMPLER_SUCCESS;
}

// ---- ncnn_moe_hip_sampler_sample_device_static: the select pass with no handle and no allocation.
// Its scratch is this file-scope device array; every GPU the library runs on holds its own copy, at its
// own address, until the process ends.  The name `scratch` is only a host-side stand-in for it: host code
// takes the device address once per device with hipGetSymbolAddress and uses that pointer everywhere.
constexpr uint32_t kStaticMaxRows = NCNN_MOE_STATIC_MAX_ROWS;
constexpr uint32_t kStaticSplitRows = kWholeRowBatch - 1; // larger batches stream whole rows and keep no records
constexpr int kStaticMaxDevices = 64;

struct StaticScratchLayout
{
    float segment_values[static_cast<size_t>(kStaticSplitRows) * kMaxSegments * kSegmentRecordSlots];
    int32_t segment_indices[static_cast<size_t>(kStaticSplitRows) * kMaxSegments * kSegmentRecordSlots];
    uint32_t segment_counts[static_cast<size_t>(kStaticSplitRows) * kMaxSegments];
    unsigned long long row_counter[kStaticMaxRows];
    uint32_t row_flags[kStaticMaxRows];
    uint32_t row_state[kStaticMaxRows];
    unsigned long long split_records[static_cast<size_t>(kStaticSplitRows) * kSplitMaxSegments * kSplitRecordSlots];
    uint32_t row_epoch[kStaticMaxRows];
};
static_assert(kStaticMaxRows >= kStaticSplitRows, "a split batch must fit the per-row words");

static __device__ __align__(256) unsigned char scratch[sizeof(StaticScratchLayout)];

std::mutex g_static_mutex;
StaticScratchLayout* g_static_scratch[kStaticMaxDevices] = {}; // device address of `scratch`, per device
thread_local char g_static_error[256] = "";

int static_fail(int rc, const char* message, const char* detail = "")
{
    std::snprintf(g_static_error, sizeof(g_static_error), "%s%s%s", message, detail[0] != 0 ? ": " : "", detail);
    return rc;
}

// The words that a launch expects to find at zero (the kernels return them to zero themselves).
__global__ void static_scratch_clear_kernel(StaticScratchLayout* layout)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < kStaticMaxRows)
    {
        layout->row_counter[i] = 0ull;
        layout->row_flags[i] = 0u;
        layout->row_state[i] = 0u;
        layout->row_epoch[i] = 1u;
    }
    if (i < kStaticSplitRows * kMaxSegments)
        layout->segment_counts[i] = 0u;
    if (i < kStaticSplitRows * kSplitMaxSegments)
    {
        for (uint32_t entry = 0; entry < static_cast<uint32_t>(kSplitRecordSlots); ++entry)
            layout->split_records[static_cast<size_t>(i) * kSplitRecordSlots + entry] = 0ull; // epoch 0 tags nothing
    }
}

} // namespace

extern "C" {

int ncnn_moe_hip_sampler_device_count(void)
{
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess)
        return 0;
    return count;
}

int ncnn_moe_hip_sampler_create(int device, uint32_t max_rows, uint32_t max_vocab, ncnn_moe_hip_sampler** out)
{
    if (out == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    *out = nullptr;
    if (max_rows == 0 || max_vocab == 0 || max_rows > NCNN_MOE_SAMPLER_MAX_ROWS)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT; // the kernels put rows on a grid dimension
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count == 0)
        return NCNN_MOE_SAMPLER_NO_DEVICE;
    if (device < 0 || device >= count)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;

    ncnn_moe_hip_sampler* s = new (std::nothrow) ncnn_moe_hip_sampler();
    if (s == nullptr)
        return NCNN_MOE_SAMPLER_HIP_ERROR;
    s->device = device;
    s->max_rows = max_rows;
    s->max_vocab = max_vocab;
    s->max_segments = static_cast<uint32_t>(std::min<uint64_t>(
        static_cast<uint64_t>(kMaxSegments), (static_cast<uint64_t>(max_vocab) + 7 + kSegmentValuesF32 - 1) / kSegmentValuesF32));
    s->logits_stride_f32 = round_up(max_vocab, 8);
    s->sort_stride = round_up(max_vocab, 4);

    auto destroy_and_return = [&](hipError_t error, const char* what) {
        std::fprintf(stderr, "ncnn_moe_hip_sampler_create: %s: %s\n", what, hipGetErrorString(error));
        ncnn_moe_hip_sampler_destroy(s);
        return NCNN_MOE_SAMPLER_HIP_ERROR;
    };
#define CREATE_CHECK(call)                            \
    do                                                \
    {                                                 \
        const hipError_t error_ = (call);             \
        if (error_ != hipSuccess)                     \
            return destroy_and_return(error_, #call); \
    } while (0)

    CREATE_CHECK(hipSetDevice(device));
    CREATE_CHECK(hipStreamCreate(&s->stream));
    CREATE_CHECK(hipStreamCreateWithFlags(&s->side_stream, hipStreamNonBlocking));
    CREATE_CHECK(hipEventCreateWithFlags(&s->side_fork, hipEventDisableTiming));
    CREATE_CHECK(hipEventCreateWithFlags(&s->side_join, hipEventDisableTiming));
    CREATE_CHECK(hipEventCreateWithFlags(&s->cut_done, hipEventDisableTiming));
    const size_t rows = max_rows;
    const size_t slots = rows * s->max_segments;
    CREATE_CHECK(hipMalloc(&s->logits, rows * s->logits_stride_f32 * sizeof(float)));
    CREATE_CHECK(hipMalloc(&s->params, rows * sizeof(ncnn_moe_sample_params)));
    CREATE_CHECK(hipMalloc(&s->uniforms, rows * sizeof(float)));
    CREATE_CHECK(hipMalloc(&s->results, rows * sizeof(ncnn_moe_sample_result)));
    s->input_uniforms_offset = rows * sizeof(ncnn_moe_sample_params);
    s->input_stops_offset = s->input_uniforms_offset + rows * sizeof(float);
    // room for stop ids: 64 per row, or one list as long as the vocabulary, whichever is more
    s->input_stop_capacity = static_cast<uint32_t>(std::min<uint64_t>(std::max<uint64_t>(rows * 64, max_vocab), 1u << 28));
    const size_t input_bytes = s->input_stops_offset + static_cast<size_t>(s->input_stop_capacity) * sizeof(int32_t);
    CREATE_CHECK(hipHostMalloc(&s->input_block_host, input_bytes, hipHostMallocDefault));
    CREATE_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&s->input_block_mapped), s->input_block_host, 0));
    CREATE_CHECK(hipHostMalloc(&s->results_host, rows * sizeof(ncnn_moe_sample_result), hipHostMallocDefault));
    CREATE_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&s->results_host_device), s->results_host, 0));
    CREATE_CHECK(hipMalloc(&s->segment_values, slots * kSegmentRecordSlots * sizeof(float)));
    CREATE_CHECK(hipMalloc(&s->segment_indices, slots * kSegmentRecordSlots * sizeof(int32_t)));
    CREATE_CHECK(hipMalloc(&s->segment_counts, slots * sizeof(uint32_t)));
    CREATE_CHECK(hipMalloc(&s->row_counter, rows * sizeof(unsigned long long)));
    CREATE_CHECK(hipMalloc(&s->row_flags, rows * sizeof(uint32_t)));
    CREATE_CHECK(hipMalloc(&s->row_state, rows * sizeof(uint32_t)));
    // split path: records start untagged (epoch 0 tags nothing), every row at epoch 1
    const size_t split_rows = std::min<size_t>(rows, static_cast<size_t>(kWholeRowBatch) - 1);
    CREATE_CHECK(hipMalloc(&s->split_records, split_rows * kSplitMaxSegments * kSplitRecordSlots * sizeof(unsigned long long)));
    CREATE_CHECK(hipMemset(s->split_records, 0, split_rows * kSplitMaxSegments * kSplitRecordSlots * sizeof(unsigned long long)));
    CREATE_CHECK(hipMalloc(&s->row_epoch, rows * sizeof(uint32_t)));
    CREATE_CHECK(hipMemsetD32(reinterpret_cast<hipDeviceptr_t>(s->row_epoch), 1, rows));
    CREATE_CHECK(hipMemset(s->segment_counts, 0, slots * sizeof(uint32_t)));
    CREATE_CHECK(hipMemset(s->row_counter, 0, rows * sizeof(unsigned long long)));
    CREATE_CHECK(hipMemset(s->row_flags, 0, rows * sizeof(uint32_t)));
    CREATE_CHECK(hipMemset(s->row_state, 0, rows * sizeof(uint32_t)));
    for (int i = 0; i < 2; ++i)
    {
        CREATE_CHECK(hipMalloc(&s->sort_keys[i], rows * s->sort_stride * sizeof(uint32_t)));
        CREATE_CHECK(hipMalloc(&s->sort_indices[i], rows * s->sort_stride * sizeof(uint32_t)));
    }
    CREATE_CHECK(hipMalloc(&s->row_list, (static_cast<size_t>(rows) + 1) * sizeof(uint32_t)));
    CREATE_CHECK(hipMalloc(&s->sort_cuts, 4 * static_cast<size_t>(rows) * sizeof(uint32_t)));
    CREATE_CHECK(hipMalloc(&s->sort_part_counts, rows * kMaxSortParts * 256 * sizeof(uint32_t)));
    s->term_sum_parts = (max_vocab + kTermsThreads * kTermsPerThread - 1) / (kTermsThreads * kTermsPerThread);
    s->chunk_capacity = max_vocab / kReplayChunk + 1;
    CREATE_CHECK(hipMalloc(&s->term_sums, rows * s->term_sum_parts * sizeof(double)));
    CREATE_CHECK(hipMalloc(&s->chunk_steps, rows * s->chunk_capacity * sizeof(uint4)));
    CREATE_CHECK(hipMalloc(&s->distribution_ids, static_cast<size_t>(max_vocab) * sizeof(int32_t)));
    CREATE_CHECK(hipMalloc(&s->distribution_probabilities, static_cast<size_t>(max_vocab) * sizeof(float)));
    CREATE_CHECK(hipMalloc(&s->distribution_count, sizeof(uint32_t)));
    constexpr size_t kVerifyRows = 2 * NCNN_MOE_MAX_DRAFT_TOKENS + 1;
    CREATE_CHECK(hipMalloc(&s->verify_ids, kVerifyRows * kVerifyCap * sizeof(int32_t)));
    CREATE_CHECK(hipMalloc(&s->verify_probabilities, kVerifyRows * kVerifyCap * sizeof(float)));
    CREATE_CHECK(hipMalloc(&s->verify_counts, kVerifyRows * sizeof(uint32_t)));
    // lists that hold whole rows and two dense vectors over the vocabulary, for steps whose filtered
    // distributions are longer than kVerifyCap (a handle for fewer rows than a step needs never gets there)
    if (max_rows >= 3)
    {
        const size_t long_rows = std::min<size_t>(kVerifyRows, rows);
        CREATE_CHECK(hipMalloc(&s->verify_long_ids, long_rows * max_vocab * sizeof(int32_t)));
        CREATE_CHECK(hipMalloc(&s->verify_long_probabilities, long_rows * max_vocab * sizeof(float)));
        CREATE_CHECK(hipMalloc(&s->verify_dense, 2 * static_cast<size_t>(max_vocab) * sizeof(float)));
    }
    CREATE_CHECK(hipHostMalloc(&s->verify_input_host, sizeof(ncnn_moe_hip_sampler::VerifyInput), hipHostMallocDefault));
    CREATE_CHECK(hipHostMalloc(&s->verify_output_host, sizeof(ncnn_moe_hip_sampler::VerifyOutput), hipHostMallocDefault));
    CREATE_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&s->verify_input_mapped), s->verify_input_host, 0));
    CREATE_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&s->verify_output_mapped), s->verify_output_host, 0));
    CREATE_CHECK(hipMalloc(&s->single_params, sizeof(ncnn_moe_sample_params)));
    CREATE_CHECK(hipMalloc(&s->single_uniform, sizeof(float)));
    CREATE_CHECK(hipMalloc(&s->single_result, sizeof(ncnn_moe_sample_result)));
    CREATE_CHECK(hipDeviceSynchronize());
#undef CREATE_CHECK
    *out = s;
    return NCNN_MOE_SAMPLER_SUCCESS;
}

void ncnn_moe_hip_sampler_destroy(ncnn_moe_hip_sampler* s)
{
    if (s == nullptr)
        return;
    (void)hipSetDevice(s->device);
    if (s->stream != nullptr)
    {
        (void)hipStreamSynchronize(s->stream);
        (void)hipStreamDestroy(s->stream);
    }
    if (s->side_stream != nullptr)
    {
        (void)hipStreamSynchronize(s->side_stream);
        (void)hipStreamDestroy(s->side_stream);
    }
    if (s->side_fork != nullptr)
        (void)hipEventDestroy(s->side_fork);
    if (s->side_join != nullptr)
        (void)hipEventDestroy(s->side_join);
    if (s->cut_done != nullptr)
        (void)hipEventDestroy(s->cut_done);
    void* buffers[] = {
        s->logits, s->params, s->uniforms, s->results, s->segment_values, s->segment_indices,
        s->segment_counts, s->row_counter, s->row_flags, s->row_state, s->split_records, s->row_epoch, s->sort_keys[0], s->sort_keys[1],
        s->sort_indices[0], s->sort_indices[1], s->sort_part_counts, s->row_list, s->sort_cuts, s->term_sums, s->chunk_steps, s->distribution_ids, s->distribution_probabilities,
        s->distribution_count, s->single_params, s->single_uniform, s->single_result, s->verify_ids,
        s->verify_probabilities, s->verify_counts, s->verify_long_ids, s->verify_long_probabilities, s->verify_dense};
    for (void* buffer : buffers)
    {
        if (buffer != nullptr)
            (void)hipFree(buffer);
    }
    if (s->input_block_host != nullptr)
        (void)hipHostFree(s->input_block_host);
    if (s->results_host != nullptr)
        (void)hipHostFree(s->results_host);
    if (s->verify_input_host != nullptr)
        (void)hipHostFree(s->verify_input_host);
    if (s->verify_output_host != nullptr)
        (void)hipHostFree(s->verify_output_host);
    delete s;
}

int ncnn_moe_hip_sampler_logits_buffer(
    ncnn_moe_hip_sampler* s, int dtype, uint32_t rows, uint32_t vocab,
    void** device_logits, uint64_t* row_stride)
{
    if (s == nullptr || device_logits == nullptr || row_stride == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    const int rc = check_shape(s, dtype, rows, vocab);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return rc;
    s->logits_dtype = dtype;
    s->logits_rows = rows;
    s->logits_vocab = vocab;
    // rows start on 16-byte boundaries: 4 fp32 or 8 bf16 elements
    s->logits_stride = round_up(vocab, dtype == NCNN_MOE_LOGITS_F32 ? 4 : 8);
    *device_logits = s->logits;
    *row_stride = s->logits_stride;
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_upload_logits(
    ncnn_moe_hip_sampler* s, const void* host_logits, int dtype,
    uint32_t rows, uint32_t vocab, uint64_t row_stride)
{
    if (s == nullptr || host_logits == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    void* device_logits = nullptr;
    uint64_t device_stride = 0;
    const int rc = ncnn_moe_hip_sampler_logits_buffer(s, dtype, rows, vocab, &device_logits, &device_stride);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return rc;
    if (row_stride < vocab)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "row_stride is smaller than vocab");
    if (vocab == 0)
        return NCNN_MOE_SAMPLER_SUCCESS;
    const size_t element = dtype == NCNN_MOE_LOGITS_F32 ? 4 : 2;
    SAMPLER_HIP_CHECK(s, hipSetDevice(s->device));
    SAMPLER_HIP_CHECK(s, hipMemcpy2DAsync(
        device_logits, device_stride * element, host_logits, row_stride * element,
        static_cast<size_t>(vocab) * element, rows, hipMemcpyHostToDevice, s->stream));
    SAMPLER_HIP_CHECK(s, hipStreamSynchronize(s->stream));
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_sample(
    ncnn_moe_hip_sampler* s, uint32_t rows,
    const ncnn_moe_sample_params* params, const float* uniforms,
    const int32_t* stop_ids, uint32_t stop_id_count,
    ncnn_moe_sample_result* results)
{
    if (s == nullptr || params == nullptr || uniforms == nullptr || results == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    if (rows == 0 || rows > s->logits_rows)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "rows exceeds the rows of the logits buffer");
    if (stop_id_count > 0 && stop_ids == nullptr)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "stop_id_count is positive and stop_ids is null");
    for (uint32_t row = 0; row < rows; ++row)
    {
        const uint64_t end = static_cast<uint64_t>(params[row].stop_begin) + params[row].stop_count;
        if (params[row].stop_count != 0 && (stop_ids == nullptr || end > stop_id_count))
            return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "a row's stop-id slice lies outside stop_ids");
    }
    if (s->logits_vocab == 0)
    {
        // src/engine/session.cpp:397-400
        for (uint32_t row = 0; row < rows; ++row)
        {
            results[row] = ncnn_moe_sample_result{-1, 0.0f, 0u, NCNN_MOE_ROW_EMPTY_LOGITS, 0, 0, 0};
        }
        return NCNN_MOE_SAMPLER_SUCCESS;
    }
    SAMPLER_HIP_CHECK(s, hipSetDevice(s->device));
    // params, uniforms and stop ids are staged in one pinned block that the kernels read in place (a few
    // dozen bytes per workgroup over the host link, behind the first logits loads); the block has room for
    // max(64 * max_rows, max_vocab) stop ids, and a call with more is refused (nothing is allocated here)
    const ncnn_moe_sample_params* device_params = reinterpret_cast<const ncnn_moe_sample_params*>(s->input_block_mapped);
    const float* device_uniforms = reinterpret_cast<const float*>(s->input_block_mapped + s->input_uniforms_offset);
    const int32_t* device_stops = nullptr;
    std::memcpy(s->input_block_host, params, rows * sizeof(ncnn_moe_sample_params));
    std::memcpy(s->input_block_host + s->input_uniforms_offset, uniforms, rows * sizeof(float));
    if (stop_id_count > 0 && stop_id_count <= s->input_stop_capacity)
    {
        std::memcpy(s->input_block_host + s->input_stops_offset, stop_ids, static_cast<size_t>(stop_id_count) * sizeof(int32_t));
        device_stops = reinterpret_cast<const int32_t*>(s->input_block_mapped + s->input_stops_offset);
    }
    else if (stop_id_count > 0)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "more stop ids than the handle holds (max(64 * max_rows, max_vocab))");
    // the host sees the options: the later passes are enqueued only if some row needs them
    SamplerPasses passes;
    passes.full_order = s->force_general != 0;
    uint32_t wide_rows = 0;
    uint32_t full_order_rows = 0;
    for (uint32_t row = 0; row < rows; ++row)
    {
        const bool beyond_select = row_left_pending(params[row], s->logits_vocab, kSelectTopK);
        const bool beyond_fast = !beyond_select && row_left_pending(params[row], s->logits_vocab, kFastTopK);
        passes.wide_select = passes.wide_select || beyond_fast;
        passes.full_order = passes.full_order || beyond_select;
        wide_rows += beyond_fast ? 1u : 0u;
        full_order_rows += beyond_select ? 1u : 0u;
    }
    // enough rows of each kind for the two passes to be worth the hand-over between two streams
    passes.side_by_side = wide_rows >= kSideBySideRows && full_order_rows >= kSideBySideRows;
    const bool full_order = passes.full_order;
    int rc = launch_sampler(
        s, s->logits, s->logits_dtype, rows, s->logits_vocab, s->logits_stride,
        device_params, device_uniforms, device_stops, s->results_host_device, DistributionExport{}, passes, s->stream);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return rc;
    SAMPLER_HIP_CHECK(s, hipStreamSynchronize(s->stream));
    if (!full_order)
    {
        // a row whose ties overflowed the select buffers is finished by the full-order kernels
        bool pending = false;
        for (uint32_t row = 0; row < rows && !pending; ++row)
            pending = s->results_host[row].status == NCNN_MOE_ROW_NEEDS_FULL_ORDER;
        if (pending)
        {
            SamplerPasses retry;
            retry.select = false;
            retry.full_order = true;
            rc = launch_sampler(
                s, s->logits, s->logits_dtype, rows, s->logits_vocab, s->logits_stride,
                device_params, device_uniforms, device_stops, s->results_host_device, DistributionExport{}, retry, s->stream);
            if (rc != NCNN_MOE_SAMPLER_SUCCESS)
                return rc;
            SAMPLER_HIP_CHECK(s, hipStreamSynchronize(s->stream));
        }
    }
    std::memcpy(results, s->results_host, rows * sizeof(ncnn_moe_sample_result));
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_sample_device(
    ncnn_moe_hip_sampler* s,
    const void* device_logits, int dtype, uint32_t rows, uint32_t vocab, uint64_t row_stride,
    const ncnn_moe_sample_params* device_params, const float* device_uniforms,
    const int32_t* device_stop_ids,
    ncnn_moe_sample_result* device_results, int may_need_full_order, void* stream)
{
    if (s == nullptr || device_logits == nullptr || device_params == nullptr || device_uniforms == nullptr ||
        device_results == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    const int rc = check_shape(s, dtype, rows, vocab);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return rc;
    if (vocab == 0)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "vocab must be positive");
    if (row_stride < vocab)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "row_stride is smaller than vocab");
    SAMPLER_HIP_CHECK(s, hipSetDevice(s->device));
    SamplerPasses passes;
    passes.wide_select = may_need_full_order != 0 && (may_need_full_order & NCNN_MOE_PASSES_NO_WIDE_WINDOWS) == 0;
    passes.full_order = may_need_full_order != 0 || s->force_general != 0;
    passes.side_by_side = passes.wide_select && (may_need_full_order & NCNN_MOE_PASSES_SIDE_BY_SIDE) != 0;
    return launch_sampler(
        s, device_logits, dtype, rows, vocab, row_stride, device_params, device_uniforms, device_stop_ids,
        device_results, DistributionExport{}, passes, static_cast<hipStream_t>(stream));
}

int ncnn_moe_hip_sampler_sample_device_static(
    int device,
    const void* device_logits, int dtype, uint32_t rows, uint32_t vocab, uint64_t row_stride,
    const ncnn_moe_sample_params* device_params, const float* device_uniforms,
    const int32_t* device_stop_ids,
    ncnn_moe_sample_result* device_results, void* stream)
{
    g_static_error[0] = 0;
    if (device_logits == nullptr || device_params == nullptr || device_uniforms == nullptr || device_results == nullptr)
        return static_fail(NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "a device pointer is null");
    if (dtype != NCNN_MOE_LOGITS_F32 && dtype != NCNN_MOE_LOGITS_BF16)
        return static_fail(NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "unknown logits dtype");
    if (rows == 0 || rows > kStaticMaxRows)
        return static_fail(NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "rows must be in [1, NCNN_MOE_STATIC_MAX_ROWS]");
    if (vocab == 0)
        return static_fail(NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "vocab must be positive");
    if (row_stride < vocab)
        return static_fail(NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "row_stride is smaller than vocab");
    if (device < 0 || device >= kStaticMaxDevices)
        return static_fail(NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "device index out of range");
    hipError_t error = hipSetDevice(device);
    if (error != hipSuccess)
        return static_fail(NCNN_MOE_SAMPLER_HIP_ERROR, "hipSetDevice", hipGetErrorString(error));
    const hipStream_t on = static_cast<hipStream_t>(stream);
    StaticScratchLayout* layout = nullptr;
    {
        // Set-up, once per device, with that device current: this GPU's address of the array.
        std::lock_guard<std::mutex> lock(g_static_mutex);
        if (g_static_scratch[device] == nullptr)
        {
            void* address = nullptr;
            error = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
            if (error != hipSuccess || address == nullptr)
                return static_fail(NCNN_MOE_SAMPLER_HIP_ERROR, "hipGetSymbolAddress(scratch)", hipGetErrorString(error));
            constexpr uint32_t kClearThreads = 256;
            constexpr uint32_t kClearWords = std::max<uint32_t>(kStaticSplitRows * kSplitMaxSegments, kStaticMaxRows);
            hipLaunchKernelGGL(static_scratch_clear_kernel, dim3((kClearWords + kClearThreads - 1) / kClearThreads), dim3(kClearThreads), 0, on,
                               static_cast<StaticScratchLayout*>(address));
            error = hipGetLastError();
            // The first call on a device waits for the clearing kernel: a second caller, on another stream,
            // finds the pointer only once the array is in the state every launch expects.
            if (error == hipSuccess)
                error = hipStreamSynchronize(on);
            if (error != hipSuccess)
                return static_fail(NCNN_MOE_SAMPLER_HIP_ERROR, "clearing the static scratch", hipGetErrorString(error));
            g_static_scratch[device] = static_cast<StaticScratchLayout*>(address);
        }
        layout = g_static_scratch[device];
    }
    SamplerArgs a;
    std::memset(&a, 0, sizeof(a));
    a.logits = device_logits;
    a.row_stride = row_stride;
    a.rows = rows;
    a.vocab = vocab;
    a.params = device_params;
    a.uniforms = device_uniforms;
    a.stop_ids = device_stop_ids;
    a.results = device_results;
    use_select_scratch(a, SelectScratch{layout->segment_values, layout->segment_indices, layout->segment_counts,
                                        layout->row_counter, layout->row_flags, layout->row_state,
                                        layout->split_records, layout->row_epoch});
    const SelectGeometry geometry = select_geometry(dtype, logits_span(vocab, dtype, device_logits, row_stride), rows, false);
    if (geometry.segments > 1 && rows > kStaticSplitRows)
        return static_fail(NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "the batch shape needs more segment records than the static scratch holds");
    if (dtype == NCNN_MOE_LOGITS_F32)
        launch_select<NCNN_MOE_LOGITS_F32>(geometry, rows, on, a, false, false);
    else
        launch_select<NCNN_MOE_LOGITS_BF16>(geometry, rows, on, a, false, false);
    error = hipGetLastError();
    if (error != hipSuccess)
        return static_fail(NCNN_MOE_SAMPLER_HIP_ERROR, "select kernel launch", hipGetErrorString(error));
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_distribution(
    ncnn_moe_hip_sampler* s, uint32_t row, const ncnn_moe_sample_params* params,
    uint32_t cap, int32_t* ids, float* probabilities, uint32_t* count, uint32_t* status)
{
    if (s == nullptr || params == nullptr || count == nullptr || status == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    if (cap > 0 && (ids == nullptr || probabilities == nullptr))
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    if (row >= s->logits_rows)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "row lies outside the logits buffer");
    *count = 0;
    if (s->logits_vocab == 0)
    {
        *status = NCNN_MOE_ROW_EMPTY_LOGITS;
        return NCNN_MOE_SAMPLER_SUCCESS;
    }
    SAMPLER_HIP_CHECK(s, hipSetDevice(s->device));
    ncnn_moe_sample_params single = *params;
    single.stop_begin = 0;
    single.stop_count = 0;
    const float uniform = 0.5f;
    SAMPLER_HIP_CHECK(s, hipMemcpyAsync(s->single_params, &single, sizeof(single), hipMemcpyHostToDevice, s->stream));
    SAMPLER_HIP_CHECK(s, hipMemcpyAsync(s->single_uniform, &uniform, sizeof(uniform), hipMemcpyHostToDevice, s->stream));
    const size_t element = s->logits_dtype == NCNN_MOE_LOGITS_F32 ? 4 : 2;
    const char* row_logits = static_cast<const char*>(s->logits) + static_cast<size_t>(row) * s->logits_stride * element;
    SamplerPasses distribution_passes;
    distribution_passes.full_order = true;
    DistributionExport single_row_export;
    single_row_export.ids = s->distribution_ids;
    single_row_export.probabilities = s->distribution_probabilities;
    single_row_export.count = s->distribution_count;
    single_row_export.cap = s->max_vocab;
    const int rc = launch_sampler(
        s, row_logits, s->logits_dtype, 1, s->logits_vocab, s->logits_stride,
        s->single_params, s->single_uniform, nullptr, s->single_result, single_row_export, distribution_passes, s->stream);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return rc;
    ncnn_moe_sample_result result;
    uint32_t kept = 0;
    SAMPLER_HIP_CHECK(s, hipMemcpyAsync(&result, s->single_result, sizeof(result), hipMemcpyDeviceToHost, s->stream));
    SAMPLER_HIP_CHECK(s, hipMemcpyAsync(&kept, s->distribution_count, sizeof(kept), hipMemcpyDeviceToHost, s->stream));
    SAMPLER_HIP_CHECK(s, hipStreamSynchronize(s->stream));
    *status = result.status;
    *count = kept;
    const uint32_t n = kept < cap ? kept : cap;
    if (n > 0)
    {
        SAMPLER_HIP_CHECK(s, hipMemcpy(ids, s->distribution_ids, static_cast<size_t>(n) * sizeof(int32_t), hipMemcpyDeviceToHost));
        SAMPLER_HIP_CHECK(s, hipMemcpy(probabilities, s->distribution_probabilities, static_cast<size_t>(n) * sizeof(float), hipMemcpyDeviceToHost));
    }
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_speculative_verify(
    ncnn_moe_hip_sampler* s, uint32_t draft_count,
    const ncnn_moe_sample_params* options, const int32_t* proposed_token_ids, const float* uniforms,
    float* accepted_probabilities, ncnn_moe_verify_result* result)
{
    if (s == nullptr || options == nullptr || proposed_token_ids == nullptr || uniforms == nullptr ||
        accepted_probabilities == nullptr || result == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    if (draft_count == 0 || draft_count > NCNN_MOE_MAX_DRAFT_TOKENS)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "draft_count must be in [1, NCNN_MOE_MAX_DRAFT_TOKENS]");
    const uint32_t rows = 2u * draft_count + 1u;
    if (s->logits_rows != rows)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "the logits buffer must hold 2 * draft_count + 1 rows");
    *result = ncnn_moe_verify_result{0u, -1, 0.0f, NCNN_MOE_VERIFY_OK, NCNN_MOE_ROW_OK, 0u, 0u, 0u};
    if (s->logits_vocab == 0)
    {
        // every row reports "cannot sample empty logits" (src/engine/session.cpp:397-400)
        result->status = NCNN_MOE_VERIFY_ROW_ERROR;
        result->row_status = NCNN_MOE_ROW_EMPTY_LOGITS;
        return NCNN_MOE_SAMPLER_SUCCESS;
    }
    ncnn_moe_sample_params row_options = *options;
    row_options.stop_begin = 0;
    row_options.stop_count = 0;
    SAMPLER_HIP_CHECK(s, hipSetDevice(s->device));
    ncnn_moe_hip_sampler::VerifyInput& in = *s->verify_input_host;
    for (uint32_t row = 0; row < rows; ++row)
    {
        in.params[row] = row_options;
        in.row_uniforms[row] = 0.0f;
    }
    in.row_uniforms[draft_count] = uniforms[draft_count]; // the draw of the row after the last drafted token
    std::memcpy(in.proposed, proposed_token_ids, draft_count * sizeof(int32_t));
    std::memcpy(in.uniforms, uniforms, (draft_count + 1) * sizeof(float));
    // The small operands are read by the kernels from the pinned block itself and the outcome is written
    // into the other one: no copy is enqueued on either side of the two launches.
    DistributionExport export_to;
    export_to.ids = s->verify_ids;
    export_to.probabilities = s->verify_probabilities;
    export_to.count = s->verify_counts;
    export_to.cap = kVerifyCap;
    VerifyArgs v;
    v.draft_count = draft_count;
    v.temperature = row_options.temperature;
    v.row_results = s->results;
    v.distribution_ids = s->verify_ids;
    v.distribution_probabilities = s->verify_probabilities;
    v.distribution_count = s->verify_counts;
    v.proposed = s->verify_input_mapped->proposed;
    v.uniforms = s->verify_input_mapped->uniforms;
    v.accepted_probabilities = s->verify_output_mapped->accepted;
    v.result = &s->verify_output_mapped->result;
    // the host sees the options: the later passes are enqueued only if the rows can need them; a row whose
    // ties overflow the select lists reports that, and the step is run again with the full-order kernels
    SamplerPasses passes;
    passes.full_order = s->force_general != 0 || row_left_pending(row_options, s->logits_vocab, kSelectTopK);
    passes.wide_select = !passes.full_order && row_left_pending(row_options, s->logits_vocab, kFastTopK);
    bool dense = s->verify_dense_known && std::memcmp(&s->verify_dense_options, &row_options, sizeof(row_options)) == 0;
    for (int attempt = 0; attempt < 2 && !dense; ++attempt)
    {
        const int rc = launch_sampler(
            s, s->logits, s->logits_dtype, rows, s->logits_vocab, s->logits_stride,
            s->verify_input_mapped->params, s->verify_input_mapped->row_uniforms, nullptr, s->results, export_to, passes, s->stream);
        if (rc != NCNN_MOE_SAMPLER_SUCCESS)
            return rc;
        hipLaunchKernelGGL(speculative_verify_kernel, dim3(1), dim3(kVerifyThreads), 0, s->stream, v);
        SAMPLER_HIP_CHECK(s, hipGetLastError());
        SAMPLER_HIP_CHECK(s, hipStreamSynchronize(s->stream));
        const ncnn_moe_verify_result& outcome = s->verify_output_host->result;
        const bool row_pending = outcome.status == NCNN_MOE_VERIFY_ROW_ERROR && outcome.row_status == NCNN_MOE_ROW_NEEDS_FULL_ORDER;
        if (!row_pending || passes.full_order)
            break;
        passes = SamplerPasses{};
        passes.select = false;
        passes.full_order = true;
    }
    if (!dense && s->verify_output_host->result.status == NCNN_MOE_VERIFY_UNSUPPORTED_WINDOW)
    {
        dense = true;
        s->verify_dense_known = true;
        s->verify_dense_options = row_options;
    }
    if (dense)
    {
        // A filtered distribution longer than the lists above: the step is run (again) with lists that
        // hold a whole row each and the kernel that builds the residual as a dense vector.
        export_to.ids = s->verify_long_ids;
        export_to.probabilities = s->verify_long_probabilities;
        export_to.cap = s->logits_vocab;
        VerifyDenseArgs d;
        d.step = v;
        d.step.distribution_ids = s->verify_long_ids;
        d.step.distribution_probabilities = s->verify_long_probabilities;
        d.list_cap = s->logits_vocab;
        d.vocab = s->logits_vocab;
        d.dense_draft = s->verify_dense;
        d.dense_residual = s->verify_dense + s->max_vocab;
        SamplerPasses every_pass;
        every_pass.wide_select = row_left_pending(row_options, s->logits_vocab, kFastTopK);
        every_pass.full_order = true;
        const int rc = launch_sampler(
            s, s->logits, s->logits_dtype, rows, s->logits_vocab, s->logits_stride,
            s->verify_input_mapped->params, s->verify_input_mapped->row_uniforms, nullptr, s->results, export_to, every_pass, s->stream);
        if (rc != NCNN_MOE_SAMPLER_SUCCESS)
            return rc;
        hipLaunchKernelGGL(speculative_verify_dense_kernel, dim3(1), dim3(kReplayThreads), 0, s->stream, d);
        SAMPLER_HIP_CHECK(s, hipGetLastError());
        SAMPLER_HIP_CHECK(s, hipStreamSynchronize(s->stream));
    }
    *result = s->verify_output_host->result;
    std::memcpy(accepted_probabilities, s->verify_output_host->accepted, draft_count * sizeof(float));
    return NCNN_MOE_SAMPLER_SUCCESS;
}

const char* ncnn_moe_hip_sampler_verify_status_message(int verify_status)
{
    switch (verify_status)
    {
    case NCNN_MOE_VERIFY_OK: return "";
    case NCNN_MOE_VERIFY_ROW_ERROR: return "a sampled row failed";
    case NCNN_MOE_VERIFY_ZERO_DRAFT_PROBABILITY: return "sampled draft token has zero probability";
    case NCNN_MOE_VERIFY_RESIDUAL_EMPTY: return "speculative residual distribution is empty";
    case NCNN_MOE_VERIFY_RESIDUAL_FAILED: return "speculative residual sampling failed";
    case NCNN_MOE_VERIFY_UNSUPPORTED_WINDOW: return "a filtered distribution exceeds the verification lists";
    default: return "unknown verification status";
    }
}

const char* ncnn_moe_hip_sampler_last_error(const ncnn_moe_hip_sampler* s)
{
    return s == nullptr ? g_static_error : s->last_error.c_str();
}

const char* ncnn_moe_hip_sampler_status_message(int row_status)
{
    switch (row_status)
    {
    case NCNN_MOE_ROW_OK: return "";
    case NCNN_MOE_ROW_EMPTY_LOGITS: return "cannot sample empty logits";
    case NCNN_MOE_ROW_BAD_TEMPERATURE: return "temperature must be finite and non-negative";
    case NCNN_MOE_ROW_BAD_TOP_P: return "top_p must be in the range (0, 1]";
    case NCNN_MOE_ROW_BAD_MIN_P: return "min_p must be in the range [0, 1]";
    case NCNN_MOE_ROW_NO_FINITE_LOGIT: return "sampling requires at least one finite logit";
    case NCNN_MOE_ROW_INVALID_DISTRIBUTION: return "sampling distribution is invalid";
    default: return "unknown row status";
    }
}

// ---- test hooks (include/ncnn_moe_hip_sampler_testing.h): compiled into the testing build of the library only
#ifdef NCNN_MOE_TESTING
int ncnn_moe_hip_sampler_debug_force_general(ncnn_moe_hip_sampler* s, int enabled)
{
    if (s == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    s->force_general = enabled ? 1 : 0;
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_debug_spread_sort(ncnn_moe_hip_sampler* s, int enabled)
{
    if (s == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    s->spread_sort = enabled ? 1 : 0;
    return NCNN_MOE_SAMPLER_SUCCESS;
}

// Full-order fp32 rows sorted only as far as their terms can move a sum (the default), or always whole.
int ncnn_moe_hip_sampler_debug_partial_sort(ncnn_moe_hip_sampler* s, int enabled)
{
    if (s == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    s->partial_sort = enabled ? 1 : 0;
    return NCNN_MOE_SAMPLER_SUCCESS;
}

// The spread sort of full-order fp32 rows in three passes and a touch-up of the lowest byte (the default), or in four.
int ncnn_moe_hip_sampler_debug_skip_low_digit(ncnn_moe_hip_sampler* s, int enabled)
{
    if (s == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    s->skip_low_digit = enabled ? 1 : 0;
    return NCNN_MOE_SAMPLER_SUCCESS;
}

// The wide select's bound for windows wider than 512: from a sample of the whole row (the default) or from the first chunk.
int ncnn_moe_hip_sampler_debug_wide_sampled_bound(ncnn_moe_hip_sampler* s, int enabled)
{
    if (s == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    s->wide_sampled_bound = enabled ? 1 : 0;
    return NCNN_MOE_SAMPLER_SUCCESS;
}

// Which rows of the last call the touch-up of the lowest byte could not put in order (1; they were sorted whole).
int ncnn_moe_hip_sampler_debug_disordered_rows(ncnn_moe_hip_sampler* s, uint32_t* flags, uint32_t rows)
{
    if (s == nullptr || flags == nullptr || rows > s->max_rows)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    SAMPLER_HIP_CHECK(s, hipSetDevice(s->device));
    SAMPLER_HIP_CHECK(s, hipStreamSynchronize(s->stream));
    SAMPLER_HIP_CHECK(s, hipMemcpy(flags, s->sort_cuts + 3 * static_cast<size_t>(s->max_rows), rows * sizeof(uint32_t), hipMemcpyDeviceToHost));
    for (uint32_t row = 0; row < rows; ++row)
        flags[row] &= 1u; // (bit 1 marks the rows that were in no list of the call)
    return NCNN_MOE_SAMPLER_SUCCESS;
}

// The rows' sort lengths of the last call (0xffffffff: the row was, or is to be, sorted whole).
int ncnn_moe_hip_sampler_debug_sort_lengths(ncnn_moe_hip_sampler* s, uint32_t* lengths, uint32_t rows)
{
    if (s == nullptr || lengths == nullptr || rows > s->max_rows)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    SAMPLER_HIP_CHECK(s, hipSetDevice(s->device));
    SAMPLER_HIP_CHECK(s, hipStreamSynchronize(s->stream));
    std::vector<uint32_t> last_keys(rows);
    SAMPLER_HIP_CHECK(s, hipMemcpy(lengths, s->sort_cuts, rows * sizeof(uint32_t), hipMemcpyDeviceToHost));
    SAMPLER_HIP_CHECK(s, hipMemcpy(last_keys.data(), s->sort_cuts + s->max_rows, rows * sizeof(uint32_t), hipMemcpyDeviceToHost));
    for (uint32_t row = 0; row < rows; ++row)
    {
        if (last_keys[row] == 0xffffffffu)
            lengths[row] = 0xffffffffu;
    }
    return NCNN_MOE_SAMPLER_SUCCESS;
}

// Sets the launch number (epoch) of every row, of a handle's split records or, with a null handle, of the
// static scratch of `device` (which must have served a call before): tests start a few launches in front
// of the point where the epochs start over.
int ncnn_moe_hip_sampler_debug_set_row_epochs(ncnn_moe_hip_sampler* s, int device, uint32_t epoch)
{
    if (epoch == 0u || epoch > kSplitLastEpoch)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    uint32_t* epochs = nullptr;
    size_t count = 0;
    if (s != nullptr)
    {
        if (hipSetDevice(s->device) != hipSuccess)
            return NCNN_MOE_SAMPLER_HIP_ERROR;
        epochs = s->row_epoch;
        count = s->max_rows;
    }
    else
    {
        std::lock_guard<std::mutex> lock(g_static_mutex);
        if (device < 0 || device >= kStaticMaxDevices || g_static_scratch[device] == nullptr || hipSetDevice(device) != hipSuccess)
            return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
        epochs = g_static_scratch[device]->row_epoch;
        count = kStaticMaxRows;
    }
    if (hipDeviceSynchronize() != hipSuccess ||
        hipMemsetD32(reinterpret_cast<hipDeviceptr_t>(epochs), static_cast<int>(epoch), count) != hipSuccess ||
        hipDeviceSynchronize() != hipSuccess)
        return NCNN_MOE_SAMPLER_HIP_ERROR;
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_debug_fused_bf16(ncnn_moe_hip_sampler* s, int enabled)
{
    if (s == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    s->fused_bf16 = enabled ? 1 : 0;
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_debug_chunk_steps(ncnn_moe_hip_sampler* s, int enabled)
{
    if (s == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    s->chunk_steps_enabled = enabled ? 1 : 0;
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_debug_scatter_segments(ncnn_moe_hip_sampler* s, int enabled)
{
    if (s == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    s->scatter_segments = enabled ? 1 : 0;
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_debug_select_geometry(
    int dtype, uint32_t rows, uint32_t vocab, uint32_t* segments, uint32_t* chunks_per_segment, uint32_t* variant)
{
    if (segments == nullptr || chunks_per_segment == nullptr || variant == nullptr || rows == 0 || vocab == 0 ||
        (dtype != NCNN_MOE_LOGITS_F32 && dtype != NCNN_MOE_LOGITS_BF16))
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    const SelectGeometry g = select_geometry(dtype, vocab, rows, false);
    *segments = g.segments;
    *chunks_per_segment = g.chunks_per_segment;
    *variant = g.segments == 1 ? 0u : (g.looped ? 2u : 1u);
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_debug_stream_only(
    ncnn_moe_hip_sampler* s, const void* device_logits, int dtype, uint32_t rows, uint32_t vocab, uint64_t row_stride, void* stream)
{
    if (s == nullptr || device_logits == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    const int rc = check_shape(s, dtype, rows, vocab);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return rc;
    const SelectGeometry g = select_geometry(dtype, vocab, rows, false);
    if (g.looped || g.segments < 2 || row_stride < vocab)
        return fail(s, NCNN_MOE_SAMPLER_INVALID_ARGUMENT, "the stream-only probe has the split kernel's geometry: rows of 2 to 16 chunks in a batch below 256 rows");
    SAMPLER_HIP_CHECK(s, hipSetDevice(s->device));
    SamplerArgs a{};
    a.logits = device_logits;
    a.rows = rows;
    a.vocab = vocab;
    a.row_stride = row_stride;
    a.segments = g.segments;
    a.xcd_grouped = 1;
    // the sink: one word per wave, in the (unused here) segment records of the looped variant
    uint32_t* sink = reinterpret_cast<uint32_t*>(s->segment_values);
    const dim3 grid(((rows + 7u) / 8u) * 8u * g.segments, 1, 1);
    if (dtype == NCNN_MOE_LOGITS_F32)
        hipLaunchKernelGGL((split_stream_only_kernel<NCNN_MOE_LOGITS_F32>), grid, dim3(kScanThreads), 0, static_cast<hipStream_t>(stream), a, sink);
    else
        hipLaunchKernelGGL((split_stream_only_kernel<NCNN_MOE_LOGITS_BF16>), grid, dim3(kScanThreads), 0, static_cast<hipStream_t>(stream), a, sink);
    SAMPLER_HIP_CHECK(s, hipGetLastError());
    return NCNN_MOE_SAMPLER_SUCCESS;
}

int ncnn_moe_hip_sampler_debug_expf(ncnn_moe_hip_sampler* s, const float* in, float* out, size_t n)
{
    if (s == nullptr || in == nullptr || out == nullptr)
        return NCNN_MOE_SAMPLER_INVALID_ARGUMENT;
    if (n == 0)
        return NCNN_MOE_SAMPLER_SUCCESS;
    SAMPLER_HIP_CHECK(s, hipSetDevice(s->device));
    float* device_in = nullptr;
    float* device_out = nullptr;
    SAMPLER_HIP_CHECK(s, hipMalloc(&device_in, n * sizeof(float)));
    hipError_t error = hipMalloc(&device_out, n * sizeof(float));
    if (error == hipSuccess)
        error = hipMemcpy(device_in, in, n * sizeof(float), hipMemcpyHostToDevice);
    if (error == hipSuccess)
    {
        const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
        hipLaunchKernelGGL(expf_probe_kernel, dim3(blocks), dim3(256), 0, s->stream, device_in, device_out, n);
        error = hipGetLastError();
    }
    if (error == hipSuccess)
        error = hipStreamSynchronize(s->stream);
    if (error == hipSuccess)
        error = hipMemcpy(out, device_out, n * sizeof(float), hipMemcpyDeviceToHost);
    (void)hipFree(device_in);
    if (device_out != nullptr)
        (void)hipFree(device_out);
    if (error != hipSuccess)
        return hip_fail(s, error, "debug_expf");
    return NCNN_MOE_SAMPLER_SUCCESS;
}

#ifdef NCNN_MOE_TIMELINE
// Only in the library built with -DNCNN_MOE_TIMELINE: the wall-clock stamps (100 MHz ticks) that the split
// kernel's workgroups left, [64 rows][16 segments][16 slots].
int ncnn_moe_hip_sampler_debug_timeline(unsigned long long* out, size_t count)
{
    const size_t bytes = std::min(count * sizeof(unsigned long long), sizeof(unsigned long long) * kTimelineRows * kMaxSegments * kTimelineSlots);
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(ncnn_moe_hip::g_timeline), bytes) == hipSuccess ? NCNN_MOE_SAMPLER_SUCCESS : NCNN_MOE_SAMPLER_HIP_ERROR;
}

// ... and the stamps of the rows' last waves inside the epilogue, [64 rows][16 slots].
int ncnn_moe_hip_sampler_debug_timeline_rows(unsigned long long* out, size_t count)
{
    const size_t bytes = std::min(count * sizeof(unsigned long long), sizeof(unsigned long long) * kTimelineRows * kTimelineSlots);
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(ncnn_moe_hip::g_timeline_rows), bytes) == hipSuccess ? NCNN_MOE_SAMPLER_SUCCESS : NCNN_MOE_SAMPLER_HIP_ERROR;
}
#endif

void ncnn_moe_hip_sampler_debug_exp2_table(uint64_t out[32])
{
    static const uint64_t table[32] = {NCNN_MOE_EXP2_TABLE_VALUES};
    std::memcpy(out, table, sizeof(table));
}

#endif // NCNN_MOE_TESTING

} // extern "C"
