/*
 * Test hooks of the MI355X generation sampler library: exported by the same shared library, used by this
 * repository's tests only, and not part of the boundary that the runtime binds (no counterpart in the
 * runtime).
 */
#ifndef NCNN_MOE_HIP_SAMPLER_TESTING_H
#define NCNN_MOE_HIP_SAMPLER_TESTING_H

#include "ncnn_moe_hip_sampler.h"

#ifdef __cplusplus
extern "C" {
#endif

/* force_general routes every non-greedy row through the full-order path; scatter_segments launches
 * split rows without the XCD-aware numbering of the workgroups, so that the segments of a row run on
 * several XCDs and the merge finds their records outside its L2; expf evaluates the device exponential
 * on n host values. */
int ncnn_moe_hip_sampler_debug_force_general(ncnn_moe_hip_sampler* sampler, int enabled);
int ncnn_moe_hip_sampler_debug_scatter_segments(ncnn_moe_hip_sampler* sampler, int enabled);
/* A launch with the split select kernel's grid and loads and nothing behind them (each wave stores one word that
 * depends on its share of the chunk): what streaming the logits alone costs at that shape.  For the benchmark's
 * detail; batches below 256 rows with rows of 2 to 16 chunks. */
int ncnn_moe_hip_sampler_debug_stream_only(
    ncnn_moe_hip_sampler* sampler, const void* device_logits, int dtype, uint32_t rows, uint32_t vocab, uint64_t row_stride, void* stream);
/* chunk_steps (on by default): the composed steps of the whole chunks of a sorted fp32 row's terms are worked out by
 * a kernel of their own before the replay, which then adds such a chunk in one step; off, the replay runs every chunk's
 * round itself.  Same results either way. */
int ncnn_moe_hip_sampler_debug_chunk_steps(ncnn_moe_hip_sampler* sampler, int enabled);
/* spread_sort (on by default): the radix sort of a long full-order row runs on several workgroups; off,
 * every row is sorted by one workgroup. */
int ncnn_moe_hip_sampler_debug_spread_sort(ncnn_moe_hip_sampler* sampler, int enabled);
/* fused_bf16 (on by default): a bf16 full-order row is counted and walked by one kernel, its runs staying in LDS; off,
 * by the counting kernel and the replay kernel, with the runs in device memory between them.  Same results either way. */
int ncnn_moe_hip_sampler_debug_fused_bf16(ncnn_moe_hip_sampler* sampler, int enabled);
/* partial_sort (on by default): a full-order fp32 row whose sort is spread over the GPU is sorted only as far as its
 * terms can move one of the sampler's sums (a kernel guesses how far, the walk checks the guess against its exact sums
 * and has a row whose guess was too short sorted whole by a second launch); off, every row is sorted whole.  Same
 * results either way.  sort_lengths copies out, for the first `rows` rows of the last call, the number of elements that
 * were sorted (0xffffffff: the whole row; only rows that took the spread sort with partial_sort on are written). */
int ncnn_moe_hip_sampler_debug_partial_sort(ncnn_moe_hip_sampler* sampler, int enabled);
int ncnn_moe_hip_sampler_debug_sort_lengths(ncnn_moe_hip_sampler* sampler, uint32_t* lengths, uint32_t rows);
/* skip_low_digit (on by default, with partial_sort): that sort takes three passes, over the keys' upper 24 bits, and
 * the kernel that computes the terms puts the neighbours that agree in those bits in order; a row in which it cannot
 * (more such keys in a row than it looks at, and out of order) is sorted whole by the second launch.  Off: four passes.
 * Same results either way.  disordered_rows copies out, for the first `rows` rows of the last call, 1 for a row that
 * was handed to the second launch for this reason (written for the rows that partial_sort serves). */
int ncnn_moe_hip_sampler_debug_skip_low_digit(ncnn_moe_hip_sampler* sampler, int enabled);
int ncnn_moe_hip_sampler_debug_disordered_rows(ncnn_moe_hip_sampler* sampler, uint32_t* flags, uint32_t rows);
/* wide_sampled_bound (on by default): a row of four chunks or more whose Top-K window is wider than 512 gets the bound
 * under which the wide select collects its candidates from a sample of the whole row (a row whose list then ends short
 * of the window is handed to the full-order kernels); off, from the row's first chunk.  Same results either way. */
int ncnn_moe_hip_sampler_debug_wide_sampled_bound(ncnn_moe_hip_sampler* sampler, int enabled);
/* Sets the per-row launch numbers (epochs, 1 .. 8191) that tag the split kernel's hand-over records: of the
 * handle, or with a null handle of the static scratch of `device` (after it has served a call).  Tests start a
 * few launches in front of the point where the epochs start over. */
int ncnn_moe_hip_sampler_debug_set_row_epochs(ncnn_moe_hip_sampler* sampler, int device, uint32_t epoch);
int ncnn_moe_hip_sampler_debug_expf(ncnn_moe_hip_sampler* sampler, const float* in, float* out, size_t n);
void ncnn_moe_hip_sampler_debug_exp2_table(uint64_t out[32]);

/* How the first select kernel covers a batch of this shape (rows aligned to 16 bytes): workgroups per
 * row, chunks each of them streams, and the kernel variant (0: one workgroup streams and finishes a whole
 * row; 1: a row is split into one-chunk workgroups; 2: into workgroups that stream several chunks).  No
 * GPU needed. */
int ncnn_moe_hip_sampler_debug_select_geometry(
    int dtype, uint32_t rows, uint32_t vocab, uint32_t* segments, uint32_t* chunks_per_segment, uint32_t* variant);

#ifdef __cplusplus
}
#endif

#endif /* NCNN_MOE_HIP_SAMPLER_TESTING_H */
