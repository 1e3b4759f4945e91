/*
 * C ABI of the MI355X (gfx950) generation sampler.
 *
 * This is the boundary a maintainer of the runtime binds from src/backends/hip: plain pointers and
 * sizes, POD structs, no exceptions.  One handle serves one device; a handle is not re-entrant
 * (use one handle per scheduler worker, or serialise calls), matching the per-Session mutex of the
 * CPU sampler (src/engine/session.cpp:452-456).
 *
 * The sampler computes, per row of a [rows, vocab] logits matrix, exactly what the CPU path
 * Session::sample computes for one Session (src/engine/session.cpp:393-443, :76-136): option
 * validation, greedy argmax over finite logits, or the stable (logit descending, index ascending)
 * ordering, Top-K, softmax in that order with sequential fp32 sums, Min-P, Top-P, renormalisation
 * and the inverse-CDF draw, plus the stop-token test of the callers
 * (src/engine/session.cpp:60-63, examples/internal/run_model.cpp:790).  The uniform draw is
 * supplied per row by the caller, which owns the Session RNG (include/ncnn/moe/session.h:303).
 */
#ifndef NCNN_MOE_HIP_SAMPLER_H
#define NCNN_MOE_HIP_SAMPLER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ncnn_moe_hip_sampler ncnn_moe_hip_sampler;

/* Logits element type.  The runtime's logits tensor is fp32 (src/compiler/graph_builder.cpp:586-594);
 * bf16 rows are widened with bits << 16 (src/kernels/cpu_ops.cpp:26-32) before any arithmetic. */
enum ncnn_moe_logits_dtype
{
    NCNN_MOE_LOGITS_F32 = 0,
    NCNN_MOE_LOGITS_BF16 = 1
};

/* Call-level return codes.  Errors map to ErrorCode::InternalError (include/ncnn/moe/result.h:12-25)
 * except NCNN_MOE_SAMPLER_INVALID_ARGUMENT, which maps to ErrorCode::InvalidArgument. */
enum ncnn_moe_sampler_rc
{
    NCNN_MOE_SAMPLER_SUCCESS = 0,
    NCNN_MOE_SAMPLER_INVALID_ARGUMENT = 1,
    NCNN_MOE_SAMPLER_HIP_ERROR = 2,
    NCNN_MOE_SAMPLER_NO_DEVICE = 3
};

/* Per-row status: one value per fixed InvalidArgument message of the CPU sampler
 * (src/engine/session.cpp:68, :70, :72, :85 and :421, :103, :399).  A bad row does not fail the batch. */
enum ncnn_moe_row_status
{
    NCNN_MOE_ROW_OK = 0,
    NCNN_MOE_ROW_EMPTY_LOGITS = 1,
    NCNN_MOE_ROW_BAD_TEMPERATURE = 2,
    NCNN_MOE_ROW_BAD_TOP_P = 3,
    NCNN_MOE_ROW_BAD_MIN_P = 4,
    NCNN_MOE_ROW_NO_FINITE_LOGIT = 5,
    NCNN_MOE_ROW_INVALID_DISTRIBUTION = 6,
    /* Not a CPU-sampler error.  Only ncnn_moe_hip_sampler_sample_device called with
     * may_need_full_order = 0 reports it, for a row that the first select kernel cannot serve:
     * its Top-K window is absent or wider than 64, or its ties overflowed the select buffers.
     * Call again with may_need_full_order = 1. */
    NCNN_MOE_ROW_NEEDS_FULL_ORDER = 7
};

/* Bits of ncnn_moe_sample_result::flags. */
enum ncnn_moe_row_flags
{
    NCNN_MOE_ROW_FLAG_HAS_NAN = 1,       /* the row held a NaN; NaN logits are skipped, as greedy does */
    NCNN_MOE_ROW_FLAG_GENERAL_PATH = 2,  /* served by the full-order path rather than the Top-K select */
    NCNN_MOE_ROW_FLAG_FALLBACK = 4       /* the Top-K select overflowed its candidate buffers (heavy ties) */
};

/* SamplingOptions (include/ncnn/moe/session.h:49-55) plus the row's slice of the stop-id array
 * (GenerationOptions::stop_tokens, include/ncnn/moe/session.h:76-84). */
typedef struct ncnn_moe_sample_params
{
    float temperature;
    uint32_t top_k;
    float top_p;
    float min_p;
    uint32_t stop_begin;
    uint32_t stop_count;
} ncnn_moe_sample_params;

/* SampledToken (include/ncnn/moe/session.h:57-61) plus StreamToken::is_stop_token (:63-72). */
typedef struct ncnn_moe_sample_result
{
    int32_t token_id;      /* -1 unless status is NCNN_MOE_ROW_OK */
    float probability;
    uint32_t kept_count;   /* candidates left after Top-K, Min-P and Top-P; 1 for greedy */
    uint8_t status;        /* enum ncnn_moe_row_status */
    uint8_t is_stop;
    uint8_t draw_consumed; /* 1 iff the CPU sampler would have advanced the Session RNG (session.cpp:429-433) */
    uint8_t flags;         /* enum ncnn_moe_row_flags */
} ncnn_moe_sample_result;

/* Replaces nothing on the CPU side (the CPU sampler holds no state); plays the role of the static
 * create() of the runtime's backend operators (src/backends/ncnn/ncnn_linear.h:45-71).  Allocates the
 * device logits buffer and every scratch buffer up front for max_rows x max_vocab, so that sampling
 * itself allocates nothing. */
#define NCNN_MOE_SAMPLER_MAX_ROWS 65535 /* create() refuses more rows per handle */
int ncnn_moe_hip_sampler_create(int device, uint32_t max_rows, uint32_t max_vocab, ncnn_moe_hip_sampler** out);
void ncnn_moe_hip_sampler_destroy(ncnn_moe_hip_sampler* sampler);

/* Device-resident hand-off replacing the host copy of the LM-head output
 * (src/engine/cpu_executor.cpp:2449-2455, :2978-2999; src/kernels/cpu_ops.cpp:1166-1172): the decode
 * step writes [rows, vocab] logits of `dtype` at *device_logits with *row_stride elements per row. */
int ncnn_moe_hip_sampler_logits_buffer(
    ncnn_moe_hip_sampler* sampler, int dtype, uint32_t rows, uint32_t vocab,
    void** device_logits, uint64_t* row_stride);

/* Host rows -> the handle's logits buffer (LogitsOutput::values, include/ncnn/moe/session.h:30-33),
 * for callers whose logits still live on the host.  row_stride is in elements. */
int ncnn_moe_hip_sampler_upload_logits(
    ncnn_moe_hip_sampler* sampler, const void* host_logits, int dtype,
    uint32_t rows, uint32_t vocab, uint64_t row_stride);

/* The batched form of Session::sample (include/ncnn/moe/session.h:326, src/engine/session.cpp:452-456)
 * over the handle's logits buffer: replaces the serial per-session loop of
 * examples/internal/run_model.cpp:776-809.  All pointers are host memory; the call returns when
 * results[] is filled.  uniforms[row] is the draw the row's Session RNG would produce next.  At most
 * max(64 * max_rows, max_vocab) stop ids per call (they are staged in memory sized by create()). */
int ncnn_moe_hip_sampler_sample(
    ncnn_moe_hip_sampler* sampler, uint32_t rows,
    const ncnn_moe_sample_params* params, const float* uniforms,
    const int32_t* stop_ids, uint32_t stop_id_count,
    ncnn_moe_sample_result* results);

/* Same computation with every operand already in device memory and no host synchronisation:
 * kernels are enqueued on `stream` (a hipStream_t, or null for the default stream) and the call
 * returns at once.  device_logits may be any device matrix (row_stride in elements), not only the
 * handle's buffer.  This is the entry the decode step calls in its own stream.
 * may_need_full_order: pass 0 when the caller knows from its host-side SamplingOptions that every
 * row is greedy or has 1 <= top_k <= 64 (then one kernel is enqueued); pass 1 otherwise (a select
 * kernel for Top-K windows up to 1024 and the full-order kernels are enqueued as well and pick up
 * the rows that need them); pass 3 (1 | NCNN_MOE_PASSES_SIDE_BY_SIDE) when the caller knows that the
 * batch holds both rows with 64 < top_k <= 1024 and rows with a wider or no window: the two later
 * passes, each of which keeps one workgroup per row busy, then run side by side, one of them on a
 * second stream of the handle that forks from and joins `stream` (worth its two stream hand-overs,
 * some 30 us, from about a hundred rows of each kind; a row with top_k <= 64 whose ties overflow the
 * first kernel's lists is then finished by the full-order kernels rather than by the select kernel for
 * wider windows: same result, NCNN_MOE_ROW_FLAG_GENERAL_PATH set); add NCNN_MOE_PASSES_NO_WIDE_WINDOWS when the
 * caller knows that no row has 64 < top_k <= 1024: the select kernel for such windows is then not
 * enqueued (a row that has one after all is served by the full-order kernels: slower, same result).
 * Calls on one handle share its scratch memory and must not overlap. */
#define NCNN_MOE_PASSES_FULL_ORDER 1
#define NCNN_MOE_PASSES_SIDE_BY_SIDE 2
#define NCNN_MOE_PASSES_NO_WIDE_WINDOWS 4
int ncnn_moe_hip_sampler_sample_device(
    ncnn_moe_hip_sampler* sampler,
    const void* device_logits, int dtype, uint32_t rows, uint32_t vocab, uint64_t row_stride,
    const ncnn_moe_sample_params* device_params, const float* device_uniforms,
    const int32_t* device_stop_ids,
    ncnn_moe_sample_result* device_results, int may_need_full_order, void* stream);

/* No counterpart in the reference.  For callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  The select pass of
 * ncnn_moe_hip_sampler_sample_device (may_need_full_order = 0) without a handle: the call allocates
 * nothing, on the device or through any library; its scratch (the segments' candidate records and the
 * per-row hand-over words, 18.8 MB) is a static device array that every GPU the library runs on holds
 * from its first call until the process ends.  Greedy rows and rows with 1 <= top_k <= 64 are final;
 * any other row comes back NCNN_MOE_ROW_NEEDS_FULL_ORDER.  Limits: rows <= NCNN_MOE_STATIC_MAX_ROWS,
 * any vocab; a larger batch is rejected with NCNN_MOE_SAMPLER_INVALID_ARGUMENT and the reason is
 * ncnn_moe_hip_sampler_last_error(NULL) on the calling thread.  `device` is made current.  All calls on
 * one GPU share the one array: calls that overlap on a GPU (two streams, two threads) race; calls in
 * one stream, or otherwise ordered, do not.  The first call on a device looks the array up and
 * clears it on `stream`: make that call outside stream capture. */
#define NCNN_MOE_STATIC_MAX_ROWS 1024
int ncnn_moe_hip_sampler_sample_device_static(
    int device,
    const void* device_logits, int dtype, uint32_t rows, uint32_t vocab, uint64_t row_stride,
    const ncnn_moe_sample_params* device_params, const float* device_uniforms,
    const int32_t* device_stop_ids,
    ncnn_moe_sample_result* device_results, void* stream);

/* sampling_distribution (src/engine/session.cpp:76-136) for one row of the handle's logits buffer:
 * the filtered, renormalised (token id, probability) list in the CPU order.  Writes min(*count, cap)
 * entries.  Used by parity tests and by speculative verification (src/engine/session.cpp:799-804).
 * Returns the row status in *status (a greedy row yields NCNN_MOE_ROW_OK with its single token). */
int ncnn_moe_hip_sampler_distribution(
    ncnn_moe_hip_sampler* sampler, uint32_t row, const ncnn_moe_sample_params* params,
    uint32_t cap, int32_t* ids, float* probabilities, uint32_t* count, uint32_t* status);

/* Outcome of one speculative verification step. */
enum ncnn_moe_verify_status
{
    NCNN_MOE_VERIFY_OK = 0,
    /* a sampling error of a row that the accept loop reached; row_status holds the ncnn_moe_row_status
     * (the target row's error wins over the draft row's, src/engine/session.cpp:805-813) */
    NCNN_MOE_VERIFY_ROW_ERROR = 1,
    NCNN_MOE_VERIFY_ZERO_DRAFT_PROBABILITY = 2, /* "sampled draft token has zero probability" (:822-830) */
    NCNN_MOE_VERIFY_RESIDUAL_EMPTY = 3,         /* "speculative residual distribution is empty" (:170-175) */
    NCNN_MOE_VERIFY_RESIDUAL_FAILED = 4,        /* "speculative residual sampling failed" (:199-201) */
    /* Not a CPU-sampler error, and not returned by ncnn_moe_hip_sampler_speculative_verify: its first
     * kernel reports a filtered distribution (after Top-K, Min-P, Top-P) of more than 1024 candidates
     * with it, and the entry then runs the step again through the kernel that holds whole rows. */
    NCNN_MOE_VERIFY_UNSUPPORTED_WINDOW = 5
};

typedef struct ncnn_moe_verify_result
{
    uint32_t accepted;            /* draft tokens accepted, 0..draft_count */
    int32_t next_token_id;        /* the token emitted after them; -1 unless status is NCNN_MOE_VERIFY_OK */
    float next_probability;
    uint32_t status;              /* enum ncnn_moe_verify_status */
    uint32_t row_status;          /* enum ncnn_moe_row_status when status is NCNN_MOE_VERIFY_ROW_ERROR */
    uint32_t accept_draws;        /* uniforms[0 .. accept_draws) were consumed by the accept tests (:833-837) */
    uint32_t final_draw_consumed; /* 1 iff uniforms[accept_draws] was consumed by the last token's draw */
    uint32_t next_is_residual;    /* 1 iff the last token came from the residual distribution (:865-869) */
} ncnn_moe_verify_result;

enum { NCNN_MOE_MAX_DRAFT_TOKENS = 16 };

/* The verification step of speculative generation (src/engine/session.cpp:776-874 with
 * candidate_probability :138-148 and sample_residual_distribution :150-202) in one device pass.
 * The handle's logits buffer holds 2 * draft_count + 1 rows: rows [0, draft_count] are the target
 * model's logits after the anchor and after each proposed token, rows [draft_count + 1,
 * 2 * draft_count] the draft model's logits that proposed_token_ids[i] was sampled from.
 * options: one SamplingOptions for every row (the stop slice is ignored).  uniforms: the next
 * draft_count + 1 draws of the Session RNG in order; the accept test of position i uses uniforms[i],
 * the last token's draw uses the one after the last accept test.  accepted_probabilities receives
 * the probability reported for each accepted token (:839-841, 1.0 for greedy :795).
 * 1 <= draft_count <= NCNN_MOE_MAX_DRAFT_TOKENS.  All pointers are host memory. */
int ncnn_moe_hip_sampler_speculative_verify(
    ncnn_moe_hip_sampler* sampler, uint32_t draft_count,
    const ncnn_moe_sample_params* options, const int32_t* proposed_token_ids, const float* uniforms,
    float* accepted_probabilities, ncnn_moe_verify_result* result);

/* The fixed message of a verification status (src/engine/session.cpp:174, :201, :829). */
const char* ncnn_moe_hip_sampler_verify_status_message(int verify_status);

/* Error text of the last failed call on this handle (Error::message, include/ncnn/moe/result.h:21-25);
 * with a null handle, of the calling thread's last failed ncnn_moe_hip_sampler_sample_device_static. */
const char* ncnn_moe_hip_sampler_last_error(const ncnn_moe_hip_sampler* sampler);

/* The CPU sampler's fixed message for a row status (src/engine/session.cpp:68,70,72,85,103,399). */
const char* ncnn_moe_hip_sampler_status_message(int row_status);

/* Number of HIP devices visible, 0 if none (no counterpart: the CPU sampler needs no device). */
int ncnn_moe_hip_sampler_device_count(void);

#ifdef __cplusplus
}
#endif

#endif /* NCNN_MOE_HIP_SAMPLER_H */
