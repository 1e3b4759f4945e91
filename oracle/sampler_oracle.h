/*
 * CPU oracle for the generation sampler -- TEST INFRASTRUCTURE ONLY.
 *
 * This is a CPU restatement of the reference sampler's arithmetic, written to be the
 * checker for the HIP sampler.  It is never part of the shipped path: only tests,
 * the smoke check and the benchmark's cpu_baseline leg may load it.
 *
 * Every function cites the reference lines it restates (paths relative to the
 * reference checkout).  What pins each function is listed in sampler_oracle.cpp.
 */
#ifndef SAMPLER_ORACLE_H
#define SAMPLER_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* include/ncnn/moe/session.h:49-55 (SamplingOptions) */
typedef struct oracle_sampling_options
{
    float temperature;
    uint32_t top_k;
    float top_p;
    float min_p;
} oracle_sampling_options;

/* One status per fixed error message of src/engine/session.cpp:68,70,72,85,103,399,421 */
enum oracle_status
{
    ORACLE_OK = 0,
    ORACLE_EMPTY_LOGITS = 1,         /* "cannot sample empty logits" */
    ORACLE_BAD_TEMPERATURE = 2,      /* "temperature must be finite and non-negative" */
    ORACLE_BAD_TOP_P = 3,            /* "top_p must be in the range (0, 1]" */
    ORACLE_BAD_MIN_P = 4,            /* "min_p must be in the range [0, 1]" */
    ORACLE_NO_FINITE_LOGIT = 5,      /* "sampling requires at least one finite logit" */
    ORACLE_INVALID_DISTRIBUTION = 6  /* "sampling distribution is invalid" */
};

/* Per-row batch parameters: SamplingOptions plus a slice of a shared stop-id array. */
typedef struct oracle_row_params
{
    float temperature;
    uint32_t top_k;
    float top_p;
    float min_p;
    uint32_t stop_begin;
    uint32_t stop_count;
} oracle_row_params;

typedef struct oracle_row_result
{
    int32_t token_id;      /* SampledToken::token_id, -1 on error */
    float probability;     /* SampledToken::probability */
    uint32_t kept_count;   /* candidates left after Top-K / Min-P / Top-P (1 for greedy) */
    uint8_t status;        /* enum oracle_status */
    uint8_t is_stop;       /* token_id is in the row's stop list */
    uint8_t draw_consumed; /* the reference would have advanced the Session RNG */
    uint8_t has_nan;       /* row held a NaN (treated as skipped) */
    float cdf_gap;         /* min |u - CDF boundary| over the kept list (diagnostic) */
    float top_p_gap;       /* |final cumulative - top_p| when the Top-P scan stopped (diagnostic) */
} oracle_row_result;

const char* oracle_status_message(int status);

/* src/engine/session.cpp:65-74 */
int oracle_validate_sampling_options(const oracle_sampling_options* options);

/* src/engine/session.cpp:76-136.  Writes min(count, cap) entries; *count is the kept length. */
int oracle_sampling_distribution(
    const float* logits, size_t vocab,
    const oracle_sampling_options* options,
    int32_t* ids, float* probabilities, size_t cap, size_t* count);

/* src/engine/session.cpp:393-443 with the uniform supplied by the caller. */
int oracle_sample(
    const float* logits, size_t vocab,
    const oracle_sampling_options* options,
    float uniform,
    oracle_row_result* result);

/*
 * examples/internal/run_model.cpp:776-809: one sample() per row plus the stop-token test
 * (src/engine/session.cpp:60-63).  dtype 0 = fp32, 1 = bf16 widened by bits << 16
 * (src/kernels/cpu_ops.cpp:26-32).  threads > 1 partitions rows over std::thread.
 */
int oracle_sample_batch(
    const void* logits, int dtype, uint32_t rows, uint32_t vocab, uint64_t row_stride,
    const oracle_row_params* params, const float* uniforms,
    const int32_t* stop_ids,
    oracle_row_result* results, int threads);

/* Speculative verification.  Statuses beyond the row statuses of the accept loop. */
enum oracle_verify_status
{
    ORACLE_VERIFY_OK = 0,
    ORACLE_VERIFY_ROW_ERROR = 1,              /* row_status holds the failing row's oracle_status */
    ORACLE_VERIFY_ZERO_DRAFT_PROBABILITY = 2, /* "sampled draft token has zero probability" */
    ORACLE_VERIFY_RESIDUAL_EMPTY = 3,         /* "speculative residual distribution is empty" */
    ORACLE_VERIFY_RESIDUAL_FAILED = 4         /* "speculative residual sampling failed" */
};

typedef struct oracle_verify_result
{
    uint32_t accepted;
    int32_t next_token_id;
    float next_probability;
    uint32_t status;
    uint32_t row_status;
    uint32_t accept_draws;
    uint32_t final_draw_consumed;
    uint32_t next_is_residual;
} oracle_verify_result;

/* src/engine/session.cpp:138-148 */
float oracle_candidate_probability(const int32_t* ids, const float* probabilities, size_t count, int32_t token_id);

/* src/engine/session.cpp:150-202 with the canonical draw in [0, 1) supplied by the caller
 * (uniform_real_distribution<float>(0, normalizer) returns canonical * normalizer). */
int oracle_sample_residual_distribution(
    const int32_t* target_ids, const float* target_probabilities, size_t target_count,
    const int32_t* draft_ids, const float* draft_probabilities, size_t draft_count,
    size_t vocab, float canonical_uniform, int32_t* token_id, float* probability);

/* src/engine/session.cpp:776-874: the accept loop over draft_count proposed tokens and the token
 * that follows.  target_logits holds draft_count + 1 rows, draft_logits draft_count rows, uniforms
 * the next draft_count + 1 canonical draws of the Session RNG. */
int oracle_speculative_verify(
    const float* target_logits, const float* draft_logits, size_t vocab, uint32_t draft_count,
    const oracle_sampling_options* options, const int32_t* proposed_token_ids, const float* uniforms,
    float* accepted_probabilities, oracle_verify_result* result);

/* src/kernels/cpu_ops.cpp:26-40 */
float oracle_bfloat16_to_float(uint16_t value);
uint16_t oracle_float_to_bfloat16(float value);
void oracle_quantize_bfloat16(const float* in, uint16_t* out, size_t n);

/*
 * Session RNG in lock-step: std::mt19937_64(seed) (src/engine/session.cpp:291) and
 * std::uniform_real_distribution<float>(0, 1) (src/engine/session.cpp:432-433).
 */
void* oracle_rng_create(uint64_t seed);
void oracle_rng_destroy(void* rng);
float oracle_rng_uniform(void* rng);

/* libm expf, and the table-driven restatement the device code uses; must agree bit for bit. */
float oracle_expf_libm(float x);
float oracle_expf_restated(float x);
void oracle_expf_libm_array(const float* in, float* out, size_t n);
/* Returns the number of mismatching bit patterns in [first_bits, last_bits]. */
uint64_t oracle_expf_compare_range(uint32_t first_bits, uint32_t last_bits, uint32_t stride);

#ifdef __cplusplus
}
#endif

#endif /* SAMPLER_ORACLE_H */
