/*
 * CPU oracle for the generation sampler -- TEST INFRASTRUCTURE ONLY, never shipped or measured
 * as the product.  Loaded by tests, the smoke check and the benchmark's cpu_baseline leg.
 *
 * It restates src/engine/session.cpp:20-36, 60-136, 393-456 of the reference in the same
 * evaluation order: a full stable sort of the vocabulary by (logit descending, index ascending),
 * sequential fp32 sums, libm expf, IEEE fp32 division.  Build with -ffp-contract=off and without
 * -ffast-math so that every operation rounds once, as in the reference's default build.
 *
 * What pins each function (see tests/test_oracle_*.py):
 *   oracle_validate_sampling_options   reference known answers (top_p = 0, T = -0.0, T = 1e-39) and,
 *                                      where the reference library builds, the reference itself.
 *   greedy branch of oracle_sample     closed form: first maximum over finite logits; the reference's
 *                                      own vectors {1,2,3}->2, {3,NaN,3}->0, {NaN,+inf}->error.
 *   oracle_sampling_distribution       brute-force selection on small inputs, fp64 softmax over the
 *                                      kept set, the known answers recorded from the reference, and
 *                                      the reference's file-static function itself (where it builds).
 *   oracle_sample (draw)               inverse-CDF definition; the reference's Session::sample in
 *                                      RNG lock-step (where it builds); committed golden vectors.
 *   oracle_candidate_probability,      the reference's file-static functions themselves (where it builds):
 *   oracle_sample_residual_distribution  random distributions with a real mt19937_64 in lock-step; brute force
 *                                      in fp64 on small cases; committed golden vectors.
 *   oracle_speculative_verify          the accept loop is inline in the reference's generate(): pinned by the
 *                                      two functions above plus the identity that fixes the algorithm (the
 *                                      emitted token follows the target distribution whatever the draft is),
 *                                      integrated over a grid of uniforms; greedy reduces to arg-max equality.
 *   oracle_rng_uniform                 2000-draw lock-step against the reference Session; golden draws.
 *   oracle_*_bfloat16                  exhaustive 65536-value round trip and round-to-nearest-even
 *                                      checks against the definition.
 *   oracle_expf_restated               all 2^32 bit patterns equal libm expf (one-off run), dense
 *                                      sample in the test-suite.
 *
 * NaN in a non-greedy row: the reference comparator is not a strict weak order there, so its
 * result depends on where the NaN sits.  The oracle defines NaN as skipped (it sorts after -inf),
 * which is what the reference does for a NaN that is not the first element of the row.
 */
#include "sampler_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <numeric>
#include <random>
#include <thread>
#include <vector>

namespace {

struct Candidate
{
    int32_t token_id;
    float probability;
};

/* src/engine/session.cpp:26-36 (LogitOrder), with NaN made the lowest value. */
struct LogitOrder
{
    const float* values;

    bool operator()(int32_t left, int32_t right) const
    {
        const float a = values[left];
        const float b = values[right];
        const bool a_nan = a != a;
        const bool b_nan = b != b;
        if (a_nan || b_nan)
        {
            if (a_nan == b_nan)
                return left < right;
            return b_nan;
        }
        if (a == b)
            return left < right;
        return a > b;
    }
};

/* src/engine/session.cpp:76-136 */
int sampling_distribution(
    const float* logits, size_t vocab,
    const oracle_sampling_options& options,
    std::vector<Candidate>& candidates,
    float* top_p_gap)
{
    std::vector<int32_t> token_ids(vocab);
    std::iota(token_ids.begin(), token_ids.end(), 0);
    std::stable_sort(token_ids.begin(), token_ids.end(), LogitOrder{logits});

    if (!std::isfinite(logits[token_ids.front()]))
        return ORACLE_NO_FINITE_LOGIT;
    if (options.top_k > 0 && options.top_k < token_ids.size())
        token_ids.resize(options.top_k);

    const float maximum = logits[token_ids.front()] / options.temperature;
    candidates.clear();
    candidates.reserve(token_ids.size());
    float normalizer = 0.0f;
    for (int32_t token_id : token_ids)
    {
        const float logit = logits[token_id];
        if (!std::isfinite(logit))
            continue;
        const float probability = std::exp(logit / options.temperature - maximum);
        candidates.push_back(Candidate{token_id, probability});
        normalizer += probability;
    }
    if (candidates.empty() || !std::isfinite(normalizer) || normalizer <= 0.0f)
        return ORACLE_INVALID_DISTRIBUTION;
    for (Candidate& candidate : candidates)
        candidate.probability /= normalizer;

    if (options.min_p > 0.0f)
    {
        const float threshold = candidates.front().probability * options.min_p;
        size_t count = 0;
        for (const Candidate& candidate : candidates)
        {
            if (candidate.probability >= threshold)
                candidates[count++] = candidate;
        }
        candidates.resize(count);
    }

    float cumulative = 0.0f;
    size_t top_p_count = 0;
    float gap = std::numeric_limits<float>::infinity();
    for (const Candidate& candidate : candidates)
    {
        cumulative += candidate.probability;
        ++top_p_count;
        gap = std::min(gap, std::fabs(cumulative - options.top_p));
        if (cumulative >= options.top_p)
            break;
    }
    candidates.resize(top_p_count);
    if (top_p_gap)
        *top_p_gap = gap;

    normalizer = 0.0f;
    for (const Candidate& candidate : candidates)
        normalizer += candidate.probability;
    for (Candidate& candidate : candidates)
        candidate.probability /= normalizer;
    return ORACLE_OK;
}

bool row_has_nan(const float* logits, size_t vocab)
{
    for (size_t i = 0; i < vocab; ++i)
    {
        if (logits[i] != logits[i])
            return true;
    }
    return false;
}

/* src/engine/session.cpp:393-443 */
int sample_row(
    const float* logits, size_t vocab,
    const oracle_sampling_options& options,
    float uniform,
    oracle_row_result& result)
{
    result.token_id = -1;
    result.probability = 0.0f;
    result.kept_count = 0;
    result.status = ORACLE_OK;
    result.is_stop = 0;
    result.draw_consumed = 0;
    result.has_nan = 0;
    result.cdf_gap = std::numeric_limits<float>::infinity();
    result.top_p_gap = std::numeric_limits<float>::infinity();

    if (vocab == 0)
        return result.status = ORACLE_EMPTY_LOGITS;
    const int valid = oracle_validate_sampling_options(&options);
    if (valid != ORACLE_OK)
        return result.status = static_cast<uint8_t>(valid);
    result.has_nan = row_has_nan(logits, vocab) ? 1 : 0;

    if (options.temperature == 0.0f)
    {
        int32_t selected_token = -1;
        float selected_logit = -std::numeric_limits<float>::infinity();
        for (size_t token_id = 0; token_id < vocab; ++token_id)
        {
            const float logit = logits[token_id];
            if (!std::isfinite(logit))
                continue;
            if (selected_token < 0 || logit > selected_logit)
            {
                selected_token = static_cast<int32_t>(token_id);
                selected_logit = logit;
            }
        }
        if (selected_token < 0)
            return result.status = ORACLE_NO_FINITE_LOGIT;
        result.token_id = selected_token;
        result.probability = 1.0f;
        result.kept_count = 1;
        return ORACLE_OK;
    }

    std::vector<Candidate> candidates;
    const int status = sampling_distribution(logits, vocab, options, candidates, &result.top_p_gap);
    if (status != ORACLE_OK)
        return result.status = static_cast<uint8_t>(status);
    result.kept_count = static_cast<uint32_t>(candidates.size());

    if (candidates.size() == 1)
    {
        result.token_id = candidates.front().token_id;
        result.probability = 1.0f;
        return ORACLE_OK;
    }

    result.draw_consumed = 1;
    float cumulative = 0.0f;
    for (const Candidate& candidate : candidates)
    {
        cumulative += candidate.probability;
        result.cdf_gap = std::min(result.cdf_gap, std::fabs(uniform - cumulative));
        if (uniform < cumulative)
        {
            result.token_id = candidate.token_id;
            result.probability = candidate.probability;
            return ORACLE_OK;
        }
    }
    result.token_id = candidates.back().token_id;
    result.probability = candidates.back().probability;
    return ORACLE_OK;
}

/* src/engine/session.cpp:138-148 */
float candidate_probability(const std::vector<Candidate>& candidates, int32_t token_id)
{
    for (const Candidate& candidate : candidates)
    {
        if (candidate.token_id == token_id)
            return candidate.probability;
    }
    return 0.0f;
}

/* src/engine/session.cpp:150-202.  The reference draws uniform_real_distribution<float>(0, normalizer),
 * which libstdc++ evaluates as canonical * (normalizer - 0) + 0 in fp32. */
int sample_residual_distribution(
    const std::vector<Candidate>& target, const std::vector<Candidate>& draft, size_t vocab,
    float canonical_uniform, int32_t& token_id, float& probability)
{
    std::vector<float> residual(vocab, 0.0f);
    for (const Candidate& candidate : target)
        residual[candidate.token_id] = candidate.probability;
    for (const Candidate& candidate : draft)
        residual[candidate.token_id] = std::max(0.0f, residual[candidate.token_id] - candidate.probability);
    const float normalizer = std::accumulate(residual.begin(), residual.end(), 0.0f);
    if (!std::isfinite(normalizer) || normalizer <= 0.0f)
        return ORACLE_VERIFY_RESIDUAL_EMPTY;
    const float sample_value = canonical_uniform * (normalizer - 0.0f) + 0.0f;
    float cumulative = 0.0f;
    for (size_t id = 0; id < residual.size(); ++id)
    {
        cumulative += residual[id];
        if (sample_value < cumulative)
        {
            token_id = static_cast<int32_t>(id);
            probability = residual[id] / normalizer;
            return ORACLE_VERIFY_OK;
        }
    }
    for (size_t id = residual.size(); id != 0; --id)
    {
        if (residual[id - 1] > 0.0f)
        {
            token_id = static_cast<int32_t>(id - 1);
            probability = residual[id - 1] / normalizer;
            return ORACLE_VERIFY_OK;
        }
    }
    return ORACLE_VERIFY_RESIDUAL_FAILED;
}

/* Table-driven expf: 2^(k/32) table, degree-3 polynomial evaluated in double, one final rounding. */
struct Exp2fTable
{
    uint64_t entry[32];

    Exp2fTable()
    {
        for (int i = 0; i < 32; ++i)
        {
            const double value = static_cast<double>(exp2l(static_cast<long double>(i) / 32.0L));
            uint64_t bits = 0;
            std::memcpy(&bits, &value, sizeof(bits));
            entry[i] = bits - (static_cast<uint64_t>(i) << 47);
        }
    }
};

const Exp2fTable exp2f_table;

inline uint32_t float_bits(float value)
{
    uint32_t bits = 0;
    std::memcpy(&bits, &value, sizeof(bits));
    return bits;
}

inline float bits_float(uint32_t bits)
{
    float value = 0.0f;
    std::memcpy(&value, &bits, sizeof(value));
    return value;
}

} // namespace

extern "C" {

const char* oracle_status_message(int status)
{
    switch (status)
    {
    case ORACLE_OK: return "";
    case ORACLE_EMPTY_LOGITS: return "cannot sample empty logits";
    case ORACLE_BAD_TEMPERATURE: return "temperature must be finite and non-negative";
    case ORACLE_BAD_TOP_P: return "top_p must be in the range (0, 1]";
    case ORACLE_BAD_MIN_P: return "min_p must be in the range [0, 1]";
    case ORACLE_NO_FINITE_LOGIT: return "sampling requires at least one finite logit";
    case ORACLE_INVALID_DISTRIBUTION: return "sampling distribution is invalid";
    default: return "unknown status";
    }
}

/* src/engine/session.cpp:65-74 */
int oracle_validate_sampling_options(const oracle_sampling_options* options)
{
    if (!std::isfinite(options->temperature) || options->temperature < 0.0f)
        return ORACLE_BAD_TEMPERATURE;
    if (!std::isfinite(options->top_p) || options->top_p <= 0.0f || options->top_p > 1.0f)
        return ORACLE_BAD_TOP_P;
    if (!std::isfinite(options->min_p) || options->min_p < 0.0f || options->min_p > 1.0f)
        return ORACLE_BAD_MIN_P;
    return ORACLE_OK;
}

int oracle_sampling_distribution(
    const float* logits, size_t vocab,
    const oracle_sampling_options* options,
    int32_t* ids, float* probabilities, size_t cap, size_t* count)
{
    *count = 0;
    if (vocab == 0)
        return ORACLE_EMPTY_LOGITS;
    const int valid = oracle_validate_sampling_options(options);
    if (valid != ORACLE_OK)
        return valid;
    std::vector<Candidate> candidates;
    const int status = sampling_distribution(logits, vocab, *options, candidates, nullptr);
    if (status != ORACLE_OK)
        return status;
    *count = candidates.size();
    const size_t n = std::min(cap, candidates.size());
    for (size_t i = 0; i < n; ++i)
    {
        ids[i] = candidates[i].token_id;
        probabilities[i] = candidates[i].probability;
    }
    return ORACLE_OK;
}

int oracle_sample(
    const float* logits, size_t vocab,
    const oracle_sampling_options* options,
    float uniform,
    oracle_row_result* result)
{
    return sample_row(logits, vocab, *options, uniform, *result);
}

int oracle_sample_batch(
    const void* logits, int dtype, uint32_t rows, uint32_t vocab, uint64_t row_stride,
    const oracle_row_params* params, const float* uniforms,
    const int32_t* stop_ids,
    oracle_row_result* results, int threads)
{
    if (dtype != 0 && dtype != 1)
        return -1;
    auto run_rows = [&](uint32_t begin, uint32_t end) {
        std::vector<float> widened;
        for (uint32_t row = begin; row < end; ++row)
        {
            const float* row_logits = nullptr;
            if (dtype == 0)
            {
                row_logits = static_cast<const float*>(logits) + static_cast<size_t>(row) * row_stride;
            }
            else
            {
                const uint16_t* source = static_cast<const uint16_t*>(logits) + static_cast<size_t>(row) * row_stride;
                widened.resize(vocab);
                for (uint32_t i = 0; i < vocab; ++i)
                    widened[i] = oracle_bfloat16_to_float(source[i]);
                row_logits = widened.data();
            }
            const oracle_row_params& p = params[row];
            const oracle_sampling_options options{p.temperature, p.top_k, p.top_p, p.min_p};
            sample_row(row_logits, vocab, options, uniforms[row], results[row]);
            /* src/engine/session.cpp:60-63 and examples/internal/run_model.cpp:790 */
            if (results[row].status == ORACLE_OK && stop_ids != nullptr)
            {
                const int32_t* begin_stop = stop_ids + p.stop_begin;
                const int32_t* end_stop = begin_stop + p.stop_count;
                results[row].is_stop = std::find(begin_stop, end_stop, results[row].token_id) != end_stop ? 1 : 0;
            }
        }
    };
    if (threads <= 1 || rows <= 1)
    {
        run_rows(0, rows);
        return 0;
    }
    const uint32_t workers = std::min<uint32_t>(static_cast<uint32_t>(threads), rows);
    std::vector<std::thread> pool;
    pool.reserve(workers);
    for (uint32_t w = 0; w < workers; ++w)
    {
        const uint32_t begin = static_cast<uint32_t>(static_cast<uint64_t>(rows) * w / workers);
        const uint32_t end = static_cast<uint32_t>(static_cast<uint64_t>(rows) * (w + 1) / workers);
        pool.emplace_back(run_rows, begin, end);
    }
    for (std::thread& worker : pool)
        worker.join();
    return 0;
}

float oracle_candidate_probability(const int32_t* ids, const float* probabilities, size_t count, int32_t token_id)
{
    std::vector<Candidate> candidates(count);
    for (size_t i = 0; i < count; ++i)
        candidates[i] = Candidate{ids[i], probabilities[i]};
    return candidate_probability(candidates, token_id);
}

int oracle_sample_residual_distribution(
    const int32_t* target_ids, const float* target_probabilities, size_t target_count,
    const int32_t* draft_ids, const float* draft_probabilities, size_t draft_count,
    size_t vocab, float canonical_uniform, int32_t* token_id, float* probability)
{
    std::vector<Candidate> target(target_count), draft(draft_count);
    for (size_t i = 0; i < target_count; ++i)
        target[i] = Candidate{target_ids[i], target_probabilities[i]};
    for (size_t i = 0; i < draft_count; ++i)
        draft[i] = Candidate{draft_ids[i], draft_probabilities[i]};
    *token_id = -1;
    *probability = 0.0f;
    return sample_residual_distribution(target, draft, vocab, canonical_uniform, *token_id, *probability);
}

/* src/engine/session.cpp:776-874 */
int oracle_speculative_verify(
    const float* target_logits, const float* draft_logits, size_t vocab, uint32_t draft_count,
    const oracle_sampling_options* options, const int32_t* proposed_token_ids, const float* uniforms,
    float* accepted_probabilities, oracle_verify_result* result)
{
    oracle_verify_result r;
    std::memset(&r, 0, sizeof(r));
    r.next_token_id = -1;
    auto fail_row = [&](int row_status) {
        r.status = ORACLE_VERIFY_ROW_ERROR;
        r.row_status = static_cast<uint32_t>(row_status);
        *result = r;
        return static_cast<int>(r.status);
    };
    std::vector<Candidate> rejected_target, rejected_draft;
    uint32_t accepted = 0;
    while (accepted < draft_count)
    {
        const float* target_row = target_logits + static_cast<size_t>(accepted) * vocab;
        const float* draft_row = draft_logits + static_cast<size_t>(accepted) * vocab;
        if (options->temperature == 0.0f)
        {
            oracle_row_result target_token;
            if (sample_row(target_row, vocab, *options, 0.0f, target_token) != ORACLE_OK)
            {
                r.accepted = accepted;
                return fail_row(target_token.status);
            }
            if (target_token.token_id != proposed_token_ids[accepted])
                break;
            accepted_probabilities[accepted] = 1.0f;
        }
        else
        {
            /* sampling_distribution is reached only with options that an earlier sample() call of the
             * generation loop has validated; the oracle reports unvalidated ones as the row's error */
            const int valid = vocab == 0 ? ORACLE_EMPTY_LOGITS : oracle_validate_sampling_options(options);
            std::vector<Candidate> target_distribution, draft_distribution;
            const int target_status = valid != ORACLE_OK ? valid
                : sampling_distribution(target_row, vocab, *options, target_distribution, nullptr);
            const int draft_status = valid != ORACLE_OK ? valid
                : sampling_distribution(draft_row, vocab, *options, draft_distribution, nullptr);
            if (target_status != ORACLE_OK || draft_status != ORACLE_OK)
            {
                r.accepted = accepted;
                return fail_row(target_status != ORACLE_OK ? target_status : draft_status);
            }
            const int32_t token_id = proposed_token_ids[accepted];
            const float target_probability = candidate_probability(target_distribution, token_id);
            const float draft_probability = candidate_probability(draft_distribution, token_id);
            if (draft_probability <= 0.0f)
            {
                r.accepted = accepted;
                r.status = ORACLE_VERIFY_ZERO_DRAFT_PROBABILITY;
                *result = r;
                return static_cast<int>(r.status);
            }
            const float acceptance_probability = std::min(1.0f, target_probability / draft_probability);
            const float uniform = uniforms[r.accept_draws++];
            if (uniform >= acceptance_probability)
            {
                rejected_target = std::move(target_distribution);
                rejected_draft = std::move(draft_distribution);
                break;
            }
            accepted_probabilities[accepted] = target_probability;
        }
        ++accepted;
    }
    r.accepted = accepted;
    if (accepted < draft_count && options->temperature > 0.0f)
    {
        r.next_is_residual = 1;
        int32_t token_id = -1;
        float probability = 0.0f;
        const int status = sample_residual_distribution(
            rejected_target, rejected_draft, vocab, uniforms[r.accept_draws], token_id, probability);
        r.status = static_cast<uint32_t>(status);
        /* the reference draws before the walk: the draw is consumed unless the distribution was empty */
        r.final_draw_consumed = status == ORACLE_VERIFY_RESIDUAL_EMPTY ? 0u : 1u;
        if (status == ORACLE_VERIFY_OK)
        {
            r.next_token_id = token_id;
            r.next_probability = probability;
        }
        *result = r;
        return status;
    }
    oracle_row_result next;
    if (sample_row(target_logits + static_cast<size_t>(accepted) * vocab, vocab, *options, uniforms[r.accept_draws], next) != ORACLE_OK)
        return fail_row(next.status);
    r.next_token_id = next.token_id;
    r.next_probability = next.probability;
    r.final_draw_consumed = next.draw_consumed;
    *result = r;
    return ORACLE_VERIFY_OK;
}

/* src/kernels/cpu_ops.cpp:26-32 */
float oracle_bfloat16_to_float(uint16_t value)
{
    return bits_float(static_cast<uint32_t>(value) << 16);
}

/* src/kernels/cpu_ops.cpp:34-40 */
uint16_t oracle_float_to_bfloat16(float value)
{
    const uint32_t bits = float_bits(value);
    const uint32_t rounding = 0x7fffu + ((bits >> 16) & 1u);
    return static_cast<uint16_t>((bits + rounding) >> 16);
}

void oracle_quantize_bfloat16(const float* in, uint16_t* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = oracle_float_to_bfloat16(in[i]);
}

struct OracleRng
{
    std::mt19937_64 generator;
};

void* oracle_rng_create(uint64_t seed)
{
    return new OracleRng{std::mt19937_64(seed)};
}

void oracle_rng_destroy(void* rng)
{
    delete static_cast<OracleRng*>(rng);
}

float oracle_rng_uniform(void* rng)
{
    std::uniform_real_distribution<float> distribution(0.0f, 1.0f);
    return distribution(static_cast<OracleRng*>(rng)->generator);
}

float oracle_expf_libm(float x)
{
    return std::exp(x);
}

void oracle_expf_libm_array(const float* in, float* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = std::exp(in[i]);
}

float oracle_expf_restated(float x)
{
    const uint32_t bits = float_bits(x);
    const uint32_t abstop = (bits >> 20) & 0x7ffu;
    if (abstop >= (0x42b00000u >> 20)) /* |x| >= 88 or not finite */
    {
        if (bits == 0xff800000u)
            return 0.0f;
        if (abstop >= (0x7f800000u >> 20))
            return x + x;
        if (x > 0x1.62e42ep6f)
            return std::numeric_limits<float>::infinity();
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
    uint64_t ki = 0;
    std::memcpy(&ki, &kd, sizeof(ki));
    kd -= shift;
    const double r = std::fma(inverse_ln2_scaled, xd, -kd);
    const uint64_t scale_bits = exp2f_table.entry[ki % 32] + (ki << 47);
    double scale = 0.0;
    std::memcpy(&scale, &scale_bits, sizeof(scale));
    const double p = std::fma(c0, r, c1);
    const double r2 = r * r;
    double y = std::fma(c2, r, 1.0);
    y = std::fma(p, r2, y);
    y = y * scale;
    return static_cast<float>(y);
}

uint64_t oracle_expf_compare_range(uint32_t first_bits, uint32_t last_bits, uint32_t stride)
{
    uint64_t mismatches = 0;
    if (stride == 0)
        stride = 1;
    for (uint64_t bits = first_bits; bits <= last_bits; bits += stride)
    {
        const float x = bits_float(static_cast<uint32_t>(bits));
        const float a = std::exp(x);
        const float b = oracle_expf_restated(x);
        const bool both_nan = (a != a) && (b != b);
        if (!both_nan && float_bits(a) != float_bits(b))
            ++mismatches;
    }
    return mismatches;
}

} // extern "C"
