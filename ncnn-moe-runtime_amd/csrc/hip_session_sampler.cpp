// Host-side C++ face of the gfx950 generation sampler (see hip_session_sampler.h).
#include "hip_session_sampler.h"

#include "ncnn_moe_hip_sampler.h"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <condition_variable>
#include <deque>
#include <limits>
#include <thread>
#include <unordered_map>

namespace ncnn {
namespace moe {

namespace {

Error invalid_argument(const char* message)
{
    return Error{ErrorCode::InvalidArgument, message};
}

// Row status -> the CPU sampler's Error (src/engine/session.cpp:68,70,72,85,103,399).
Error error_of_row_status(int status)
{
    return Error{ErrorCode::InvalidArgument, ncnn_moe_hip_sampler_status_message(status)};
}

Error error_of_call(int rc, const ncnn_moe_hip_sampler* handle)
{
    const char* text = handle != nullptr ? ncnn_moe_hip_sampler_last_error(handle) : "";
    if (rc == NCNN_MOE_SAMPLER_INVALID_ARGUMENT)
        return Error{ErrorCode::InvalidArgument, std::string("hip sampler: ") + text};
    return Error{ErrorCode::InternalError, std::string("hip sampler: ") + text};
}

// Wall time of one device call, added to the statistics of the Sessions that took part in it.
struct SampleTimer
{
    std::chrono::steady_clock::time_point started = std::chrono::steady_clock::now();

    void charge(SamplingStatistics& statistics, uint64_t tokens) const
    {
        const auto elapsed = std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - started);
        statistics.sample_calls += 1;
        statistics.sampled_tokens += tokens;
        statistics.sample_time_microseconds += static_cast<uint64_t>(elapsed.count());
    }
};

// Locks the Sessions in ascending pointer order (src/engine/session.cpp:1249-1265); empty when the
// list holds a null or a duplicate.
template <typename Mutex>
bool lock_in_pointer_order(std::vector<std::pair<const void*, Mutex*>> order, std::vector<std::unique_lock<Mutex>>& locks)
{
    std::sort(order.begin(), order.end());
    for (size_t i = 0; i < order.size(); ++i)
    {
        if (order[i].first == nullptr || (i > 0 && order[i].first == order[i - 1].first))
            return false;
    }
    locks.reserve(order.size());
    for (const auto& entry : order)
        locks.emplace_back(*entry.second);
    return true;
}

template <typename T>
std::vector<Result<T>> every_row(size_t rows, const Error& error)
{
    std::vector<Result<T>> results;
    results.reserve(rows);
    for (size_t i = 0; i < rows; ++i)
        results.emplace_back(error);
    return results;
}

} // namespace

Result<bool> validate_sampling_options(const SamplingOptions& options)
{
    if (!std::isfinite(options.temperature) || options.temperature < 0.0f)
        return invalid_argument("temperature must be finite and non-negative");
    if (!std::isfinite(options.top_p) || options.top_p <= 0.0f || options.top_p > 1.0f)
        return invalid_argument("top_p must be in the range (0, 1]");
    if (!std::isfinite(options.min_p) || options.min_p < 0.0f || options.min_p > 1.0f)
        return invalid_argument("min_p must be in the range [0, 1]");
    return true;
}

uint32_t hip_sampler_capabilities()
{
    return ncnn_moe_hip_sampler_device_count() > 0 ? static_cast<uint32_t>(RuntimeCapabilityHipSampler) : 0u;
}

float peek_uniform(const std::mt19937_64& generator, std::mt19937_64& advanced)
{
    advanced = generator;
    std::uniform_real_distribution<float> distribution(0.0f, 1.0f);
    return distribution(advanced);
}

struct HipSampler::Impl
{
    ncnn_moe_hip_sampler* handle = nullptr;
    uint32_t max_rows = 0;
    uint32_t max_vocab = 0;
    std::vector<float> staging;
    std::vector<ncnn_moe_sample_params> params;
    std::vector<int32_t> stop_ids;
    std::vector<ncnn_moe_sample_result> results;
    uint32_t resident_rows = 0; // rows x vocab the logits buffer was last laid out for
    uint32_t resident_vocab = 0;
    bool resident_overwritten = false; // a sample() of host logits has used the buffer since

    // The verification step over the 2 D + 1 rows the logits buffer holds.  The caller holds the sampler's mutex.
    Result<SpeculativeVerification> verify_rows(
        std::span<const int32_t> proposed_token_ids, const SamplingOptions& options, std::span<const float> uniforms,
        uint32_t& draws_consumed, uint32_t* accept_draws, bool* failed_behind_an_empty_accept_loop);

    // Samples the rows the logits buffer holds.  The caller holds the sampler's mutex.
    std::vector<Result<BatchSampledToken>> sample_rows(
        size_t rows, std::span<const SamplingOptions> options, std::span<const float> uniforms,
        std::span<const std::vector<int32_t>> stop_tokens, std::vector<uint8_t>& draw_consumed);

    ~Impl()
    {
        if (handle != nullptr)
            ncnn_moe_hip_sampler_destroy(handle);
    }
};

HipSampler::HipSampler() : impl_(std::make_unique<Impl>()) {}

HipSampler::~HipSampler() = default;

std::shared_ptr<HipSampler> HipSampler::create(int device, uint32_t max_rows, uint32_t max_vocab)
{
    std::shared_ptr<HipSampler> sampler(new HipSampler());
    if (ncnn_moe_hip_sampler_create(device, max_rows, max_vocab, &sampler->impl_->handle) != NCNN_MOE_SAMPLER_SUCCESS)
        return nullptr;
    sampler->impl_->max_rows = max_rows;
    sampler->impl_->max_vocab = max_vocab;
    return sampler;
}

uint32_t HipSampler::max_rows() const noexcept
{
    return impl_->max_rows;
}

uint32_t HipSampler::max_vocab() const noexcept
{
    return impl_->max_vocab;
}

std::vector<Result<BatchSampledToken>> HipSampler::sample(
    std::span<const std::span<const float>> logits,
    std::span<const SamplingOptions> options,
    std::span<const float> uniforms,
    std::span<const std::vector<int32_t>> stop_tokens,
    std::vector<uint8_t>& draw_consumed)
{
    const size_t rows = logits.size();
    draw_consumed.assign(rows, 0);
    if (rows == 0 || options.size() != rows || uniforms.size() != rows || (!stop_tokens.empty() && stop_tokens.size() != rows))
        return every_row<BatchSampledToken>(rows, invalid_argument("sample batch operands differ in length"));
    if (rows > impl_->max_rows)
        return every_row<BatchSampledToken>(rows, invalid_argument("sample batch exceeds the sampler's max_rows"));
    const size_t vocab = logits[0].size();
    for (const std::span<const float>& row : logits)
    {
        if (row.size() != vocab)
            return every_row<BatchSampledToken>(rows, invalid_argument("sample batch rows differ in length"));
    }
    if (vocab > impl_->max_vocab)
        return every_row<BatchSampledToken>(rows, invalid_argument("logits exceed the sampler's max_vocab"));

    const std::lock_guard<std::mutex> lock(mutex_);
    Impl& impl = *impl_;
    impl.staging.resize(rows * vocab);
    for (size_t row = 0; row < rows; ++row)
        std::copy(logits[row].begin(), logits[row].end(), impl.staging.begin() + row * vocab);
    const int rc = ncnn_moe_hip_sampler_upload_logits(
        impl.handle, impl.staging.data(), NCNN_MOE_LOGITS_F32, static_cast<uint32_t>(rows), static_cast<uint32_t>(vocab), vocab);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return every_row<BatchSampledToken>(rows, error_of_call(rc, impl.handle));
    // the buffer now holds this call's rows: what device_logits() laid out before is gone
    impl.resident_rows = 0;
    impl.resident_vocab = 0;
    impl.resident_overwritten = true;
    return impl.sample_rows(rows, options, uniforms, stop_tokens, draw_consumed);
}

std::vector<Result<BatchSampledToken>> HipSampler::Impl::sample_rows(
    size_t rows, std::span<const SamplingOptions> options, std::span<const float> uniforms,
    std::span<const std::vector<int32_t>> stop_tokens, std::vector<uint8_t>& draw_consumed)
{
    draw_consumed.assign(rows, 0);
    params.resize(rows);
    stop_ids.clear();
    for (size_t row = 0; row < rows; ++row)
    {
        ncnn_moe_sample_params& p = params[row];
        p.temperature = options[row].temperature;
        p.top_k = options[row].top_k;
        p.top_p = options[row].top_p;
        p.min_p = options[row].min_p;
        p.stop_begin = static_cast<uint32_t>(stop_ids.size());
        p.stop_count = 0;
        if (!stop_tokens.empty())
        {
            p.stop_count = static_cast<uint32_t>(stop_tokens[row].size());
            stop_ids.insert(stop_ids.end(), stop_tokens[row].begin(), stop_tokens[row].end());
        }
    }
    results.resize(rows);
    const int rc = ncnn_moe_hip_sampler_sample(
        handle, static_cast<uint32_t>(rows), params.data(), uniforms.data(),
        stop_ids.empty() ? nullptr : stop_ids.data(), static_cast<uint32_t>(stop_ids.size()), results.data());
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return every_row<BatchSampledToken>(rows, error_of_call(rc, handle));

    std::vector<Result<BatchSampledToken>> out;
    out.reserve(rows);
    for (size_t row = 0; row < rows; ++row)
    {
        const ncnn_moe_sample_result& r = results[row];
        if (r.status != NCNN_MOE_ROW_OK)
        {
            out.emplace_back(error_of_row_status(r.status));
            continue;
        }
        draw_consumed[row] = r.draw_consumed;
        BatchSampledToken token;
        token.token.token_id = r.token_id;
        token.token.probability = r.probability;
        token.is_stop_token = r.is_stop != 0;
        token.kept_count = r.kept_count;
        out.emplace_back(token);
    }
    return out;
}

Result<DeviceLogitsRows> HipSampler::device_logits(uint32_t rows, uint32_t vocab, bool bf16)
{
    if (rows == 0 || vocab == 0)
        return invalid_argument("cannot sample empty logits");
    if (rows > impl_->max_rows)
        return invalid_argument("sample batch exceeds the sampler's max_rows");
    if (vocab > impl_->max_vocab)
        return invalid_argument("logits exceed the sampler's max_vocab");
    const std::lock_guard<std::mutex> lock(mutex_);
    DeviceLogitsRows out;
    const int rc = ncnn_moe_hip_sampler_logits_buffer(
        impl_->handle, bf16 ? NCNN_MOE_LOGITS_BF16 : NCNN_MOE_LOGITS_F32, rows, vocab, &out.data, &out.row_stride);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return error_of_call(rc, impl_->handle);
    out.rows = rows;
    out.vocab = vocab;
    out.bf16 = bf16;
    impl_->resident_rows = rows;
    impl_->resident_vocab = vocab;
    impl_->resident_overwritten = false;
    return out;
}

Result<DeviceLogitsRows> HipSampler::upload_resident(std::span<const std::span<const float>> logits)
{
    const size_t rows = logits.size();
    if (rows == 0 || logits[0].empty())
        return invalid_argument("cannot sample empty logits");
    if (rows > impl_->max_rows)
        return invalid_argument("sample batch exceeds the sampler's max_rows");
    const size_t vocab = logits[0].size();
    for (const std::span<const float>& row : logits)
    {
        if (row.size() != vocab)
            return invalid_argument("sample batch rows differ in length");
    }
    if (vocab > impl_->max_vocab)
        return invalid_argument("logits exceed the sampler's max_vocab");
    const std::lock_guard<std::mutex> lock(mutex_);
    Impl& impl = *impl_;
    impl.staging.resize(rows * vocab);
    for (size_t row = 0; row < rows; ++row)
        std::copy(logits[row].begin(), logits[row].end(), impl.staging.begin() + row * vocab);
    int rc = ncnn_moe_hip_sampler_upload_logits(
        impl.handle, impl.staging.data(), NCNN_MOE_LOGITS_F32, static_cast<uint32_t>(rows), static_cast<uint32_t>(vocab), vocab);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return error_of_call(rc, impl.handle);
    DeviceLogitsRows out;
    rc = ncnn_moe_hip_sampler_logits_buffer(
        impl.handle, NCNN_MOE_LOGITS_F32, static_cast<uint32_t>(rows), static_cast<uint32_t>(vocab), &out.data, &out.row_stride);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return error_of_call(rc, impl.handle);
    out.rows = static_cast<uint32_t>(rows);
    out.vocab = static_cast<uint32_t>(vocab);
    impl.resident_rows = out.rows;
    impl.resident_vocab = out.vocab;
    impl.resident_overwritten = false;
    return out;
}

std::vector<Result<BatchSampledToken>> HipSampler::sample_resident(
    std::span<const SamplingOptions> options, std::span<const float> uniforms,
    std::span<const std::vector<int32_t>> stop_tokens, std::vector<uint8_t>& draw_consumed,
    std::span<const uint32_t> device_rows)
{
    const size_t rows = options.size();
    draw_consumed.assign(rows, 0);
    if (rows == 0 || uniforms.size() != rows || (!stop_tokens.empty() && stop_tokens.size() != rows) ||
        (!device_rows.empty() && device_rows.size() != rows))
        return every_row<BatchSampledToken>(rows, invalid_argument("sample batch operands differ in length"));
    const std::lock_guard<std::mutex> lock(mutex_);
    if (impl_->resident_overwritten)
        return every_row<BatchSampledToken>(rows, invalid_argument("the rows laid out by device_logits were overwritten by a sample() of host logits"));
    if (device_rows.empty())
    {
        if (rows != impl_->resident_rows)
            return every_row<BatchSampledToken>(rows, invalid_argument("sample batch differs from the rows laid out by device_logits"));
        return impl_->sample_rows(rows, options, uniforms, stop_tokens, draw_consumed);
    }
    // Named rows, in any order: the device call covers rows 0 .. the largest one named.  A row that nobody
    // named carries options that fail validation at once (its workgroups leave before they look at a logit)
    // and its result is dropped.
    uint32_t covered = 0;
    for (uint32_t row : device_rows)
    {
        if (row >= impl_->resident_rows)
            return every_row<BatchSampledToken>(rows, invalid_argument("sample request names a row beyond those laid out by device_logits"));
        covered = std::max(covered, row + 1u);
    }
    std::vector<uint8_t> named(covered, 0);
    for (uint32_t row : device_rows)
    {
        if (named[row])
            return every_row<BatchSampledToken>(rows, invalid_argument("sample batch names a device row twice"));
        named[row] = 1;
    }
    SamplingOptions unused;
    unused.temperature = std::numeric_limits<float>::quiet_NaN();
    std::vector<SamplingOptions> all_options(covered, unused);
    std::vector<float> all_uniforms(covered, 0.0f);
    std::vector<std::vector<int32_t>> all_stop_tokens(stop_tokens.empty() ? 0 : covered);
    for (size_t i = 0; i < rows; ++i)
    {
        all_options[device_rows[i]] = options[i];
        all_uniforms[device_rows[i]] = uniforms[i];
        if (!stop_tokens.empty())
            all_stop_tokens[device_rows[i]] = stop_tokens[i];
    }
    std::vector<uint8_t> all_consumed;
    std::vector<Result<BatchSampledToken>> all = impl_->sample_rows(covered, all_options, all_uniforms, all_stop_tokens, all_consumed);
    std::vector<Result<BatchSampledToken>> out;
    out.reserve(rows);
    for (size_t i = 0; i < rows; ++i)
    {
        out.push_back(all[device_rows[i]]);
        draw_consumed[i] = all_consumed.size() > device_rows[i] ? all_consumed[device_rows[i]] : 0;
    }
    return out;
}

Result<std::vector<TokenProbability>> HipSampler::distribution(std::span<const float> logits, const SamplingOptions& options)
{
    if (logits.empty())
        return invalid_argument("cannot sample empty logits");
    if (logits.size() > impl_->max_vocab)
        return invalid_argument("logits exceed the sampler's max_vocab");
    const std::lock_guard<std::mutex> lock(mutex_);
    Impl& impl = *impl_;
    int rc = ncnn_moe_hip_sampler_upload_logits(
        impl.handle, logits.data(), NCNN_MOE_LOGITS_F32, 1, static_cast<uint32_t>(logits.size()), logits.size());
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return error_of_call(rc, impl.handle);
    ncnn_moe_sample_params p{options.temperature, options.top_k, options.top_p, options.min_p, 0, 0};
    std::vector<int32_t> ids(logits.size());
    std::vector<float> probabilities(logits.size());
    uint32_t count = 0;
    uint32_t status = 0;
    rc = ncnn_moe_hip_sampler_distribution(
        impl.handle, 0, &p, static_cast<uint32_t>(logits.size()), ids.data(), probabilities.data(), &count, &status);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return error_of_call(rc, impl.handle);
    if (status != NCNN_MOE_ROW_OK)
        return error_of_row_status(static_cast<int>(status));
    std::vector<TokenProbability> candidates(count);
    for (uint32_t i = 0; i < count; ++i)
        candidates[i] = TokenProbability{ids[i], probabilities[i]};
    return candidates;
}

Result<SpeculativeVerification> HipSampler::verify_speculative(
    std::span<const std::span<const float>> target_logits,
    std::span<const std::span<const float>> draft_logits,
    std::span<const int32_t> proposed_token_ids,
    const SamplingOptions& options,
    std::span<const float> uniforms,
    uint32_t& draws_consumed,
    uint32_t* accept_draws,
    bool* failed_behind_an_empty_accept_loop)
{
    draws_consumed = 0;
    if (accept_draws != nullptr)
        *accept_draws = 0;
    if (failed_behind_an_empty_accept_loop != nullptr)
        *failed_behind_an_empty_accept_loop = false;
    const size_t drafts = proposed_token_ids.size();
    if (drafts == 0 || drafts > NCNN_MOE_MAX_DRAFT_TOKENS)
        return invalid_argument("speculative verification takes 1 to 16 proposed tokens");
    if (target_logits.size() != drafts + 1 || draft_logits.size() != drafts || uniforms.size() != drafts + 1)
        return invalid_argument("speculative verification operands differ in length");
    const size_t rows = 2 * drafts + 1;
    if (rows > impl_->max_rows)
        return invalid_argument("speculative verification exceeds the sampler's max_rows");
    const size_t vocab = target_logits[0].size();
    if (vocab == 0)
        return invalid_argument("cannot sample empty logits");
    if (vocab > impl_->max_vocab)
        return invalid_argument("logits exceed the sampler's max_vocab");
    for (const std::span<const float>& row : target_logits)
    {
        if (row.size() != vocab)
            return invalid_argument("speculative verification rows differ in length");
    }
    for (const std::span<const float>& row : draft_logits)
    {
        if (row.size() != vocab)
            return invalid_argument("speculative verification rows differ in length");
    }

    const std::lock_guard<std::mutex> lock(mutex_);
    Impl& impl = *impl_;
    impl.staging.resize(rows * vocab);
    for (size_t row = 0; row <= drafts; ++row)
        std::copy(target_logits[row].begin(), target_logits[row].end(), impl.staging.begin() + row * vocab);
    for (size_t row = 0; row < drafts; ++row)
        std::copy(draft_logits[row].begin(), draft_logits[row].end(), impl.staging.begin() + (drafts + 1 + row) * vocab);
    const int rc = ncnn_moe_hip_sampler_upload_logits(
        impl.handle, impl.staging.data(), NCNN_MOE_LOGITS_F32, static_cast<uint32_t>(rows), static_cast<uint32_t>(vocab), vocab);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return error_of_call(rc, impl.handle);
    impl.resident_rows = 0;
    impl.resident_vocab = 0;
    impl.resident_overwritten = true;
    return impl.verify_rows(proposed_token_ids, options, uniforms, draws_consumed, accept_draws, failed_behind_an_empty_accept_loop);
}

Result<SpeculativeVerification> HipSampler::verify_speculative_resident(
    std::span<const int32_t> proposed_token_ids, const SamplingOptions& options, std::span<const float> uniforms,
    uint32_t& draws_consumed, uint32_t* accept_draws, bool* failed_behind_an_empty_accept_loop)
{
    draws_consumed = 0;
    if (accept_draws != nullptr)
        *accept_draws = 0;
    if (failed_behind_an_empty_accept_loop != nullptr)
        *failed_behind_an_empty_accept_loop = false;
    const size_t drafts = proposed_token_ids.size();
    if (drafts == 0 || drafts > NCNN_MOE_MAX_DRAFT_TOKENS)
        return invalid_argument("speculative verification takes 1 to 16 proposed tokens");
    if (uniforms.size() != drafts + 1)
        return invalid_argument("speculative verification operands differ in length");
    const std::lock_guard<std::mutex> lock(mutex_);
    if (impl_->resident_overwritten)
        return invalid_argument("the rows laid out by device_logits were overwritten by a sample() of host logits");
    if (impl_->resident_rows != 2 * drafts + 1)
        return invalid_argument("speculative verification needs the 2 D + 1 rows of its step laid out by device_logits");
    return impl_->verify_rows(proposed_token_ids, options, uniforms, draws_consumed, accept_draws, failed_behind_an_empty_accept_loop);
}

Result<SpeculativeVerification> HipSampler::Impl::verify_rows(
    std::span<const int32_t> proposed_token_ids, const SamplingOptions& options, std::span<const float> uniforms,
    uint32_t& draws_consumed, uint32_t* accept_draws, bool* failed_behind_an_empty_accept_loop)
{
    const size_t drafts = proposed_token_ids.size();
    const ncnn_moe_sample_params p{options.temperature, options.top_k, options.top_p, options.min_p, 0, 0};
    std::vector<float> accepted_probabilities(drafts, 0.0f);
    ncnn_moe_verify_result verified{};
    const int rc = ncnn_moe_hip_sampler_speculative_verify(
        handle, static_cast<uint32_t>(drafts), &p, proposed_token_ids.data(), uniforms.data(),
        accepted_probabilities.data(), &verified);
    if (rc != NCNN_MOE_SAMPLER_SUCCESS)
        return error_of_call(rc, handle);
    draws_consumed = verified.accept_draws + verified.final_draw_consumed;
    if (accept_draws != nullptr)
        *accept_draws = verified.accept_draws;
    if (verified.status != NCNN_MOE_VERIFY_OK && failed_behind_an_empty_accept_loop != nullptr && verified.accepted == 0)
    {
        // The accept loop fails at a position before that position's draw; once a draw has rejected the first
        // proposal (sampled rows), or the first proposal differed from the target's choice (greedy rows), the
        // loop has ended and what failed is the draw of the next token.
        const bool sampled_row = options.temperature != 0.0f;
        const bool residual_stage = verified.status == NCNN_MOE_VERIFY_RESIDUAL_EMPTY || verified.status == NCNN_MOE_VERIFY_RESIDUAL_FAILED;
        *failed_behind_an_empty_accept_loop = residual_stage || (sampled_row && verified.status == NCNN_MOE_VERIFY_ROW_ERROR && verified.accept_draws > 0);
    }
    switch (verified.status)
    {
    case NCNN_MOE_VERIFY_OK:
        break;
    case NCNN_MOE_VERIFY_ROW_ERROR:
        return error_of_row_status(static_cast<int>(verified.row_status));
    case NCNN_MOE_VERIFY_UNSUPPORTED_WINDOW:
        return Error{ErrorCode::InvalidArgument, ncnn_moe_hip_sampler_verify_status_message(static_cast<int>(verified.status))};
    default: // the reference reports these three as InternalError (src/engine/session.cpp:172-175, :199-201, :826-830)
        return Error{ErrorCode::InternalError, ncnn_moe_hip_sampler_verify_status_message(static_cast<int>(verified.status))};
    }
    SpeculativeVerification out;
    out.accepted.reserve(verified.accepted);
    for (uint32_t i = 0; i < verified.accepted; ++i)
        out.accepted.push_back(SampledToken{proposed_token_ids[i], accepted_probabilities[i]});
    out.next = SampledToken{verified.next_token_id, verified.next_probability};
    out.next_from_residual = verified.next_is_residual != 0;
    return out;
}

SamplingSession::SamplingSession(HipSamplerPtr sampler, const SamplingSessionOptions& options)
    : sampler_(std::move(sampler)), logits_output_mode_(options.logits_output_mode), random_generator_(options.sampling_seed)
{
}

Result<SamplingSessionPtr> create_sampling_session(const HipSamplerPtr& sampler, const SamplingSessionOptions& options)
{
    // src/engine/runtime.cpp:575-582 accepts FullLogits only; the device sampler adds SampledToken
    if (options.logits_output_mode == LogitsOutputMode::SampledToken && !sampler)
        return Error{ErrorCode::UnsupportedModel, "the current executor supports full logits output only"};
    if (options.logits_output_mode == LogitsOutputMode::TopKCandidates)
        return Error{ErrorCode::UnsupportedModel, "the current executor supports full logits and sampled token output only"};
    return std::make_shared<SamplingSession>(sampler, options);
}

float SamplingSession::uniform_ahead(size_t position)
{
    while (drawn_ahead_.size() <= position)
    {
        std::uniform_real_distribution<float> distribution(0.0f, 1.0f);
        drawn_ahead_.push_back(distribution(random_generator_));
    }
    return drawn_ahead_[position];
}

void SamplingSession::consume_uniforms(size_t count)
{
    drawn_ahead_.erase(drawn_ahead_.begin(), drawn_ahead_.begin() + static_cast<std::ptrdiff_t>(std::min(count, drawn_ahead_.size())));
}

Result<SampledToken> SamplingSession::sample(const LogitsOutput& logits, const SamplingOptions& options)
{
    const std::lock_guard<std::mutex> lock(mutex_);
    if (logits_output_mode_ != LogitsOutputMode::FullLogits)
        return invalid_argument("session output mode is SampledToken: its logits stay in device memory");
    if (logits.values.empty())
        return invalid_argument("cannot sample empty logits");
    if (!sampler_)
        return Error{ErrorCode::InternalError, "hip sampler is unavailable (no GPU, or create() failed)"};
    const float uniform = uniform_ahead(0);
    const std::span<const float> row(logits.values);
    std::vector<uint8_t> draw_consumed;
    const SampleTimer timer;
    auto results = sampler_->sample(
        std::span<const std::span<const float>>(&row, 1), std::span<const SamplingOptions>(&options, 1),
        std::span<const float>(&uniform, 1), {}, draw_consumed);
    timer.charge(statistics_, results[0] ? 1 : 0);
    if (!results[0])
        return results[0].error();
    if (draw_consumed[0])
        consume_uniforms(1);
    return results[0].value().token;
}

SamplingStatistics SamplingSession::statistics() const
{
    const std::lock_guard<std::mutex> lock(mutex_);
    return statistics_;
}

Result<SpeculativeVerification> SamplingSession::verify_speculative(
    std::span<const LogitsOutput> target_logits, std::span<const LogitsOutput> draft_logits,
    std::span<const int32_t> proposed_token_ids, const SamplingOptions& options)
{
    return verify_speculative(target_logits, draft_logits, proposed_token_ids, options, true);
}

Result<SpeculativeVerification> SamplingSession::verify_speculative(
    std::span<const LogitsOutput> target_logits, std::span<const LogitsOutput> draft_logits,
    std::span<const int32_t> proposed_token_ids, const SamplingOptions& options, bool state_cache_transactions)
{
    const std::lock_guard<std::mutex> lock(mutex_);
    if (!sampler_)
        return Error{ErrorCode::InternalError, "hip sampler is unavailable (no GPU, or create() failed)"};
    std::vector<std::span<const float>> target_rows, draft_rows;
    for (const LogitsOutput& row : target_logits)
        target_rows.emplace_back(row.values);
    for (const LogitsOutput& row : draft_logits)
        draft_rows.emplace_back(row.values);
    // the draws the loop could consume, in the generator's order; only the consumed ones are committed
    std::vector<float> uniforms(proposed_token_ids.size() + 1);
    for (size_t i = 0; i < uniforms.size(); ++i)
        uniforms[i] = uniform_ahead(i);
    uint32_t draws_consumed = 0;
    uint32_t accept_draws = 0;
    bool failed_behind_an_empty_accept_loop = false;
    auto verified = sampler_->verify_speculative(target_rows, draft_rows, proposed_token_ids, options, uniforms, draws_consumed, &accept_draws,
                                                 &failed_behind_an_empty_accept_loop);
    if (!state_cache_transactions && ((verified && verified.value().accepted.empty()) || failed_behind_an_empty_accept_loop))
    {
        // src/engine/session.cpp:843-857: nothing accepted and no cache transactions to keep part of the
        // step: roll back and leave speculative mode before the next token is drawn.  The device computed
        // that token as well; it is dropped and its draw stays unconsumed.
        consume_uniforms(accept_draws);
        SpeculativeVerification fallen_back;
        fallen_back.fell_back = true;
        return fallen_back;
    }
    consume_uniforms(draws_consumed);
    return verified;
}

std::vector<Result<BatchSampledToken>> SessionBatchSampler::sample(
    const HipSamplerPtr& sampler, std::span<const SampleBatchRequest> requests)
{
    const size_t rows = requests.size();
    if (rows == 0)
        return {};
    if (!sampler)
        return every_row<BatchSampledToken>(rows, Error{ErrorCode::InternalError, "hip sampler is unavailable (no GPU, or create() failed)"});
    std::vector<SamplingSession*> ordered;
    ordered.reserve(rows);
    for (const SampleBatchRequest& request : requests)
    {
        if (request.session == nullptr || request.logits == nullptr)
            return every_row<BatchSampledToken>(rows, invalid_argument("sample batch contains a null session or logits"));
        ordered.push_back(request.session);
    }
    std::sort(ordered.begin(), ordered.end());
    if (std::adjacent_find(ordered.begin(), ordered.end()) != ordered.end())
        return every_row<BatchSampledToken>(rows, invalid_argument("sample batch contains duplicate sessions"));
    for (const SampleBatchRequest& request : requests)
    {
        if (request.session->logits_output_mode_ != LogitsOutputMode::FullLogits)
            return every_row<BatchSampledToken>(rows, invalid_argument("session output mode is SampledToken: its logits stay in device memory"));
    }
    std::vector<std::unique_lock<std::mutex>> locks;
    locks.reserve(rows);
    for (SamplingSession* session : ordered)
        locks.emplace_back(session->mutex_);

    // rows with empty logits fail on their own (session.cpp:397-400); the others go to the device together
    std::vector<size_t> active;
    std::vector<std::span<const float>> logits;
    std::vector<SamplingOptions> options;
    std::vector<float> uniforms;
    std::vector<std::vector<int32_t>> stop_tokens;
    for (size_t i = 0; i < rows; ++i)
    {
        if (requests[i].logits->values.empty())
            continue;
        active.push_back(i);
        logits.emplace_back(requests[i].logits->values);
        options.push_back(requests[i].sampling);
        uniforms.push_back(requests[i].session->uniform_ahead(0));
        stop_tokens.push_back(requests[i].stop_tokens);
    }
    std::vector<Result<BatchSampledToken>> out = every_row<BatchSampledToken>(rows, invalid_argument("cannot sample empty logits"));
    if (active.empty())
        return out;
    std::vector<uint8_t> draw_consumed;
    const SampleTimer timer;
    auto sampled = sampler->sample(logits, options, uniforms, stop_tokens, draw_consumed);
    for (size_t j = 0; j < active.size(); ++j)
    {
        const size_t i = active[j];
        out[i] = sampled[j];
        timer.charge(requests[i].session->statistics_, sampled[j] ? 1 : 0);
        if (sampled[j] && draw_consumed[j])
            requests[i].session->consume_uniforms(1);
    }
    return out;
}

std::vector<Result<BatchSampledToken>> SessionBatchSampler::sample_resident(
    const HipSamplerPtr& sampler, std::span<const SampleBatchRequest> requests)
{
    const size_t rows = requests.size();
    if (rows == 0)
        return {};
    if (!sampler)
        return every_row<BatchSampledToken>(rows, Error{ErrorCode::InternalError, "hip sampler is unavailable (no GPU, or create() failed)"});
    std::vector<std::pair<const void*, std::mutex*>> order;
    for (const SampleBatchRequest& request : requests)
    {
        if (request.session == nullptr)
            return every_row<BatchSampledToken>(rows, invalid_argument("sample batch contains a null session or logits"));
        if (request.logits != nullptr || request.session->logits_output_mode_ != LogitsOutputMode::SampledToken)
            return every_row<BatchSampledToken>(rows, invalid_argument("session output mode is FullLogits: pass its logits to sample()"));
        order.emplace_back(request.session, &request.session->mutex_);
    }
    std::vector<std::unique_lock<std::mutex>> locks;
    if (!lock_in_pointer_order(std::move(order), locks))
        return every_row<BatchSampledToken>(rows, invalid_argument("sample batch contains duplicate sessions"));
    // either every request names its device row, or none does and request i samples row i
    size_t named_rows = 0;
    for (const SampleBatchRequest& request : requests)
        named_rows += request.device_row != SampleBatchRequest::kRowByPosition ? 1 : 0;
    if (named_rows != 0 && named_rows != rows)
        return every_row<BatchSampledToken>(rows, invalid_argument("sample batch names the device row of some requests only"));
    std::vector<SamplingOptions> options;
    std::vector<float> uniforms;
    std::vector<std::vector<int32_t>> stop_tokens;
    std::vector<uint32_t> device_rows;
    for (const SampleBatchRequest& request : requests)
    {
        options.push_back(request.sampling);
        uniforms.push_back(request.session->uniform_ahead(0));
        stop_tokens.push_back(request.stop_tokens);
        if (named_rows != 0)
            device_rows.push_back(request.device_row);
    }
    std::vector<uint8_t> draw_consumed;
    const SampleTimer timer;
    auto sampled = sampler->sample_resident(options, uniforms, stop_tokens, draw_consumed, device_rows);
    for (size_t i = 0; i < rows; ++i)
    {
        timer.charge(requests[i].session->statistics_, sampled[i] ? 1 : 0);
        if (sampled[i] && draw_consumed[i])
            requests[i].session->consume_uniforms(1);
    }
    return sampled;
}

// ---- BatchSampleScheduler -----------------------------------------------------------------------------------

class BatchSampleScheduler::Implementation
{
public:
    using Results = std::vector<Result<BatchSampledToken>>;

    Implementation(std::vector<HipSamplerPtr> samplers, const SampleSchedulerOptions& options)
        : samplers_(std::move(samplers)), window_(options.cross_call_window_microseconds)
    {
        spin_microseconds_ = options.worker_spin_microseconds;
        if (samplers_.empty())
            samplers_.push_back(nullptr); // (a scheduler without a sampler answers every request with InternalError)
        const uint32_t hardware_threads = std::max(1u, std::thread::hardware_concurrency());
        worker_count_ = options.worker_count == 0 ? std::min(4u, hardware_threads) : std::min(options.worker_count, 1024u);
        max_collected_ = options.cross_call_max_batch_size != 0 ? options.cross_call_max_batch_size
                                                                : (samplers_.front() ? samplers_.front()->max_rows() : 1u);
        for (uint32_t i = 0; i < worker_count_; ++i)
            workers_.emplace_back([this] { worker_loop(); });
        if (window_ != 0)
            collector_ = std::thread([this] { collector_loop(); });
    }

    ~Implementation()
    {
        {
            const std::lock_guard<std::mutex> lock(mutex_);
            stopping_ = true;
        }
        work_ready_.notify_all();
        single_ready_.notify_all();
        if (collector_.joinable())
            collector_.join();
        for (std::thread& worker : workers_)
            worker.join();
    }

    std::future<Results> submit(std::vector<SampleBatchRequest> requests)
    {
        submitted_batches_.fetch_add(1, std::memory_order_relaxed);
        submitted_requests_.fetch_add(requests.size(), std::memory_order_relaxed);
        update_max(max_batch_size_, requests.size());
        std::promise<Results> promise;
        std::future<Results> future = promise.get_future();
        const auto reject = [&](const char* message) {
            rejected_requests_.fetch_add(requests.size(), std::memory_order_relaxed);
            promise.set_value(every_row<BatchSampledToken>(requests.size(), invalid_argument(message)));
            return std::move(future);
        };
        if (requests.empty())
        {
            promise.set_value({});
            return future;
        }
        std::vector<const SamplingSession*> named;
        for (const SampleBatchRequest& request : requests)
        {
            if (request.session == nullptr)
                return reject("sample batch contains a null session or logits");
            named.push_back(request.session);
        }
        std::sort(named.begin(), named.end());
        if (std::adjacent_find(named.begin(), named.end()) != named.end())
            return reject("sample batch contains duplicate sessions");
        // A batch is of one kind.  Device-resident requests sample rows of ONE sampler's buffer, which they all
        // name; a request that names no row takes the row of its place in the batch, so such a batch runs as it
        // was submitted and is never merged with others.
        const bool resident = requests.front().logits == nullptr;
        bool rows_named = true;
        for (const SampleBatchRequest& request : requests)
        {
            if ((request.logits == nullptr) != resident)
                return reject("sample batch mixes host logits and device-resident rows");
            if (resident && request.resident_sampler != requests.front().resident_sampler)
                return reject("sample batch names device rows of several samplers");
            if (resident && request.resident_sampler >= samplers_.size())
                return reject("sample request names a sampler the scheduler does not have");
            rows_named = rows_named && request.device_row != SampleBatchRequest::kRowByPosition;
        }
        const bool collectable = requests.size() == 1 && collector_.joinable() && (!resident || rows_named);
        {
            const std::lock_guard<std::mutex> lock(mutex_);
            // the place of every request in its Session's order is fixed here, whichever way it travels
            std::vector<uint64_t> tickets;
            for (const SampleBatchRequest& request : requests)
            {
                std::deque<uint64_t>& order = session_order_[request.session];
                if (!order.empty())
                    serialized_session_requests_.fetch_add(1, std::memory_order_relaxed);
                order.push_back(next_ticket_);
                tickets.push_back(next_ticket_++);
            }
            if (collectable)
            {
                singles_.push_back(Single{std::move(requests.front()), tickets.front(), std::move(promise), std::chrono::steady_clock::now()});
                single_ready_.notify_one();
                return future;
            }
            queue_.push_back(Batch{std::move(requests), std::move(tickets), {}, std::move(promise)});
            queue_changes_.fetch_add(1, std::memory_order_release);
        }
        work_ready_.notify_one();
        return future;
    }

    size_t sampler_count() const noexcept { return samplers_.size(); }
    HipSamplerPtr sampler(size_t index) const { return index < samplers_.size() ? samplers_[index] : nullptr; }

    SampleSchedulerStatistics statistics() const noexcept
    {
        SampleSchedulerStatistics out;
        out.submitted_batches = submitted_batches_.load(std::memory_order_relaxed);
        out.submitted_requests = submitted_requests_.load(std::memory_order_relaxed);
        out.completed_requests = completed_requests_.load(std::memory_order_relaxed);
        out.rejected_requests = rejected_requests_.load(std::memory_order_relaxed);
        out.max_batch_size = max_batch_size_.load(std::memory_order_relaxed);
        out.serialized_session_requests = serialized_session_requests_.load(std::memory_order_relaxed);
        out.cross_call_collected_batches = collected_batches_.load(std::memory_order_relaxed);
        out.cross_call_collected_requests = collected_requests_.load(std::memory_order_relaxed);
        out.cross_call_collection_timeouts = collection_timeouts_.load(std::memory_order_relaxed);
        out.device_calls = device_calls_.load(std::memory_order_relaxed);
        out.overlapped_device_calls = overlapped_calls_.load(std::memory_order_relaxed);
        out.worker_count = worker_count_;
        return out;
    }

private:
    struct Single
    {
        SampleBatchRequest request;
        uint64_t ticket = 0;
        std::promise<Results> promise;
        std::chrono::steady_clock::time_point submitted_at;
    };

    // One device call's worth of requests.  A collected batch answers one promise per request.
    struct Batch
    {
        std::vector<SampleBatchRequest> requests;
        std::vector<uint64_t> tickets; // one per request: its place in its Session's order
        std::vector<std::promise<Results>> single_promises;
        std::promise<Results> promise;
    };

    static void update_max(std::atomic<uint64_t>& slot, uint64_t value)
    {
        uint64_t seen = slot.load(std::memory_order_relaxed);
        while (seen < value && !slot.compare_exchange_weak(seen, value, std::memory_order_relaxed))
        {
        }
    }

    // Host-logits batches keep off the first sampler while there are others: its buffer is where a decode
    // step that knows of one sampler only (resident_sampler 0) leaves its rows, and a sample() of host
    // logits would overwrite them.
    size_t host_lane(uint64_t turn) const
    {
        return samplers_.size() > 1 ? 1 + static_cast<size_t>(turn % (samplers_.size() - 1)) : 0;
    }

    // mutex_ held.  The first batch every request of which is the oldest unfinished one of its Session:
    // requests of a Session run in the order of their submission and never two at a time.  (A batch waits
    // only for requests with smaller tickets, so some batch can always run.)
    bool take_runnable_locked(Batch& out)
    {
        for (auto batch = queue_.begin(); batch != queue_.end(); ++batch)
        {
            bool runnable = true;
            for (size_t i = 0; i < batch->requests.size() && runnable; ++i)
                runnable = session_order_[batch->requests[i].session].front() == batch->tickets[i];
            if (runnable)
            {
                out = std::move(*batch);
                queue_.erase(batch);
                return true;
            }
        }
        return false;
    }

    void worker_loop()
    {
        for (;;)
        {
            Batch batch;
            if (spin_microseconds_ != 0)
            {
                // look for work without sleeping for a while: queue_changes_ moves on with every submission and
                // every completed batch, so the mutex is taken only when there is something new to look at
                const auto give_up = std::chrono::steady_clock::now() + std::chrono::microseconds(spin_microseconds_);
                uint64_t seen = queue_changes_.load(std::memory_order_acquire) - 1;
                while (batch.requests.empty() && std::chrono::steady_clock::now() < give_up)
                {
                    const uint64_t now = queue_changes_.load(std::memory_order_acquire);
                    if (now == seen)
                        continue;
                    seen = now;
                    const std::lock_guard<std::mutex> lock(mutex_);
                    if (stopping_)
                        break;
                    take_runnable_locked(batch);
                }
            }
            if (batch.requests.empty())
            {
                std::unique_lock<std::mutex> lock(mutex_);
                work_ready_.wait(lock, [&] { return take_runnable_locked(batch) || (stopping_ && queue_.empty() && singles_.empty() && !collecting_); });
                if (batch.requests.empty())
                    return;
            }
            Results results;
            try
            {
                // a device-resident batch runs on the sampler that holds its rows; a batch of host logits on the
                // next sampler in turn, so that batches which different workers run at once meet on different ones
                const bool resident = batch.requests.front().logits == nullptr;
                const size_t lane = resident ? batch.requests.front().resident_sampler
                                             : host_lane(next_host_lane_.fetch_add(1, std::memory_order_relaxed));
                if (running_calls_.fetch_add(1, std::memory_order_acq_rel) != 0)
                    overlapped_calls_.fetch_add(1, std::memory_order_relaxed);
                results = resident ? SessionBatchSampler::sample_resident(samplers_[lane], batch.requests)
                                   : SessionBatchSampler::sample(samplers_[lane], batch.requests);
                running_calls_.fetch_sub(1, std::memory_order_acq_rel);
                device_calls_.fetch_add(1, std::memory_order_relaxed);
            }
            catch (const std::exception& error)
            {
                results = every_row<BatchSampledToken>(batch.requests.size(), Error{ErrorCode::InternalError, std::string("sample batch failed: ") + error.what()});
            }
            completed_requests_.fetch_add(batch.requests.size(), std::memory_order_relaxed);
            {
                const std::lock_guard<std::mutex> lock(mutex_);
                for (const SampleBatchRequest& request : batch.requests)
                {
                    auto order = session_order_.find(request.session);
                    order->second.pop_front(); // this request was the Session's oldest
                    if (order->second.empty())
                        session_order_.erase(order);
                }
                queue_changes_.fetch_add(1, std::memory_order_release);
            }
            work_ready_.notify_all(); // a batch that waited for one of these Sessions may run now
            if (batch.single_promises.empty())
                batch.promise.set_value(std::move(results));
            else
            {
                for (size_t i = 0; i < batch.single_promises.size(); ++i)
                {
                    Results one;
                    one.push_back(std::move(results[i]));
                    batch.single_promises[i].set_value(std::move(one));
                }
            }
        }
    }

    // Gathers single-request submissions: waits, from the oldest one's submission, up to the window for a
    // request of another Session to come in, then takes one request per Session, oldest first, into a batch.
    void collector_loop()
    {
        for (;;)
        {
            Batch batch;
            {
                std::unique_lock<std::mutex> lock(mutex_);
                single_ready_.wait(lock, [&] { return stopping_ || !singles_.empty(); });
                if (singles_.empty())
                    return;
                collecting_ = true;
                const auto distinct_sessions = [&] {
                    std::vector<const SamplingSession*> seen;
                    for (const Single& single : singles_)
                    {
                        if (std::find(seen.begin(), seen.end(), single.request.session) == seen.end())
                            seen.push_back(single.request.session);
                    }
                    return seen.size();
                };
                const auto deadline = singles_.front().submitted_at + std::chrono::microseconds(window_);
                size_t seen_before = distinct_sessions();
                // every new Session extends nothing: the window runs from the oldest submission
                while (!stopping_ && seen_before < max_collected_ && std::chrono::steady_clock::now() < deadline)
                {
                    single_ready_.wait_until(lock, deadline);
                    seen_before = distinct_sessions();
                }
                std::vector<const SamplingSession*> taken;
                for (auto single = singles_.begin(); single != singles_.end() && batch.requests.size() < max_collected_;)
                {
                    const bool resident = single->request.logits == nullptr;
                    const bool same_kind = batch.requests.empty() ||
                        (resident == (batch.requests.front().logits == nullptr) &&
                         (!resident || single->request.resident_sampler == batch.requests.front().resident_sampler));
                    bool row_taken = false;
                    for (const SampleBatchRequest& other : batch.requests)
                        row_taken = row_taken || (resident && other.device_row == single->request.device_row);
                    if (!same_kind || row_taken || std::find(taken.begin(), taken.end(), single->request.session) != taken.end())
                    {
                        ++single;
                        continue;
                    }
                    taken.push_back(single->request.session);
                    batch.tickets.push_back(single->ticket);
                    batch.requests.push_back(std::move(single->request));
                    batch.single_promises.push_back(std::move(single->promise));
                    single = singles_.erase(single);
                }
                if (batch.requests.size() > 1)
                {
                    collected_batches_.fetch_add(1, std::memory_order_relaxed);
                    collected_requests_.fetch_add(batch.requests.size(), std::memory_order_relaxed);
                    update_max(max_batch_size_, batch.requests.size());
                }
                else
                    collection_timeouts_.fetch_add(1, std::memory_order_relaxed);
                queue_.push_back(std::move(batch));
                queue_changes_.fetch_add(1, std::memory_order_release);
                collecting_ = !singles_.empty();
            }
            work_ready_.notify_one();
        }
    }

    std::vector<HipSamplerPtr> samplers_;
    std::atomic<uint64_t> next_host_lane_{0};
    std::atomic<uint64_t> queue_changes_{1};
    uint32_t spin_microseconds_ = 0;
    std::atomic<uint32_t> running_calls_{0};
    std::atomic<uint64_t> overlapped_calls_{0};
    uint32_t window_ = 0;
    uint32_t worker_count_ = 1;
    size_t max_collected_ = 1;
    std::vector<std::thread> workers_;
    std::thread collector_;
    mutable std::mutex mutex_;
    std::condition_variable work_ready_;
    std::condition_variable single_ready_;
    std::deque<Batch> queue_;
    std::deque<Single> singles_;
    std::unordered_map<const SamplingSession*, std::deque<uint64_t>> session_order_; // unfinished requests, oldest first
    uint64_t next_ticket_ = 1;
    bool stopping_ = false;
    bool collecting_ = false;
    std::atomic<uint64_t> submitted_batches_{0}, submitted_requests_{0}, completed_requests_{0}, rejected_requests_{0};
    std::atomic<uint64_t> max_batch_size_{0}, serialized_session_requests_{0}, collected_batches_{0}, collected_requests_{0};
    std::atomic<uint64_t> collection_timeouts_{0}, device_calls_{0};
};

BatchSampleScheduler::BatchSampleScheduler(HipSamplerPtr sampler, const SampleSchedulerOptions& options)
    : implementation_(std::make_unique<Implementation>(std::vector<HipSamplerPtr>{std::move(sampler)}, options))
{
}

BatchSampleScheduler::BatchSampleScheduler(std::vector<HipSamplerPtr> samplers, const SampleSchedulerOptions& options)
    : implementation_(std::make_unique<Implementation>(std::move(samplers), options))
{
}

size_t BatchSampleScheduler::sampler_count() const noexcept
{
    return implementation_->sampler_count();
}

HipSamplerPtr BatchSampleScheduler::sampler(size_t index) const
{
    return implementation_->sampler(index);
}

BatchSampleScheduler::~BatchSampleScheduler() = default;

std::future<std::vector<Result<BatchSampledToken>>> BatchSampleScheduler::submit_sample(std::vector<SampleBatchRequest> requests)
{
    return implementation_->submit(std::move(requests));
}

SampleSchedulerStatistics BatchSampleScheduler::statistics() const noexcept
{
    return implementation_->statistics();
}

Result<std::vector<GenerationResult>> BatchGenerationLoop::generate(
    const HipSamplerPtr& sampler, std::span<SamplingSession* const> sessions, IDeviceLogitsSource& source,
    std::span<const GenerationOptions> options, const BatchTokenCallback& on_token, const TokenTextDecoder& decode_text)
{
    const size_t count = sessions.size();
    if (count == 0)
        return invalid_argument("generation batch is empty");
    if (!sampler)
        return Error{ErrorCode::InternalError, "hip sampler is unavailable (no GPU, or create() failed)"};
    if (options.size() != 1 && options.size() != count)
        return invalid_argument("generation options must hold one entry, or one per session");
    if (count > sampler->max_rows())
        return invalid_argument("generation batch exceeds the sampler's max_rows");
    const uint32_t vocab = source.vocabulary_size();
    const bool bf16 = source.bf16_logits();
    std::vector<std::pair<const void*, std::mutex*>> order;
    for (SamplingSession* session : sessions)
        order.emplace_back(session, session != nullptr ? &session->mutex_ : nullptr);
    std::vector<std::unique_lock<std::mutex>> locks;
    if (!lock_in_pointer_order(std::move(order), locks))
        return invalid_argument("generation batch contains a null or duplicate session");
    const auto options_of = [&](size_t session_index) -> const GenerationOptions& {
        return options[options.size() == 1 ? 0 : session_index];
    };
    for (size_t i = 0; i < count; ++i)
    {
        // Session::generate checks these before it decodes anything (src/engine/session.cpp:461-473)
        if (options_of(i).max_new_tokens == 0)
            return invalid_argument("max_new_tokens must be non-zero");
        const float threshold = options_of(i).speculative_confidence_threshold;
        if (!std::isfinite(threshold) || threshold < 0.0f || threshold > 1.0f)
            return invalid_argument("speculative_confidence_threshold must be in the range [0, 1]");
        auto valid = validate_sampling_options(options_of(i).sampling);
        if (!valid)
            return valid.error();
    }
    auto* const speculative = dynamic_cast<ISpeculativeLogitsSource*>(&source);
    const uint32_t block_size = speculative != nullptr ? std::min<uint32_t>(speculative->speculative_block_size(), NCNN_MOE_MAX_DRAFT_TOKENS) : 0u;
    const bool state_cache_transactions = speculative != nullptr && speculative->state_cache_transactions();
    if (block_size != 0 && 2u * block_size + 1u > sampler->max_rows())
        return invalid_argument("speculative verification exceeds the sampler's max_rows");

    std::vector<GenerationResult> results(count);
    // enable_speculative_context of session.cpp:503-506, and whether the Session is still in speculative mode
    std::vector<uint8_t> speculative_context(count, 0), speculative_active(count, 0), finished(count, 0);
    for (size_t i = 0; i < count; ++i)
        speculative_context[i] = speculative_active[i] = (block_size != 0 && options_of(i).enable_speculative) ? 1 : 0;

    // One token of Session i goes out: text, callback, and the three reasons to stop in the order of
    // src/engine/session.cpp:1000-1013 (callback, stop token, token budget).  False: the Session has finished.
    const auto emit = [&](uint32_t i, int32_t token_id, float probability, bool is_stop_token) {
        StreamToken token;
        token.index = static_cast<uint32_t>(results[i].tokens.size());
        token.token_id = token_id;
        token.probability = probability;
        token.is_stop_token = is_stop_token;
        if (decode_text)
            token.text = decode_text(token.token_id);
        const bool continue_generation = !on_token || on_token(i, token);
        results[i].tokens.push_back(std::move(token));
        if (!continue_generation)
            results[i].stopped_by_callback = true;
        else if (results[i].tokens.back().is_stop_token)
            results[i].stopped_by_stop_token = true;
        else if (results[i].tokens.size() < options_of(i).max_new_tokens)
            return true;
        finished[i] = 1;
        return false;
    };
    const auto is_stop = [&](uint32_t i, int32_t token_id) {
        const std::vector<int32_t>& stops = options_of(i).stop_tokens;
        return std::find(stops.begin(), stops.end(), token_id) != stops.end();
    };

    std::vector<SamplingOptions> row_options;
    std::vector<float> uniforms;
    std::vector<std::vector<int32_t>> stop_tokens;
    std::vector<uint8_t> draw_consumed;
    // Samples the rows the buffer holds, row r for Session members[r], consuming each Session's draw where the
    // sampler took it.  A row that failed fails the call before anything of the step is committed: no draw is
    // taken from a generator, no callback runs and no token is appended for the Sessions in front of it.
    const auto sample_members = [&](const std::vector<uint32_t>& members, bool with_stop_tokens) -> Result<std::vector<BatchSampledToken>> {
        row_options.clear();
        uniforms.clear();
        stop_tokens.resize(with_stop_tokens ? members.size() : 0);
        for (size_t row = 0; row < members.size(); ++row)
        {
            const uint32_t i = members[row];
            row_options.push_back(options_of(i).sampling);
            uniforms.push_back(sessions[i]->uniform_ahead(0));
            if (with_stop_tokens)
                stop_tokens[row] = options_of(i).stop_tokens; // assignment reuses the row's storage from the last step
        }
        const SampleTimer timer;
        auto sampled = sampler->sample_resident(row_options, uniforms, stop_tokens, draw_consumed);
        std::vector<BatchSampledToken> tokens;
        tokens.reserve(members.size());
        for (size_t row = 0; row < members.size(); ++row)
        {
            if (!sampled[row])
                return sampled[row].error();
        }
        for (size_t row = 0; row < members.size(); ++row)
        {
            timer.charge(sessions[members[row]]->statistics_, 1);
            if (draw_consumed[row])
                sessions[members[row]]->consume_uniforms(1);
            tokens.push_back(sampled[row].value());
        }
        return tokens;
    };

    // ---- token 0 of every Session, from the prefill's logits
    std::vector<uint32_t> everyone(count);
    for (size_t i = 0; i < count; ++i)
        everyone[i] = static_cast<uint32_t>(i);
    auto rows = sampler->device_logits(static_cast<uint32_t>(count), vocab, bf16);
    if (!rows)
        return rows.error();
    auto prefilled = source.prefill(everyone, rows.value());
    if (!prefilled)
        return prefilled.error();
    {
        auto first = sample_members(everyone, true);
        if (!first)
            return first.error();
        for (uint32_t i : everyone)
            emit(i, first.value()[i].token.token_id, first.value()[i].token.probability, first.value()[i].is_stop_token);
    }

    std::vector<uint32_t> stepping, proposing;
    std::vector<DecodeSlot> slots;
    std::vector<std::vector<int32_t>> proposals(count);
    for (;;)
    {
        // The Sessions that take a plain step now (decode the last token, sample the next): those outside
        // speculative mode and those with one token left (session.cpp:586).  The others propose.
        stepping.clear();
        proposing.clear();
        for (uint32_t i = 0; i < count; ++i)
        {
            if (finished[i])
                continue;
            const size_t remaining = options_of(i).max_new_tokens - results[i].tokens.size();
            if (speculative_context[i] && speculative_active[i] && remaining > 1)
                proposing.push_back(i);
            else
                stepping.push_back(i);
        }
        if (stepping.empty() && proposing.empty())
            break;
        if (!stepping.empty())
        {
            slots.clear();
            for (uint32_t i : stepping)
                slots.push_back(DecodeSlot{i, results[i].tokens.back().token_id});
            rows = sampler->device_logits(static_cast<uint32_t>(stepping.size()), vocab, bf16);
            if (!rows)
                return rows.error();
            auto decoded = source.decode(slots, rows.value());
            if (!decoded)
                return decoded.error();
            auto sampled = sample_members(stepping, true);
            if (!sampled)
                return sampled.error();
            for (size_t row = 0; row < stepping.size(); ++row)
            {
                const uint32_t i = stepping[row];
                emit(i, sampled.value()[row].token.token_id, sampled.value()[row].token.probability, sampled.value()[row].is_stop_token);
            }
        }
        if (proposing.empty())
            continue;

        // ---- propose: the block's draft tokens, each sampled with the Session's own options and generator as
        // the executor's sampler callback does (session.cpp:634-652), one device call per draft index
        for (uint32_t i : proposing)
            proposals[i].clear();
        for (uint32_t draft_index = 0; draft_index < block_size; ++draft_index)
        {
            slots.clear();
            for (uint32_t i : proposing)
                slots.push_back(DecodeSlot{i, draft_index == 0 ? results[i].tokens.back().token_id : proposals[i].back()});
            rows = sampler->device_logits(static_cast<uint32_t>(proposing.size()), vocab, bf16);
            if (!rows)
                return rows.error();
            auto drafted = speculative->draft(slots, draft_index, rows.value());
            if (!drafted)
                return drafted.error();
            auto sampled = sample_members(proposing, false);
            if (!sampled)
                return sampled.error();
            for (size_t row = 0; row < proposing.size(); ++row)
                proposals[proposing[row]].push_back(sampled.value()[row].token.token_id);
        }

        // ---- cut and verify, Session by Session
        for (uint32_t i : proposing)
        {
            const GenerationOptions& session_options = options_of(i);
            const size_t remaining = session_options.max_new_tokens - results[i].tokens.size();
            size_t draft_count = std::min<size_t>(proposals[i].size(), remaining - 1);
            if (session_options.speculative_max_draft_tokens != 0)
                draft_count = std::min<size_t>(draft_count, session_options.speculative_max_draft_tokens);
            if (session_options.speculative_confidence_threshold > 0.0f)
            {
                for (size_t index = 0; index < draft_count; ++index)
                {
                    const float confidence = 1.0f / (1.0f + std::exp(-speculative->confidence_logit(i, static_cast<uint32_t>(index))));
                    if (confidence < session_options.speculative_confidence_threshold)
                    {
                        draft_count = index;
                        break;
                    }
                }
            }
            if (draft_count == 0)
            {
                // nothing worth verifying: the proposal is dropped and the Session leaves speculative mode (session.cpp:690-694)
                auto dropped = speculative->commit(i, {});
                if (!dropped)
                    return dropped.error();
                speculative_active[i] = 0;
                continue;
            }
            const int32_t anchor = results[i].tokens.back().token_id;
            const std::span<const int32_t> proposed(proposals[i].data(), draft_count);
            rows = sampler->device_logits(static_cast<uint32_t>(2 * draft_count + 1), vocab, bf16);
            if (!rows)
                return rows.error();
            auto written = speculative->verify(i, anchor, proposed, rows.value());
            if (!written)
                return written.error();
            uniforms.resize(draft_count + 1);
            for (size_t k = 0; k <= draft_count; ++k)
                uniforms[k] = sessions[i]->uniform_ahead(k);
            uint32_t draws_consumed = 0, accept_draws = 0;
            bool failed_behind_an_empty_accept_loop = false;
            const SampleTimer timer;
            auto verified = sampler->verify_speculative_resident(proposed, session_options.sampling, uniforms, draws_consumed, &accept_draws,
                                                                 &failed_behind_an_empty_accept_loop);
            SamplingStatistics& statistics = sessions[i]->statistics_;
            statistics.speculative_steps += 1;
            statistics.speculative_verify_time_microseconds += static_cast<uint64_t>(
                std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - timer.started).count());
            if (!state_cache_transactions && ((verified && verified.value().accepted.empty()) || failed_behind_an_empty_accept_loop))
            {
                // session.cpp:843-857: roll the step back, leave speculative mode; only the accept test's draw is gone
                sessions[i]->consume_uniforms(accept_draws);
                auto rolled_back = speculative->commit(i, {});
                if (!rolled_back)
                    return rolled_back.error();
                speculative_active[i] = 0;
                continue;
            }
            if (!verified)
                return verified.error();
            sessions[i]->consume_uniforms(draws_consumed);
            std::vector<int32_t> emitted;
            bool continues = true;
            for (const SampledToken& accepted : verified.value().accepted)
            {
                emitted.push_back(accepted.token_id);
                continues = emit(i, accepted.token_id, accepted.probability, is_stop(i, accepted.token_id));
                if (!continues)
                    break;
            }
            if (continues)
            {
                const SampledToken& next = verified.value().next;
                emitted.push_back(next.token_id);
                emit(i, next.token_id, next.probability, is_stop(i, next.token_id));
            }
            statistics.sampled_tokens += emitted.size();
            statistics.speculative_accepted_tokens += emitted.size() - 1;
            auto committed = speculative->commit(i, emitted);
            if (!committed)
                return committed.error();
        }
    }
    return results;
}

} // namespace moe
} // namespace ncnn
