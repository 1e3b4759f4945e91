// Tests of the C++ host face of the HIP sampler, written in the manner of the runtime's own test
// binary (hand-rolled check()/check_near(), one function per topic, "all ... passed" at the end).
// The first group mirrors the runtime's sampler test (tests/test_runtime.cpp:4320-4362); the rest
// cover what that test leaves out: draws, RNG bookkeeping, batches, stop tokens, error text.
//
//   test_session_sampler            all tests (needs a GPU)
//   test_session_sampler --host     only the tests that need no GPU
#include "hip_session_sampler.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <limits>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

using namespace ncnn::moe;

#define check(condition)                                                                              \
    do                                                                                                \
    {                                                                                                 \
        if (!(condition))                                                                             \
            throw std::runtime_error(std::string(__FILE__) + ":" + std::to_string(__LINE__) + ": check failed: " #condition); \
    } while (0)

static void check_near(float actual, float expected, float tolerance)
{
    if (!(std::fabs(actual - expected) <= tolerance))
        throw std::runtime_error("check_near failed: " + std::to_string(actual) + " vs " + std::to_string(expected));
}

static LogitsOutput logits_of(std::vector<float> values)
{
    LogitsOutput output;
    output.values = std::move(values);
    return output;
}

// ---- host only ------------------------------------------------------------------------------

static void test_option_validation_messages()
{
    SamplingOptions options;
    check(static_cast<bool>(validate_sampling_options(options)));
    options.top_p = 0.0f;
    auto invalid = validate_sampling_options(options);
    check(!invalid);
    check(invalid.error().code == ErrorCode::InvalidArgument);
    check(invalid.error().message == "top_p must be in the range (0, 1]");
    options = SamplingOptions{};
    options.temperature = -1.0f;
    check(validate_sampling_options(options).error().message == "temperature must be finite and non-negative");
    options.temperature = std::numeric_limits<float>::infinity();
    check(!validate_sampling_options(options));
    options = SamplingOptions{};
    options.temperature = -0.0f;
    check(static_cast<bool>(validate_sampling_options(options)));
    options.min_p = 1.5f;
    check(validate_sampling_options(options).error().message == "min_p must be in the range [0, 1]");
    options.min_p = std::numeric_limits<float>::quiet_NaN();
    check(!validate_sampling_options(options));
}

static void test_defaults_match_the_runtime()
{
    const SamplingOptions options;
    check(options.temperature == 1.0f && options.top_k == 0 && options.top_p == 1.0f && options.min_p == 0.0f);
    const SampledToken token;
    check(token.token_id == -1 && token.probability == 0.0f);
    const SamplingSessionOptions session_options;
    check(session_options.sampling_seed == 0);
}

static void test_peek_uniform_does_not_advance()
{
    std::mt19937_64 generator(1234);
    std::mt19937_64 shadow(1234);
    std::mt19937_64 advanced;
    const float first = peek_uniform(generator, advanced);
    check(generator == shadow);
    std::uniform_real_distribution<float> distribution(0.0f, 1.0f);
    check(first == distribution(shadow));
    check(advanced == shadow);
    check(first >= 0.0f && first < 1.0f);
}

static void test_missing_sampler_fails_loudly()
{
    SamplingSession session(nullptr);
    auto sampled = session.sample(logits_of({1.0f, 2.0f}));
    check(!sampled);
    check(sampled.error().code == ErrorCode::InternalError);
    SampleBatchRequest request;
    LogitsOutput logits = logits_of({1.0f, 2.0f});
    request.session = &session;
    request.logits = &logits;
    auto batch = SessionBatchSampler::sample(nullptr, std::span<const SampleBatchRequest>(&request, 1));
    check(batch.size() == 1 && !batch[0] && batch[0].error().code == ErrorCode::InternalError);
}

// ---- GPU ------------------------------------------------------------------------------------

static void test_sampling_like_the_runtime_test(const HipSamplerPtr& sampler)
{
    SamplingSessionOptions session_options;
    session_options.sampling_seed = 1234;
    SamplingSession session(sampler, session_options);

    LogitsOutput logits = logits_of({1.0f, 2.0f, 3.0f});
    SamplingOptions greedy_options;
    greedy_options.temperature = 0.0f;
    auto greedy = session.sample(logits, greedy_options);
    check(static_cast<bool>(greedy));
    check(greedy.value().token_id == 2);
    check_near(greedy.value().probability, 1.0f, 1e-6f);

    logits.values = {3.0f, std::numeric_limits<float>::quiet_NaN(), 3.0f};
    greedy = session.sample(logits, greedy_options);
    check(static_cast<bool>(greedy));
    check(greedy.value().token_id == 0);

    logits.values = {std::numeric_limits<float>::quiet_NaN(), std::numeric_limits<float>::infinity()};
    greedy = session.sample(logits, greedy_options);
    check(!greedy);
    check(greedy.error().code == ErrorCode::InvalidArgument);
    check(greedy.error().message == "sampling requires at least one finite logit");

    logits.values = {1.0f, 2.0f, 3.0f};
    SamplingOptions top_k_options;
    top_k_options.top_k = 1;
    auto top_k = session.sample(logits, top_k_options);
    check(static_cast<bool>(top_k));
    check(top_k.value().token_id == 2);

    SamplingOptions invalid_options;
    invalid_options.top_p = 0.0f;
    auto invalid = session.sample(logits, invalid_options);
    check(!invalid);
    check(invalid.error().code == ErrorCode::InvalidArgument);
    check(invalid.error().message == "top_p must be in the range (0, 1]");

    logits.values.clear();
    auto empty = session.sample(logits);
    check(!empty);
    check(empty.error().message == "cannot sample empty logits");

    logits.values = {1.0f, 2.0f};
    SamplingOptions tiny;
    tiny.temperature = 1e-39f;
    auto overflowed = session.sample(logits, tiny);
    check(!overflowed);
    check(overflowed.error().message == "sampling distribution is invalid");
}

// {0,5,5,-1}, Top-K 2: token 1 iff u < 0.5, with u from a shadow generator; calls that keep one
// candidate, greedy calls and failing calls must not advance the Session generator.
static void test_rng_bookkeeping(const HipSamplerPtr& sampler)
{
    SamplingSessionOptions session_options;
    session_options.sampling_seed = 1234;
    SamplingSession session(sampler, session_options);
    std::mt19937_64 shadow(1234);
    std::uniform_real_distribution<float> distribution(0.0f, 1.0f);
    const LogitsOutput logits = logits_of({0.0f, 5.0f, 5.0f, -1.0f});
    SamplingOptions two;
    two.top_k = 2;
    SamplingOptions one;
    one.top_k = 1;
    SamplingOptions greedy;
    greedy.temperature = 0.0f;
    SamplingOptions invalid;
    invalid.min_p = 2.0f;
    for (int call = 0; call < 200; ++call)
    {
        const float u = distribution(shadow);
        auto sampled = session.sample(logits, two);
        check(static_cast<bool>(sampled));
        check(sampled.value().token_id == (u < 0.5f ? 1 : 2));
        check(sampled.value().probability == 0.5f);
        auto single = session.sample(logits, one);
        check(static_cast<bool>(single) && single.value().token_id == 1 && single.value().probability == 1.0f);
        check(static_cast<bool>(session.sample(logits, greedy)));
        check(!session.sample(logits, invalid));
    }
}

static void test_distribution_known_answers(const HipSamplerPtr& sampler)
{
    SamplingOptions options;
    options.temperature = 0.5f;
    options.top_k = 3;
    options.top_p = 0.9f;
    options.min_p = 0.05f;
    const std::vector<float> logits = {1.0f, 2.0f, 3.0f, 4.0f, 5.0f};
    auto candidates = sampler->distribution(logits, options);
    check(static_cast<bool>(candidates));
    check(candidates.value().size() == 2);
    check(candidates.value()[0].token_id == 4 && candidates.value()[1].token_id == 3);
    check_near(candidates.value()[0].probability, 0.880797088f, 1e-7f);
    check_near(candidates.value()[1].probability, 0.119202919f, 1e-7f);

    SamplingOptions ties;
    ties.top_k = 2;
    const std::vector<float> tied = {5.0f, 7.0f, 7.0f, 7.0f};
    candidates = sampler->distribution(tied, ties);
    check(static_cast<bool>(candidates) && candidates.value().size() == 2);
    check(candidates.value()[0].token_id == 1 && candidates.value()[1].token_id == 2);
    check(candidates.value()[0].probability == 0.5f && candidates.value()[1].probability == 0.5f);
}

// A batch over distinct Sessions equals the same Sessions sampled one by one, RNG states included.
static void test_batch_equals_serial(const HipSamplerPtr& sampler)
{
    const int sessions = 24;
    const int vocab = 5000;
    std::mt19937_64 data(99);
    std::normal_distribution<float> normal(0.0f, 2.0f);
    std::vector<LogitsOutput> logits(sessions);
    for (LogitsOutput& row : logits)
    {
        row.values.resize(vocab);
        for (float& value : row.values)
            value = normal(data);
    }
    std::vector<SamplingOptions> options(sessions);
    std::vector<std::vector<int32_t>> stops(sessions);
    for (int i = 0; i < sessions; ++i)
    {
        options[i].temperature = (i % 5 == 0) ? 0.0f : 0.3f + 0.1f * static_cast<float>(i % 7);
        options[i].top_k = (i % 4 == 0) ? 0 : (i % 4 == 1) ? 1 : (i % 4 == 2) ? 20 : 100;
        options[i].top_p = 0.6f + 0.05f * static_cast<float>(i % 8);
        options[i].min_p = (i % 3 == 0) ? 0.05f : 0.0f;
        if (i == 7)
            options[i].top_p = 0.0f; // one bad row must not fail the others
    }
    for (int step = 0; step < 3; ++step)
    {
        std::vector<std::unique_ptr<SamplingSession>> serial;
        std::vector<std::unique_ptr<SamplingSession>> batched;
        for (int i = 0; i < sessions; ++i)
        {
            SamplingSessionOptions so;
            so.sampling_seed = 1000 + i;
            serial.push_back(std::make_unique<SamplingSession>(sampler, so));
            batched.push_back(std::make_unique<SamplingSession>(sampler, so));
        }
        // two rounds so that the committed generator states matter
        for (int round = 0; round < 2; ++round)
        {
            std::vector<Result<SampledToken>> expected;
            for (int i = 0; i < sessions; ++i)
                expected.push_back(serial[i]->sample(logits[i], options[i]));
            std::vector<SampleBatchRequest> requests(sessions);
            for (int i = 0; i < sessions; ++i)
            {
                requests[i].session = batched[i].get();
                requests[i].logits = &logits[i];
                requests[i].sampling = options[i];
                if (expected[i])
                    stops[i] = (i % 2 == 0) ? std::vector<int32_t>{-5, expected[i].value().token_id} : std::vector<int32_t>{-5, -6};
                requests[i].stop_tokens = stops[i];
            }
            auto got = SessionBatchSampler::sample(sampler, requests);
            check(got.size() == static_cast<size_t>(sessions));
            for (int i = 0; i < sessions; ++i)
            {
                check(static_cast<bool>(got[i]) == static_cast<bool>(expected[i]));
                if (!expected[i])
                {
                    check(got[i].error().code == ErrorCode::InvalidArgument);
                    check(got[i].error().message == expected[i].error().message);
                    continue;
                }
                check(got[i].value().token.token_id == expected[i].value().token_id);
                check(got[i].value().token.probability == expected[i].value().probability);
                check(got[i].value().is_stop_token == (i % 2 == 0));
            }
        }
    }
}

static void test_batch_rejects_bad_requests(const HipSamplerPtr& sampler)
{
    SamplingSession a(sampler), b(sampler);
    LogitsOutput logits = logits_of({1.0f, 2.0f, 3.0f});
    LogitsOutput shorter = logits_of({1.0f, 2.0f});
    LogitsOutput empty;
    std::vector<SampleBatchRequest> requests(2);
    requests[0].session = &a;
    requests[0].logits = &logits;
    requests[1].session = &a;
    requests[1].logits = &logits;
    auto duplicate = SessionBatchSampler::sample(sampler, requests);
    check(duplicate.size() == 2 && !duplicate[0] && !duplicate[1]);
    check(duplicate[0].error().code == ErrorCode::InvalidArgument);
    check(duplicate[0].error().message == "sample batch contains duplicate sessions");
    requests[1].session = &b;
    requests[1].logits = &shorter;
    auto ragged = SessionBatchSampler::sample(sampler, requests);
    check(!ragged[0] && ragged[0].error().message == "sample batch rows differ in length");
    requests[1].logits = &empty;
    auto with_empty = SessionBatchSampler::sample(sampler, requests);
    check(static_cast<bool>(with_empty[0]));
    check(!with_empty[1] && with_empty[1].error().message == "cannot sample empty logits");
    requests[1].logits = nullptr;
    check(!SessionBatchSampler::sample(sampler, requests)[0]);
    check(SessionBatchSampler::sample(sampler, {}).empty());
}

// The verification step of speculative generation (src/engine/session.cpp:776-874): what is accepted,
// what follows, which error text comes back, and that the Session's generator advances by exactly the
// draws the step consumed.
static void test_speculative_verification(const HipSamplerPtr& sampler)
{
    const std::vector<float> ramp = {0.0f, 1.0f, 2.0f, 3.0f, 2.5f, -1.0f};
    // greedy: the first two proposals are the target's own choices, the third is not
    {
        SamplingSession session(sampler, SamplingSessionOptions{7});
        std::vector<LogitsOutput> target = {logits_of(ramp), logits_of({5, 0, 0, 0, 0, 0}), logits_of({0, 0, 9, 0, 0, 0}),
                                            logits_of({0, 7, 0, 0, 0, 0})};
        std::vector<LogitsOutput> draft = {logits_of(ramp), logits_of(ramp), logits_of(ramp)};
        const std::vector<int32_t> proposed = {3, 0, 4};
        SamplingOptions greedy;
        greedy.temperature = 0.0f;
        auto verified = session.verify_speculative(target, draft, proposed, greedy);
        check(static_cast<bool>(verified));
        check(verified.value().accepted.size() == 2);
        check(verified.value().accepted[0].token_id == 3 && verified.value().accepted[0].probability == 1.0f);
        check(verified.value().accepted[1].token_id == 0);
        check(verified.value().next.token_id == 2 && verified.value().next.probability == 1.0f);
        check(!verified.value().next_from_residual);
        // no draw was consumed: the next sampled token is decided by the generator's first output
        std::mt19937_64 shadow(7);
        const float u = std::uniform_real_distribution<float>(0.0f, 1.0f)(shadow);
        SamplingOptions two;
        two.top_k = 2;
        auto sampled = session.sample(logits_of({0, 5, 5, -1}), two);
        check(static_cast<bool>(sampled));
        check(sampled.value().token_id == (u < 0.5f ? 1 : 2));
    }
    // identical target and draft distributions: every proposal stands (ratio 1), D accept draws and
    // one draw for the row behind the last proposal
    {
        SamplingSession session(sampler, SamplingSessionOptions{11});
        std::vector<LogitsOutput> target = {logits_of(ramp), logits_of(ramp), logits_of({0, 5, 5, -1, -1, -1})};
        std::vector<LogitsOutput> draft = {logits_of(ramp), logits_of(ramp)};
        SamplingOptions options;
        options.top_k = 4;
        auto verified = session.verify_speculative(target, draft, std::vector<int32_t>{2, 4}, options);
        check(static_cast<bool>(verified));
        check(verified.value().accepted.size() == 2 && !verified.value().next_from_residual);
        std::mt19937_64 shadow(11);
        std::uniform_real_distribution<float> canonical(0.0f, 1.0f);
        canonical(shadow);
        canonical(shadow);
        const float u_final = canonical(shadow);
        check(verified.value().next.token_id == (u_final < 0.5f ? 1 : 2));
        const float u_next = canonical(shadow);
        SamplingOptions two;
        two.top_k = 2;
        auto sampled = session.sample(logits_of({0, 5, 5, -1}), two);
        check(sampled.value().token_id == (u_next < 0.5f ? 1 : 2));
    }
    // a draft that is sure of a token the target rates low: rejected, the next token comes from the residual
    {
        std::vector<float> sure = ramp;
        sure[5] = 40.0f;
        int rejected = 0;
        for (uint64_t seed = 0; seed < 8; ++seed)
        {
            SamplingSession session(sampler, SamplingSessionOptions{seed});
            std::vector<LogitsOutput> target = {logits_of(ramp), logits_of(ramp)};
            std::vector<LogitsOutput> draft = {logits_of(sure)};
            SamplingOptions options;
            options.top_k = 6;
            auto verified = session.verify_speculative(target, draft, std::vector<int32_t>{5}, options);
            check(static_cast<bool>(verified));
            if (verified.value().accepted.empty())
            {
                ++rejected;
                check(verified.value().next_from_residual);
                check(verified.value().next.token_id != 5 && verified.value().next.probability > 0.0f);
            }
        }
        check(rejected >= 7); // the target gives token 5 about 0.8 % of the mass
    }
    // error text
    {
        SamplingSession session(sampler);
        std::vector<LogitsOutput> target = {logits_of(ramp), logits_of(ramp)};
        std::vector<LogitsOutput> draft = {logits_of(ramp)};
        SamplingOptions options;
        options.top_k = 2;
        auto outside = session.verify_speculative(target, draft, std::vector<int32_t>{0}, options);
        check(!outside && outside.error().code == ErrorCode::InternalError);
        check(outside.error().message == "sampled draft token has zero probability");
        // a flat vocabulary of 3000 tokens with no filter: distributions longer than the entry holds
        std::vector<LogitsOutput> long_target = {logits_of(std::vector<float>(3000, 0.5f)), logits_of(std::vector<float>(3000, 0.5f))};
        std::vector<LogitsOutput> long_draft = {logits_of(std::vector<float>(3000, 0.5f))};
        auto window = session.verify_speculative(long_target, long_draft, std::vector<int32_t>{3}, SamplingOptions{});
        check(!window && window.error().code == ErrorCode::InvalidArgument);
        // the same options over a short vocabulary are served
        auto whole = session.verify_speculative(target, draft, std::vector<int32_t>{3}, SamplingOptions{});
        check(static_cast<bool>(whole));
        std::vector<LogitsOutput> broken = {logits_of(std::vector<float>(6, -std::numeric_limits<float>::infinity())), logits_of(ramp)};
        auto no_finite = session.verify_speculative(broken, draft, std::vector<int32_t>{3}, options);
        check(!no_finite && no_finite.error().message == "sampling requires at least one finite logit");
        auto lengths = session.verify_speculative(target, draft, std::vector<int32_t>{3, 3}, options);
        check(!lengths && lengths.error().code == ErrorCode::InvalidArgument);
    }
}

int main(int argc, char** argv)
{
    const bool host_only = argc > 1 && std::strcmp(argv[1], "--host") == 0;
    try
    {
        test_option_validation_messages();
        test_defaults_match_the_runtime();
        test_peek_uniform_does_not_advance();
        test_missing_sampler_fails_loudly();
        if (host_only)
        {
            std::printf("all host-side session sampler tests passed\n");
            return 0;
        }
        HipSamplerPtr sampler = HipSampler::create(0, 64, 8192);
        if (!sampler)
        {
            std::fprintf(stderr, "HipSampler::create failed: no usable GPU\n");
            return 2;
        }
        test_sampling_like_the_runtime_test(sampler);
        test_rng_bookkeeping(sampler);
        test_distribution_known_answers(sampler);
        test_batch_equals_serial(sampler);
        test_batch_rejects_bad_requests(sampler);
        test_speculative_verification(sampler);
    }
    catch (const std::exception& error)
    {
        std::fprintf(stderr, "FAILED: %s\n", error.what());
        return 1;
    }
    std::printf("all session sampler tests passed\n");
    return 0;
}
