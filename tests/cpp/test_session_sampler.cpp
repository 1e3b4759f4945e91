// Tests of the C++ host face of the HIP sampler, written in the manner of the runtime's own test
// binary (hand-rolled check()/check_near(), one function per topic, "all ... passed" at the end).
// The first group mirrors the runtime's sampler test (tests/test_runtime.cpp:4320-4362); the rest
// cover what that test leaves out: draws, RNG bookkeeping, batches, stop tokens, error text.
//
//   test_session_sampler                      all tests (needs a GPU)
//   test_session_sampler --host               only the tests that need no GPU
//   test_session_sampler --generation-bench SESSIONS VOCAB STEPS   times the batched generation loop
//   test_session_sampler --generation-trace   runs the batched generation loop on the synthetic
//                                             model below and prints every emitted token, for a
//                                             checker that recomputes the run with the CPU sampler
#include "hip_session_sampler.h"
#include "synthetic_model.h"
#include "worker_wire.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <bit>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <future>
#include <limits>
#include <random>
#include <stdexcept>
#include <string>
#include <thread>
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

// Worker threads that share one sampler, each with Sessions of its own (the runtime's scheduler
// workers and std::async callers, src/engine/scheduler.cpp:87-104): every thread must see exactly
// what it would have seen alone, single calls and batched calls interleaved.
static void test_threads_share_a_sampler(const HipSamplerPtr& sampler)
{
    const int threads = 8;
    const int steps = 30;
    const int vocab = 3000;
    std::vector<std::vector<LogitsOutput>> logits(threads, std::vector<LogitsOutput>(steps));
    std::vector<SamplingOptions> options(threads);
    for (int t = 0; t < threads; ++t)
    {
        std::mt19937_64 data(500 + t);
        std::normal_distribution<float> normal(0.0f, 2.5f);
        for (LogitsOutput& row : logits[t])
        {
            row.values.resize(vocab);
            for (float& value : row.values)
                value = normal(data);
        }
        options[t].temperature = 0.4f + 0.15f * static_cast<float>(t);
        options[t].top_k = (t % 4 == 0) ? 0 : (t % 4 == 1) ? 40 : (t % 4 == 2) ? 200 : 8;
        options[t].top_p = 0.7f + 0.03f * static_cast<float>(t);
        options[t].min_p = (t % 2 == 0) ? 0.01f : 0.0f;
    }
    // thread t: step s is a single call on Session A when s is even, a batch over Sessions A and B when odd
    const auto run = [&](int t, std::vector<SampledToken>& out) {
        SamplingSessionOptions so;
        so.sampling_seed = 7000 + t;
        SamplingSession a(sampler, so);
        so.sampling_seed = 8000 + t;
        SamplingSession b(sampler, so);
        for (int step = 0; step < steps; ++step)
        {
            if (step % 2 == 0)
            {
                auto sampled = a.sample(logits[t][step], options[t]);
                check(static_cast<bool>(sampled));
                out.push_back(sampled.value());
                continue;
            }
            std::vector<SampleBatchRequest> requests(2);
            requests[0].session = &a;
            requests[0].logits = &logits[t][step];
            requests[0].sampling = options[t];
            requests[1].session = &b;
            requests[1].logits = &logits[t][step - 1];
            requests[1].sampling = options[(t + 1) % threads];
            auto sampled = SessionBatchSampler::sample(sampler, requests);
            check(sampled.size() == 2 && sampled[0] && sampled[1]);
            out.push_back(sampled[0].value().token);
            out.push_back(sampled[1].value().token);
        }
    };
    std::vector<std::vector<SampledToken>> expected(threads);
    for (int t = 0; t < threads; ++t)
        run(t, expected[t]);
    std::vector<std::vector<SampledToken>> got(threads);
    std::vector<std::string> failures(threads);
    std::vector<std::thread> workers;
    for (int t = 0; t < threads; ++t)
        workers.emplace_back([&, t] {
            try
            {
                run(t, got[t]);
            }
            catch (const std::exception& error)
            {
                failures[t] = error.what();
            }
        });
    for (std::thread& worker : workers)
        worker.join();
    for (int t = 0; t < threads; ++t)
    {
        if (!failures[t].empty())
            throw std::runtime_error("thread " + std::to_string(t) + ": " + failures[t]);
        check(got[t].size() == expected[t].size());
        for (size_t i = 0; i < got[t].size(); ++i)
        {
            check(got[t][i].token_id == expected[t][i].token_id);
            check(std::bit_cast<uint32_t>(got[t][i].probability) == std::bit_cast<uint32_t>(expected[t][i].probability));
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
        // a flat vocabulary of 3000 tokens with no filter: distributions longer than the fast kernel's
        // lists are served by the dense one (equal target and draft: the token is always accepted)
        std::vector<LogitsOutput> long_target = {logits_of(std::vector<float>(3000, 0.5f)), logits_of(std::vector<float>(3000, 0.5f))};
        std::vector<LogitsOutput> long_draft = {logits_of(std::vector<float>(3000, 0.5f))};
        auto window = session.verify_speculative(long_target, long_draft, std::vector<int32_t>{3}, SamplingOptions{});
        check(static_cast<bool>(window));
        check(window.value().accepted.size() == 1 && window.value().accepted[0].token_id == 3);
        check(!window.value().next_from_residual && window.value().next.token_id >= 0 && window.value().next.token_id < 3000);
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

// ---- the scheduler's batched-sample entry, output modes, capability bit ---------------------------

static void test_scheduler_and_modes_without_a_sampler()
{
    // Runtime::create_session (src/engine/runtime.cpp:575-582): without the device sampler only full logits
    auto full = create_sampling_session(nullptr, SamplingSessionOptions{3, LogitsOutputMode::FullLogits});
    check(static_cast<bool>(full) && full.value()->logits_output_mode() == LogitsOutputMode::FullLogits);
    auto sampled_only = create_sampling_session(nullptr, SamplingSessionOptions{3, LogitsOutputMode::SampledToken});
    check(!sampled_only && sampled_only.error().code == ErrorCode::UnsupportedModel);
    check(sampled_only.error().message == "the current executor supports full logits output only");
    auto candidates = create_sampling_session(nullptr, SamplingSessionOptions{3, LogitsOutputMode::TopKCandidates});
    check(!candidates && candidates.error().code == ErrorCode::UnsupportedModel);
    check(RuntimeCapabilityHipSampler == (UINT32_C(1) << 18)); // the runtime's own flags end at bit 17
    check((hip_sampler_capabilities() & ~static_cast<uint32_t>(RuntimeCapabilityHipSampler)) == 0);

    // the scheduler without a sampler: every row of every submission reports the missing device
    BatchSampleScheduler scheduler(nullptr, SampleSchedulerOptions{2, 100, 0});
    SamplingSession a(nullptr), b(nullptr);
    const LogitsOutput logits = logits_of({1.0f, 2.0f, 3.0f});
    std::vector<SampleBatchRequest> pair = {SampleBatchRequest{&a, &logits, {}, {}}, SampleBatchRequest{&b, &logits, {}, {}}};
    auto results = scheduler.submit_sample(pair).get();
    check(results.size() == 2 && !results[0] && !results[1]);
    check(results[0].error().code == ErrorCode::InternalError);
    auto single = scheduler.submit_sample({SampleBatchRequest{&a, &logits, {}, {}}}).get();
    check(single.size() == 1 && !single[0] && single[0].error().code == ErrorCode::InternalError);
    // rejected at submission: a Session named twice (src/engine/session.cpp:1257-1265), a null Session
    auto duplicate = scheduler.submit_sample({SampleBatchRequest{&a, &logits, {}, {}}, SampleBatchRequest{&a, &logits, {}, {}}}).get();
    check(duplicate.size() == 2 && !duplicate[0] && duplicate[0].error().code == ErrorCode::InvalidArgument);
    check(duplicate[0].error().message == "sample batch contains duplicate sessions");
    auto missing = scheduler.submit_sample({SampleBatchRequest{nullptr, &logits, {}, {}}}).get();
    check(missing.size() == 1 && !missing[0] && missing[0].error().code == ErrorCode::InvalidArgument);
    check(scheduler.submit_sample({}).get().empty());
    const SampleSchedulerStatistics statistics = scheduler.statistics();
    check(statistics.worker_count == 2);
    check(statistics.submitted_batches == 5 && statistics.submitted_requests == 6);
    check(statistics.rejected_requests == 3 && statistics.completed_requests == 3);
}

// One Session per thread, each sampling its own row again and again through the scheduler: the rows of
// different threads share device calls, and every Session sees the tokens it would have drawn alone.
static void test_scheduler_collects_across_calls(const HipSamplerPtr& sampler)
{
    constexpr int kSessions = 12, kSteps = 10;
    const uint32_t vocab = 5000;
    SamplingOptions options;
    options.temperature = 0.9f;
    options.top_k = 40;
    options.top_p = 0.95f;
    std::vector<std::vector<SampledToken>> alone(kSessions), together(kSessions);
    for (int s = 0; s < kSessions; ++s)
    {
        SamplingSession session(sampler, SamplingSessionOptions{static_cast<uint64_t>(100 + s)});
        for (int step = 0; step < kSteps; ++step)
        {
            auto token = session.sample(logits_of(synthetic_logits(vocab, s, step, 17)), options);
            check(static_cast<bool>(token));
            alone[s].push_back(token.value());
        }
    }
    std::deque<SamplingSession> sessions;
    for (int s = 0; s < kSessions; ++s)
        sessions.emplace_back(sampler, SamplingSessionOptions{static_cast<uint64_t>(100 + s)});
    BatchSampleScheduler scheduler(sampler, SampleSchedulerOptions{3, 2000, 0});
    std::vector<std::thread> threads;
    std::vector<std::string> failures(kSessions);
    for (int s = 0; s < kSessions; ++s)
    {
        threads.emplace_back([&, s] {
            for (int step = 0; step < kSteps; ++step)
            {
                const LogitsOutput logits = logits_of(synthetic_logits(vocab, s, step, 17));
                auto results = scheduler.submit_sample({SampleBatchRequest{&sessions[s], &logits, options, {}}}).get();
                if (results.size() != 1 || !results[0])
                {
                    failures[s] = results.empty() ? "no result" : results[0].error().message;
                    return;
                }
                together[s].push_back(results[0].value().token);
            }
        });
    }
    for (std::thread& thread : threads)
        thread.join();
    for (int s = 0; s < kSessions; ++s)
    {
        check(failures[s].empty());
        check(together[s].size() == alone[s].size());
        for (int step = 0; step < kSteps; ++step)
        {
            check(together[s][step].token_id == alone[s][step].token_id);
            check(std::bit_cast<uint32_t>(together[s][step].probability) == std::bit_cast<uint32_t>(alone[s][step].probability));
        }
    }
    const SampleSchedulerStatistics statistics = scheduler.statistics();
    check(statistics.completed_requests == kSessions * kSteps && statistics.rejected_requests == 0);
    check(statistics.device_calls <= static_cast<uint64_t>(kSessions * kSteps));
    check(statistics.cross_call_collected_requests + statistics.cross_call_collection_timeouts >= statistics.device_calls);
    std::printf("scheduler: %d requests in %llu device calls (largest batch %llu, %llu requests collected across calls)\n", kSessions * kSteps,
                static_cast<unsigned long long>(statistics.device_calls), static_cast<unsigned long long>(statistics.max_batch_size),
                static_cast<unsigned long long>(statistics.cross_call_collected_requests));
}

// Requests of one Session keep their order (its generator's draws go to them in that order), alone
// or mixed into batches with other Sessions; a multi-request submission is one device call.
static void test_scheduler_keeps_a_sessions_order(const HipSamplerPtr& sampler)
{
    const uint32_t vocab = 3000;
    SamplingOptions options;
    options.top_k = 30;
    constexpr int kRequests = 9;
    std::vector<LogitsOutput> rows;
    for (int i = 0; i < kRequests; ++i)
        rows.push_back(logits_of(synthetic_logits(vocab, 5, i, 3)));
    SamplingSession serial(sampler, SamplingSessionOptions{77});
    std::vector<SampledToken> expected;
    for (int i = 0; i < kRequests; ++i)
        expected.push_back(serial.sample(rows[i], options).value());
    SamplingSession session(sampler, SamplingSessionOptions{77});
    SamplingSession other(sampler, SamplingSessionOptions{78});
    BatchSampleScheduler scheduler(sampler, SampleSchedulerOptions{4, 300, 0}); // after the Sessions: its workers stop first
    std::vector<std::future<std::vector<Result<BatchSampledToken>>>> futures;
    for (int i = 0; i < kRequests; ++i)
    {
        if (i % 3 == 1) // in a batch with another Session
            futures.push_back(scheduler.submit_sample({SampleBatchRequest{&other, &rows[0], options, {}}, SampleBatchRequest{&session, &rows[i], options, {}}}));
        else
            futures.push_back(scheduler.submit_sample({SampleBatchRequest{&session, &rows[i], options, {}}}));
    }
    for (int i = 0; i < kRequests; ++i)
    {
        auto results = futures[i].get();
        const Result<BatchSampledToken>& mine = results.back();
        check(static_cast<bool>(mine));
        check(mine.value().token.token_id == expected[i].token_id);
        check(std::bit_cast<uint32_t>(mine.value().token.probability) == std::bit_cast<uint32_t>(expected[i].probability));
    }
    check(scheduler.statistics().serialized_session_requests >= 1);
}

// Sessions in SampledToken mode: the rows are written into the sampler's device buffer (here with a copy,
// by a decode step in the runtime) and only tokens come back; same tokens as the full-logits Sessions.
static void test_sampled_token_mode(const HipSamplerPtr& sampler)
{
    const uint32_t vocab = 4001, count = 6;
    check(hip_sampler_capabilities() == RuntimeCapabilityHipSampler);
    SamplingOptions options;
    options.temperature = 0.8f;
    options.top_k = 25;
    std::vector<SamplingSessionPtr> resident, full;
    for (uint32_t i = 0; i < count; ++i)
    {
        auto a = create_sampling_session(sampler, SamplingSessionOptions{500 + i, LogitsOutputMode::SampledToken});
        auto b = create_sampling_session(sampler, SamplingSessionOptions{500 + i, LogitsOutputMode::FullLogits});
        check(static_cast<bool>(a) && static_cast<bool>(b));
        resident.push_back(a.value());
        full.push_back(b.value());
    }
    auto host_entry = resident[0]->sample(logits_of({1.0f, 2.0f}), options);
    check(!host_entry && host_entry.error().code == ErrorCode::InvalidArgument);
    for (uint32_t step = 0; step < 3; ++step)
    {
        auto rows = sampler->device_logits(count, vocab);
        check(static_cast<bool>(rows));
        std::vector<LogitsOutput> host_rows;
        for (uint32_t i = 0; i < count; ++i)
        {
            host_rows.push_back(logits_of(synthetic_logits(vocab, i, step, 9)));
            check(hipMemcpy(static_cast<float*>(rows.value().data) + static_cast<size_t>(i) * rows.value().row_stride, host_rows[i].values.data(),
                            vocab * sizeof(float), hipMemcpyHostToDevice) == hipSuccess);
        }
        std::vector<SampleBatchRequest> requests, full_requests;
        for (uint32_t i = 0; i < count; ++i)
        {
            requests.push_back(SampleBatchRequest{resident[i].get(), nullptr, options, {}});
            full_requests.push_back(SampleBatchRequest{full[i].get(), &host_rows[i], options, {}});
        }
        auto got = SessionBatchSampler::sample_resident(sampler, requests);
        auto expected = SessionBatchSampler::sample(sampler, full_requests);
        check(got.size() == count && expected.size() == count);
        // that sample() of host logits used the buffer: the rows laid out before are gone, and say so
        auto stale = SessionBatchSampler::sample_resident(sampler, requests);
        check(stale.size() == count && !stale[0] && stale[0].error().code == ErrorCode::InvalidArgument &&
              stale[0].error().message.find("overwritten") != std::string::npos);
        for (uint32_t i = 0; i < count; ++i)
        {
            check(static_cast<bool>(got[i]) && static_cast<bool>(expected[i]));
            check(got[i].value().token.token_id == expected[i].value().token.token_id);
            check(std::bit_cast<uint32_t>(got[i].value().token.probability) == std::bit_cast<uint32_t>(expected[i].value().token.probability));
        }
    }
    // the two kinds do not mix
    const LogitsOutput row = logits_of({1.0f, 2.0f, 3.0f});
    auto mixed = SessionBatchSampler::sample(sampler, std::vector<SampleBatchRequest>{SampleBatchRequest{resident[0].get(), &row, options, {}}});
    check(mixed.size() == 1 && !mixed[0] && mixed[0].error().code == ErrorCode::InvalidArgument);
    auto wrong = SessionBatchSampler::sample_resident(sampler, std::vector<SampleBatchRequest>{SampleBatchRequest{full[0].get(), nullptr, options, {}}});
    check(wrong.size() == 1 && !wrong[0] && wrong[0].error().code == ErrorCode::InvalidArgument);
}

// SampledToken-mode requests that travel alone through the scheduler, one serving thread per Session, in an
// order that has nothing to do with the decode step's: each names the device row that holds its logits.  Tokens
// per Session against SessionBatchSampler::sample_resident on the whole batch in layout order.
static void test_resident_requests_through_the_scheduler(const HipSamplerPtr& sampler)
{
    const uint32_t vocab = 4001, count = 8;
    SamplingOptions options;
    options.temperature = 0.9f;
    options.top_k = 30;
    options.top_p = 0.95f;
    std::vector<SamplingSessionPtr> scheduled, direct;
    for (uint32_t i = 0; i < count; ++i)
    {
        scheduled.push_back(create_sampling_session(sampler, SamplingSessionOptions{900 + i, LogitsOutputMode::SampledToken}).value());
        direct.push_back(create_sampling_session(sampler, SamplingSessionOptions{900 + i, LogitsOutputMode::SampledToken}).value());
    }
    SampleSchedulerOptions scheduler_options;
    scheduler_options.worker_count = 4;
    scheduler_options.cross_call_window_microseconds = 3000;
    BatchSampleScheduler scheduler(sampler, scheduler_options);
    for (uint32_t step = 0; step < 4; ++step)
    {
        auto rows = sampler->device_logits(count, vocab);
        check(static_cast<bool>(rows));
        for (uint32_t i = 0; i < count; ++i)
        {
            const std::vector<float> values = synthetic_logits(vocab, i, step, 17);
            check(hipMemcpy(static_cast<float*>(rows.value().data) + static_cast<size_t>(i) * rows.value().row_stride, values.data(),
                            vocab * sizeof(float), hipMemcpyHostToDevice) == hipSuccess);
        }
        std::vector<SampleBatchRequest> whole;
        for (uint32_t i = 0; i < count; ++i)
            whole.push_back(SampleBatchRequest{direct[i].get(), nullptr, options, {}});
        auto expected = SessionBatchSampler::sample_resident(sampler, whole);
        std::vector<std::future<std::vector<Result<BatchSampledToken>>>> futures(count);
        std::vector<std::thread> threads;
        for (uint32_t k = 0; k < count; ++k)
        {
            const uint32_t i = (k * 5 + step) % count; // Session i's thread starts k-th
            threads.emplace_back([&, i] {
                SampleBatchRequest request{scheduled[i].get(), nullptr, options, {}};
                request.device_row = i;
                futures[i] = scheduler.submit_sample(std::vector<SampleBatchRequest>{request});
            });
        }
        for (std::thread& thread : threads)
            thread.join();
        for (uint32_t i = 0; i < count; ++i)
        {
            auto got = futures[i].get();
            check(got.size() == 1 && static_cast<bool>(got[0]) && static_cast<bool>(expected[i]));
            check(got[0].value().token.token_id == expected[i].value().token.token_id);
            check(std::bit_cast<uint32_t>(got[0].value().token.probability) == std::bit_cast<uint32_t>(expected[i].value().token.probability));
        }
    }
    check(scheduler.statistics().cross_call_collected_requests > 0);
    // a subset of the rows, named in descending order, directly
    {
        std::vector<SampleBatchRequest> whole, some;
        for (uint32_t i = 0; i < count; ++i)
            whole.push_back(SampleBatchRequest{direct[i].get(), nullptr, options, {}});
        for (uint32_t i : {6u, 3u, 1u})
        {
            SampleBatchRequest request{scheduled[i].get(), nullptr, options, {}};
            request.device_row = i;
            some.push_back(request);
        }
        auto got = SessionBatchSampler::sample_resident(sampler, some);
        auto expected = SessionBatchSampler::sample_resident(sampler, whole);
        const uint32_t named[3] = {6, 3, 1};
        for (size_t j = 0; j < 3; ++j)
        {
            check(static_cast<bool>(got[j]) && got[j].value().token.token_id == expected[named[j]].value().token.token_id);
            check(std::bit_cast<uint32_t>(got[j].value().token.probability) == std::bit_cast<uint32_t>(expected[named[j]].value().token.probability));
        }
        // (the Sessions of `scheduled` that were not named keep their generators: bring them level again)
        std::vector<SampleBatchRequest> rest;
        for (uint32_t i : {0u, 2u, 4u, 5u, 7u})
        {
            SampleBatchRequest request{scheduled[i].get(), nullptr, options, {}};
            request.device_row = i;
            rest.push_back(request);
        }
        auto level = SessionBatchSampler::sample_resident(sampler, rest);
        check(level.size() == 5 && static_cast<bool>(level[0]));
        // a row named twice, a row beyond the layout, rows named for some requests only
        some[1].device_row = 6;
        auto twice = SessionBatchSampler::sample_resident(sampler, some);
        check(!twice[0] && twice[0].error().message.find("twice") != std::string::npos);
        some[1].device_row = count;
        auto beyond = SessionBatchSampler::sample_resident(sampler, some);
        check(!beyond[0] && beyond[0].error().message.find("beyond") != std::string::npos);
        some[1].device_row = SampleBatchRequest::kRowByPosition;
        auto partly = SessionBatchSampler::sample_resident(sampler, some);
        check(!partly[0] && partly[0].error().code == ErrorCode::InvalidArgument);
    }
    // a request that names no row and travels alone is a batch of one: row 0 of a one-row layout, never merged
    {
        auto one = sampler->device_logits(1, vocab);
        check(static_cast<bool>(one));
        const std::vector<float> values = synthetic_logits(vocab, 3, 9, 17);
        check(hipMemcpy(one.value().data, values.data(), vocab * sizeof(float), hipMemcpyHostToDevice) == hipSuccess);
        const uint64_t collected_before = scheduler.statistics().cross_call_collected_requests;
        auto alone = scheduler.submit_sample(std::vector<SampleBatchRequest>{SampleBatchRequest{scheduled[0].get(), nullptr, options, {}}}).get();
        auto same = SessionBatchSampler::sample_resident(sampler, std::vector<SampleBatchRequest>{SampleBatchRequest{direct[0].get(), nullptr, options, {}}});
        check(alone.size() == 1 && static_cast<bool>(alone[0]) && alone[0].value().token.token_id == same[0].value().token.token_id);
        check(scheduler.statistics().cross_call_collected_requests == collected_before);
    }
    // the two kinds in one batch, and a sampler the scheduler does not have
    {
        const LogitsOutput row = logits_of({1.0f, 2.0f, 3.0f});
        SamplingSession host_session(sampler, SamplingSessionOptions{5});
        std::vector<SampleBatchRequest> mixed = {SampleBatchRequest{scheduled[0].get(), nullptr, options, {}},
                                                 SampleBatchRequest{&host_session, &row, options, {}}};
        auto rejected = scheduler.submit_sample(mixed).get();
        check(rejected.size() == 2 && !rejected[0] && rejected[0].error().message.find("mixes") != std::string::npos);
        SampleBatchRequest elsewhere{scheduled[0].get(), nullptr, options, {}};
        elsewhere.resident_sampler = 3;
        auto missing = scheduler.submit_sample(std::vector<SampleBatchRequest>{elsewhere}).get();
        check(missing.size() == 1 && !missing[0] && missing[0].error().code == ErrorCode::InvalidArgument);
    }
}

// A scheduler over three samplers: batches of host logits that its workers run at the same time go to
// different samplers (buffers and streams of their own) and overlap on the GPU, while a device-resident batch
// runs on the sampler that holds its rows.  Every batch bit-equal to the same batch sampled alone.
static void test_scheduler_over_several_samplers(const HipSamplerPtr& first)
{
    const uint32_t vocab = 6007, batches = 18, per_batch = 5;
    std::vector<HipSamplerPtr> samplers = {first, HipSampler::create(0, 64, 8192), HipSampler::create(0, 64, 8192)};
    check(samplers[1] != nullptr && samplers[2] != nullptr);
    SamplingOptions options;
    options.temperature = 0.8f;
    options.top_k = 40;
    options.top_p = 0.9f;
    std::deque<SamplingSession> through, alone;
    std::vector<std::vector<LogitsOutput>> rows(batches);
    for (uint32_t b = 0; b < batches; ++b)
    {
        for (uint32_t i = 0; i < per_batch; ++i)
        {
            through.emplace_back(first, SamplingSessionOptions{3000 + b * per_batch + i});
            alone.emplace_back(first, SamplingSessionOptions{3000 + b * per_batch + i});
            rows[b].push_back(logits_of(synthetic_logits(vocab, b * per_batch + i, 2, 41)));
        }
    }
    SampleSchedulerOptions scheduler_options;
    scheduler_options.worker_count = 3;
    scheduler_options.cross_call_window_microseconds = 0;
    BatchSampleScheduler scheduler(samplers, scheduler_options);
    check(scheduler.sampler_count() == 3 && scheduler.sampler(0) == first && scheduler.sampler(3) == nullptr);
    // rows on the first sampler's buffer, for a resident batch in the middle of the host batches
    std::deque<SamplingSession> resident_through, resident_alone;
    auto laid_out = scheduler.sampler(0)->device_logits(4, vocab);
    check(static_cast<bool>(laid_out));
    for (uint32_t i = 0; i < 4; ++i)
    {
        resident_through.emplace_back(first, SamplingSessionOptions{7000 + i, LogitsOutputMode::SampledToken});
        resident_alone.emplace_back(first, SamplingSessionOptions{7000 + i, LogitsOutputMode::SampledToken});
        const std::vector<float> values = synthetic_logits(vocab, 100 + i, 0, 41);
        check(hipMemcpy(static_cast<float*>(laid_out.value().data) + static_cast<size_t>(i) * laid_out.value().row_stride, values.data(),
                        vocab * sizeof(float), hipMemcpyHostToDevice) == hipSuccess);
    }
    std::vector<std::future<std::vector<Result<BatchSampledToken>>>> futures;
    std::future<std::vector<Result<BatchSampledToken>>> resident_future;
    for (uint32_t b = 0; b < batches; ++b)
    {
        std::vector<SampleBatchRequest> requests;
        for (uint32_t i = 0; i < per_batch; ++i)
            requests.push_back(SampleBatchRequest{&through[b * per_batch + i], &rows[b][i], options, {}});
        futures.push_back(scheduler.submit_sample(std::move(requests)));
        if (b == batches / 2)
        {
            std::vector<SampleBatchRequest> resident;
            for (uint32_t i = 0; i < 4; ++i)
                resident.push_back(SampleBatchRequest{&resident_through[i], nullptr, options, {}});
            resident_future = scheduler.submit_sample(std::move(resident));
        }
    }
    for (uint32_t b = 0; b < batches; ++b)
    {
        auto got = futures[b].get();
        std::vector<SampleBatchRequest> requests;
        for (uint32_t i = 0; i < per_batch; ++i)
            requests.push_back(SampleBatchRequest{&alone[b * per_batch + i], &rows[b][i], options, {}});
        auto expected = SessionBatchSampler::sample(samplers[1], requests);
        check(got.size() == per_batch);
        for (uint32_t i = 0; i < per_batch; ++i)
        {
            check(static_cast<bool>(got[i]) && static_cast<bool>(expected[i]));
            check(got[i].value().token.token_id == expected[i].value().token.token_id);
            check(std::bit_cast<uint32_t>(got[i].value().token.probability) == std::bit_cast<uint32_t>(expected[i].value().token.probability));
        }
    }
    // no host batch ran on the first sampler: its rows are still there, for the scheduler's batch and for this one
    auto resident_got = resident_future.get();
    std::vector<SampleBatchRequest> resident;
    for (uint32_t i = 0; i < 4; ++i)
        resident.push_back(SampleBatchRequest{&resident_alone[i], nullptr, options, {}});
    auto resident_expected = SessionBatchSampler::sample_resident(first, resident);
    for (uint32_t i = 0; i < 4; ++i)
    {
        check(static_cast<bool>(resident_got[i]) && static_cast<bool>(resident_expected[i]));
        check(resident_got[i].value().token.token_id == resident_expected[i].value().token.token_id);
    }
    const SampleSchedulerStatistics statistics = scheduler.statistics();
    check(statistics.device_calls == batches + 1 && statistics.completed_requests == batches * per_batch + 4);
    std::printf("scheduler over 3 samplers: %llu of %llu device calls began while another was running\n",
                static_cast<unsigned long long>(statistics.overlapped_device_calls), static_cast<unsigned long long>(statistics.device_calls));
}

// A state without cache transactions: a step in which nothing is accepted falls back before the next token
// is drawn (src/engine/session.cpp:843-857); only the accept test's draw is consumed.
static void test_speculative_fallback(const HipSamplerPtr& sampler)
{
    const std::vector<float> ramp = {0.0f, 1.0f, 2.0f, 3.0f, 2.5f, -1.0f};
    SamplingOptions two;
    two.top_k = 2;
    // sampled: the target's window (Top-2: tokens 3 and 4) does not hold the proposed token, so the
    // accept test fails whatever the draw is
    {
        std::vector<float> draft_row = ramp;
        draft_row[0] = 9.0f;
        SamplingSession session(sampler, SamplingSessionOptions{21});
        std::vector<LogitsOutput> target = {logits_of(ramp), logits_of(ramp)};
        std::vector<LogitsOutput> draft = {logits_of(draft_row)};
        auto verified = session.verify_speculative(target, draft, std::vector<int32_t>{0}, two, false);
        check(static_cast<bool>(verified));
        check(verified.value().fell_back && verified.value().accepted.empty() && verified.value().next.token_id == -1);
        std::mt19937_64 shadow(21);
        std::uniform_real_distribution<float> canonical(0.0f, 1.0f);
        canonical(shadow); // the accept test's draw; the residual's draw was not taken
        const float u = canonical(shadow);
        auto sampled = session.sample(logits_of({0, 5, 5, -1}), two);
        check(sampled.value().token_id == (u < 0.5f ? 1 : 2));
        // with cache transactions the same step draws the next token from the residual
        SamplingSession transactional(sampler, SamplingSessionOptions{21});
        auto kept = transactional.verify_speculative(target, draft, std::vector<int32_t>{0}, two, true);
        check(static_cast<bool>(kept) && !kept.value().fell_back && kept.value().next_from_residual && kept.value().next.token_id >= 0);
        canonical(shadow);
    }
    // greedy: the proposal differs from the target's choice; no draw at all
    {
        SamplingSession session(sampler, SamplingSessionOptions{22});
        SamplingOptions greedy;
        greedy.temperature = 0.0f;
        std::vector<LogitsOutput> target = {logits_of(ramp), logits_of(ramp)};
        std::vector<LogitsOutput> draft = {logits_of(ramp)};
        auto verified = session.verify_speculative(target, draft, std::vector<int32_t>{1}, greedy, false);
        check(static_cast<bool>(verified) && verified.value().fell_back);
        std::mt19937_64 shadow(22);
        const float u = std::uniform_real_distribution<float>(0.0f, 1.0f)(shadow);
        auto sampled = session.sample(logits_of({0, 5, 5, -1}), two);
        check(sampled.value().token_id == (u < 0.5f ? 1 : 2));
        // something accepted: no fall-back even without cache transactions
        auto accepted = session.verify_speculative(target, draft, std::vector<int32_t>{3}, greedy, false);
        check(static_cast<bool>(accepted) && !accepted.value().fell_back && accepted.value().accepted.size() == 1);
    }
}

// ---- worker wire format (host only) -----------------------------------------------------------

static void test_wire_generate_request_defaults_and_fields()
{
    // the request tools/ncnn_moe_protocol.py sends
    const std::string line =
        "{\"op\": \"generate\", \"request_id\": \"r1\", \"session_id\": \"s\", \"prompt_tokens\": [1, 2, 3], "
        "\"max_new_tokens\": 16, \"temperature\": 0.7, \"top_k\": 20, \"top_p\": 0.8, \"min_p\": 0.0, "
        "\"stop_tokens\": [5, 151645], \"enable_speculative\": true, \"speculative_confidence\": 0.5, "
        "\"speculative_max_draft\": 0, \"metrics_enabled\": true, \"metrics_interval_ms\": 1000}";
    const wire::GenerateRequest parsed = wire::parse_generate_request(line);
    check(parsed.request_id == "r1" && parsed.session_id == "s");
    check(parsed.prompt_tokens == std::vector<int32_t>({1, 2, 3}));
    check(parsed.options.max_new_tokens == 16);
    check(parsed.options.sampling.temperature == 0.7f && parsed.options.sampling.top_k == 20);
    check(parsed.options.sampling.top_p == 0.8f && parsed.options.sampling.min_p == 0.0f);
    check(parsed.options.stop_tokens == std::vector<int32_t>({5, 151645}));

    // what the worker assumes for absent fields: greedy, one token, the default ids
    const wire::GenerateRequest bare = wire::parse_generate_request("{\"op\":\"generate\",\"prompt_tokens\":[7]}");
    check(bare.request_id == "generate" && bare.session_id == "main");
    check(bare.options.max_new_tokens == 1 && bare.options.sampling.temperature == 0.0f);
    check(bare.options.sampling.top_k == 0 && bare.options.sampling.top_p == 1.0f && bare.options.sampling.min_p == 0.0f);
    check(bare.options.stop_tokens.empty());

    // top_k is read from an integer literal only; a temperature may be written as an integer
    const wire::GenerateRequest odd = wire::parse_generate_request("{\"prompt_tokens\":[7],\"top_k\":20.0,\"temperature\":1}");
    check(odd.options.sampling.top_k == 0 && odd.options.sampling.temperature == 1.0f);

    const auto message_of = [](const char* text) {
        try
        {
            (void)wire::parse_generate_request(text);
        }
        catch (const std::invalid_argument& error)
        {
            return std::string(error.what());
        }
        return std::string();
    };
    check(message_of("{\"op\":\"generate\"}") == "prompt_tokens must be an integer array");
    check(message_of("{\"prompt_tokens\":[]}") == "prompt_tokens must not be empty");
    check(message_of("{\"prompt_tokens\":[1, \"a\"]}") == "prompt_tokens must be an integer array");
    check(message_of("{\"prompt_tokens\":[1],\"stop_tokens\":[4294967296]}") == "stop_tokens contains an out-of-range token ID");
    check(message_of("{\"prompt_tokens\":[1],\"top_k\":-1}") == "top_k is outside the uint32 range");
    check(message_of("{\"prompt_tokens\":[1],\"max_new_tokens\":4294967296}") == "max_new_tokens is outside the uint32 range");
    check(!message_of("[1, 2]").empty());
}

static void test_wire_events()
{
    StreamToken token;
    token.index = 3;
    token.token_id = 151645;
    token.probability = 0.33816584944725037f;
    token.is_stop_token = true;
    check(wire::token_event("r\"1", "main", token, 0.125) ==
          "{\"event\":\"token\",\"request_id\":\"r\\\"1\",\"session_id\":\"main\",\"index\":3,\"token_id\":151645,"
          "\"probability\":0.3381658494,\"is_stop_token\":true,\"elapsed_seconds\":0.125}");
    token.probability = 1.0f;
    token.token_id = -1;
    token.is_stop_token = false;
    check(wire::token_event("g", "s", token, 2.0).find("\"token_id\":-1,\"probability\":1,\"is_stop_token\":false,\"elapsed_seconds\":2}") != std::string::npos);
    token.probability = 1.0e-7f;
    check(wire::token_event("g", "s", token, 0.0).find("\"probability\":1.000000012e-07,") != std::string::npos);
    token.probability = std::numeric_limits<float>::quiet_NaN();
    check(wire::token_event("g", "s", token, 0.0).find("\"probability\":null,") != std::string::npos);

    check(wire::error_event("r1", "top_p must be in the range (0, 1]", wire::error_code_name(ErrorCode::InvalidArgument)) ==
          "{\"event\":\"error\",\"request_id\":\"r1\",\"code\":\"invalid_argument\",\"message\":\"top_p must be in the range (0, 1]\"}");
    check(wire::error_event("", "line\nbreak") == "{\"event\":\"error\",\"code\":\"invalid_request\",\"message\":\"line\\nbreak\"}");
    check(std::string(wire::error_code_name(ErrorCode::InternalError)) == "internal_error");
    check(std::string(wire::error_code_name(ErrorCode::InvalidModel)) == "invalid_model");

    GenerationResult generation;
    generation.tokens.resize(4);
    generation.stopped_by_stop_token = true;
    SamplingStatistics statistics{4, 4, 180};
    check(wire::done_event("r1", "main", generation, false, 0.5, 9, statistics) ==
          "{\"event\":\"done\",\"request_id\":\"r1\",\"session_id\":\"main\",\"ok\":true,\"metrics_enabled\":false,"
          "\"generated_tokens\":4,\"stopped_by_stop_token\":true,\"stopped_by_callback\":false,\"cancelled\":false,"
          "\"elapsed_seconds\":0.5,\"tokens_per_second\":8,\"sequence_length\":9,"
          "\"sampling\":{\"sampled_tokens\":4,\"sample_calls\":4,\"sample_time_microseconds\":180}}");
}

static void test_wire_request_fields()
{
    const wire::RequestFields fields(
        " { \"a\" : \"x\\ty\\u0041\" , \"n\":-12, \"f\": 2.5e-1, \"t\":true, \"z\":null, \"arr\":[ 1 ,2,\n3 ], "
        "\"nested\":{\"a\":\"inner\",\"arr\":[9]}, \"empty\":[] } ");
    check(fields.string("a").value() == "x\tyA");
    check(fields.integer("n").value() == -12 && fields.number("n").value() == -12.0);
    check(!fields.integer("f") && fields.number("f").value() == 0.25);
    check(fields.boolean("t").value() && !fields.boolean("n"));
    check(!fields.string("z") && !fields.number("z") && !fields.string("missing"));
    check(fields.integer_array("arr").value() == std::vector<int64_t>({1, 2, 3}));
    check(fields.integer_array("empty").value().empty());
    check(!fields.integer_array("a") && !fields.integer_array("nested"));
    check(!fields.string("inner")); // members of nested objects are not members of the request
    bool thrown = false;
    try
    {
        wire::RequestFields broken("{\"a\": [1, 2");
    }
    catch (const std::invalid_argument&)
    {
        thrown = true;
    }
    check(thrown);
}

// ---- batched generation loop ----------------------------------------------------------------

class SyntheticSource : public IDeviceLogitsSource
{
public:
    SyntheticSource(uint32_t vocab, uint32_t sessions) : vocab_(vocab), positions_(sessions, 0) {}

    uint32_t vocabulary_size() const override { return vocab_; }

    Result<bool> prefill(std::span<const uint32_t> session_indices, const DeviceLogitsRows& rows) override
    {
        for (size_t row = 0; row < session_indices.size(); ++row)
        {
            positions_[session_indices[row]] = 0;
            auto written = write_row(rows, row, synthetic_logits(vocab_, session_indices[row], 0, -1));
            if (!written)
                return written;
        }
        ++prefill_calls;
        return true;
    }

    Result<bool> decode(std::span<const DecodeSlot> slots, const DeviceLogitsRows& rows) override
    {
        if (fail_decode_at != 0 && decode_calls + 1 == fail_decode_at)
            return Error{ErrorCode::InternalError, "synthetic decode failure"};
        for (size_t row = 0; row < slots.size(); ++row)
        {
            const uint32_t position = ++positions_[slots[row].session_index];
            auto written = write_row(rows, row, synthetic_logits(vocab_, slots[row].session_index, position, slots[row].token_id));
            if (!written)
                return written;
        }
        ++decode_calls;
        decoded_rows += static_cast<uint32_t>(slots.size());
        return true;
    }

    uint32_t prefill_calls = 0;
    uint32_t decode_calls = 0;
    uint32_t decoded_rows = 0;
    uint32_t fail_decode_at = 0;

private:
    Result<bool> write_row(const DeviceLogitsRows& rows, size_t row, const std::vector<float>& values)
    {
        if (rows.bf16 || rows.vocab != vocab_ || row >= rows.rows || rows.row_stride < vocab_)
            return Error{ErrorCode::InternalError, "synthetic source: unexpected device rows"};
        float* target = static_cast<float*>(rows.data) + row * rows.row_stride;
        if (hipMemcpy(target, values.data(), values.size() * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
            return Error{ErrorCode::InternalError, "synthetic source: hipMemcpy failed"};
        return true;
    }

    uint32_t vocab_;
    std::vector<uint32_t> positions_;
};

// The same model with a draft head: a proposal's row k predicts the token k places behind the anchor from the
// row the target will have there, shifted by 0.75 at every fifth token (exact in fp32), so that proposals are
// mostly but not always accepted; its confidence logit is low at some positions.  The verification rows are the
// target's rows for the anchor and the proposed tokens and the draft rows the tokens were sampled from.
inline std::vector<float> synthetic_draft_logits(uint32_t vocab, uint32_t session, uint32_t position, int32_t fed_token, uint32_t draft_index)
{
    std::vector<float> row = synthetic_logits(vocab, session, position, fed_token);
    for (uint32_t v = (session + draft_index) % 5u; v < vocab; v += 5u)
        row[v] += 0.75f;
    return row;
}

inline float synthetic_confidence_logit(uint32_t session, uint32_t position)
{
    return (session * 7u + position * 3u) % 11u == 0u ? -0.5f : 2.0f;
}

class SyntheticSpeculativeSource : public ISpeculativeLogitsSource
{
public:
    SyntheticSpeculativeSource(uint32_t vocab, uint32_t sessions, uint32_t block_size, bool transactions)
        : vocab_(vocab), block_size_(block_size), transactions_(transactions), positions_(sessions, 0), proposal_rows_(sessions)
    {
    }

    uint32_t vocabulary_size() const override { return vocab_; }
    uint32_t speculative_block_size() const override { return block_size_; }
    bool state_cache_transactions() const override { return transactions_; }

    Result<bool> prefill(std::span<const uint32_t> session_indices, const DeviceLogitsRows& rows) override
    {
        for (size_t row = 0; row < session_indices.size(); ++row)
        {
            positions_[session_indices[row]] = 0;
            auto written = write_row(rows, row, synthetic_logits(vocab_, session_indices[row], 0, -1));
            if (!written)
                return written;
        }
        return true;
    }

    Result<bool> decode(std::span<const DecodeSlot> slots, const DeviceLogitsRows& rows) override
    {
        for (size_t row = 0; row < slots.size(); ++row)
        {
            const uint32_t position = ++positions_[slots[row].session_index];
            auto written = write_row(rows, row, synthetic_logits(vocab_, slots[row].session_index, position, slots[row].token_id));
            if (!written)
                return written;
        }
        ++decode_calls;
        return true;
    }

    Result<bool> draft(std::span<const DecodeSlot> slots, uint32_t draft_index, const DeviceLogitsRows& rows) override
    {
        for (size_t row = 0; row < slots.size(); ++row)
        {
            const uint32_t session = slots[row].session_index;
            if (draft_index == 0)
                proposal_rows_[session].clear();
            if (proposal_rows_[session].size() != draft_index)
                return Error{ErrorCode::InternalError, "synthetic source: draft rows out of order"};
            proposal_rows_[session].push_back(
                synthetic_draft_logits(vocab_, session, positions_[session] + 1 + draft_index, slots[row].token_id, draft_index));
            auto written = write_row(rows, row, proposal_rows_[session].back());
            if (!written)
                return written;
        }
        ++draft_calls;
        return true;
    }

    float confidence_logit(uint32_t session_index, uint32_t draft_index) const override
    {
        return synthetic_confidence_logit(session_index, positions_[session_index] + 1 + draft_index);
    }

    Result<bool> verify(uint32_t session_index, int32_t anchor, std::span<const int32_t> proposed, const DeviceLogitsRows& rows) override
    {
        const uint32_t drafts = static_cast<uint32_t>(proposed.size());
        if (rows.rows != 2 * drafts + 1 || proposal_rows_[session_index].size() < drafts)
            return Error{ErrorCode::InternalError, "synthetic source: unexpected verification rows"};
        for (uint32_t k = 0; k <= drafts; ++k)
        {
            auto written = write_row(rows, k, synthetic_logits(vocab_, session_index, positions_[session_index] + 1 + k, k == 0 ? anchor : proposed[k - 1]));
            if (!written)
                return written;
        }
        for (uint32_t k = 0; k < drafts; ++k)
        {
            auto written = write_row(rows, drafts + 1 + k, proposal_rows_[session_index][k]);
            if (!written)
                return written;
        }
        ++verify_calls;
        return true;
    }

    Result<bool> commit(uint32_t session_index, std::span<const int32_t> emitted) override
    {
        positions_[session_index] += static_cast<uint32_t>(emitted.size());
        committed_tokens += static_cast<uint32_t>(emitted.size());
        rolled_back_steps += emitted.empty() ? 1u : 0u;
        return true;
    }

    uint32_t decode_calls = 0, draft_calls = 0, verify_calls = 0, committed_tokens = 0, rolled_back_steps = 0;

private:
    Result<bool> write_row(const DeviceLogitsRows& rows, size_t row, const std::vector<float>& values)
    {
        if (rows.bf16 || rows.vocab != vocab_ || row >= rows.rows || rows.row_stride < vocab_)
            return Error{ErrorCode::InternalError, "synthetic source: unexpected device rows"};
        float* target = static_cast<float*>(rows.data) + row * rows.row_stride;
        if (hipMemcpy(target, values.data(), values.size() * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
            return Error{ErrorCode::InternalError, "synthetic source: hipMemcpy failed"};
        return true;
    }

    uint32_t vocab_;
    uint32_t block_size_;
    bool transactions_;
    std::vector<uint32_t> positions_;
    std::vector<std::vector<std::vector<float>>> proposal_rows_;
};

struct LoopCase
{
    uint64_t seed;
    GenerationOptions options;
};

static std::vector<LoopCase> loop_cases()
{
    std::vector<LoopCase> cases;
    const auto add = [&](uint64_t seed, uint32_t max_new_tokens, float temperature, uint32_t top_k, float top_p, float min_p,
                         std::vector<int32_t> stop_tokens) {
        LoopCase entry;
        entry.seed = seed;
        entry.options.max_new_tokens = max_new_tokens;
        entry.options.sampling = SamplingOptions{temperature, top_k, top_p, min_p};
        entry.options.stop_tokens = std::move(stop_tokens);
        cases.push_back(std::move(entry));
    };
    std::vector<int32_t> many_stops;
    for (int32_t id = 0; id < 3000; id += 7)
        many_stops.push_back(id); // a seventh of the vocabulary stops this Session early
    add(11, 24, 0.0f, 0, 1.0f, 0.0f, {});           // greedy
    add(12, 24, 0.7f, 20, 0.8f, 0.0f, {});          // the headline options
    add(13, 17, 1.0f, 0, 0.9f, 0.0f, {});           // no Top-K window: the full-order kernels
    add(14, 24, 1.3f, 300, 1.0f, 0.001f, {});       // the wide select kernel
    add(15, 24, 0.9f, 40, 0.95f, 0.0f, many_stops); // stops early
    add(16, 1, 0.8f, 8, 1.0f, 0.0f, {});            // one token only
    add(17, 24, 0.5f, 1, 1.0f, 0.0f, {});           // single survivor: the generator is never advanced
    add(18, 9, 1.0f, 64, 0.5f, 0.05f, {5, 6, 7});
    return cases;
}

constexpr uint32_t kLoopVocab = 3000;

static std::vector<GenerationResult> run_loop(const HipSamplerPtr& sampler, const std::vector<LoopCase>& cases,
                                              std::deque<SamplingSession>& sessions, SyntheticSource& source,
                                              const BatchTokenCallback& on_token = {})
{
    std::vector<SamplingSession*> pointers;
    std::vector<GenerationOptions> options;
    for (size_t i = 0; i < cases.size(); ++i)
    {
        pointers.push_back(&sessions[i]);
        options.push_back(cases[i].options);
    }
    auto generated = BatchGenerationLoop::generate(sampler, pointers, source, options, on_token);
    if (!generated)
        throw std::runtime_error("generation loop failed: " + generated.error().message);
    return std::move(generated).value();
}

// a deque: Sessions hold a mutex and do not move
static void make_sessions(const HipSamplerPtr& sampler, const std::vector<LoopCase>& cases, std::deque<SamplingSession>& sessions)
{
    for (const LoopCase& entry : cases)
        sessions.emplace_back(sampler, SamplingSessionOptions{entry.seed});
}

// The loop against each Session generating alone through SamplingSession::sample on host logits:
// the order of Session::generate (src/engine/session.cpp:978-1020).
static void test_generation_loop_equals_serial(const HipSamplerPtr& sampler)
{
    const std::vector<LoopCase> cases = loop_cases();
    std::deque<SamplingSession> sessions;
    make_sessions(sampler, cases, sessions);
    SyntheticSource source(kLoopVocab, static_cast<uint32_t>(cases.size()));
    const std::vector<GenerationResult> batched = run_loop(sampler, cases, sessions, source);
    check(batched.size() == cases.size());
    check(source.prefill_calls == 1);
    uint32_t expected_decoded_rows = 0;
    uint32_t longest = 0;
    for (size_t i = 0; i < cases.size(); ++i)
    {
        SamplingSession alone(sampler, SamplingSessionOptions{cases[i].seed});
        const GenerationOptions& options = cases[i].options;
        GenerationResult serial;
        int32_t fed = -1;
        for (uint32_t index = 0; index < options.max_new_tokens; ++index)
        {
            auto sampled = alone.sample(logits_of(synthetic_logits(kLoopVocab, static_cast<uint32_t>(i), index, fed)), options.sampling);
            check(static_cast<bool>(sampled));
            StreamToken token;
            token.index = index;
            token.token_id = sampled.value().token_id;
            token.probability = sampled.value().probability;
            token.is_stop_token = std::find(options.stop_tokens.begin(), options.stop_tokens.end(), token.token_id) != options.stop_tokens.end();
            serial.tokens.push_back(token);
            if (token.is_stop_token)
            {
                serial.stopped_by_stop_token = true;
                break;
            }
            fed = token.token_id;
        }
        check(batched[i].tokens.size() == serial.tokens.size());
        check(batched[i].stopped_by_stop_token == serial.stopped_by_stop_token);
        check(!batched[i].stopped_by_callback);
        for (size_t t = 0; t < serial.tokens.size(); ++t)
        {
            check(batched[i].tokens[t].index == serial.tokens[t].index);
            check(batched[i].tokens[t].token_id == serial.tokens[t].token_id);
            check(std::memcmp(&batched[i].tokens[t].probability, &serial.tokens[t].probability, sizeof(float)) == 0);
            check(batched[i].tokens[t].is_stop_token == serial.tokens[t].is_stop_token);
        }
        // both generators stand at the same draw afterwards
        const LogitsOutput probe = logits_of(synthetic_logits(kLoopVocab, 99, 0, -1));
        auto next_batched = sessions[i].sample(probe, SamplingOptions{1.0f, 50, 1.0f, 0.0f});
        auto next_serial = alone.sample(probe, SamplingOptions{1.0f, 50, 1.0f, 0.0f});
        check(next_batched && next_serial && next_batched.value().token_id == next_serial.value().token_id);
        const SamplingStatistics statistics = sessions[i].statistics();
        check(statistics.sampled_tokens == serial.tokens.size() + 1);
        check(statistics.sample_calls == serial.tokens.size() + 1);
        check(statistics.sample_time_microseconds > 0);
        const uint32_t emitted = static_cast<uint32_t>(serial.tokens.size());
        expected_decoded_rows += serial.stopped_by_stop_token ? emitted - 1 : emitted - 1;
        longest = std::max(longest, emitted);
    }
    check(source.decoded_rows == expected_decoded_rows); // a stopped Session is never decoded again
    check(source.decode_calls == longest - 1);
    check(batched[4].stopped_by_stop_token);                // the Session with many stop tokens
    check(batched[4].tokens.size() < 24);
    check(batched[5].tokens.size() == 1);
}

static void test_generation_loop_callback_and_errors(const HipSamplerPtr& sampler)
{
    const std::vector<LoopCase> cases = loop_cases();
    {
        // the callback declines Session 2's fourth token: it stops there, the others run on
        std::deque<SamplingSession> sessions;
    make_sessions(sampler, cases, sessions);
        SyntheticSource source(kLoopVocab, static_cast<uint32_t>(cases.size()));
        uint32_t seen = 0;
        const auto results = run_loop(sampler, cases, sessions, source, [&](uint32_t session_index, const StreamToken& token) {
            ++seen;
            return !(session_index == 2 && token.index == 3);
        });
        check(results[2].stopped_by_callback && results[2].tokens.size() == 4);
        check(!results[1].stopped_by_callback && results[1].tokens.size() == 24);
        uint32_t total = 0;
        for (const GenerationResult& result : results)
            total += static_cast<uint32_t>(result.tokens.size());
        check(seen == total);
    }
    {
        std::deque<SamplingSession> sessions;
    make_sessions(sampler, cases, sessions);
        SyntheticSource source(kLoopVocab, static_cast<uint32_t>(cases.size()));
        std::vector<SamplingSession*> pointers = {&sessions[0], &sessions[1]};
        std::vector<GenerationOptions> options = {cases[0].options};
        // one shared options entry
        auto shared = BatchGenerationLoop::generate(sampler, pointers, source, options);
        check(shared && shared.value().size() == 2 && shared.value()[1].tokens.size() == 24);
        // errors before anything is decoded
        const uint32_t prefills = source.prefill_calls;
        GenerationOptions bad = cases[1].options;
        bad.sampling.top_p = 0.0f;
        auto invalid = BatchGenerationLoop::generate(sampler, pointers, source, std::vector<GenerationOptions>{bad});
        check(!invalid && invalid.error().message == "top_p must be in the range (0, 1]");
        bad = cases[1].options;
        bad.max_new_tokens = 0;
        invalid = BatchGenerationLoop::generate(sampler, pointers, source, std::vector<GenerationOptions>{bad});
        check(!invalid && invalid.error().message == "max_new_tokens must be non-zero");
        std::vector<SamplingSession*> twice = {&sessions[0], &sessions[0]};
        invalid = BatchGenerationLoop::generate(sampler, twice, source, options);
        check(!invalid && invalid.error().code == ErrorCode::InvalidArgument);
        std::vector<SamplingSession*> with_null = {&sessions[0], nullptr};
        invalid = BatchGenerationLoop::generate(sampler, with_null, source, options);
        check(!invalid && invalid.error().code == ErrorCode::InvalidArgument);
        invalid = BatchGenerationLoop::generate(sampler, pointers, source, std::vector<GenerationOptions>(3, cases[0].options));
        check(!invalid && invalid.error().code == ErrorCode::InvalidArgument);
        invalid = BatchGenerationLoop::generate(nullptr, pointers, source, options);
        check(!invalid && invalid.error().code == ErrorCode::InternalError);
        check(source.prefill_calls == prefills);
        // a decode failure ends the run with the model's error
        source.fail_decode_at = source.decode_calls + 3;
        auto failed = BatchGenerationLoop::generate(sampler, pointers, source, options);
        check(!failed && failed.error().message == "synthetic decode failure");
    }
}

constexpr uint32_t kSpeculativeBlock = 4;

static std::vector<LoopCase> speculative_cases()
{
    std::vector<LoopCase> cases;
    const auto add = [&](uint64_t seed, uint32_t max_new_tokens, float temperature, uint32_t top_k, float top_p, float min_p,
                         std::vector<int32_t> stop_tokens, bool enable, float confidence, uint32_t max_draft) {
        LoopCase entry;
        entry.seed = seed;
        entry.options.max_new_tokens = max_new_tokens;
        entry.options.sampling = SamplingOptions{temperature, top_k, top_p, min_p};
        entry.options.stop_tokens = std::move(stop_tokens);
        entry.options.enable_speculative = enable;
        entry.options.speculative_confidence_threshold = confidence;
        entry.options.speculative_max_draft_tokens = max_draft;
        cases.push_back(std::move(entry));
    };
    std::vector<int32_t> many_stops;
    for (int32_t id = 0; id < 3000; id += 11)
        many_stops.push_back(id);
    add(31, 30, 0.0f, 0, 1.0f, 0.0f, {}, true, 0.5f, 0);            // greedy: proposals stand while they are the target's choice
    add(32, 30, 0.7f, 20, 0.8f, 0.0f, {}, true, 0.5f, 0);           // the headline options: ratio tests, residual draws
    add(33, 30, 0.7f, 20, 0.8f, 0.0f, {}, false, 0.5f, 0);          // speculation switched off for this Session
    add(34, 23, 1.0f, 50, 0.95f, 0.0f, {}, true, 0.0f, 2);          // no confidence cut, two drafts a step at most
    add(35, 30, 0.9f, 40, 0.9f, 0.0f, many_stops, true, 0.3f, 0);   // stops on a stop token, possibly an accepted one
    add(36, 2, 0.8f, 8, 1.0f, 0.0f, {}, true, 0.5f, 0);             // two tokens: the second by a plain step (one token left)
    add(37, 30, 0.5f, 1, 1.0f, 0.0f, {}, true, 0.5f, 0);            // single survivor: ratio 1, no residual, few draws
    add(38, 17, 1.2f, 64, 0.6f, 0.02f, {}, true, 1.0f, 0);          // threshold 1: every finite confidence falls short, nothing is ever verified
    return cases;
}

static std::vector<GenerationResult> run_speculative(const HipSamplerPtr& sampler, const std::vector<LoopCase>& cases, bool transactions,
                                                     SyntheticSpeculativeSource** source_out = nullptr, const TokenTextDecoder& decode_text = {})
{
    static std::deque<SyntheticSpeculativeSource> sources; // (kept for the caller to read the counters)
    std::deque<SamplingSession> sessions;
    make_sessions(sampler, cases, sessions);
    sources.emplace_back(kLoopVocab, static_cast<uint32_t>(cases.size()), kSpeculativeBlock, transactions);
    if (source_out != nullptr)
        *source_out = &sources.back();
    std::vector<SamplingSession*> pointers;
    std::vector<GenerationOptions> options;
    for (size_t i = 0; i < cases.size(); ++i)
    {
        pointers.push_back(&sessions[i]);
        options.push_back(cases[i].options);
    }
    auto generated = BatchGenerationLoop::generate(sampler, pointers, sources.back(), options, {}, decode_text);
    if (!generated)
        throw std::runtime_error("speculative generation failed: " + generated.error().message);
    if (source_out != nullptr)
    {
        const SamplingStatistics statistics = sessions[1].statistics();
        check(statistics.speculative_steps > 0 && statistics.speculative_verify_time_microseconds > 0);
    }
    return std::move(generated).value();
}

// The speculative loop: structure (every Session gets its tokens, budgets and stop tokens hold, a Session with
// speculation off equals the plain loop), the text decoder, option errors.  The tokens themselves are checked by
// tests/test_gpu_generation_loop.py, which replays every Session with the CPU oracle.
static void test_speculative_generation_loop(const HipSamplerPtr& sampler)
{
    const std::vector<LoopCase> cases = speculative_cases();
    for (const bool transactions : {true, false})
    {
        SyntheticSpeculativeSource* source = nullptr;
        uint32_t decoded = 0;
        const std::vector<GenerationResult> results = run_speculative(sampler, cases, transactions, &source, [&](int32_t token_id) {
            ++decoded;
            return "<" + std::to_string(token_id) + ">";
        });
        check(results.size() == cases.size());
        size_t tokens = 0;
        for (size_t i = 0; i < results.size(); ++i)
        {
            check(!results[i].tokens.empty() && results[i].tokens.size() <= cases[i].options.max_new_tokens);
            check(results[i].stopped_by_stop_token || results[i].tokens.size() == cases[i].options.max_new_tokens);
            for (size_t k = 0; k < results[i].tokens.size(); ++k)
            {
                const StreamToken& token = results[i].tokens[k];
                check(token.index == k && token.text == "<" + std::to_string(token.token_id) + ">");
                const bool stop = std::find(cases[i].options.stop_tokens.begin(), cases[i].options.stop_tokens.end(), token.token_id) != cases[i].options.stop_tokens.end();
                check(token.is_stop_token == stop && (!stop || k + 1 == results[i].tokens.size()));
            }
            tokens += results[i].tokens.size();
        }
        check(decoded == tokens);
        check(source->verify_calls > 0 && source->draft_calls > 0 && source->committed_tokens > 0);
        check(transactions || source->rolled_back_steps > 0);
        // the Session with speculation off generates what the plain loop generates
        std::deque<SamplingSession> plain_sessions;
        plain_sessions.emplace_back(sampler, SamplingSessionOptions{cases[2].seed});
        SyntheticSource plain(kLoopVocab, 3);
        // (Session index 2 of the synthetic model: two idle Sessions in front keep its index)
        std::deque<SamplingSession> idle;
        idle.emplace_back(sampler, SamplingSessionOptions{1});
        idle.emplace_back(sampler, SamplingSessionOptions{2});
        std::vector<SamplingSession*> pointers = {&idle[0], &idle[1], &plain_sessions[0]};
        GenerationOptions one_token;
        one_token.sampling.temperature = 0.0f;
        std::vector<GenerationOptions> options = {one_token, one_token, cases[2].options};
        auto alone = BatchGenerationLoop::generate(sampler, pointers, plain, options);
        check(static_cast<bool>(alone) && alone.value()[2].tokens.size() == results[2].tokens.size());
        for (size_t k = 0; k < results[2].tokens.size(); ++k)
        {
            check(alone.value()[2].tokens[k].token_id == results[2].tokens[k].token_id);
            check(std::bit_cast<uint32_t>(alone.value()[2].tokens[k].probability) == std::bit_cast<uint32_t>(results[2].tokens[k].probability));
        }
    }
    // the threshold is checked before anything runs (src/engine/session.cpp:462-470)
    std::deque<SamplingSession> sessions;
    sessions.emplace_back(sampler, SamplingSessionOptions{1});
    std::vector<SamplingSession*> pointers = {&sessions[0]};
    SyntheticSpeculativeSource source(kLoopVocab, 1, kSpeculativeBlock, true);
    GenerationOptions bad;
    bad.speculative_confidence_threshold = 1.5f;
    auto rejected = BatchGenerationLoop::generate(sampler, pointers, source, std::vector<GenerationOptions>{bad});
    check(!rejected && rejected.error().code == ErrorCode::InvalidArgument &&
          rejected.error().message == "speculative_confidence_threshold must be in the range [0, 1]");
    check(source.draft_calls == 0);
}

static void print_trace_lines(const std::vector<LoopCase>& cases, const std::vector<GenerationResult>& results)
{
    for (size_t i = 0; i < results.size(); ++i)
    {
        const GenerationOptions& options = cases[i].options;
        std::printf("session %zu seed %llu max_new_tokens %u temperature_bits %u top_k %u top_p_bits %u min_p_bits %u "
                    "speculative %d confidence_bits %u max_draft %u stops",
                    i, static_cast<unsigned long long>(cases[i].seed), options.max_new_tokens,
                    std::bit_cast<uint32_t>(options.sampling.temperature), options.sampling.top_k,
                    std::bit_cast<uint32_t>(options.sampling.top_p), std::bit_cast<uint32_t>(options.sampling.min_p),
                    options.enable_speculative ? 1 : 0, std::bit_cast<uint32_t>(options.speculative_confidence_threshold),
                    options.speculative_max_draft_tokens);
        for (int32_t id : options.stop_tokens)
            std::printf(" %d", id);
        std::printf("\n");
        for (const StreamToken& token : results[i].tokens)
            std::printf("token %zu %u %d %u %d\n", i, token.index, token.token_id, std::bit_cast<uint32_t>(token.probability),
                        token.is_stop_token ? 1 : 0);
        std::printf("result %zu tokens %zu stopped_by_stop_token %d stopped_by_callback %d\n", i, results[i].tokens.size(),
                    results[i].stopped_by_stop_token ? 1 : 0, results[i].stopped_by_callback ? 1 : 0);
    }
}

// --speculative-trace 0|1: the speculative loop without / with state cache transactions, printed like --generation-trace
static int print_speculative_trace(const HipSamplerPtr& sampler, bool transactions)
{
    const std::vector<LoopCase> cases = speculative_cases();
    const std::vector<GenerationResult> results = run_speculative(sampler, cases, transactions);
    print_trace_lines(cases, results);
    std::printf("vocab %u\nblock %u\ntransactions %d\n", kLoopVocab, kSpeculativeBlock, transactions ? 1 : 0);
    return 0;
}

// Prints "session index token_id probability_bits is_stop" per emitted token and a summary line per
// Session; tests/test_gpu_generation_loop.py recomputes the run with the CPU sampler.
static int print_generation_trace(const HipSamplerPtr& sampler)
{
    const std::vector<LoopCase> cases = loop_cases();
    std::deque<SamplingSession> sessions;
    make_sessions(sampler, cases, sessions);
    SyntheticSource source(kLoopVocab, static_cast<uint32_t>(cases.size()));
    const std::vector<GenerationResult> results = run_loop(sampler, cases, sessions, source);
    for (size_t i = 0; i < results.size(); ++i)
    {
        const GenerationOptions& options = cases[i].options;
        std::printf("session %zu seed %llu max_new_tokens %u temperature_bits %u top_k %u top_p_bits %u min_p_bits %u stops",
                    i, static_cast<unsigned long long>(cases[i].seed), options.max_new_tokens,
                    std::bit_cast<uint32_t>(options.sampling.temperature), options.sampling.top_k,
                    std::bit_cast<uint32_t>(options.sampling.top_p), std::bit_cast<uint32_t>(options.sampling.min_p));
        for (int32_t id : options.stop_tokens)
            std::printf(" %d", id);
        std::printf("\n");
        for (const StreamToken& token : results[i].tokens)
            std::printf("token %zu %u %d %u %d\n", i, token.index, token.token_id, std::bit_cast<uint32_t>(token.probability),
                        token.is_stop_token ? 1 : 0);
        std::printf("result %zu tokens %zu stopped_by_stop_token %d stopped_by_callback %d\n", i, results[i].tokens.size(),
                    results[i].stopped_by_stop_token ? 1 : 0, results[i].stopped_by_callback ? 1 : 0);
    }
    std::printf("vocab %u\n", kLoopVocab);
    return 0;
}

// A model whose decode step costs nothing: the rows written at prefill stay in the buffer, as if a
// decode step on the GPU had just produced them.  What remains is the loop itself: one device call per
// token index over device-resident logits, and the host bookkeeping around it.
class ResidentSource : public IDeviceLogitsSource
{
public:
    explicit ResidentSource(uint32_t vocab) : vocab_(vocab) {}
    uint32_t vocabulary_size() const override { return vocab_; }

    Result<bool> prefill(std::span<const uint32_t> session_indices, const DeviceLogitsRows& rows) override
    {
        const auto started = std::chrono::steady_clock::now();
        for (size_t row = 0; row < session_indices.size(); ++row)
        {
            const std::vector<float> values = synthetic_logits(vocab_, session_indices[row], 0, -1);
            float* target = static_cast<float*>(rows.data) + row * rows.row_stride;
            if (hipMemcpy(target, values.data(), values.size() * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
                return Error{ErrorCode::InternalError, "resident source: hipMemcpy failed"};
        }
        prefill_seconds += std::chrono::duration<double>(std::chrono::steady_clock::now() - started).count();
        return true;
    }

    Result<bool> decode(std::span<const DecodeSlot>, const DeviceLogitsRows&) override { return true; }

    double prefill_seconds = 0.0;

private:
    uint32_t vocab_;
};

// --generation-bench SESSIONS VOCAB STEPS: times BatchGenerationLoop::generate and prints one line.
static int generation_bench(uint32_t session_count, uint32_t vocab, uint32_t steps)
{
    HipSamplerPtr sampler = HipSampler::create(0, session_count, vocab);
    if (!sampler)
    {
        std::fprintf(stderr, "HipSampler::create failed: no usable GPU\n");
        return 2;
    }
    GenerationOptions options;
    options.sampling = SamplingOptions{0.7f, 20, 0.8f, 0.0f};
    double seconds = 0.0;
    double prefill_seconds = 0.0;
    uint64_t tokens = 0;
    uint64_t sample_time_microseconds = 0;
    int32_t first_token = -1;
    uint32_t first_probability_bits = 0;
    for (int pass = 0; pass < 2; ++pass) // the first pass warms up
    {
        std::deque<SamplingSession> sessions;
        std::vector<SamplingSession*> pointers;
        for (uint32_t i = 0; i < session_count; ++i)
            pointers.push_back(&sessions.emplace_back(sampler, SamplingSessionOptions{1000 + i}));
        options.max_new_tokens = pass == 0 ? 20 : steps;
        ResidentSource source(vocab);
        const auto started = std::chrono::steady_clock::now();
        auto generated = BatchGenerationLoop::generate(sampler, pointers, source, std::vector<GenerationOptions>{options});
        seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - started).count();
        if (!generated)
        {
            std::fprintf(stderr, "generation failed: %s\n", generated.error().message.c_str());
            return 1;
        }
        prefill_seconds = source.prefill_seconds;
        tokens = 0;
        for (const GenerationResult& result : generated.value())
            tokens += result.tokens.size();
        sample_time_microseconds = sessions.front().statistics().sample_time_microseconds;
        first_token = generated.value()[0].tokens[0].token_id;
        first_probability_bits = std::bit_cast<uint32_t>(generated.value()[0].tokens[0].probability);
    }
    std::printf("generation_bench sessions %u vocab %u steps %u tokens %llu seconds %.6f prefill_seconds %.6f "
                "sample_time_microseconds %llu first_token %d first_probability_bits %u\n",
                session_count, vocab, steps, static_cast<unsigned long long>(tokens), seconds, prefill_seconds,
                static_cast<unsigned long long>(sample_time_microseconds), first_token, first_probability_bits);
    return 0;
}

// --scheduler-bench ROWS VOCAB SAMPLERS STEPS: batches of ROWS device-resident rows through BatchSampleScheduler
// over SAMPLERS samplers (a worker each), as many batches in flight as there are samplers, every batch one
// synchronous device call of the worker that runs it.  Prints one line; the tokens of the first batch are there
// for a check against the CPU oracle (row i of sampler 0: synthetic_logits(VOCAB, i, 0, -1), seed 5000 + i).
static int scheduler_bench(uint32_t rows, uint32_t vocab, uint32_t sampler_count, uint32_t steps)
{
    std::vector<HipSamplerPtr> samplers;
    std::deque<SamplingSession> sessions;
    for (uint32_t lane = 0; lane < sampler_count; ++lane)
    {
        samplers.push_back(HipSampler::create(0, rows, vocab));
        if (!samplers.back())
        {
            std::fprintf(stderr, "HipSampler::create failed: no usable GPU\n");
            return 2;
        }
        std::vector<std::vector<float>> values;
        std::vector<std::span<const float>> spans;
        for (uint32_t i = 0; i < rows; ++i)
            values.push_back(synthetic_logits(vocab, i, lane, -1));
        for (const std::vector<float>& row : values)
            spans.emplace_back(row);
        auto uploaded = samplers.back()->upload_resident(spans);
        if (!uploaded)
        {
            std::fprintf(stderr, "upload_resident failed: %s\n", uploaded.error().message.c_str());
            return 1;
        }
        for (uint32_t i = 0; i < rows; ++i)
            sessions.emplace_back(samplers.back(), SamplingSessionOptions{5000 + lane * rows + i, LogitsOutputMode::SampledToken});
    }
    SamplingOptions options{0.7f, 20, 0.8f, 0.0f};
    SampleSchedulerOptions scheduler_options;
    scheduler_options.worker_count = sampler_count;
    scheduler_options.cross_call_window_microseconds = 0;
    BatchSampleScheduler scheduler(samplers, scheduler_options);
    const auto batch_of = [&](uint32_t lane) {
        std::vector<SampleBatchRequest> requests;
        for (uint32_t i = 0; i < rows; ++i)
        {
            SampleBatchRequest request{&sessions[lane * rows + i], nullptr, options, {}};
            request.resident_sampler = lane;
            requests.push_back(std::move(request));
        }
        return requests;
    };
    std::vector<std::future<std::vector<Result<BatchSampledToken>>>> in_flight(sampler_count);
    std::vector<Result<BatchSampledToken>> first_batch;
    double seconds = 0.0;
    for (int pass = 0; pass < 2; ++pass) // the first pass warms up (and keeps the first batch's tokens)
    {
        const uint32_t count = pass == 0 ? 4 * sampler_count : steps;
        const auto started = std::chrono::steady_clock::now();
        for (uint32_t step = 0; step < count; ++step)
        {
            const uint32_t lane = step % sampler_count;
            if (in_flight[lane].valid())
            {
                while (in_flight[lane].wait_for(std::chrono::seconds(0)) != std::future_status::ready)
                {
                } // (the serving thread keeps awake as well)
                auto done = in_flight[lane].get();
                if (first_batch.empty())
                    first_batch = std::move(done);
            }
            in_flight[lane] = scheduler.submit_sample(batch_of(lane));
        }
        for (auto& future : in_flight)
        {
            if (future.valid())
            {
                auto done = future.get();
                for (const auto& row : done)
                {
                    if (!row)
                    {
                        std::fprintf(stderr, "a row failed: %s\n", row.error().message.c_str());
                        return 1;
                    }
                }
            }
        }
        seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - started).count();
    }
    const SampleSchedulerStatistics statistics = scheduler.statistics();
    std::printf("scheduler_bench rows %u vocab %u samplers %u steps %u seconds %.6f device_calls %llu overlapped_device_calls %llu first_batch",
                rows, vocab, sampler_count, steps, seconds, static_cast<unsigned long long>(statistics.device_calls),
                static_cast<unsigned long long>(statistics.overlapped_device_calls));
    for (const auto& row : first_batch)
        std::printf(" %d:%u", row ? row.value().token.token_id : -1, row ? std::bit_cast<uint32_t>(row.value().token.probability) : 0u);
    std::printf("\n");
    return 0;
}

int main(int argc, char** argv)
{
    if (argc == 6 && std::strcmp(argv[1], "--scheduler-bench") == 0)
        return scheduler_bench(static_cast<uint32_t>(std::atoi(argv[2])), static_cast<uint32_t>(std::atoi(argv[3])),
                               static_cast<uint32_t>(std::atoi(argv[4])), static_cast<uint32_t>(std::atoi(argv[5])));
    if (argc == 5 && std::strcmp(argv[1], "--generation-bench") == 0)
        return generation_bench(static_cast<uint32_t>(std::atoi(argv[2])), static_cast<uint32_t>(std::atoi(argv[3])),
                                static_cast<uint32_t>(std::atoi(argv[4])));
    const bool host_only = argc > 1 && std::strcmp(argv[1], "--host") == 0;
    const bool trace_only = argc > 1 && std::strcmp(argv[1], "--generation-trace") == 0;
    const bool speculative_trace = argc > 2 && std::strcmp(argv[1], "--speculative-trace") == 0;
    try
    {
        test_option_validation_messages();
        test_defaults_match_the_runtime();
        test_peek_uniform_does_not_advance();
        test_missing_sampler_fails_loudly();
        test_scheduler_and_modes_without_a_sampler();
        test_wire_generate_request_defaults_and_fields();
        test_wire_events();
        test_wire_request_fields();
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
        if (trace_only)
            return print_generation_trace(sampler);
        if (speculative_trace)
            return print_speculative_trace(sampler, std::atoi(argv[2]) != 0);
        test_sampling_like_the_runtime_test(sampler);
        test_rng_bookkeeping(sampler);
        test_distribution_known_answers(sampler);
        test_batch_equals_serial(sampler);
        test_threads_share_a_sampler(sampler);
        test_batch_rejects_bad_requests(sampler);
        test_speculative_verification(sampler);
        test_speculative_fallback(sampler);
        test_scheduler_collects_across_calls(sampler);
        test_scheduler_keeps_a_sessions_order(sampler);
        test_sampled_token_mode(sampler);
        test_resident_requests_through_the_scheduler(sampler);
        test_scheduler_over_several_samplers(sampler);
        test_generation_loop_equals_serial(sampler);
        test_generation_loop_callback_and_errors(sampler);
        test_speculative_generation_loop(sampler);
    }
    catch (const std::exception& error)
    {
        std::fprintf(stderr, "FAILED: %s\n", error.what());
        return 1;
    }
    std::printf("all session sampler tests passed\n");
    return 0;
}
