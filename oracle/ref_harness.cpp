/*
 * Driver around the REFERENCE library, built only where the reference checkout is present.
 * TEST INFRASTRUCTURE ONLY.
 *
 * The reference's sources are compiled from where they lie (see oracle/Makefile); nothing from
 * them is copied here.  This translation unit textually includes the reference's
 * src/engine/session.cpp so that its file-static sampling_distribution() (session.cpp:76-136) and
 * validate_sampling_options() (session.cpp:65-74) can be called directly, and it reaches
 * Session::sample (session.cpp:452-456) through a real Session created by the reference Runtime on
 * the reference's own 4-token fixture model (tests/fixture_model_adapter.cpp, the package layout of
 * tests/test_runtime.cpp:166-271).  The sampler never checks logits.size() against the model
 * vocabulary (session.cpp:393-400), so rows of any length can be sampled through that Session.
 */
#include "engine/session.cpp"

#include "fixture_model_adapter.h"
#include "kernels/cpu_ops.h"
#include "ncnn/moe/expert_dispatcher.h"
#include "ncnn/moe/runtime.h"

#include <cstdio>
#include <cstring>
#include <filesystem>
#include <fstream>
#include <memory>
#include <string>
#include <thread>
#include <unistd.h>

namespace {

using namespace ncnn::moe;

class HarnessRuntime final : public Runtime
{
public:
    HarnessRuntime()
    {
        register_adapter(std::make_shared<FixtureModelAdapter>());
    }
};

/* The fixture package: a manifest for model_type "test_moe" and 40 fp32 weights. */
std::filesystem::path write_fixture_package()
{
    static int serial = 0;
    const std::filesystem::path directory = std::filesystem::temp_directory_path() /
        ("sampler_ref_harness_" + std::to_string(::getpid()) + "_" + std::to_string(serial++));
    std::filesystem::create_directories(directory);
    {
        std::ofstream manifest(directory / "config.json", std::ios::binary);
        manifest << "{\"model_type\": \"test_moe\", \"vocabulary_size\": 4, \"hidden_size\": 2, "
                    "\"intermediate_size\": 2, \"layer_count\": 1, \"expert_count\": 2, "
                    "\"experts_per_token\": 1, \"expert_activation\": \"relu\", "
                    "\"expert_layout\": \"up_down\", \"normalize_topk_weights\": true, "
                    "\"use_expert_bias\": false, \"norm_epsilon\": 0.00001, "
                    "\"weights_file\": \"model.test.bin\"}\n";
    }
    {
        const float weights[40] = {
            1, 0, 0, 1, 1, 1, -1, 0, 1, 1, 1, -1, -1, 1, 1, 0, 0, 1, 1, 0,
            0, 1, 1, 0, 0, 1, 2, 0, 0, 2, 1, 1, 1, 0, 0, 1, 1, 1, -1, 0};
        std::ofstream file(directory / "model.test.bin", std::ios::binary);
        file.write(reinterpret_cast<const char*>(weights), sizeof(weights));
    }
    return directory;
}

struct RefSession
{
    std::unique_ptr<HarnessRuntime> runtime;
    ModelPtr model;
    SessionPtr session;
    std::filesystem::path package;

    ~RefSession()
    {
        session.reset();
        model.reset();
        runtime.reset();
        std::error_code ignored;
        std::filesystem::remove_all(package, ignored);
    }
};

void copy_message(const std::string& message, char* out, size_t cap)
{
    if (out == nullptr || cap == 0)
        return;
    std::snprintf(out, cap, "%s", message.c_str());
}

} // namespace

extern "C" {

void* ref_session_create(uint64_t seed, char* message, size_t message_cap)
{
    auto holder = std::make_unique<RefSession>();
    holder->package = write_fixture_package();
    holder->runtime = std::make_unique<HarnessRuntime>();
    auto model = holder->runtime->load_model(holder->package);
    if (!model)
    {
        copy_message(model.error().message, message, message_cap);
        return nullptr;
    }
    holder->model = model.value();
    SessionOptions options;
    options.sampling_seed = seed;
    auto session = holder->runtime->create_session(holder->model, options);
    if (!session)
    {
        copy_message(session.error().message, message, message_cap);
        return nullptr;
    }
    holder->session = session.value();
    return holder.release();
}

void ref_session_destroy(void* handle)
{
    delete static_cast<RefSession*>(handle);
}

/* Returns 0 on success, 1 + ErrorCode on a reference error (message filled). */
int ref_session_sample(
    void* handle, const float* logits, size_t vocab,
    float temperature, uint32_t top_k, float top_p, float min_p,
    int32_t* token_id, float* probability, char* message, size_t message_cap)
{
    RefSession* holder = static_cast<RefSession*>(handle);
    LogitsOutput output;
    output.values.assign(logits, logits + vocab);
    SamplingOptions options;
    options.temperature = temperature;
    options.top_k = top_k;
    options.top_p = top_p;
    options.min_p = min_p;
    auto sampled = holder->session->sample(output, options);
    if (!sampled)
    {
        copy_message(sampled.error().message, message, message_cap);
        *token_id = -1;
        *probability = 0.0f;
        return 1 + static_cast<int>(sampled.error().code);
    }
    *token_id = sampled.value().token_id;
    *probability = sampled.value().probability;
    return 0;
}

/* session.cpp:65-74 followed by session.cpp:76-136, exactly as sample_unlocked orders them. */
int ref_sampling_distribution(
    const float* logits, size_t vocab,
    float temperature, uint32_t top_k, float top_p, float min_p,
    int32_t* ids, float* probabilities, size_t cap, size_t* count,
    char* message, size_t message_cap)
{
    *count = 0;
    SamplingOptions options;
    options.temperature = temperature;
    options.top_k = top_k;
    options.top_p = top_p;
    options.min_p = min_p;
    auto valid = validate_sampling_options(options);
    if (!valid)
    {
        copy_message(valid.error().message, message, message_cap);
        return 1 + static_cast<int>(valid.error().code);
    }
    auto candidates = sampling_distribution(std::span<const float>(logits, vocab), options);
    if (!candidates)
    {
        copy_message(candidates.error().message, message, message_cap);
        return 1 + static_cast<int>(candidates.error().code);
    }
    *count = candidates.value().size();
    const size_t n = std::min(cap, candidates.value().size());
    for (size_t i = 0; i < n; ++i)
    {
        ids[i] = candidates.value()[i].token_id;
        probabilities[i] = candidates.value()[i].probability;
    }
    return 0;
}

/*
 * The serial caller loop of examples/internal/run_model.cpp:776-809: one Session per row, one
 * Session::sample per row, the stop test of session.cpp:60-63.  Used as the timed CPU baseline.
 * sessions[] holds `rows` handles from ref_session_create.  threads > 1 partitions the rows over
 * std::thread, the reference's own concurrency model (one Session per worker thread).
 */
int ref_sample_rows(
    void* const* sessions, const float* logits, uint32_t rows, uint32_t vocab, uint64_t row_stride,
    const float* temperature, const uint32_t* top_k, const float* top_p, const float* min_p,
    const int32_t* stop_ids, const uint32_t* stop_begin, const uint32_t* stop_count,
    int32_t* token_ids, float* probabilities, uint8_t* is_stop, int32_t* status, int threads)
{
    auto run_rows = [&](uint32_t begin, uint32_t end) {
        LogitsOutput output;
        for (uint32_t row = begin; row < end; ++row)
        {
            RefSession* holder = static_cast<RefSession*>(sessions[row]);
            const float* source = logits + static_cast<size_t>(row) * row_stride;
            output.values.assign(source, source + vocab);
            SamplingOptions options;
            options.temperature = temperature[row];
            options.top_k = top_k[row];
            options.top_p = top_p[row];
            options.min_p = min_p[row];
            auto sampled = holder->session->sample(output, options);
            if (!sampled)
            {
                token_ids[row] = -1;
                probabilities[row] = 0.0f;
                is_stop[row] = 0;
                status[row] = 1 + static_cast<int>(sampled.error().code);
                continue;
            }
            token_ids[row] = sampled.value().token_id;
            probabilities[row] = sampled.value().probability;
            status[row] = 0;
            std::vector<int32_t> stops;
            if (stop_ids != nullptr)
                stops.assign(stop_ids + stop_begin[row], stop_ids + stop_begin[row] + stop_count[row]);
            is_stop[row] = contains_token(stops, token_ids[row]) ? 1 : 0;
        }
    };
    if (threads <= 1 || rows <= 1)
    {
        run_rows(0, rows);
        return 0;
    }
    const uint32_t workers = std::min<uint32_t>(static_cast<uint32_t>(threads), rows);
    std::vector<std::thread> pool;
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

/* candidate_probability, file-static at src/engine/session.cpp:138-148. */
float ref_candidate_probability(const int32_t* ids, const float* probabilities, size_t count, int32_t token_id)
{
    std::vector<SamplingCandidate> candidates(count);
    for (size_t i = 0; i < count; ++i)
    {
        candidates[i].token_id = ids[i];
        candidates[i].probability = probabilities[i];
    }
    return candidate_probability(candidates, token_id);
}

/*
 * sample_residual_distribution, file-static at src/engine/session.cpp:150-202, driven by a
 * std::mt19937_64 seeded with `seed` and advanced by `discard` draws first.  *draws receives the
 * number of 64-bit outputs the call consumed.
 */
int ref_sample_residual_distribution(
    const int32_t* target_ids, const float* target_probabilities, size_t target_count,
    const int32_t* draft_ids, const float* draft_probabilities, size_t draft_count,
    size_t vocab, uint64_t seed, uint64_t discard,
    int32_t* token_id, float* probability, uint64_t* draws,
    char* message, size_t message_cap)
{
    std::vector<SamplingCandidate> target(target_count), draft(draft_count);
    for (size_t i = 0; i < target_count; ++i)
    {
        target[i].token_id = target_ids[i];
        target[i].probability = target_probabilities[i];
    }
    for (size_t i = 0; i < draft_count; ++i)
    {
        draft[i].token_id = draft_ids[i];
        draft[i].probability = draft_probabilities[i];
    }
    std::mt19937_64 generator(seed);
    generator.discard(discard);
    std::mt19937_64 shadow = generator;
    *token_id = -1;
    *probability = 0.0f;
    auto sampled = sample_residual_distribution(target, draft, vocab, generator);
    uint64_t consumed = 0;
    while (!(shadow == generator) && consumed < 16)
    {
        shadow.discard(1);
        ++consumed;
    }
    *draws = consumed;
    if (!sampled)
    {
        copy_message(sampled.error().message, message, message_cap);
        return 1 + static_cast<int>(sampled.error().code);
    }
    *token_id = sampled.value().token_id;
    *probability = sampled.value().probability;
    return 0;
}

/*
 * ExpertDispatcher::dispatch (src/graph/expert_dispatcher.cpp:76-157) or, with use_dispatch_into != 0,
 * dispatch_into (:159-301), through the reference's public class.  The plan comes back flat: routes
 * grouped by expert in the order of plan.batches, expert_offsets[e] .. expert_offsets[e + 1] for every
 * expert id (expert_count + 1 entries).  Returns 0, or 1 + ErrorCode with the message.
 */
int ref_router_dispatch(
    const float* router_logits, uint32_t token_count,
    uint32_t expert_count, uint32_t top_k, uint32_t score_function, uint32_t normalization, uint32_t flags,
    float routed_scaling_factor, const float* selection_bias, const uint32_t* explicit_expert_ids,
    int use_dispatch_into, uint32_t* expert_offsets, uint32_t* route_tokens, uint32_t* route_ranks, float* route_weights,
    uint64_t* assignment_count, char* message, size_t message_cap)
{
    ExpertDispatchOptions options;
    options.expert_count = expert_count;
    options.top_k = top_k;
    options.score_function = static_cast<RouterScoreFunction>(score_function);
    options.normalization = static_cast<RouterNormalization>(normalization);
    options.routed_scaling_factor = routed_scaling_factor;
    options.flags = flags;
    if (selection_bias != nullptr)
        options.selection_bias = std::span<const float>(selection_bias, expert_count);
    if (explicit_expert_ids != nullptr)
        options.explicit_expert_ids = std::span<const uint32_t>(explicit_expert_ids, static_cast<size_t>(token_count) * top_k);
    const std::span<const float> logits(router_logits, static_cast<size_t>(token_count) * expert_count);
    ExpertDispatcher dispatcher;
    ExpertDispatchPlan plan;
    if (use_dispatch_into)
    {
        auto status = dispatcher.dispatch_into(logits, token_count, options, plan);
        if (!status)
        {
            copy_message(status.error().message, message, message_cap);
            return 1 + static_cast<int>(status.error().code);
        }
    }
    else
    {
        auto dispatched = dispatcher.dispatch(logits, token_count, options);
        if (!dispatched)
        {
            copy_message(dispatched.error().message, message, message_cap);
            return 1 + static_cast<int>(dispatched.error().code);
        }
        plan = std::move(dispatched).value();
    }
    *assignment_count = plan.assignment_count;
    uint32_t written = 0;
    size_t batch = 0;
    for (uint32_t expert_id = 0; expert_id < expert_count; ++expert_id)
    {
        expert_offsets[expert_id] = written;
        if (batch < plan.batches.size() && plan.batches[batch].expert_id == expert_id)
        {
            for (const ExpertRoute& route : plan.batches[batch].routes)
            {
                route_tokens[written] = route.token_index;
                route_ranks[written] = route.rank;
                route_weights[written] = route.weight;
                ++written;
            }
            ++batch;
        }
    }
    expert_offsets[expert_count] = written;
    return batch == plan.batches.size() ? 0 : -1; /* -1: batches were not in ascending expert order */
}

float ref_bfloat16_to_float(uint16_t value)
{
    return bfloat16_to_float(value);
}

uint16_t ref_float_to_bfloat16(float value)
{
    return float_to_bfloat16(value);
}

} // extern "C"
