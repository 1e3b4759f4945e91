// A worker that speaks the sampling slice of the runtime's JSON-lines protocol (one request object per
// line on stdin, one event object per line on stdout) over the HIP sampler and the synthetic model of
// these tests.  It exists so that the wire format can be exercised end to end: the requests are the ones
// tools/ncnn_moe_protocol.py sends, the events carry the fields its clients read.
//
//   {"op":"create_session","session_id":"a","seed":7}   -> {"event":"session_created",...}
//   {"op":"generate","session_id":"a","prompt_tokens":[1,2],"max_new_tokens":8,"temperature":0.7,...}
//                                                       -> {"event":"token",...} ... {"event":"done",...}
//   {"op":"stats","session_id":"a"}                     -> {"event":"stats",...}
//   {"op":"shutdown"}                                   -> {"event":"shutdown"}
//
// Sessions are numbered in creation order; the logits after position p of Session n, when token t was
// fed last, are synthetic_logits(vocab, n, p, t).
#include "hip_session_sampler.h"
#include "synthetic_model.h"
#include "worker_wire.h"

#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstdio>
#include <iostream>
#include <map>
#include <memory>
#include <string>

using namespace ncnn::moe;

namespace {

constexpr uint32_t kVocab = 4096;

struct WorkerSession
{
    uint32_t number = 0;
    std::unique_ptr<SamplingSession> sampling;
    uint64_t sequence_length = 0;
};

// One Session's prompt and decode steps as device rows.
class WorkerSource : public IDeviceLogitsSource
{
public:
    WorkerSource(WorkerSession& session, const std::vector<int32_t>& prompt) : session_(session), prompt_(prompt) {}
    uint32_t vocabulary_size() const override { return kVocab; }

    Result<bool> prefill(std::span<const uint32_t>, const DeviceLogitsRows& rows) override
    {
        session_.sequence_length += prompt_.size();
        return write(rows, prompt_.back());
    }

    Result<bool> decode(std::span<const DecodeSlot> slots, const DeviceLogitsRows& rows) override
    {
        session_.sequence_length += 1;
        return write(rows, slots[0].token_id);
    }

private:
    Result<bool> write(const DeviceLogitsRows& rows, int32_t fed)
    {
        const std::vector<float> values =
            synthetic_logits(kVocab, session_.number, static_cast<uint32_t>(session_.sequence_length - 1), fed);
        if (rows.bf16 || rows.vocab != kVocab || rows.rows != 1)
            return Error{ErrorCode::InternalError, "worker source: unexpected device rows"};
        if (hipMemcpy(rows.data, values.data(), values.size() * sizeof(float), hipMemcpyHostToDevice) != hipSuccess)
            return Error{ErrorCode::InternalError, "worker source: hipMemcpy failed"};
        return true;
    }

    WorkerSession& session_;
    const std::vector<int32_t>& prompt_;
};

void emit(const std::string& line)
{
    std::cout << line << '\n' << std::flush;
}

} // namespace

int main()
{
    HipSamplerPtr sampler = HipSampler::create(0, 4, kVocab);
    if (!sampler)
    {
        emit(wire::error_event("", "hip sampler is unavailable (no GPU, or create() failed)", "internal_error"));
        return 2;
    }
    emit(wire::JsonLine().add_string("event", "ready").add_uint("vocabulary_size", kVocab).finish());
    std::map<std::string, WorkerSession> sessions;
    std::string line;
    while (std::getline(std::cin, line))
    {
        if (line.empty())
            continue;
        std::string request_id;
        try
        {
            const wire::RequestFields fields(line);
            request_id = fields.string("request_id").value_or("");
            const std::string op = fields.string("op").value_or("");
            if (op == "shutdown")
            {
                emit(wire::JsonLine().add_string("event", "shutdown").finish());
                return 0;
            }
            if (op == "create_session")
            {
                const auto session_id = fields.string("session_id");
                if (!session_id || session_id->empty())
                    throw std::invalid_argument("create_session requires a non-empty session_id");
                if (sessions.count(*session_id) != 0)
                    throw std::invalid_argument("session already exists: " + *session_id);
                WorkerSession& session = sessions[*session_id];
                session.number = static_cast<uint32_t>(sessions.size() - 1);
                SamplingSessionOptions options;
                options.sampling_seed = static_cast<uint64_t>(fields.integer("seed").value_or(0));
                session.sampling = std::make_unique<SamplingSession>(sampler, options);
                emit(wire::JsonLine().add_string("event", "session_created").add_string("session_id", *session_id)
                         .add_uint("sequence_length", 0).finish());
                continue;
            }
            if (op == "stats")
            {
                const std::string session_id = fields.string("session_id").value_or("main");
                const auto found = sessions.find(session_id);
                if (found == sessions.end())
                    throw std::invalid_argument("unknown session: " + session_id);
                const SamplingStatistics statistics = found->second.sampling->statistics();
                emit(wire::JsonLine().add_string("event", "stats").add_string("session_id", session_id)
                         .add_uint("sequence_length", found->second.sequence_length)
                         .add_uint("sampled_tokens", statistics.sampled_tokens).add_uint("sample_calls", statistics.sample_calls)
                         .add_uint("sample_time_microseconds", statistics.sample_time_microseconds).finish());
                continue;
            }
            if (op == "generate")
            {
                const wire::GenerateRequest request = wire::parse_generate_request(line);
                request_id = request.request_id;
                const auto found = sessions.find(request.session_id);
                if (found == sessions.end())
                    throw std::invalid_argument("unknown session: " + request.session_id);
                WorkerSession& session = found->second;
                WorkerSource source(session, request.prompt_tokens);
                SamplingSession* pointer = session.sampling.get();
                const auto started = std::chrono::steady_clock::now();
                const auto elapsed = [&]() { return std::chrono::duration<double>(std::chrono::steady_clock::now() - started).count(); };
                auto generated = BatchGenerationLoop::generate(
                    sampler, std::span<SamplingSession* const>(&pointer, 1), source, std::span<const GenerationOptions>(&request.options, 1),
                    [&](uint32_t, const StreamToken& token) {
                        emit(wire::token_event(request.request_id, request.session_id, token, elapsed()));
                        return true;
                    });
                if (!generated)
                    emit(wire::error_event(request.request_id, generated.error().message, wire::error_code_name(generated.error().code)));
                else
                    emit(wire::done_event(request.request_id, request.session_id, generated.value()[0], false, elapsed(),
                                          session.sequence_length, session.sampling->statistics()));
                continue;
            }
            throw std::invalid_argument("unknown op: " + op);
        }
        catch (const std::exception& error)
        {
            emit(wire::error_event(request_id, error.what()));
        }
    }
    return 0;
}
