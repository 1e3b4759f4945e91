// The sampling slice of the worker's JSON-lines protocol (examples/ncnn_moe_worker.cpp): how a
// `generate` request names its sampling options, and how tokens, completion and errors are reported.
// A front end that speaks these lines (tools/ncnn_moe_protocol.py, the CLI and TUI above it) reaches
// the GPU sampler unchanged.
//
//   parse_generate_request   the fields handle_generate reads (examples/ncnn_moe_worker.cpp:1031-1058),
//                            with its defaults: temperature 0 when absent, top_k only from an integer
//                            literal, max_new_tokens 1, request_id "generate", session_id "main"
//   token_event              the `token` line (examples/ncnn_moe_worker.cpp:870-886)
//   done_event               the sampling fields of the `done` line (:895-905, :912) plus the
//                            Session's sampling statistics
//   error_event              emit_error (:727-736) and error_code_name (:163-174)
#ifndef NCNN_MOE_HIP_WORKER_WIRE_H
#define NCNN_MOE_HIP_WORKER_WIRE_H

#include "hip_session_sampler.h"

#include <optional>
#include <stdexcept>
#include <string>
#include <string_view>
#include <vector>

namespace ncnn {
namespace moe {
namespace wire {

// One JSON object on a line, written key by key in call order (the worker's JsonObject).
class JsonLine
{
public:
    JsonLine& add_string(std::string_view name, std::string_view value);
    JsonLine& add_uint(std::string_view name, uint64_t value);
    JsonLine& add_int(std::string_view name, int64_t value);
    JsonLine& add_bool(std::string_view name, bool value);
    JsonLine& add_double(std::string_view name, double value); // 10 significant digits; null when not finite
    JsonLine& add_null(std::string_view name);
    JsonLine& add_raw(std::string_view name, std::string_view json);
    std::string finish() const;

private:
    void key(std::string_view name);
    std::string text_ = "{";
    bool first_ = true;
};

std::string json_escape(std::string_view value);

// The members of one flat request object, each kept as the raw text of its value.
class RequestFields
{
public:
    // Throws std::invalid_argument when the line is not a JSON object.
    explicit RequestFields(std::string_view line);

    std::optional<std::string> string(std::string_view key) const;
    std::optional<int64_t> integer(std::string_view key) const;   // an integer literal only: 20.0 is not one
    std::optional<double> number(std::string_view key) const;
    std::optional<bool> boolean(std::string_view key) const;
    std::optional<std::vector<int64_t>> integer_array(std::string_view key) const;

private:
    const std::string* find(std::string_view key) const;
    std::vector<std::pair<std::string, std::string>> members_;
};

struct GenerateRequest
{
    std::string request_id;
    std::string session_id;
    std::vector<int32_t> prompt_tokens;
    GenerationOptions options;
};

// Throws std::invalid_argument with the worker's messages ("prompt_tokens must be an integer array",
// "prompt_tokens must not be empty", "stop_tokens contains an out-of-range token ID",
// "top_k is outside the uint32 range", ...).
GenerateRequest parse_generate_request(std::string_view line);

std::string token_event(std::string_view request_id, std::string_view session_id, const StreamToken& token, double elapsed_seconds);

std::string done_event(std::string_view request_id, std::string_view session_id, const GenerationResult& generation,
                       bool cancelled, double elapsed_seconds, uint64_t sequence_length, const SamplingStatistics& sampling);

std::string error_event(std::string_view request_id, std::string_view message, std::string_view code = "invalid_request");

const char* error_code_name(ErrorCode code) noexcept;

} // namespace wire
} // namespace moe
} // namespace ncnn

#endif // NCNN_MOE_HIP_WORKER_WIRE_H
