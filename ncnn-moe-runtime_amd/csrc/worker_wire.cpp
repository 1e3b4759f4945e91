// The sampling slice of the worker's JSON-lines protocol (see worker_wire.h).
#include "worker_wire.h"

#include <charconv>
#include <cmath>
#include <cstdlib>
#include <iomanip>
#include <limits>
#include <sstream>

namespace ncnn {
namespace moe {
namespace wire {

std::string json_escape(std::string_view value)
{
    std::string out = "\"";
    for (const char c : value)
    {
        switch (c)
        {
        case '"': out += "\\\""; break;
        case '\\': out += "\\\\"; break;
        case '\b': out += "\\b"; break;
        case '\f': out += "\\f"; break;
        case '\n': out += "\\n"; break;
        case '\r': out += "\\r"; break;
        case '\t': out += "\\t"; break;
        default: out += static_cast<unsigned char>(c) < 0x20 ? '?' : c; break; // other control characters are not sent
        }
    }
    out += '"';
    return out;
}

void JsonLine::key(std::string_view name)
{
    if (!first_)
        text_ += ',';
    first_ = false;
    text_ += json_escape(name);
    text_ += ':';
}

JsonLine& JsonLine::add_string(std::string_view name, std::string_view value)
{
    key(name);
    text_ += json_escape(value);
    return *this;
}

JsonLine& JsonLine::add_uint(std::string_view name, uint64_t value)
{
    key(name);
    text_ += std::to_string(value);
    return *this;
}

JsonLine& JsonLine::add_int(std::string_view name, int64_t value)
{
    key(name);
    text_ += std::to_string(value);
    return *this;
}

JsonLine& JsonLine::add_bool(std::string_view name, bool value)
{
    key(name);
    text_ += value ? "true" : "false";
    return *this;
}

JsonLine& JsonLine::add_double(std::string_view name, double value)
{
    key(name);
    if (!std::isfinite(value))
    {
        text_ += "null";
        return *this;
    }
    std::ostringstream stream;
    stream << std::setprecision(10) << value;
    text_ += stream.str();
    return *this;
}

JsonLine& JsonLine::add_null(std::string_view name)
{
    key(name);
    text_ += "null";
    return *this;
}

JsonLine& JsonLine::add_raw(std::string_view name, std::string_view json)
{
    key(name);
    text_ += json;
    return *this;
}

std::string JsonLine::finish() const
{
    return text_ + "}";
}

namespace {

bool is_space(char c)
{
    return c == ' ' || c == '\t' || c == '\r' || c == '\n';
}

struct Scanner
{
    std::string_view text;
    size_t at = 0;

    void skip_space()
    {
        while (at < text.size() && is_space(text[at]))
            ++at;
    }

    [[noreturn]] void fail(const char* what) const
    {
        throw std::invalid_argument(std::string("malformed request: ") + what);
    }

    // A string literal, unescaped.
    std::string string_literal()
    {
        if (at >= text.size() || text[at] != '"')
            fail("expected a string");
        std::string out;
        for (++at; at < text.size(); ++at)
        {
            const char c = text[at];
            if (c == '"')
            {
                ++at;
                return out;
            }
            if (c != '\\')
            {
                out += c;
                continue;
            }
            if (++at >= text.size())
                break;
            switch (text[at])
            {
            case '"': out += '"'; break;
            case '\\': out += '\\'; break;
            case '/': out += '/'; break;
            case 'b': out += '\b'; break;
            case 'f': out += '\f'; break;
            case 'n': out += '\n'; break;
            case 'r': out += '\r'; break;
            case 't': out += '\t'; break;
            case 'u':
            {
                if (at + 4 >= text.size())
                    fail("truncated \\u escape");
                unsigned code = 0;
                const auto parsed = std::from_chars(text.data() + at + 1, text.data() + at + 5, code, 16);
                if (parsed.ec != std::errc() || parsed.ptr != text.data() + at + 5)
                    fail("bad \\u escape");
                at += 4;
                // ids and names on this protocol are ASCII; anything else is kept as UTF-8 of the code unit
                if (code < 0x80)
                    out += static_cast<char>(code);
                else if (code < 0x800)
                {
                    out += static_cast<char>(0xC0 | (code >> 6));
                    out += static_cast<char>(0x80 | (code & 0x3F));
                }
                else
                {
                    out += static_cast<char>(0xE0 | (code >> 12));
                    out += static_cast<char>(0x80 | ((code >> 6) & 0x3F));
                    out += static_cast<char>(0x80 | (code & 0x3F));
                }
                break;
            }
            default: fail("unknown escape");
            }
        }
        fail("unterminated string");
    }

    // The raw text of one value; nested arrays and objects are taken whole.
    std::string raw_value()
    {
        const size_t begin = at;
        if (at >= text.size())
            fail("missing value");
        if (text[at] == '"')
        {
            (void)string_literal();
            return std::string(text.substr(begin, at - begin));
        }
        if (text[at] == '[' || text[at] == '{')
        {
            int depth = 0;
            while (at < text.size())
            {
                const char c = text[at];
                if (c == '"')
                {
                    (void)string_literal();
                    continue;
                }
                if (c == '[' || c == '{')
                    ++depth;
                if (c == ']' || c == '}')
                    --depth;
                ++at;
                if (depth == 0)
                    return std::string(text.substr(begin, at - begin));
            }
            fail("unterminated array or object");
        }
        while (at < text.size() && text[at] != ',' && text[at] != '}' && text[at] != ']' && !is_space(text[at]))
            ++at;
        if (at == begin)
            fail("missing value");
        return std::string(text.substr(begin, at - begin));
    }
};

} // namespace

RequestFields::RequestFields(std::string_view line)
{
    Scanner scanner{line};
    scanner.skip_space();
    if (scanner.at >= line.size() || line[scanner.at] != '{')
        scanner.fail("expected an object");
    ++scanner.at;
    scanner.skip_space();
    if (scanner.at < line.size() && line[scanner.at] == '}')
        return;
    while (true)
    {
        scanner.skip_space();
        std::string name = scanner.string_literal();
        scanner.skip_space();
        if (scanner.at >= line.size() || line[scanner.at] != ':')
            scanner.fail("expected ':'");
        ++scanner.at;
        scanner.skip_space();
        members_.emplace_back(std::move(name), scanner.raw_value());
        scanner.skip_space();
        if (scanner.at < line.size() && line[scanner.at] == ',')
        {
            ++scanner.at;
            continue;
        }
        if (scanner.at < line.size() && line[scanner.at] == '}')
            return;
        scanner.fail("expected ',' or '}'");
    }
}

const std::string* RequestFields::find(std::string_view key) const
{
    for (const auto& member : members_)
    {
        if (member.first == key)
            return &member.second;
    }
    return nullptr;
}

std::optional<std::string> RequestFields::string(std::string_view key) const
{
    const std::string* raw = find(key);
    if (raw == nullptr || raw->empty() || raw->front() != '"')
        return std::nullopt;
    Scanner scanner{*raw};
    return scanner.string_literal();
}

std::optional<int64_t> RequestFields::integer(std::string_view key) const
{
    const std::string* raw = find(key);
    if (raw == nullptr)
        return std::nullopt;
    int64_t value = 0;
    const auto parsed = std::from_chars(raw->data(), raw->data() + raw->size(), value);
    if (parsed.ec != std::errc() || parsed.ptr != raw->data() + raw->size())
        return std::nullopt;
    return value;
}

std::optional<double> RequestFields::number(std::string_view key) const
{
    const std::string* raw = find(key);
    if (raw == nullptr || raw->empty() || raw->front() == '"' || raw->front() == '[' || raw->front() == '{')
        return std::nullopt;
    char* end = nullptr;
    const double value = std::strtod(raw->c_str(), &end);
    if (end == raw->c_str() || *end != '\0')
        return std::nullopt;
    return value;
}

std::optional<bool> RequestFields::boolean(std::string_view key) const
{
    const std::string* raw = find(key);
    if (raw == nullptr)
        return std::nullopt;
    if (*raw == "true")
        return true;
    if (*raw == "false")
        return false;
    return std::nullopt;
}

std::optional<std::vector<int64_t>> RequestFields::integer_array(std::string_view key) const
{
    const std::string* raw = find(key);
    if (raw == nullptr || raw->size() < 2 || raw->front() != '[' || raw->back() != ']')
        return std::nullopt;
    std::vector<int64_t> values;
    size_t at = 1;
    const size_t end = raw->size() - 1;
    while (true)
    {
        while (at < end && is_space((*raw)[at]))
            ++at;
        if (at == end)
        {
            if (values.empty())
                return values;
            return std::nullopt; // a trailing comma
        }
        size_t stop = at;
        while (stop < end && (*raw)[stop] != ',' && !is_space((*raw)[stop]))
            ++stop;
        int64_t value = 0;
        const auto parsed = std::from_chars(raw->data() + at, raw->data() + stop, value);
        if (parsed.ec != std::errc() || parsed.ptr != raw->data() + stop)
            return std::nullopt;
        values.push_back(value);
        at = stop;
        while (at < end && is_space((*raw)[at]))
            ++at;
        if (at == end)
            return values;
        if ((*raw)[at] != ',')
            return std::nullopt;
        ++at;
    }
}

namespace {

uint32_t request_uint(const RequestFields& fields, std::string_view key, uint32_t default_value)
{
    const auto value = fields.integer(key);
    if (!value)
        return default_value;
    if (*value < 0 || static_cast<uint64_t>(*value) > std::numeric_limits<uint32_t>::max())
        throw std::invalid_argument(std::string(key) + " is outside the uint32 range");
    return static_cast<uint32_t>(*value);
}

std::vector<int32_t> request_tokens(const RequestFields& fields, std::string_view key, bool required)
{
    const auto values = fields.integer_array(key);
    if (!values)
    {
        if (required)
            throw std::invalid_argument(std::string(key) + " must be an integer array");
        return {};
    }
    std::vector<int32_t> out;
    out.reserve(values->size());
    for (const int64_t value : *values)
    {
        if (value < std::numeric_limits<int32_t>::min() || value > std::numeric_limits<int32_t>::max())
            throw std::invalid_argument(std::string(key) + " contains an out-of-range token ID");
        out.push_back(static_cast<int32_t>(value));
    }
    if (required && out.empty())
        throw std::invalid_argument(std::string(key) + " must not be empty");
    return out;
}

} // namespace

GenerateRequest parse_generate_request(std::string_view line)
{
    const RequestFields fields(line);
    GenerateRequest parsed;
    parsed.request_id = fields.string("request_id").value_or("generate");
    parsed.session_id = fields.string("session_id").value_or("main");
    parsed.prompt_tokens = request_tokens(fields, "prompt_tokens", true);
    parsed.options.max_new_tokens = request_uint(fields, "max_new_tokens", parsed.options.max_new_tokens);
    parsed.options.stop_tokens = request_tokens(fields, "stop_tokens", false);
    // a request without a temperature is greedy, whatever SamplingOptions defaults to
    const auto temperature = fields.number("temperature");
    parsed.options.sampling.temperature = temperature ? static_cast<float>(*temperature) : 0.0f;
    if (fields.integer("top_k"))
        parsed.options.sampling.top_k = request_uint(fields, "top_k", 0);
    if (const auto top_p = fields.number("top_p"))
        parsed.options.sampling.top_p = static_cast<float>(*top_p);
    if (const auto min_p = fields.number("min_p"))
        parsed.options.sampling.min_p = static_cast<float>(*min_p);
    // the speculative switches of examples/ncnn_moe_worker.cpp:1040, :1053-1055
    parsed.options.enable_speculative = fields.boolean("enable_speculative").value_or(true);
    if (const auto confidence = fields.number("speculative_confidence"))
        parsed.options.speculative_confidence_threshold = static_cast<float>(*confidence);
    parsed.options.speculative_max_draft_tokens = request_uint(fields, "speculative_max_draft", 0);
    return parsed;
}

std::string token_event(std::string_view request_id, std::string_view session_id, const StreamToken& token, double elapsed_seconds)
{
    JsonLine event;
    event.add_string("event", "token");
    event.add_string("request_id", request_id);
    event.add_string("session_id", session_id);
    event.add_uint("index", token.index);
    event.add_int("token_id", token.token_id);
    event.add_double("probability", token.probability);
    event.add_bool("is_stop_token", token.is_stop_token);
    event.add_double("elapsed_seconds", elapsed_seconds);
    return event.finish();
}

std::string done_event(std::string_view request_id, std::string_view session_id, const GenerationResult& generation,
                       bool cancelled, double elapsed_seconds, uint64_t sequence_length, const SamplingStatistics& sampling)
{
    JsonLine done;
    done.add_string("event", "done");
    done.add_string("request_id", request_id);
    done.add_string("session_id", session_id);
    done.add_bool("ok", true);
    done.add_bool("metrics_enabled", false);
    done.add_uint("generated_tokens", generation.tokens.size());
    done.add_bool("stopped_by_stop_token", generation.stopped_by_stop_token);
    done.add_bool("stopped_by_callback", generation.stopped_by_callback);
    done.add_bool("cancelled", generation.stopped_by_callback && cancelled);
    done.add_double("elapsed_seconds", elapsed_seconds);
    if (elapsed_seconds > 0.0 && !generation.tokens.empty())
        done.add_double("tokens_per_second", static_cast<double>(generation.tokens.size()) / elapsed_seconds);
    else
        done.add_null("tokens_per_second");
    done.add_uint("sequence_length", sequence_length);
    JsonLine statistics;
    statistics.add_uint("sampled_tokens", sampling.sampled_tokens);
    statistics.add_uint("sample_calls", sampling.sample_calls);
    statistics.add_uint("sample_time_microseconds", sampling.sample_time_microseconds);
    done.add_raw("sampling", statistics.finish());
    return done.finish();
}

std::string error_event(std::string_view request_id, std::string_view message, std::string_view code)
{
    JsonLine event;
    event.add_string("event", "error");
    if (!request_id.empty())
        event.add_string("request_id", request_id);
    event.add_string("code", code);
    event.add_string("message", message);
    return event.finish();
}

const char* error_code_name(ErrorCode code) noexcept
{
    switch (code)
    {
    case ErrorCode::InvalidArgument: return "invalid_argument";
    case ErrorCode::IoError: return "io_error";
    case ErrorCode::InvalidModel: return "invalid_model";
    case ErrorCode::UnsupportedModel: return "unsupported_model";
    case ErrorCode::InternalError: return "internal_error";
    }
    return "unknown";
}

} // namespace wire
} // namespace moe
} // namespace ncnn
