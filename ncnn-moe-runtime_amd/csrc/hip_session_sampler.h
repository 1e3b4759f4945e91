// Host-side C++ face of the gfx950 generation sampler, shaped like the runtime's own Session
// sampling interface so that it can stand in for the CPU sampler:
//
//   SamplingOptions / SampledToken / LogitsOutput / Result<T> / Error   the runtime's public types
//       (include/ncnn/moe/session.h:30-61, include/ncnn/moe/result.h:12-71).  When this header is
//       compiled inside the runtime (NCNN_MOE_SESSION_H already defined) the runtime's own types
//       are used; a stand-alone build defines equivalents with the same names and defaults.
//   HipSampler           backend operator in the style of src/backends/ncnn/ncnn_linear.h:45-71:
//       pimpl, static create() returning a shared_ptr that is null on failure.
//   SamplingSession      the sampling slice of Session (include/ncnn/moe/session.h:288-342): the
//       seeded std::mt19937_64 (session.cpp:291), the per-Session mutex, sample().
//   SessionBatchSampler  the batched entry beside SessionBatchAccess::decode
//       (src/engine/session_batch.h:32-42): locks the Sessions in ascending pointer order and
//       rejects duplicates (src/engine/session.cpp:1249-1265), draws one uniform per row from a COPY
//       of each Session's generator, samples every row in one device call, and commits the copy back
//       only for rows whose draw was consumed (session.cpp:429-433).
//   BatchSampleScheduler the batched-sample hand-off of the batch scheduler: submit_sample() beside
//       BatchScheduler::submit_decode (include/ncnn/moe/scheduler.h:122-123), with the scheduler's worker
//       threads, per-Session order and cross-call collection (src/engine/scheduler.cpp:87-104, :416-437,
//       :975-1096, :1104-1138), so that callers that each sample one row share one device call.
//   BatchGenerationLoop  the scheduler-driven generation loop of examples/internal/run_model.cpp:726-847
//       over device-resident logits: an IDeviceLogitsSource (the model's prefill / decode) writes
//       each step's logits into the sampler's buffer and one device call samples every active Session.
//
// Everything here runs on the device through the C ABI of include/ncnn_moe_hip_sampler.h.  There is
// no CPU fallback: without a usable GPU create() returns null and sample() reports InternalError.
#ifndef NCNN_MOE_HIP_SESSION_SAMPLER_H
#define NCNN_MOE_HIP_SESSION_SAMPLER_H

#include <cstdint>
#include <functional>
#include <future>
#include <memory>
#include <mutex>
#include <random>
#include <span>
#include <string>
#include <utility>
#include <variant>
#include <vector>

#ifndef NCNN_MOE_SESSION_H

namespace ncnn {
namespace moe {

enum class ErrorCode
{
    InvalidArgument,
    IoError,
    InvalidModel,
    UnsupportedModel,
    InternalError
};

struct Error
{
    ErrorCode code = ErrorCode::InternalError;
    std::string message;
};

// Value-or-error carrier with the accessors the runtime's callers use: bool conversion, value(), error().
template <typename T>
class Result
{
public:
    Result(T value) : storage_(std::in_place_index<0>, std::move(value)) {}
    Result(Error error) : storage_(std::in_place_index<1>, std::move(error)) {}

    explicit operator bool() const noexcept { return storage_.index() == 0; }
    T& value() { return std::get<0>(storage_); }
    const T& value() const { return std::get<0>(storage_); }
    const Error& error() const { return std::get<1>(storage_); }

private:
    std::variant<T, Error> storage_;
};

struct LogitsOutput
{
    std::vector<float> values;
};

// include/ncnn/moe/types.h:304-309
enum class LogitsOutputMode
{
    FullLogits,
    TopKCandidates,
    SampledToken
};

struct SamplingOptions
{
    float temperature = 1.0f;
    uint32_t top_k = 0;
    float top_p = 1.0f;
    float min_p = 0.0f;
};

struct SampledToken
{
    int32_t token_id = -1;
    float probability = 0.0f;
};

// StreamToken, GenerationOptions, GenerationResult and TokenTextDecoder of include/ncnn/moe/session.h:63-96.
struct StreamToken
{
    uint32_t index = 0;
    int32_t token_id = -1;
    float probability = 0.0f;
    std::string text; // what the caller's TokenTextDecoder returned for the token; empty without one
    bool is_stop_token = false;
};

struct GenerationOptions
{
    uint32_t max_new_tokens = 1;
    SamplingOptions sampling;
    std::vector<int32_t> stop_tokens;
    bool enable_speculative = true;
    float speculative_confidence_threshold = 0.5f;
    uint32_t speculative_max_draft_tokens = 0;
};

using TokenTextDecoder = std::function<std::string(int32_t token_id)>;

struct GenerationResult
{
    std::vector<StreamToken> tokens;
    bool stopped_by_stop_token = false;
    bool stopped_by_callback = false;
};

} // namespace moe
} // namespace ncnn

#endif // NCNN_MOE_SESSION_H

namespace ncnn {
namespace moe {

// One sampled row of a batch: the token plus the stop flag the generation loops derive from it
// (StreamToken::is_stop_token, include/ncnn/moe/session.h:63-72).
struct BatchSampledToken
{
    SampledToken token;
    bool is_stop_token = false;
    uint32_t kept_count = 0;
};

// A candidate of the filtered distribution (sampling_distribution, src/engine/session.cpp:76-136).
struct TokenProbability
{
    int32_t token_id = -1;
    float probability = 0.0f;
};

// Outcome of one verification step of speculative generation (src/engine/session.cpp:776-874).
struct SpeculativeVerification
{
    std::vector<SampledToken> accepted; // the proposed tokens that stand, each with its reported probability
    SampledToken next;                  // the token emitted after them (residual draw, or the target's own sample)
    bool next_from_residual = false;
    // Nothing was accepted and the caller's state keeps no cache transactions: the step is rolled back and
    // speculative mode left before `next` is drawn (src/engine/session.cpp:843-857); `next` is not set and
    // only the accept test's draw was consumed.
    bool fell_back = false;
};

// The capability bit a runtime with this backend reports beside RuntimeCapabilityFlag
// (include/ncnn/moe/runtime.h:40-59; bits 0-17 are taken there).
#define NCNN_MOE_RUNTIME_CAP_HIP_SAMPLER_BIT 18
enum : uint32_t
{
    RuntimeCapabilityHipSampler = UINT32_C(1) << NCNN_MOE_RUNTIME_CAP_HIP_SAMPLER_BIT
};
// RuntimeCapabilityHipSampler if a HIP device is usable, else 0 (what Runtime::capabilities() would OR in).
uint32_t hip_sampler_capabilities();

// Rows of logits in device memory: row i starts at data + i * row_stride elements.
struct DeviceLogitsRows
{
    void* data = nullptr;
    uint64_t row_stride = 0; // in elements
    uint32_t rows = 0;
    uint32_t vocab = 0;
    bool bf16 = false;       // bfloat16 elements instead of float
};

class HipSampler
{
public:
    // Null when no GPU is usable or the device buffers for max_rows x max_vocab cannot be allocated.
    static std::shared_ptr<HipSampler> create(int device, uint32_t max_rows, uint32_t max_vocab);
    ~HipSampler();
    HipSampler(const HipSampler&) = delete;
    HipSampler& operator=(const HipSampler&) = delete;

    uint32_t max_rows() const noexcept;
    uint32_t max_vocab() const noexcept;

    // Samples rows.size() rows; logits[i] is row i (all rows must have the same length).  uniforms[i]
    // is the draw row i would consume.  draw_consumed[i] reports whether it did.  One Result per row:
    // a bad row does not fail the others.  A call-level failure yields that Error for every row.
    std::vector<Result<BatchSampledToken>> sample(
        std::span<const std::span<const float>> logits,
        std::span<const SamplingOptions> options,
        std::span<const float> uniforms,
        std::span<const std::vector<int32_t>> stop_tokens,
        std::vector<uint8_t>& draw_consumed);

    // The device-resident hand-off (ncnn_moe_hip_sampler_logits_buffer): the sampler's own logits
    // buffer laid out for rows x vocab.  A decode step writes its LM-head output there, and
    // sample_resident() reads it: the logits never become a std::vector<float>
    // (src/engine/cpu_executor.cpp:2988-2994, src/kernels/cpu_ops.cpp:1166-1172 are the copies this removes).
    Result<DeviceLogitsRows> device_logits(uint32_t rows, uint32_t vocab, bool bf16 = false);

    // sample() over the rows last laid out by device_logits(); the rows must be complete in device
    // memory when this is called.  device_rows empty: entry i of the operands samples row i (as many
    // entries as rows were laid out).  Otherwise entry i samples row device_rows[i], in any order and for
    // any subset of the rows; the rows that no entry names are left alone.  A sample() of host logits in
    // between overwrites the buffer: the next sample_resident() is then refused until device_logits() has
    // laid the rows out again.
    std::vector<Result<BatchSampledToken>> sample_resident(
        std::span<const SamplingOptions> options,
        std::span<const float> uniforms,
        std::span<const std::vector<int32_t>> stop_tokens,
        std::vector<uint8_t>& draw_consumed,
        std::span<const uint32_t> device_rows = {});

    // Copies host rows into the buffer and lays it out for them, as a decode step that runs on the CPU would
    // hand its logits over (ncnn_moe_hip_sampler_upload_logits): sample_resident() then samples them.
    Result<DeviceLogitsRows> upload_resident(std::span<const std::span<const float>> logits);

    // sampling_distribution for one row.
    Result<std::vector<TokenProbability>> distribution(std::span<const float> logits, const SamplingOptions& options);

    // The accept loop and the following token of src/engine/session.cpp:776-874 in one device pass.
    // target_logits: proposed.size() + 1 rows (after the anchor and after each proposed token);
    // draft_logits: the rows the proposed tokens were sampled from; uniforms: the Session RNG's next
    // proposed.size() + 1 draws.  draws_consumed receives how many of them the step used, in order.
    Result<SpeculativeVerification> verify_speculative(
        std::span<const std::span<const float>> target_logits,
        std::span<const std::span<const float>> draft_logits,
        std::span<const int32_t> proposed_token_ids,
        const SamplingOptions& options,
        std::span<const float> uniforms,
        uint32_t& draws_consumed,
        uint32_t* accept_draws = nullptr, // of draws_consumed, those of the accept tests (the rest is the last token's draw)
        // set when the step failed only after its accept loop had ended with nothing accepted, i.e. while the
        // next token was drawn: a caller without cache transactions leaves speculative mode in front of that
        // draw (src/engine/session.cpp:843-857) and never sees the failure
        bool* failed_behind_an_empty_accept_loop = nullptr);

    // The same over rows that are already in the sampler's buffer: rows 0 .. D the target's logits after the
    // anchor and after each of the D proposed tokens, rows D + 1 .. 2 D the draft rows those tokens were
    // sampled from (laid out by device_logits(2 D + 1, vocab)).
    Result<SpeculativeVerification> verify_speculative_resident(
        std::span<const int32_t> proposed_token_ids,
        const SamplingOptions& options,
        std::span<const float> uniforms,
        uint32_t& draws_consumed,
        uint32_t* accept_draws = nullptr,
        bool* failed_behind_an_empty_accept_loop = nullptr);

private:
    HipSampler();
    struct Impl;
    std::unique_ptr<Impl> impl_;
    std::mutex mutex_;
};

using HipSamplerPtr = std::shared_ptr<HipSampler>;

// The sampling share of SessionStatistics (include/ncnn/moe/session.h:98-160 keeps prefill/decode
// counters and times per Session; sampling had none because it was not measurable on the CPU path).
struct SamplingStatistics
{
    uint64_t sampled_tokens = 0;           // tokens this Session's sampler returned
    uint64_t sample_calls = 0;             // device calls the Session took part in
    uint64_t sample_time_microseconds = 0; // wall time of those calls (a batched call counts in full for each of its Sessions)
    // SessionStatistics::speculative_accepted_tokens and ::speculative_verify_time_microseconds (the share of the
    // verification's device call), plus the steps themselves
    uint64_t speculative_steps = 0;
    uint64_t speculative_accepted_tokens = 0;
    uint64_t speculative_verify_time_microseconds = 0;
};

struct SamplingSessionOptions
{
    uint64_t sampling_seed = 0; // SessionOptions::sampling_seed, include/ncnn/moe/session.h:280-286
    // SessionOptions::logits_output_mode.  FullLogits: the Session's logits are host vectors (LogitsOutput).
    // SampledToken: they stay in the sampler's device buffer and only tokens come back; such a Session
    // is sampled through SessionBatchSampler::sample_resident, BatchSampleScheduler or BatchGenerationLoop.
    LogitsOutputMode logits_output_mode = LogitsOutputMode::FullLogits;
};

class SamplingSession
{
public:
    SamplingSession(HipSamplerPtr sampler, const SamplingSessionOptions& options = {});

    // Session::sample, include/ncnn/moe/session.h:326.
    [[nodiscard]] Result<SampledToken> sample(const LogitsOutput& logits, const SamplingOptions& options = {});

    // The verification step of Session::generate's speculative loop (src/engine/session.cpp:776-874):
    // draws from this Session's generator exactly as that loop would.
    [[nodiscard]] Result<SpeculativeVerification> verify_speculative(
        std::span<const LogitsOutput> target_logits, std::span<const LogitsOutput> draft_logits,
        std::span<const int32_t> proposed_token_ids, const SamplingOptions& options = {});

    // state_cache_transactions = false: the model state cannot roll back part of a step, so a step in which
    // nothing is accepted falls back (SpeculativeVerification::fell_back) before the next token is drawn.
    [[nodiscard]] Result<SpeculativeVerification> verify_speculative(
        std::span<const LogitsOutput> target_logits, std::span<const LogitsOutput> draft_logits,
        std::span<const int32_t> proposed_token_ids, const SamplingOptions& options, bool state_cache_transactions);

    // Session::statistics(), the sampling share.
    [[nodiscard]] SamplingStatistics statistics() const;
    [[nodiscard]] LogitsOutputMode logits_output_mode() const noexcept { return logits_output_mode_; }

private:
    friend class SessionBatchSampler;
    friend class BatchGenerationLoop;
    HipSamplerPtr sampler_;
    LogitsOutputMode logits_output_mode_ = LogitsOutputMode::FullLogits;
    // The uniform the sampler would draw `position` draws from now, without consuming it, and the
    // consumption of the next `count` of them.  A draw that was looked at but not consumed (a greedy
    // call, Top-K 1, an error: src/engine/session.cpp:404, :425-433) stays at the head of
    // `drawn_ahead_` and is the next call's first uniform, so the sequence of uniforms the sampler
    // consumes is the generator's own; the generator itself is ahead of the CPU sampler's by the
    // entries of `drawn_ahead_` (copying its 2.5 KB state on every call to look at one draw was a
    // fifth of the generation loop's time).
    float uniform_ahead(size_t position);
    void consume_uniforms(size_t count);

    std::mt19937_64 random_generator_;
    std::vector<float> drawn_ahead_;
    SamplingStatistics statistics_;
    mutable std::mutex mutex_;
};

using SamplingSessionPtr = std::shared_ptr<SamplingSession>;

// Runtime::create_session for the sampling slice (src/engine/runtime.cpp:575-582): with a HIP sampler the
// Session may be created in SampledToken mode, which the CPU executor refuses; TopKCandidates stays
// unsupported, and without a sampler only FullLogits is accepted, with the runtime's own message.
Result<SamplingSessionPtr> create_sampling_session(const HipSamplerPtr& sampler, const SamplingSessionOptions& options = {});

struct SampleBatchRequest
{
    static constexpr uint32_t kRowByPosition = UINT32_MAX;

    SamplingSession* session = nullptr;
    const LogitsOutput* logits = nullptr; // null for a Session in SampledToken mode: its row is in the device buffer
    SamplingOptions sampling;
    std::vector<int32_t> stop_tokens; // GenerationOptions::stop_tokens
    // SampledToken mode: the row of the device buffer that holds this Session's logits (the place the decode
    // step gave it).  kRowByPosition: request i of a batch samples row i, which fits a batch that is
    // submitted whole, in the decode step's order.  A request that travels alone (one serving thread per
    // Session, collected across calls by the scheduler) names its row.
    uint32_t device_row = kRowByPosition;
    // ... and, for a scheduler over several samplers, the one whose buffer holds the row
    uint32_t resident_sampler = 0;
};

class SessionBatchSampler
{
public:
    // One device call for the whole batch; replaces the serial loop of
    // examples/internal/run_model.cpp:776-809.  Rejects empty batches, null or duplicate Sessions and
    // rows of different lengths with InvalidArgument for every row.
    static std::vector<Result<BatchSampledToken>> sample(const HipSamplerPtr& sampler, std::span<const SampleBatchRequest> requests);

    // The same for Sessions in SampledToken mode: a request samples its device_row (or, with kRowByPosition in
    // every request, request i row i) of the rows last laid out by HipSampler::device_logits (the decode
    // step wrote them there); every request's logits must be null.
    static std::vector<Result<BatchSampledToken>> sample_resident(const HipSamplerPtr& sampler, std::span<const SampleBatchRequest> requests);
};

// BatchScheduler's options and counters, as far as sampling uses them (include/ncnn/moe/scheduler.h:41-109).
struct SampleSchedulerOptions
{
    uint32_t worker_count = 0;                     // 0: min(4, hardware threads), src/engine/scheduler.cpp:87
    uint32_t cross_call_window_microseconds = 200; // zero disables cross-call collection
    uint32_t cross_call_max_batch_size = 0;        // 0: the sampler's max_rows
    // An idle worker looks for work this long before it goes to sleep on the queue's condition variable: waking a
    // sleeping thread costs more than a whole device call of the select path (tens of microseconds against 15 to
    // 30), so a serving loop that submits batch after batch keeps its workers awake in between.  0: sleep at once.
    uint32_t worker_spin_microseconds = 100;
};

struct SampleSchedulerStatistics
{
    uint64_t submitted_batches = 0;
    uint64_t submitted_requests = 0;
    uint64_t completed_requests = 0;
    uint64_t rejected_requests = 0;
    uint64_t max_batch_size = 0;
    uint64_t serialized_session_requests = 0; // requests that waited for an earlier one of their Session
    uint64_t cross_call_collected_batches = 0;
    uint64_t cross_call_collected_requests = 0;
    uint64_t cross_call_collection_timeouts = 0;
    uint64_t device_calls = 0;
    uint64_t overlapped_device_calls = 0; // device calls that began while another one of this scheduler was running
    uint32_t worker_count = 0;
};

// The batched-sample entry of the batch scheduler.  submit_sample() returns at once; worker threads run
// the batches, each as ONE device call (SessionBatchSampler::sample).  Requests of one Session run in
// the order they were submitted and never two at a time; a batch that names a Session twice is rejected
// (src/engine/session.cpp:1257-1265).  Submissions of a single request, the shape of a serving loop with one
// thread per Session, are collected across calls for up to cross_call_window_microseconds and sampled
// together, one request per Session and batch.  The Sessions and logits a request points to must stay
// alive until its future is ready.
class BatchSampleScheduler
{
public:
    explicit BatchSampleScheduler(HipSamplerPtr sampler, const SampleSchedulerOptions& options = {});
    // Several samplers, each with device buffers and a stream of its own: batches that different workers
    // run at the same time go to different samplers and overlap on the GPU (the scheduler's workers run
    // batches concurrently, src/engine/scheduler.cpp:87-104, :257-270).  A batch of host logits takes the
    // next sampler in turn; a device-resident batch runs on the sampler its requests name
    // (SampleBatchRequest::resident_sampler: the one into whose buffer the decode step wrote).
    explicit BatchSampleScheduler(std::vector<HipSamplerPtr> samplers, const SampleSchedulerOptions& options = {});
    ~BatchSampleScheduler();
    BatchSampleScheduler(const BatchSampleScheduler&) = delete;
    BatchSampleScheduler& operator=(const BatchSampleScheduler&) = delete;

    [[nodiscard]] std::future<std::vector<Result<BatchSampledToken>>> submit_sample(std::vector<SampleBatchRequest> requests);
    [[nodiscard]] SampleSchedulerStatistics statistics() const noexcept;
    [[nodiscard]] size_t sampler_count() const noexcept;
    [[nodiscard]] HipSamplerPtr sampler(size_t index) const; // null beyond sampler_count()

private:
    class Implementation;
    std::unique_ptr<Implementation> implementation_;
};

// One row of a decode step: DecodeBatchRequest of the batch scheduler ({session, token}).
struct DecodeSlot
{
    uint32_t session_index = 0;
    int32_t token_id = -1;
};

// The model side of the loop: what BatchScheduler::submit_prefill / submit_decode do, writing the
// logits into device rows instead of returning LogitsOutput vectors.  Row i belongs to the i-th
// listed Session.  The rows must be complete in device memory when a call returns.
class IDeviceLogitsSource
{
public:
    virtual ~IDeviceLogitsSource() = default;
    virtual uint32_t vocabulary_size() const = 0;
    virtual bool bf16_logits() const { return false; }
    virtual Result<bool> prefill(std::span<const uint32_t> session_indices, const DeviceLogitsRows& rows) = 0;
    virtual Result<bool> decode(std::span<const DecodeSlot> slots, const DeviceLogitsRows& rows) = 0;
};

// The draft side of a model that can speculate: what CpuExecutor::propose_speculative and the verification pass of
// Session::generate do (src/engine/cpu_executor.cpp:2105-2160, :2270-2312; src/engine/session.cpp:630-760), writing
// device rows.  A source that implements it is recognised by BatchGenerationLoop::generate.
class ISpeculativeLogitsSource : public IDeviceLogitsSource
{
public:
    // Tokens of one proposal (CompiledModel::speculative.block_size); 0: the model has no draft head.
    virtual uint32_t speculative_block_size() const = 0;
    // SpeculativeModelKind::Mtp: the model state can keep part of a step (state cache transactions); without them
    // a step that accepts nothing is rolled back and the Session leaves speculative mode (session.cpp:843-857).
    virtual bool state_cache_transactions() const = 0;
    // Draft row `draft_index` of every listed Session: the draft head's logits after slot.token_id was fed (the
    // anchor for index 0, the Session's previous draft after that).  Row i belongs to slots[i].
    virtual Result<bool> draft(std::span<const DecodeSlot> slots, uint32_t draft_index, const DeviceLogitsRows& rows) = 0;
    // CpuSpeculativeProposal::confidence_logits of the Session's current proposal (+infinity where the model has none).
    virtual float confidence_logit(uint32_t session_index, uint32_t draft_index) const = 0;
    // The verification rows of one Session's step: rows 0 .. D the target's logits after the anchor and after each
    // of the D proposed tokens, rows D + 1 .. 2 D the draft rows those tokens were sampled from.
    virtual Result<bool> verify(uint32_t session_index, int32_t anchor, std::span<const int32_t> proposed, const DeviceLogitsRows& rows) = 0;
    // The step's outcome: the tokens that were emitted (the accepted ones and the one after them), none when the
    // step was rolled back.  The state moves on by them (finish_cache_transaction, session.cpp:931-935).
    virtual Result<bool> commit(uint32_t session_index, std::span<const int32_t> emitted) = 0;
};

// Called for every token as it is sampled; returning false stops that Session (GenerationResult::stopped_by_callback).
using BatchTokenCallback = std::function<bool(uint32_t session_index, const StreamToken& token)>;

class BatchGenerationLoop
{
public:
    // The scheduler-driven generation of examples/internal/run_model.cpp:726-847 with the sampling
    // of every step as ONE device call over device-resident logits: prefill all Sessions, then per
    // token index sample the active Sessions in Session order (each with its own generator, options
    // and stop tokens), stop those that emitted a stop token, reached max_new_tokens or whose callback
    // declined, and decode the others' tokens for the next step.  `options` holds one entry for all
    // Sessions or one per Session.  Token ids, probabilities, stop flags and generator states end up
    // as Session::generate (src/engine/session.cpp:978-1020) leaves them for each Session alone.
    //
    // With a source that can speculate (ISpeculativeLogitsSource with a block size above zero) a Session whose
    // options enable it runs the speculative loop of Session::generate (src/engine/session.cpp:522-977): after its
    // first token, rounds of propose (the block's draft tokens, each sampled with the Session's own generator, one
    // device call per draft index for all such Sessions) - cut the proposal (token budget,
    // speculative_max_draft_tokens, confidence threshold) - verify (one device pass per Session: accept loop and
    // the token after it) - stream the accepted tokens and that one.  A step that proposes or, without cache
    // transactions, accepts nothing leaves speculative mode for good, and the Session goes on token by token.
    // decode_text fills StreamToken::text in front of the callback (TokenTextDecoder, session.h:96).
    static Result<std::vector<GenerationResult>> generate(
        const HipSamplerPtr& sampler, std::span<SamplingSession* const> sessions, IDeviceLogitsSource& source,
        std::span<const GenerationOptions> options, const BatchTokenCallback& on_token = {}, const TokenTextDecoder& decode_text = {});
};

// validate_sampling_options (src/engine/session.cpp:65-74) on the host, with the same messages.
Result<bool> validate_sampling_options(const SamplingOptions& options);

// The uniform std::uniform_real_distribution<float>(0, 1) would draw next from `generator`,
// without advancing it.  `advanced` receives the generator state after the draw.
float peek_uniform(const std::mt19937_64& generator, std::mt19937_64& advanced);

} // namespace moe
} // namespace ncnn

#endif // NCNN_MOE_HIP_SESSION_SAMPLER_H
