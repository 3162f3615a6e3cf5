// Host-side policy types of the step scheduler: requests, events, bounded
// event streams, and the decode backend interface the scheduler drives.
//
// Mirrors the reference's retrograd-infer crate (crates/retrograd-infer/src/
// request.rs:16-257, backend.rs:27-155, error.rs) in C++: same names, same
// argument meaning, same error behaviour.
#pragma once

#include <chrono>
#include <cstdint>
#include <deque>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace sched {

enum class ErrKind : int {
    Invalid = 1,    // the caller's request cannot be served as written
    Failed = 2,     // the scheduler or backend failed
    Overflow = 3,   // a value does not fit its native type
    QueueFull = 4,  // the admission queue is at capacity
    KvFull = 5,     // a step failed while the pool is saturated
    Cancelled = 6,  // the request was cancelled before it ran
    Backend = 7,    // the backend's step or sequence operation failed
};

struct InferError : std::runtime_error {
    ErrKind kind;
    uint64_t needed = 0, available = 0;   // KvFull
    size_t capacity = 0;                  // QueueFull
    InferError(ErrKind k, const std::string & msg) : std::runtime_error(msg), kind(k) {}
    static InferError invalid(const std::string & msg) { return InferError(ErrKind::Invalid, msg); }
    static InferError failed(const std::string & msg) { return InferError(ErrKind::Failed, msg); }
    static InferError overflow(const std::string & msg) { return InferError(ErrKind::Overflow, msg); }
    static InferError backend(const std::string & msg) { return InferError(ErrKind::Backend, msg); }
    static InferError cancelled() { return InferError(ErrKind::Cancelled, "request cancelled"); }
    static InferError queue_full(size_t capacity) {
        InferError e(ErrKind::QueueFull, "admission queue is full (capacity " + std::to_string(capacity) + ")");
        e.capacity = capacity;
        return e;
    }
    static InferError kv_full(uint64_t needed, uint64_t available) {
        InferError e(ErrKind::KvFull, "kv pool capacity: " + std::to_string(needed) + " cells needed, " +
                                          std::to_string(available) + " available");
        e.needed = needed;
        e.available = available;
        return e;
    }
};

// crates/retrograd-core/src/types.rs:1353-1374; the neutral extended values
// are those of `From<SamplingParams>` (:1400-1417).
struct SamplingParamsV2 {
    float temperature = 1.0f;
    float top_p = 1.0f;
    uint32_t max_new_tokens = 0;
    uint32_t seed = 0;
    int32_t top_k = 0;
    float min_p = 0.0f;
    float repeat_penalty = 1.0f;
    float frequency_penalty = 0.0f;
    float presence_penalty = 0.0f;
    uint32_t penalty_window = 0;
    std::vector<std::pair<int32_t, float>> logit_bias;
    std::optional<std::string> grammar_gbnf;
};

// The adapter a step row decodes under (retrograd-engine/src/step.rs:61-80):
// 0 = the context's own adapter set, -1 = the base model alone, > 0 = a
// per-row adapter id.
using RowAdapter = int32_t;
constexpr RowAdapter kAdapterContext = 0;
constexpr RowAdapter kAdapterBase = -1;

struct Retention {
    std::string key;
    std::optional<std::string> release;
};

// request.rs:16-47
struct Request {
    std::vector<int32_t> prompt;
    std::vector<SamplingParamsV2> sampling;
    std::vector<std::string> stop;
    uint32_t n_top_logprobs = 0;
    bool logprobs = false;
    std::optional<std::string> adapter;
    bool unparse_special = false;
    std::optional<Retention> retention;

    size_t n() const { return sampling.size(); }
    void validate() const;   // request.rs:101-169; throws InferError::invalid
};

enum class FinishReason : int { Eog = 0, Stop = 1, MaxTokens = 2, ContextFull = 3, Cancelled = 4 };

struct TopLogprob {
    int32_t token;
    float logprob;
    std::string piece;
};

// request.rs:227-257
struct Event {
    enum Type : int { Token = 0, End = 1, Error = 2 } type = Token;
    size_t index = 0;
    // Token
    int32_t token = 0;
    float logprob = 0.0f;
    bool has_sampled_logprob = false;
    float sampled_logprob = 0.0f;
    bool forced = false;
    std::string text;                  // Token: newly emittable text; End: the flushed tail
    std::string piece;
    std::vector<TopLogprob> top_logprobs;
    // End
    FinishReason reason = FinishReason::Eog;
    size_t cached_tokens = 0;
    // Error
    ErrKind error_kind = ErrKind::Failed;
    std::string error_message;
    uint64_t error_needed = 0, error_available = 0;
};

// The bounded channel of one request (std::sync::mpsc::sync_channel in the
// reference): `senders` counts the live sending ends, the receiver is the
// caller's handle. Dropping the receiver cancels the request.
struct Stream {
    std::deque<Event> queue;
    size_t capacity = 0;
    int senders = 0;
    bool receiver_alive = true;
    bool cancelled = false;            // the flag the scheduler checks before each step

    enum class Send { Ok, Full, Disconnected };
    Send try_send(Event && e) {
        if (!receiver_alive) return Send::Disconnected;
        if (queue.size() >= capacity) return Send::Full;
        queue.push_back(std::move(e));
        return Send::Ok;
    }
};
using StreamRef = std::shared_ptr<Stream>;

// A sending end: counted, so the stream reads as closed once every end is gone.
class Sender {
public:
    Sender() = default;
    explicit Sender(StreamRef s) : s_(std::move(s)) { if (s_) ++s_->senders; }
    Sender(const Sender & o) : s_(o.s_) { if (s_) ++s_->senders; }
    Sender(Sender && o) noexcept : s_(std::move(o.s_)) { o.s_.reset(); }
    Sender & operator=(Sender o) noexcept { std::swap(s_, o.s_); return *this; }
    ~Sender() { if (s_) --s_->senders; }
    explicit operator bool() const { return (bool)s_; }
    Stream * operator->() const { return s_.get(); }
    const StreamRef & ref() const { return s_; }
    void reset() { if (s_) --s_->senders; s_.reset(); }
private:
    StreamRef s_;
};

// One row of a step plan (retrograd-engine/src/step.rs:93-106). `tokens`
// points into the scheduler's own buffers and is valid for the step call.
struct StepRow {
    int32_t request = 0;
    int32_t slot = 0;
    const int32_t * tokens = nullptr;
    uint32_t n = 0;
    int32_t pos0 = 0;
    bool sample = false;
    const SamplingParamsV2 * sampling = nullptr;
    uint32_t n_top_logprobs = 0;
    bool want_logprob = false;
    RowAdapter adapter = kAdapterContext;
};

// step.rs:208-221
struct StepOutRow {
    int32_t token = 0;
    float logprob = 0.0f;
    bool forced = false;
    bool sampled = false;
    size_t n_top = 0;
    float sampled_logprob = 0.0f;
};

// step.rs:256-263: one output row per step row and the row-major top-logprob
// arrays of stride n_top_stride.
struct StepOutput {
    std::vector<StepOutRow> rows;
    std::vector<int32_t> top_ids;
    std::vector<float> top_logprobs;
    size_t n_top_stride = 0;
    const StepOutRow & row(size_t i) const { return rows.at(i); }
};

// step.rs:225-238
struct EngineMemory {
    uint32_t n_slots = 0;
    uint64_t cells_total = 0, cells_used = 0, kv_bytes = 0, recurrent_bytes = 0;
};

struct AdapterRowsInfo {
    uint32_t n_adapters = 0, max_rank = 0;
    uint64_t stacked_bytes = 0, unpadded_bytes = 0;
};

// kv.rs:47-63
struct KvCacheKey {
    uint64_t fingerprint = 0, weights_version = 0, settings = 0;
    bool operator==(const KvCacheKey & o) const {
        return fingerprint == o.fingerprint && weights_version == o.weights_version && settings == o.settings;
    }
};
// FNV-1a mix (kv.rs:39-44)
inline uint64_t mix(uint64_t hash, uint64_t value) {
    hash ^= value;
    hash *= 1099511628211ull;
    return hash;
}

// What the scheduler drives (backend.rs:27-155): one decode per step call plus
// the raw sequence operations, the occupancy report and the read-only queries
// the emit path needs. Every method throws InferError on failure.
struct DecodeBackend {
    virtual ~DecodeBackend() = default;
    virtual void step(const std::vector<StepRow> & rows, StepOutput & out) = 0;
    virtual void seq_rm(int32_t slot, int32_t p0, int32_t p1) = 0;
    virtual void seq_cp(int32_t src, int32_t dst, int32_t p0, int32_t p1) = 0;
    virtual std::pair<int32_t, int32_t> seq_pos(int32_t slot) = 0;
    virtual size_t seq_save_len(int32_t slot, uint32_t flags) = 0;
    virtual size_t seq_save_into(int32_t slot, uint32_t flags, uint8_t * buffer, size_t n) = 0;
    virtual size_t seq_load(int32_t slot, uint32_t flags, const uint8_t * data, size_t n) = 0;
    virtual bool kv_unified() = 0;
    virtual uint64_t weights_version() = 0;
    virtual uint64_t model_fingerprint() = 0;
    virtual bool is_hybrid() = 0;
    virtual EngineMemory memory() = 0;
    virtual void request_free(int32_t request) = 0;
    virtual bool is_eog_token(int32_t token) = 0;
    virtual std::string detokenize_bytes(const int32_t * tokens, size_t n, bool unparse_special) = 0;
    virtual uint32_t context_size() = 0;
    virtual uint32_t vocab_size() = 0;
    // backend.rs:67-77
    virtual KvCacheKey cache_key() {
        const uint64_t fingerprint = model_fingerprint();
        const uint64_t version = weights_version();
        const EngineMemory m = memory();
        const bool unified = kv_unified();
        uint64_t settings = mix(0x9e3779b97f4a7c15ull, m.cells_total);
        settings = mix(settings, (uint64_t)m.n_slots);
        settings = mix(settings, unified ? 1u : 0u);
        settings = mix(settings, (uint64_t)context_size());
        return KvCacheKey{fingerprint, version, settings};
    }
    virtual void load_adapter(const std::string &, const std::string &) {
        throw InferError::failed("this backend does not support named adapters");
    }
    virtual void activate_adapter(const std::optional<std::string> & name) {
        if (name) throw InferError::failed("this backend does not support named adapters");
    }
    virtual std::optional<std::string> active_adapter() { return std::nullopt; }
    virtual bool supports_row_adapters() { return false; }
    virtual int32_t load_row_adapter(const std::string &, float) {
        throw InferError::failed("this backend does not support per-row adapters");
    }
    virtual void unload_row_adapter(int32_t) {
        throw InferError::failed("this backend does not support per-row adapters");
    }
    virtual AdapterRowsInfo adapter_rows_info() { return AdapterRowsInfo(); }
};

}  // namespace sched
