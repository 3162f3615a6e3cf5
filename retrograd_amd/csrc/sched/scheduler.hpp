// The step scheduler: one step at a time - admit, compose, execute, emit,
// remove (reference crates/retrograd-infer/src/scheduler.rs). The plan of every
// step comes from here; its execution belongs to the DecodeBackend, a single
// decode per step. This is the synchronous driver of the reference
// (`Scheduler::submit` / `pump` / `run_until_idle`, scheduler.rs:684-815); the
// actor thread and its inbox are not part of the step path and are not built.
#pragma once

#include <chrono>
#include <deque>
#include <memory>
#include <optional>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "detok.hpp"
#include "prefix_tree.hpp"
#include "types.hpp"

namespace sched {

enum class AdmissionMode : int { Lockstep = 0, Continuous = 1 };

// scheduler.rs:86-135
struct SchedulerOptions {
    AdmissionMode mode = AdmissionMode::Lockstep;
    size_t n_batch = 512;
    size_t queue_capacity = 64;
    size_t event_capacity = 64;
    std::chrono::nanoseconds slow_client_timeout = std::chrono::seconds(5);
    bool prefix_cache = true;
    size_t min_prefix_len = 8;
    uint64_t max_snapshot_bytes = 256ull << 20;
    size_t swap_min_tokens = 256;
    size_t max_retained = 8;
    std::chrono::nanoseconds retain_ttl = std::chrono::seconds(300);
};

struct SchedulerStats {
    KvStats kv;
    EngineMemory memory;
    size_t queued = 0, live = 0;
    std::optional<std::string> adapter;
    std::vector<std::string> row_adapters;
    AdapterRowsInfo adapter_rows;
};

// The order of a lockstep wave: prompt length, prompt tokens, then the sampling
// parameters (scheduler.rs:260-293). Negative, zero or positive.
int sampling_cmp(const SamplingParamsV2 & a, const SamplingParamsV2 & b);
int canonical_cmp(const Request & a, const Request & b);

class Scheduler {
public:
    Scheduler(std::unique_ptr<DecodeBackend> backend, SchedulerOptions options);

    // One-time pool setup: reads the geometry and clears every slot.
    void initialize();
    // Queues one request; the returned stream carries its events. Throws
    // InferError (Invalid, QueueFull).
    StreamRef submit(Request request);
    // One iteration: remove cancelled sequences, admit, compose and execute one
    // step, emit, remove finished sequences. Returns whether it made progress.
    // A failed step fails every live request and is rethrown.
    bool pump();
    void run_until_idle();

    size_t queued_len() const { return queue_.size(); }
    size_t queue_capacity() const { return options_.queue_capacity; }
    size_t live_len() const;
    bool is_idle() const { return queue_.empty() && live_.empty(); }
    void fail_queued();

    KvStats kv_stats() const;
    SchedulerStats stats();
    // One pool slot outside the bookkeeping, for host work between waves: a slot that no live sequence and no
    // dormant prefix holds, with `cells` of the pool left beside the dormant prefixes; least recently used
    // prefix nodes are evicted until both fit. -1 when nothing more can be evicted. Only while no sequence
    // is live (throws otherwise); the caller leaves the slot empty before the next pump. scheduler.rs:746-777
    int32_t lend_slot(uint64_t cells);
    PinId pin_prefix(const std::vector<int32_t> & prefix);
    bool unpin(PinId id) { return kv_.unpin(id); }
    void load_adapter(const std::string & name, const std::string & path);
    void unload_adapter(const std::string & name);

    DecodeBackend & backend() { return *backend_; }
    const SchedulerOptions & options() const { return options_; }
    void set_mode(AdmissionMode mode) { options_.mode = mode; }

private:
    struct Queued {
        Request request;
        Sender events;
    };
    enum class Phase { Prefill, Terminal, Decode };
    struct LiveMember {
        int32_t slot = 0;
        int32_t request_id = 0;
        size_t index = 0;
        SamplingParamsV2 sampling;
        bool want_logprob = false;
        size_t limit = 0;
        uint64_t reserved_share = 0;
        size_t generated = 0;
        int32_t next_token = 0;
        std::vector<int32_t> history;
        bool live = true;
        uint32_t n_top_logprobs = 0;
        bool unparse_special = false;
        Detokenizer detok;
        Sender events;
        StreamRef cancel;                 // the request's stream: carries the cancellation flag
        std::optional<Retention> retention;
    };
    struct LiveGroup {
        std::vector<int32_t> prompt;
        RowAdapter adapter = kAdapterContext;
        size_t prefix_end = 0;
        size_t leader = 0;
        uint64_t reserved = 0;
        size_t cache_hit = 0;
        std::vector<LiveMember> members;
        Phase phase = Phase::Prefill;
        size_t phase_pos = 0;             // Prefill: pos; Terminal: next
    };
    struct RowKind {
        enum Kind { Decode, Prefill, Terminal } kind;
        size_t group = 0, member = 0, end = 0;
        bool has_sampled_member = false;
    };
    struct Retained {
        PinId pin;
        std::chrono::steady_clock::time_point since;
        uint64_t order;
    };
    struct Composed {
        std::vector<StepRow> rows;
        std::vector<RowKind> kinds;
        uint64_t total_tokens = 0;
    };

    bool step_once();
    Composed compose();
    void advance_phases();
    void admit();
    void admit_candidates(size_t n_ctx_seq);
    std::pair<size_t, uint64_t> capacity();
    struct Fit { size_t members; uint64_t need; std::optional<size_t> node; };
    std::optional<Fit> front_fits(size_t n_ctx_seq, size_t held_slots, uint64_t held_cells, size_t & evictions_left);
    bool evict_one_lru();
    std::optional<std::pair<size_t, size_t>> hit_candidate(Namespace ns, const std::vector<int32_t> & prompt);
    size_t apply_cache_hit(Namespace ns, const std::vector<int32_t> & prompt, int32_t leader_slot);
    void admit_group(std::vector<Queued> group, size_t n_ctx_seq);
    void emit_sampled(size_t group, size_t member, const StepOutRow & produced, size_t row_index);
    void finish_member(size_t group, size_t member, FinishReason reason);
    void remove_cancelled();
    void rollback(const std::vector<RowKind> & kinds);
    InferError classify_step_error(const InferError & error, uint64_t needed);
    void fail_all(const InferError & error);
    void refresh_key();
    void retain(const std::string & key, size_t node);
    bool release_retained(const std::string & key);
    bool release_oldest_retained();
    void release_expired_retained();
    void release_retired();
    RowAdapter row_adapter(const Request & request) const;
    std::optional<std::string> serial_adapter(const Request & request) const;
    void ensure_adapter(const std::optional<std::string> & wanted);
    bool send_bounded(Stream & events, Event event);
    void drop_dead_groups();

    std::unique_ptr<DecodeBackend> backend_;
    SchedulerOptions options_;
    std::deque<Queued> queue_;
    std::vector<LiveGroup> live_;
    size_t n_slots_ = 0;
    int32_t next_request_id_ = 1;
    StepOutput out_;
    std::vector<int32_t> scratch_;
    size_t decode_cursor_ = 0;
    bool prefill_turn_ = false;
    PrefixTree kv_;
    std::optional<KvCacheKey> kv_key_;
    KvStats kv_stats_;
    std::unordered_map<std::string, Retained> retained_;
    uint64_t retained_order_ = 0;
    std::optional<std::string> active_adapter_;
    std::unordered_map<std::string, int32_t> row_adapters_;
    std::vector<int32_t> retiring_;
    std::unordered_set<std::string> unloaded_adapters_;
};

}  // namespace sched
