#include "scheduler.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>

namespace sched {

namespace {

constexpr size_t kMaxStalledPumps = 1024;     // scheduler.rs:44

// f32::total_cmp: the IEEE total order, through the sign-magnitude to
// two's-complement transform of the bits.
int total_cmp(float a, float b) {
    int32_t x, y;
    std::memcpy(&x, &a, 4);
    std::memcpy(&y, &b, 4);
    x ^= (int32_t)((uint32_t)(x >> 31) >> 1);
    y ^= (int32_t)((uint32_t)(y >> 31) >> 1);
    return x < y ? -1 : (x > y ? 1 : 0);
}
template <typename T> int cmp(const T & a, const T & b) { return a < b ? -1 : (b < a ? 1 : 0); }

// scheduler.rs:239-255
std::optional<uint64_t> member_need(size_t prompt_len, const SamplingParamsV2 & sampling, size_t n_ctx_seq) {
    if (prompt_len >= n_ctx_seq) return std::nullopt;
    const size_t budget = std::min<size_t>(sampling.max_new_tokens, n_ctx_seq - prompt_len);
    return (uint64_t)(prompt_len + budget);
}

uint64_t sat_add(uint64_t a, uint64_t b) { return a > UINT64_MAX - b ? UINT64_MAX : a + b; }
uint64_t sat_sub(uint64_t a, uint64_t b) { return a > b ? a - b : 0; }

uint64_t reservation(const Request & request, size_t n_ctx_seq) {
    uint64_t sum = 0;
    for (const SamplingParamsV2 & sampling : request.sampling)
        sum = sat_add(sum, member_need(request.prompt.size(), sampling, n_ctx_seq).value_or(0));
    return sum;
}

// The prefix-tree namespace of an adapter (scheduler.rs:386-396).
Namespace namespace_of(RowAdapter adapter) {
    if (adapter > 0) return (Namespace)adapter;
    if (adapter == kAdapterContext) return 0;
    return UINT64_MAX;
}

Event error_event(const InferError & e) {
    Event ev;
    ev.type = Event::Error;
    // a broadcast error is a clone: the backend's own error type does not
    // clone and arrives as Failed (error.rs:43-60)
    ev.error_kind = e.kind == ErrKind::Backend ? ErrKind::Failed : e.kind;
    ev.error_message = e.what();
    ev.error_needed = e.needed;
    ev.error_available = e.available;
    return ev;
}

}  // namespace

// request.rs:101-169
void Request::validate() const {
    if (prompt.empty()) throw InferError::invalid("a request requires a non-empty prompt");
    if (sampling.empty()) throw InferError::invalid("a request requires at least one sampling entry");
    for (const SamplingParamsV2 & p : sampling)
        if (p.max_new_tokens == 0) throw InferError::invalid("max_new_tokens must be greater than zero");
    for (const SamplingParamsV2 & p : sampling)
        if (!std::isfinite(p.temperature) || p.temperature <= 0.0f)
            throw InferError::invalid("temperature must be finite and greater than zero");
    for (const SamplingParamsV2 & p : sampling)
        if (!(p.top_p > 0.0f && p.top_p <= 1.0f)) throw InferError::invalid("top_p must be in (0, 1]");
    for (const SamplingParamsV2 & p : sampling) {
        bool bad = !std::isfinite(p.min_p) || p.min_p < 0.0f || p.min_p > 1.0f || !std::isfinite(p.repeat_penalty)
                || p.repeat_penalty <= 0.0f || !std::isfinite(p.frequency_penalty) || !std::isfinite(p.presence_penalty);
        for (const auto & b : p.logit_bias) bad = bad || !std::isfinite(b.second);
        if (bad)
            throw InferError::invalid(
                "min_p must be in [0, 1], repeat_penalty finite and > 0, frequency/presence penalties and logit biases finite");
    }
    for (const SamplingParamsV2 & p : sampling)
        if (p.logit_bias.size() > 4096) throw InferError::invalid("logit_bias takes at most 4096 entries");
    for (const std::string & s : stop)
        if (s.empty()) throw InferError::invalid("stop strings must not be empty");
    if (adapter && adapter->empty()) throw InferError::invalid("an adapter name must not be empty");
    if (retention && retention->key.empty()) throw InferError::invalid("a retention key must not be empty");
}

// scheduler.rs:269-293
int sampling_cmp(const SamplingParamsV2 & a, const SamplingParamsV2 & b) {
    int c;
    if ((c = cmp(a.seed, b.seed))) return c;
    if ((c = cmp(a.max_new_tokens, b.max_new_tokens))) return c;
    if ((c = total_cmp(a.temperature, b.temperature))) return c;
    if ((c = total_cmp(a.top_p, b.top_p))) return c;
    if ((c = cmp(a.top_k, b.top_k))) return c;
    if ((c = total_cmp(a.min_p, b.min_p))) return c;
    if ((c = total_cmp(a.repeat_penalty, b.repeat_penalty))) return c;
    if ((c = total_cmp(a.frequency_penalty, b.frequency_penalty))) return c;
    if ((c = total_cmp(a.presence_penalty, b.presence_penalty))) return c;
    if ((c = cmp(a.penalty_window, b.penalty_window))) return c;
    const size_t n = std::min(a.logit_bias.size(), b.logit_bias.size());
    for (size_t i = 0; i < n; ++i) {
        if ((c = cmp(a.logit_bias[i].first, b.logit_bias[i].first))) return c;
        uint32_t x, y;
        std::memcpy(&x, &a.logit_bias[i].second, 4);
        std::memcpy(&y, &b.logit_bias[i].second, 4);
        if ((c = cmp(x, y))) return c;
    }
    if ((c = cmp(a.logit_bias.size(), b.logit_bias.size()))) return c;
    if (a.grammar_gbnf.has_value() != b.grammar_gbnf.has_value()) return a.grammar_gbnf.has_value() ? 1 : -1;
    if (a.grammar_gbnf) {
        const int s = a.grammar_gbnf->compare(*b.grammar_gbnf);
        return s < 0 ? -1 : (s > 0 ? 1 : 0);
    }
    return 0;
}

// scheduler.rs:260-267
int canonical_cmp(const Request & a, const Request & b) {
    int c;
    if ((c = cmp(a.prompt.size(), b.prompt.size()))) return c;
    if (a.prompt < b.prompt) return -1;
    if (b.prompt < a.prompt) return 1;
    return sampling_cmp(a.sampling[0], b.sampling[0]);
}

Scheduler::Scheduler(std::unique_ptr<DecodeBackend> backend, SchedulerOptions options)
    : backend_(std::move(backend)), options_(options) {
    options_.queue_capacity = std::max<size_t>(options_.queue_capacity, 1);
    scratch_.reserve(std::max<size_t>(options_.n_batch, 1));
}

// scheduler.rs:300-319: try_send in a loop until the deadline, so a full stream
// costs at most the timeout of bounded backpressure.
bool Scheduler::send_bounded(Stream & events, Event event) {
    const auto started = std::chrono::steady_clock::now();
    for (;;) {
        if (!events.receiver_alive) return false;
        if (events.queue.size() < events.capacity) {
            events.queue.push_back(std::move(event));
            return true;
        }
        if (std::chrono::steady_clock::now() - started >= options_.slow_client_timeout) return false;
        std::this_thread::sleep_for(std::chrono::milliseconds(1));
    }
}

KvStats Scheduler::kv_stats() const {
    KvStats s = kv_stats_;
    s.nodes = kv_.node_count();
    s.resident_slots = kv_.resident_slot_count();
    s.snapshot_bytes = kv_.snapshot_bytes();
    return s;
}

SchedulerStats Scheduler::stats() {
    SchedulerStats s;
    s.kv = kv_stats();
    try { s.memory = backend_->memory(); } catch (const InferError &) { s.memory = EngineMemory(); }
    s.queued = queue_.size();
    s.live = live_len();
    s.adapter = active_adapter_;
    for (const auto & kv : row_adapters_) s.row_adapters.push_back(kv.first);
    std::sort(s.row_adapters.begin(), s.row_adapters.end());
    try { s.adapter_rows = backend_->adapter_rows_info(); } catch (const InferError &) { s.adapter_rows = AdapterRowsInfo(); }
    return s;
}

// scheduler.rs:454-483
void Scheduler::load_adapter(const std::string & name, const std::string & path) {
    if (name.empty()) throw InferError::invalid("an adapter name must not be empty");
    if (backend_->supports_row_adapters()) {
        bool loaded = false;
        int32_t id = 0;
        try {
            id = backend_->load_row_adapter(path, 1.0f);
            loaded = true;
        } catch (const InferError &) {
        }
        if (loaded) {
            unloaded_adapters_.erase(name);
            auto it = row_adapters_.find(name);
            if (it != row_adapters_.end()) {
                const int32_t old = it->second;
                it->second = id;
                retiring_.push_back(old);
                release_retired();
            } else {
                row_adapters_[name] = id;
            }
            return;
        }
    }
    backend_->load_adapter(name, path);
    unloaded_adapters_.erase(name);
    auto it = row_adapters_.find(name);
    if (it != row_adapters_.end()) {
        retiring_.push_back(it->second);
        row_adapters_.erase(it);
        release_retired();
    }
}

void Scheduler::unload_adapter(const std::string & name) {
    auto it = row_adapters_.find(name);
    if (it == row_adapters_.end()) throw InferError::invalid("no per-row adapter is loaded under '" + name + "'");
    const int32_t id = it->second;
    row_adapters_.erase(it);
    unloaded_adapters_.insert(name);
    retiring_.push_back(id);
    release_retired();
}

// scheduler.rs:500-517
void Scheduler::release_retired() {
    size_t index = 0;
    while (index < retiring_.size()) {
        const int32_t id = retiring_[index];
        bool in_use = false;
        for (const LiveGroup & g : live_) in_use = in_use || g.adapter == id;
        if (in_use) {
            ++index;
            continue;
        }
        for (int32_t slot : kv_.drop_namespace(namespace_of(id))) backend_->seq_rm(slot, -1, -1);
        backend_->unload_row_adapter(id);
        retiring_[index] = retiring_.back();
        retiring_.pop_back();
    }
}

RowAdapter Scheduler::row_adapter(const Request & request) const {
    if (request.adapter) {
        auto it = row_adapters_.find(*request.adapter);
        if (it != row_adapters_.end()) return it->second;
    }
    return kAdapterContext;
}

std::optional<std::string> Scheduler::serial_adapter(const Request & request) const {
    if (request.adapter && row_adapters_.find(*request.adapter) == row_adapters_.end()) return request.adapter;
    return std::nullopt;
}

void Scheduler::ensure_adapter(const std::optional<std::string> & wanted) {
    const std::optional<std::string> current = backend_->active_adapter();
    if (current != wanted) {
        backend_->activate_adapter(wanted);
        active_adapter_ = wanted;
        refresh_key();
    }
}

PinId Scheduler::pin_prefix(const std::vector<int32_t> & prefix) {
    refresh_key();
    const auto pin = kv_.pin_at(0, prefix.data(), prefix.size());
    if (!pin) throw InferError::invalid("no resident prefix node at exactly that token path");
    return *pin;
}

// scheduler.rs:548-560
void Scheduler::refresh_key() {
    const KvCacheKey key = backend_->cache_key();
    if (!kv_key_ || !(*kv_key_ == key)) {
        for (int32_t slot : kv_.clear()) backend_->seq_rm(slot, -1, -1);
        retained_.clear();
        kv_key_ = key;
    }
}

// scheduler.rs:564-582
void Scheduler::retain(const std::string & key, size_t node) {
    auto it = retained_.find(key);
    if (it != retained_.end()) {
        kv_.unpin(it->second.pin);
        retained_.erase(it);
    }
    const size_t cap = std::min(options_.max_retained, n_slots_ / 4);
    if (cap == 0) return;
    while (retained_.size() >= cap && release_oldest_retained()) {}
    const PinId pin = kv_.pin_node(node);
    retained_[key] = Retained{pin, std::chrono::steady_clock::now(), retained_order_++};
}

bool Scheduler::release_retained(const std::string & key) {
    auto it = retained_.find(key);
    if (it == retained_.end()) return false;
    const PinId pin = it->second.pin;
    retained_.erase(it);
    return kv_.unpin(pin);
}

bool Scheduler::release_oldest_retained() {
    const std::string * oldest = nullptr;
    const Retained * best = nullptr;
    for (const auto & kv : retained_) {
        if (!best || kv.second.since < best->since || (kv.second.since == best->since && kv.second.order < best->order)) {
            best = &kv.second;
            oldest = &kv.first;
        }
    }
    if (!oldest) return false;
    const std::string key = *oldest;
    return release_retained(key);
}

void Scheduler::release_expired_retained() {
    const auto now = std::chrono::steady_clock::now();
    for (auto it = retained_.begin(); it != retained_.end();) {
        if (now - it->second.since < options_.retain_ttl) {
            ++it;
        } else {
            kv_.unpin(it->second.pin);
            it = retained_.erase(it);
        }
    }
}

void Scheduler::fail_queued() {
    while (!queue_.empty()) {
        Queued q = std::move(queue_.front());
        queue_.pop_front();
        q.events->try_send(error_event(InferError::cancelled()));
    }
}

// scheduler.rs:665-680
void Scheduler::initialize() {
    const EngineMemory memory = backend_->memory();
    if (memory.n_slots > (uint32_t)INT32_MAX) throw InferError::overflow("backend slot count exceeds signed native IDs");
    n_slots_ = memory.n_slots;
    for (size_t slot = 0; slot < n_slots_; ++slot) backend_->seq_rm((int32_t)slot, -1, -1);
    active_adapter_ = backend_->active_adapter();
}

// scheduler.rs:687-707
StreamRef Scheduler::submit(Request request) {
    request.validate();
    if (queue_.size() >= options_.queue_capacity) throw InferError::queue_full(options_.queue_capacity);
    auto stream = std::make_shared<Stream>();
    stream->capacity = std::max(options_.event_capacity, request.n() + 2);
    Queued q;
    q.request = std::move(request);
    q.events = Sender(stream);
    queue_.push_back(std::move(q));
    return stream;
}

size_t Scheduler::live_len() const {
    size_t n = 0;
    for (const LiveGroup & g : live_)
        for (const LiveMember & m : g.members) n += m.live ? 1 : 0;
    return n;
}

// scheduler.rs:736-745
bool Scheduler::pump() {
    const size_t q0 = queue_.size(), l0 = live_len();
    try {
        const bool stepped = step_once();
        return stepped || queue_.size() != q0 || live_len() != l0;
    } catch (const InferError & error) {
        fail_all(error);
        throw;
    }
}

// scheduler.rs:755-777
int32_t Scheduler::lend_slot(uint64_t cells) {
    if (!live_.empty()) throw InferError::failed("a slot can only be lent while no sequence is live");
    for (;;) {
        const auto cap = capacity();
        if (cap.first > 0 && cap.second >= cells) {
            std::vector<bool> held(n_slots_, false);
            for (int32_t slot : kv_.resident_slots())
                if (slot >= 0 && (size_t)slot < held.size()) held[(size_t)slot] = true;
            for (size_t slot = 0; slot < held.size(); ++slot)
                if (!held[slot]) return (int32_t)slot;
            return -1;
        }
        if (!evict_one_lru()) return -1;
    }
}

// scheduler.rs:783-789
void Scheduler::run_until_idle() {
    size_t stalled = 0;
    while (!is_idle()) {
        if (pump()) {
            stalled = 0;
        } else if (++stalled > kMaxStalledPumps) {
            throw InferError::failed("the scheduler made no progress with requests still queued");
        }
    }
}

void Scheduler::drop_dead_groups() {
    live_.erase(std::remove_if(live_.begin(), live_.end(), [](const LiveGroup & g) {
        for (const LiveMember & m : g.members) if (m.live) return false;
        return true;
    }), live_.end());
}

// scheduler.rs:851-921
bool Scheduler::step_once() {
    queue_.erase(std::remove_if(queue_.begin(), queue_.end(), [](const Queued & q) { return q.events->cancelled; }),
                 queue_.end());
    remove_cancelled();
    if (!retiring_.empty()) release_retired();
    admit();
    advance_phases();
    if (live_.empty()) return false;
    Composed plan = compose();
    if (plan.rows.empty()) return false;
    try {
        backend_->step(plan.rows, out_);
    } catch (const InferError & error) {
        // A failed step may have made a prefix of the submitted tokens resident:
        // clear every touched slot before reporting.
        const InferError classified = classify_step_error(error, plan.total_tokens);
        rollback(plan.kinds);
        throw classified;
    }
    for (size_t index = 0; index < plan.kinds.size(); ++index) {
        const RowKind & kind = plan.kinds[index];
        switch (kind.kind) {
            case RowKind::Decode:
                emit_sampled(kind.group, kind.member, out_.row(index), index);
                break;
            case RowKind::Terminal: {
                emit_sampled(kind.group, kind.member, out_.row(index), index);
                LiveGroup & g = live_[kind.group];
                if (g.phase == Phase::Terminal) {
                    g.phase_pos = std::max(g.phase_pos, kind.member + 1);
                    if (g.phase_pos >= g.members.size()) g.phase = Phase::Decode;
                }
                break;
            }
            case RowKind::Prefill: {
                LiveGroup & g = live_[kind.group];
                if (g.phase == Phase::Prefill) g.phase_pos = kind.end;
                if (kind.has_sampled_member) emit_sampled(kind.group, kind.member, out_.row(index), index);
                break;
            }
        }
    }
    drop_dead_groups();
    if (!retiring_.empty()) release_retired();
    return true;
}

// scheduler.rs:933-1089
Scheduler::Composed Scheduler::compose() {
    const size_t n_batch = std::max<size_t>(options_.n_batch, 1);
    size_t used = 0;
    Composed plan;
    scratch_.clear();

    bool prefill_active = false;
    for (const LiveGroup & g : live_) prefill_active = prefill_active || g.phase != Phase::Decode;
    const bool allow_decode = options_.mode == AdmissionMode::Continuous || !prefill_active;

    // Pass 1: pick the decode rows and stage their tokens.
    std::vector<std::pair<size_t, size_t>> decode_list;
    if (allow_decode) {
        for (size_t gi = 0; gi < live_.size(); ++gi) {
            if (live_[gi].phase != Phase::Decode) continue;
            for (size_t mi = 0; mi < live_[gi].members.size(); ++mi)
                if (live_[gi].members[mi].live) decode_list.emplace_back(gi, mi);
        }
    }
    // Reserve progress for prefill even when decodes fill the batch; rotate the
    // decoding members when more than fit in one step.
    size_t decode_budget;
    if (options_.mode == AdmissionMode::Continuous && prefill_active) {
        if (n_batch == 1) {
            prefill_turn_ = !prefill_turn_;
            decode_budget = prefill_turn_ ? 0 : 1;
        } else {
            decode_budget = n_batch - 1;
        }
    } else {
        decode_budget = n_batch;
    }
    if (!decode_list.empty()) {
        const size_t start = decode_cursor_ % decode_list.size();
        std::rotate(decode_list.begin(), decode_list.begin() + (ptrdiff_t)start, decode_list.end());
        const size_t count = std::min(decode_budget, decode_list.size());
        decode_cursor_ = (start + count) % decode_list.size();
        decode_list.resize(count);
    }
    // scratch_ must not reallocate once rows point into it
    scratch_.reserve(decode_list.size());
    for (const auto & gm : decode_list) scratch_.push_back(live_[gm.first].members[gm.second].next_token);
    used += decode_list.size();
    auto position = [](size_t pos) -> int32_t {
        if (pos > (size_t)INT32_MAX) throw InferError::overflow("a step position does not fit i32");
        return (int32_t)pos;
    };
    // Pass 2: build the rows.
    for (size_t offset = 0; offset < decode_list.size(); ++offset) {
        const LiveGroup & group = live_[decode_list[offset].first];
        const LiveMember & member = group.members[decode_list[offset].second];
        StepRow row;
        row.request = member.request_id;
        row.slot = member.slot;
        row.tokens = scratch_.data() + offset;
        row.n = 1;
        row.pos0 = position(group.prompt.size() + member.generated - 1);
        row.sample = true;
        row.sampling = &member.sampling;
        row.n_top_logprobs = member.n_top_logprobs;
        row.want_logprob = member.want_logprob;
        row.adapter = group.adapter;
        plan.rows.push_back(row);
        RowKind kind{RowKind::Decode, decode_list[offset].first, decode_list[offset].second, 0, false};
        plan.kinds.push_back(kind);
    }
    for (size_t gi = 0; gi < live_.size(); ++gi) {
        if (used >= n_batch) break;
        const LiveGroup & group = live_[gi];
        if (group.phase == Phase::Prefill) {
            const size_t pos = group.phase_pos;
            const size_t remaining = n_batch - used;
            const size_t chunk = std::min(remaining, group.prefix_end - pos);
            if (chunk == 0) continue;
            const size_t end = pos + chunk;
            const bool single = group.members.size() == 1;
            const bool sampled = single && end == group.prompt.size();
            const LiveMember & leader = group.members[group.leader];
            StepRow row;
            row.request = leader.request_id;
            row.slot = leader.slot;
            row.tokens = group.prompt.data() + pos;
            row.n = (uint32_t)chunk;
            row.pos0 = position(pos);
            row.sample = sampled;
            row.sampling = &leader.sampling;
            row.n_top_logprobs = sampled ? leader.n_top_logprobs : 0;
            row.want_logprob = sampled && leader.want_logprob;
            row.adapter = group.adapter;
            plan.rows.push_back(row);
            RowKind kind{RowKind::Prefill, gi, 0, end, sampled};
            plan.kinds.push_back(kind);
            used += chunk;
        } else if (group.phase == Phase::Terminal) {
            const size_t last = group.prompt.size() - 1;
            size_t mi = group.phase_pos;
            while (mi < group.members.size() && used < n_batch) {
                const LiveMember & member = group.members[mi];
                if (!member.live) {
                    ++mi;
                    continue;
                }
                StepRow row;
                row.request = member.request_id;
                row.slot = member.slot;
                row.tokens = group.prompt.data() + last;
                row.n = 1;
                row.pos0 = position(last);
                row.sample = true;
                row.sampling = &member.sampling;
                row.n_top_logprobs = member.n_top_logprobs;
                row.want_logprob = member.want_logprob;
                row.adapter = group.adapter;
                plan.rows.push_back(row);
                RowKind kind{RowKind::Terminal, gi, mi, 0, false};
                plan.kinds.push_back(kind);
                used += 1;
                ++mi;
            }
        }
    }
    plan.total_tokens = used;
    return plan;
}

// scheduler.rs:1094-1121
void Scheduler::advance_phases() {
    for (size_t gi = 0; gi < live_.size(); ++gi) {
        LiveGroup & g = live_[gi];
        const bool done = g.phase == Phase::Prefill && g.phase_pos == g.prefix_end;
        if (done) {
            if (g.members.size() > 1) {
                const int32_t leader_slot = g.members[g.leader].slot;
                std::vector<int32_t> slots;
                for (const LiveMember & m : g.members)
                    if (m.live && m.slot != leader_slot) slots.push_back(m.slot);
                if (g.prefix_end > 0)
                    for (int32_t slot : slots) backend_->seq_cp(leader_slot, slot, -1, -1);
                g.phase = Phase::Terminal;
                g.phase_pos = 0;
            } else {
                g.phase = Phase::Decode;
            }
        } else if (g.phase == Phase::Terminal) {
            bool none_live = true;
            for (size_t mi = g.phase_pos; mi < g.members.size(); ++mi) none_live = none_live && !g.members[mi].live;
            if (none_live) g.phase = Phase::Decode;
        }
    }
}

// scheduler.rs:1124-1268
void Scheduler::admit() {
    if (queue_.empty()) return;
    refresh_key();
    release_expired_retained();
    while (kv_.snapshot_bytes() > options_.max_snapshot_bytes) {
        const auto node = kv_.snapshot_eviction_candidate();
        if (!node) break;
        kv_.remove(*node);
        kv_stats_.evictions += 1;
    }
    const size_t n_ctx_seq = backend_->context_size();
    const size_t vocab = backend_->vocab_size();
    const EngineMemory memory = backend_->memory();
    n_slots_ = memory.n_slots;
    const uint64_t cells_total = memory.cells_total;

    // Refuse what can never fit: an impossible reservation is an error, not a wait.
    size_t index = 0;
    while (index < queue_.size()) {
        const Request & r = queue_[index].request;
        const bool prompt_too_long = r.prompt.size() >= n_ctx_seq;
        const bool too_many_members = r.n() > n_slots_;
        const bool top_too_wide = (size_t)r.n_top_logprobs > vocab;
        bool invalid_token = false;
        for (int32_t t : r.prompt) invalid_token = invalid_token || t < 0 || (size_t)t >= vocab;
        bool invalid_bias = false;
        for (const SamplingParamsV2 & p : r.sampling)
            for (const auto & b : p.logit_bias) invalid_bias = invalid_bias || b.first < 0 || (size_t)b.first >= vocab;
        const uint64_t need = reservation(r, n_ctx_seq);
        if (prompt_too_long || too_many_members || top_too_wide || invalid_token || invalid_bias || need > cells_total) {
            Queued q = std::move(queue_[index]);
            queue_.erase(queue_.begin() + (ptrdiff_t)index);
            std::string message;
            if (prompt_too_long) {
                message = "the prompt (" + std::to_string(q.request.prompt.size()) +
                          " tokens) leaves no room to generate in the per-sequence context (" + std::to_string(n_ctx_seq) + ")";
            } else if (too_many_members) {
                message = "the request asks for " + std::to_string(q.request.n()) + " completions but the pool has " +
                          std::to_string(n_slots_) + " slots";
            } else if (top_too_wide) {
                message = "n_top_logprobs exceeds the vocabulary (" + std::to_string(vocab) + ")";
            } else if (invalid_bias) {
                message = "logit_bias token ids must be in 0.." + std::to_string(vocab);
            } else if (invalid_token) {
                message = "prompt tokens must be in 0.." + std::to_string(vocab);
            } else {
                message = "the reservation (prompt + max_new_tokens = " + std::to_string(need) +
                          " cells) exceeds the KV pool of " + std::to_string(cells_total) + " cells";
            }
            q.events->try_send(error_event(InferError::invalid(message)));
            continue;
        }
        ++index;
    }
    if (queue_.empty()) return;

    for (auto it = queue_.begin(); it != queue_.end();) {
        if (it->request.adapter && unloaded_adapters_.count(*it->request.adapter)) {
            it->events->try_send(error_event(InferError::invalid("no adapter is loaded under '" + *it->request.adapter + "'")));
            it = queue_.erase(it);
        } else {
            ++it;
        }
    }
    if (queue_.empty()) return;

    // Serialized adapters partition the batch; per-row adapters can mix.
    const std::optional<std::string> target = live_.empty() ? serial_adapter(queue_.front().request) : active_adapter_;
    std::deque<Queued> candidates, rest;
    for (Queued & q : queue_) {
        if (serial_adapter(q.request) == target) candidates.push_back(std::move(q));
        else rest.push_back(std::move(q));
    }
    queue_.clear();
    if (live_.empty()) {
        try {
            ensure_adapter(target);
        } catch (const InferError & error) {
            while (!candidates.empty()) {
                candidates.front().events->try_send(error_event(error));
                candidates.pop_front();
            }
            queue_ = std::move(rest);
            return;
        }
    }
    queue_ = std::move(candidates);
    auto restore = [&]() {
        std::deque<Queued> leftover = std::move(queue_);
        queue_ = std::move(rest);
        for (Queued & q : leftover) queue_.push_back(std::move(q));
    };
    try {
        admit_candidates(n_ctx_seq);
    } catch (...) {
        restore();
        throw;
    }
    restore();
}

// scheduler.rs:1272-1338
void Scheduler::admit_candidates(size_t n_ctx_seq) {
    size_t evictions_left = n_slots_ + 1;
    if (options_.mode == AdmissionMode::Lockstep) {
        if (!live_.empty()) return;
        // Select the oldest fitting wave before sorting it; the node each
        // selected request hits is pinned until the wave is admitted.
        std::vector<Queued> pending;
        std::vector<PinId> wave_pins;
        size_t held_slots = 0;
        uint64_t held_cells = 0;
        while (auto fit = front_fits(n_ctx_seq, held_slots, held_cells, evictions_left)) {
            held_slots += fit->members;
            held_cells += fit->need;
            if (fit->node) wave_pins.push_back(kv_.pin_node(*fit->node));
            pending.push_back(std::move(queue_.front()));
            queue_.pop_front();
        }
        std::stable_sort(pending.begin(), pending.end(),
                         [](const Queued & a, const Queued & b) { return canonical_cmp(a.request, b.request) < 0; });
        std::exception_ptr failure;
        size_t at = 0;
        while (at < pending.size() && !failure) {
            size_t run_end = at + 1;
            while (run_end < pending.size() && pending[run_end].request.prompt == pending[at].request.prompt &&
                   pending[run_end].request.adapter == pending[at].request.adapter)
                ++run_end;
            std::vector<Queued> run;
            for (size_t i = at; i < run_end; ++i) run.push_back(std::move(pending[i]));
            at = run_end;
            try {
                admit_group(std::move(run), n_ctx_seq);
            } catch (...) {
                failure = std::current_exception();
            }
        }
        for (PinId pin : wave_pins) kv_.unpin(pin);
        if (failure) std::rethrow_exception(failure);
    } else {
        // Do not let smaller arrivals overtake a request waiting for several
        // slots or a larger cell reservation.
        while (front_fits(n_ctx_seq, 0, 0, evictions_left)) {
            std::vector<Queued> one;
            one.push_back(std::move(queue_.front()));
            queue_.pop_front();
            admit_group(std::move(one), n_ctx_seq);
        }
    }
}

// scheduler.rs:1345-1362
std::pair<size_t, uint64_t> Scheduler::capacity() {
    const EngineMemory memory = backend_->memory();
    const size_t used_slots = live_len() + kv_.resident_slot_count();
    uint64_t reserved = 0;
    for (const LiveGroup & g : live_) reserved += g.reserved;
    const uint64_t committed = std::max(memory.cells_used, sat_add(reserved, kv_.resident_cells()));
    return {n_slots_ > used_slots ? n_slots_ - used_slots : 0, sat_sub(memory.cells_total, committed)};
}

// scheduler.rs:1368-1404
std::optional<Scheduler::Fit> Scheduler::front_fits(size_t n_ctx_seq, size_t held_slots, uint64_t held_cells,
                                                    size_t & evictions_left) {
    for (;;) {
        if (queue_.empty()) return std::nullopt;
        const Request & request = queue_.front().request;
        const size_t members = request.n();
        // recomputed after every eviction: the evicted node may be the one the hit came from
        const Namespace ns = namespace_of(row_adapter(request));
        const auto hit = hit_candidate(ns, request.prompt);
        const uint64_t shared = hit ? (uint64_t)hit->second * (uint64_t)members : 0;
        const uint64_t need = sat_sub(reservation(request, n_ctx_seq), shared);
        const auto cap = capacity();
        if (held_slots + members <= cap.first && held_cells + need <= cap.second) {
            Fit fit{members, need, std::nullopt};
            if (hit) fit.node = hit->first;
            return fit;
        }
        if (evictions_left == 0) return std::nullopt;
        if (!evict_one_lru()) {
            // A retention is a hint: release the oldest and let the next pass evict it.
            if (!release_oldest_retained()) return std::nullopt;
            continue;
        }
        evictions_left -= 1;
    }
}

// scheduler.rs:1410-1437
bool Scheduler::evict_one_lru() {
    const auto candidate = kv_.eviction_candidate();
    if (!candidate) return false;
    const size_t node = *candidate;
    const int32_t slot = *kv_.slot(node);
    if (kv_.depth(node) >= options_.swap_min_tokens) {
        // a failed save only costs the swap: the node is dropped instead
        size_t save_len = 0;
        try { save_len = backend_->seq_save_len(slot, 0); } catch (const InferError &) { save_len = 0; }
        if (save_len > 0 && kv_.snapshot_bytes() + save_len <= options_.max_snapshot_bytes) {
            auto buffer = std::make_shared<std::vector<uint8_t>>(save_len);
            try {
                const size_t written = backend_->seq_save_into(slot, 0, buffer->data(), buffer->size());
                buffer->resize(written);
                kv_.attach_snapshot(node, buffer);
                kv_stats_.swaps += 1;
            } catch (const InferError &) {
            }
        }
    }
    backend_->seq_rm(slot, -1, -1);
    kv_.detach_slot(node);
    if (!kv_.snapshot(node)) kv_.remove(node);
    kv_stats_.evictions += 1;
    return true;
}

// scheduler.rs:1446-1485
std::optional<std::pair<size_t, size_t>> Scheduler::hit_candidate(Namespace ns, const std::vector<int32_t> & prompt) {
    if (!options_.prefix_cache || prompt.size() < 2) return std::nullopt;
    // A mid-sequence hit needs a partial-range copy: only on a unified pool and
    // only for a dense model.
    const bool partial_ok = backend_->kv_unified() && !backend_->is_hybrid();
    const size_t last = prompt.size() - 1;
    auto usable = [&](size_t node, size_t hit) -> bool {
        const size_t applied = std::min(hit, last);      // clamped to a strict prefix
        const size_t depth = kv_.depth(node);
        if (applied == 0 || (applied < depth && !partial_ok)) return false;
        if (const auto slot = kv_.slot(node)) {
            // the resident span must be frozen at the node's boundary
            try {
                const auto span = backend_->seq_pos(*slot);
                return span.first == 0 && span.second == (int32_t)depth - 1;
            } catch (const InferError &) {
                return false;
            }
        }
        // swapped node: restorable from its snapshot, but only at its exact boundary
        return kv_.snapshot(node) != nullptr && applied == depth;
    };
    const auto found = kv_.longest_prefix(ns, prompt.data(), prompt.size(), partial_ok, usable);
    if (!found) return std::nullopt;
    return std::make_pair(found->first, std::min(found->second, last));
}

// scheduler.rs:1491-1522
size_t Scheduler::apply_cache_hit(Namespace ns, const std::vector<int32_t> & prompt, int32_t leader_slot) {
    const auto found = hit_candidate(ns, prompt);
    if (!found) return 0;
    const size_t node = found->first, hit = found->second;
    const auto src = kv_.slot(node);
    if (src && hit == kv_.depth(node)) {
        backend_->seq_cp(*src, leader_slot, -1, -1);            // exact boundary: whole-slot copy
    } else if (src) {
        backend_->seq_cp(*src, leader_slot, 0, (int32_t)hit);   // mid-sequence: positions [0, hit)
    } else {
        const Snapshot snapshot = kv_.snapshot(node);           // swapped node at its exact boundary
        backend_->seq_load(leader_slot, 0, snapshot->data(), snapshot->size());
    }
    kv_.touch(node);
    return hit;
}

// scheduler.rs:1526-1650
void Scheduler::admit_group(std::vector<Queued> group, size_t n_ctx_seq) {
    const std::vector<int32_t> prompt = group[0].request.prompt;
    const RowAdapter adapter = row_adapter(group[0].request);
    size_t n_members = 0;
    for (const Queued & q : group) n_members += q.request.n();
    const size_t prefix_end = n_members > 1 ? prompt.size() - 1 : prompt.size();
    std::vector<LiveMember> members;
    members.reserve(n_members);
    // slots already taken, including the ones this group is taking
    std::vector<bool> used(n_slots_, false);
    for (const LiveGroup & g : live_)
        for (const LiveMember & m : g.members)
            if (m.live && (size_t)m.slot < n_slots_) used[(size_t)m.slot] = true;
    for (int32_t slot : kv_.resident_slots())
        if ((size_t)slot < n_slots_) used[(size_t)slot] = true;
    for (Queued & queued : group) {
        Request & request = queued.request;
        std::optional<Retention> retention = std::move(request.retention);
        for (size_t index = 0; index < request.sampling.size(); ++index) {
            size_t free_slot = 0;
            while (free_slot < used.size() && used[free_slot]) ++free_slot;
            if (free_slot >= used.size()) throw InferError::failed("admission checked the available slot count");
            used[free_slot] = true;
            const int32_t request_id = next_request_id_;
            // ids are reused only after wraparound, skipping all live ids
            auto bump = [&]() { next_request_id_ = next_request_id_ == INT32_MAX ? 1 : next_request_id_ + 1; };
            bump();
            auto taken = [&]() {
                for (const LiveGroup & g : live_)
                    for (const LiveMember & m : g.members)
                        if (m.live && m.request_id == next_request_id_) return true;
                for (const LiveMember & m : members)
                    if (m.live && m.request_id == next_request_id_) return true;
                return next_request_id_ == request_id;
            };
            while (taken()) bump();
            LiveMember member;
            member.slot = (int32_t)free_slot;
            member.request_id = request_id;
            member.index = index;
            member.sampling = request.sampling[index];
            member.want_logprob = request.logprobs || request.n_top_logprobs > 0;
            member.limit = std::min<size_t>(member.sampling.max_new_tokens, n_ctx_seq - prompt.size());
            member.n_top_logprobs = request.n_top_logprobs;
            member.unparse_special = request.unparse_special;
            member.detok = Detokenizer(request.stop);
            member.events = queued.events;
            member.cancel = queued.events.ref();
            if (retention) {
                member.retention = std::move(retention);
                retention.reset();
            }
            members.push_back(std::move(member));
        }
        queued.events.reset();
    }
    if (options_.mode == AdmissionMode::Lockstep) {
        std::vector<int32_t> slots;
        for (const LiveMember & m : members) slots.push_back(m.slot);
        std::sort(slots.begin(), slots.end());
        std::stable_sort(members.begin(), members.end(),
                         [](const LiveMember & a, const LiveMember & b) { return sampling_cmp(a.sampling, b.sampling) < 0; });
        for (size_t i = 0; i < members.size(); ++i) members[i].slot = slots[i];
    }
    // Prefix-cache hit into the leader's slot: the shared prefix is copied (or
    // restored from a snapshot) instead of prefilled.
    const int32_t leader_slot = members[0].slot;
    const size_t cache_hit = apply_cache_hit(namespace_of(adapter), prompt, leader_slot);
    const size_t prefill_from = std::min(cache_hit, prefix_end);
    uint64_t reserved = 0;
    for (LiveMember & m : members) {
        m.reserved_share = (uint64_t)((prompt.size() - cache_hit) + m.limit);
        reserved += m.reserved_share;
    }
    if (cache_hit > 0) kv_stats_.hits += 1;
    else kv_stats_.misses += 1;
    kv_stats_.prompt_cells += prompt.size();
    kv_stats_.prefilled_cells += prefix_end - prefill_from;
    LiveGroup g;
    g.prompt = prompt;
    g.adapter = adapter;
    g.prefix_end = prefix_end;
    g.leader = 0;
    g.reserved = reserved;
    g.cache_hit = cache_hit;
    g.members = std::move(members);
    g.phase = Phase::Prefill;
    g.phase_pos = prefill_from;
    live_.push_back(std::move(g));
}

// scheduler.rs:1654-1759
void Scheduler::emit_sampled(size_t group, size_t member, const StepOutRow & produced, size_t row_index) {
    if (live_[group].members[member].cancel->cancelled) {
        finish_member(group, member, FinishReason::Cancelled);
        return;
    }
    if (!produced.sampled) throw InferError::failed("a sampling step row produced no token");
    bool stopped = false, send_failed = false;
    {
        LiveMember & m = live_[group].members[member];
        m.generated += 1;
        m.next_token = produced.token;
        m.history.push_back(produced.token);
        // The EOG token is carried in the token events but contributes no text.
        std::string piece;
        if (!(m.unparse_special && backend_->is_eog_token(produced.token)))
            piece = backend_->detokenize_bytes(&produced.token, 1, m.unparse_special);
        auto pushed = m.detok.push_bytes(piece);
        Event ev;
        ev.type = Event::Token;
        ev.index = m.index;
        ev.token = produced.token;
        ev.logprob = produced.logprob;
        ev.has_sampled_logprob = m.want_logprob;
        ev.sampled_logprob = m.want_logprob ? produced.sampled_logprob : 0.0f;
        ev.forced = produced.forced;
        ev.text = std::move(pushed.first);
        ev.piece = piece;
        if (m.n_top_logprobs > 0) {
            for (size_t k = 0; k < produced.n_top; ++k) {
                TopLogprob top;
                top.token = out_.top_ids.at(row_index * out_.n_top_stride + k);
                top.logprob = out_.top_logprobs.at(row_index * out_.n_top_stride + k);
                try { top.piece = backend_->detokenize_bytes(&top.token, 1, m.unparse_special); } catch (const InferError &) {}
                ev.top_logprobs.push_back(std::move(top));
            }
        }
        stopped = pushed.second;
        send_failed = !send_bounded(*m.events.operator->(), std::move(ev));
    }
    std::optional<FinishReason> reason;
    if (send_failed) {
        reason = FinishReason::Cancelled;
    } else if (stopped) {
        reason = FinishReason::Stop;
    } else if (backend_->is_eog_token(produced.token)) {
        reason = FinishReason::Eog;
    } else {
        const LiveMember & m = live_[group].members[member];
        if (m.generated >= m.limit)
            reason = m.limit >= (size_t)m.sampling.max_new_tokens ? FinishReason::MaxTokens : FinishReason::ContextFull;
    }
    if (reason) finish_member(group, member, *reason);
}

// scheduler.rs:1763-1854
void Scheduler::finish_member(size_t group, size_t member, FinishReason reason) {
    const Namespace ns = namespace_of(live_[group].adapter);
    LiveGroup & g = live_[group];
    LiveMember & m = g.members[member];
    if (!m.live) return;
    g.reserved = sat_sub(g.reserved, m.reserved_share);
    m.live = false;
    const std::string text = m.detok.finish();
    std::vector<int32_t> path = g.prompt;
    path.insert(path.end(), m.history.begin(), m.history.end());
    const int32_t slot = m.slot, request_id = m.request_id;
    const size_t index = m.index;
    Sender events = std::move(m.events);
    std::optional<Retention> retention = std::move(m.retention);
    m.retention.reset();
    const size_t cached_tokens = g.cache_hit;
    // a timed-out stream is cancelled for every completion of its request
    if (reason == FinishReason::Cancelled) m.cancel->cancelled = true;
    if (reason != FinishReason::Cancelled) {
        Event ev;
        ev.type = Event::End;
        ev.index = index;
        ev.reason = reason;
        ev.text = text;
        ev.cached_tokens = cached_tokens;
        if (!send_bounded(*events.operator->(), std::move(ev))) m.cancel->cancelled = true;
    }
    // Hand the finished sequence's slot to the prefix tree as a dormant node
    // instead of releasing it. The node's depth is the resident span: the last
    // sampled token is never fed back. A span that does not start at 0 cannot be
    // shared from zero and is released.
    const auto span = backend_->seq_pos(slot);
    const size_t resident = span.first == 0 ? (size_t)(span.second + 1) : 0;
    std::optional<size_t> node;
    if (options_.prefix_cache && resident > 0 && resident >= options_.min_prefix_len && resident <= path.size()) {
        const auto inserted = kv_.insert(ns, path.data(), resident, slot);
        if (!inserted.second) backend_->seq_rm(slot, -1, -1);     // the exact path already has a node
        node = inserted.first;
    } else {
        backend_->seq_rm(slot, -1, -1);
    }
    backend_->request_free(request_id);
    if (retention && reason != FinishReason::Cancelled) {
        if (retention->release) release_retained(*retention->release);
        if (node) retain(retention->key, *node);
    }
}

// scheduler.rs:1857-1892
void Scheduler::remove_cancelled() {
    for (size_t group = 0; group < live_.size(); ++group) {
        // preserve a partially decoded shared prefix before returning its cancelled leader's slot
        LiveGroup & g = live_[group];
        if (g.phase == Phase::Prefill && g.members[g.leader].cancel->cancelled) {
            std::optional<size_t> replacement;
            for (size_t mi = 0; mi < g.members.size() && !replacement; ++mi)
                if (g.members[mi].live && !g.members[mi].cancel->cancelled) replacement = mi;
            if (replacement) {
                if (g.phase_pos > 0) backend_->seq_cp(g.members[g.leader].slot, g.members[*replacement].slot, -1, -1);
                g.leader = *replacement;
            }
        }
        std::vector<size_t> cancelled;
        for (size_t mi = 0; mi < live_[group].members.size(); ++mi)
            if (live_[group].members[mi].live && live_[group].members[mi].cancel->cancelled) cancelled.push_back(mi);
        for (size_t mi : cancelled) finish_member(group, mi, FinishReason::Cancelled);
    }
    drop_dead_groups();
}

// scheduler.rs:1896-1911
void Scheduler::rollback(const std::vector<RowKind> & kinds) {
    for (const RowKind & kind : kinds) {
        const size_t group = kind.group;
        const size_t member = kind.kind == RowKind::Prefill ? live_[group].leader : kind.member;
        const LiveMember & m = live_[group].members[member];
        try { backend_->seq_rm(m.slot, -1, -1); } catch (const InferError &) {}
        try { backend_->request_free(m.request_id); } catch (const InferError &) {}
    }
}

// scheduler.rs:1915-1926
InferError Scheduler::classify_step_error(const InferError & error, uint64_t needed) {
    if (error.kind == ErrKind::Backend) {
        try {
            const EngineMemory memory = backend_->memory();
            const uint64_t available = sat_sub(memory.cells_total, memory.cells_used);
            if (needed > available) return InferError::kv_full(needed, available);
        } catch (const InferError &) {
        }
    }
    return error;
}

// scheduler.rs:1931-1955
void Scheduler::fail_all(const InferError & error) {
    std::vector<std::pair<int32_t, int32_t>> to_release;
    for (LiveGroup & g : live_) {
        for (LiveMember & m : g.members) {
            if (!m.live) continue;
            if (m.events) {
                Sender events = std::move(m.events);
                send_bounded(*events.operator->(), error_event(error));
            }
            m.live = false;
            to_release.emplace_back(m.slot, m.request_id);
        }
    }
    for (const auto & sr : to_release) {
        try { backend_->seq_rm(sr.first, -1, -1); } catch (const InferError &) {}
        try { backend_->request_free(sr.second); } catch (const InferError &) {}
    }
    live_.clear();
}

}  // namespace sched
