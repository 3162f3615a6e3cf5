#include "fake_backend.hpp"

#include <algorithm>
#include <cstring>

namespace sched {

namespace {
constexpr uint32_t kPartialOnly = 1u;     // RETRO_STATE_SEQ_FLAGS_PARTIAL_ONLY
void put32(std::vector<uint8_t> & buf, uint32_t v) {
    for (int i = 0; i < 4; ++i) buf.push_back((uint8_t)(v >> (8 * i)));
}
uint32_t get32(const uint8_t * p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }
}  // namespace

FakeBackend::FakeBackend(uint32_t n_slots, uint32_t n_ctx_seq, uint64_t cells_total, uint32_t vocab, int32_t eos,
                         std::vector<std::string> pieces)
    : n_slots_(n_slots), n_ctx_seq_(n_ctx_seq), cells_total_(cells_total), vocab_(vocab), eos_(eos),
      pieces_(std::move(pieces)), slots_(n_slots) {}

void FakeBackend::register_adapter(const std::string & name, const std::string & path) {
    adapters_[name] = path;
    adapter_ops.emplace_back("load", name);
}

// fake.rs:153-173: activation clears the pool and bumps the weights version.
void FakeBackend::apply_adapter(const std::optional<std::string> & name) {
    if (!name) {
        active_adapter_.reset();
    } else if (adapters_.count(*name)) {
        active_adapter_ = *name;
    } else {
        throw InferError::invalid("no adapter registered under '" + *name + "'");
    }
    adapter_ops.emplace_back("activate", active_adapter_.value_or(""));
    for (auto & slot : slots_) slot.reset();
    bump_weights_version();
}

std::optional<std::vector<uint8_t>> FakeBackend::encode_snapshot(int32_t slot, uint32_t flags) const {
    if (slot < 0 || (size_t)slot >= slots_.size() || !slots_[(size_t)slot]) return std::nullopt;
    std::vector<uint8_t> buf;
    put32(buf, 0x5EED);
    put32(buf, flags);
    put32(buf, (uint32_t)slots_[(size_t)slot]->first);
    put32(buf, (uint32_t)slots_[(size_t)slot]->second);
    return buf;
}

uint64_t FakeBackend::cells_used() const {
    uint64_t sum = 0;
    for (const auto & s : slots_) if (s) sum += (uint64_t)(s->second - s->first + 1);
    return sum;
}

// fake.rs:217-230
int32_t FakeBackend::sample_token(int32_t request, size_t generated) const {
    if (eog_after && *eog_after == generated) return eos_;
    if (!script.empty()) return script[generated % script.size()];
    const int64_t vocab = std::max<int64_t>((int64_t)(vocab_ > 0 ? vocab_ - 1 : 0), 1);
    const int64_t mixed = (int64_t)request * 31 + ((int64_t)generated * 7 + 1);
    int64_t r = mixed % vocab;
    if (r < 0) r += vocab;
    return (int32_t)r;
}

// fake.rs:234-352
void FakeBackend::step(const std::vector<StepRow> & rows, StepOutput & out) {
    if (rows.empty()) throw InferError::invalid("a step requires at least one row");
    uint64_t total = 0;
    for (const StepRow & row : rows) total += row.n;
    if (total == 0) throw InferError::invalid("a step row requires tokens");
    std::vector<RowLog> log;
    std::vector<RowAdapter> adapters;
    for (const StepRow & row : rows) {
        log.push_back(RowLog{row.slot, row.n, row.sample ? row.request : -1});
        adapters.push_back(row.adapter);
    }
    steps.push_back(std::move(log));
    step_adapters.push_back(std::move(adapters));
    for (const StepRow & row : rows)
        if (row.adapter > 0 && !row_adapters_.count(row.adapter))
            throw InferError::invalid("step row adapter " + std::to_string(row.adapter) + " is not a loaded per-row adapter");
    // validate spans and capacity before mutating anything
    uint64_t used = cells_used();
    for (const StepRow & row : rows) {
        if (row.slot < 0 || row.slot >= (int32_t)n_slots_) throw InferError::invalid("step row slot out of range");
        if (row.n == 0) throw InferError::invalid("a step row requires at least one token");
        if (row.n > (uint32_t)INT32_MAX) throw InferError::overflow("a step row's token count does not fit i32");
        const int64_t end64 = (int64_t)row.pos0 + (int64_t)row.n;
        if (end64 > INT32_MAX) throw InferError::overflow("position range overflows i32");
        const int32_t end = (int32_t)end64;
        if (end > (int32_t)n_ctx_seq_) throw InferError::invalid("a step row decodes past the per-sequence context");
        const auto & span = slots_[(size_t)row.slot];
        if (!span) used += row.n;
        else if (row.pos0 == span->second + 1) used += row.n;
        else if (row.pos0 >= span->first && end - 1 <= span->second) {}
        else throw InferError::invalid("a step row leaves a gap in its slot's resident span");
        if (row.sample && row.request < 0) throw InferError::invalid("a sampling step row requires a request id >= 0");
    }
    if (used > cells_total_) throw InferError::backend("the fake KV pool is full");
    // commit: extend spans, then sample
    size_t stride = 0;
    for (const StepRow & row : rows) stride = std::max<size_t>(stride, row.n_top_logprobs);
    out.rows.assign(rows.size(), StepOutRow());
    out.n_top_stride = stride;
    out.top_ids.assign(rows.size() * stride, 0);
    out.top_logprobs.assign(rows.size() * stride, 0.0f);
    for (size_t index = 0; index < rows.size(); ++index) {
        const StepRow & row = rows[index];
        const int32_t end = row.pos0 + (int32_t)row.n;
        auto & slot = slots_[(size_t)row.slot];
        if (!slot) slot = std::make_pair(row.pos0, end - 1);
        else slot = std::make_pair(std::min(slot->first, row.pos0), std::max(slot->second, end - 1));
        if (!row.sample) continue;
        const size_t generated = requests_.count(row.request) ? requests_[row.request] : 0;
        if (std::find(request_order.begin(), request_order.end(), row.request) == request_order.end())
            request_order.push_back(row.request);
        const int32_t token = sample_token(row.request, generated);
        requests_[row.request] = generated + 1;
        const size_t n_top = std::min<size_t>(row.n_top_logprobs, vocab_);
        for (size_t k = 0; k < n_top; ++k) {
            out.top_ids[index * stride + k] = (int32_t)k;
            out.top_logprobs[index * stride + k] = -1.0f - (float)k;
        }
        StepOutRow & o = out.rows[index];
        o.token = token;
        o.logprob = -0.5f;
        o.forced = false;
        o.sampled = true;
        o.n_top = n_top;
        o.sampled_logprob = row.want_logprob ? -0.7f : 0.0f;
    }
    if (fail_after_steps == 0) {
        fail_after_steps = -1;
        throw InferError::backend("partial decode failure");
    }
    if (fail_after_steps > 0) --fail_after_steps;
}

// fake.rs:354-370
void FakeBackend::seq_rm(int32_t slot, int32_t p0, int32_t p1) {
    if (slot < 0 || slot >= (int32_t)n_slots_) throw InferError::invalid("seq_rm slot out of range");
    removed.push_back(slot);
    auto & span = slots_[(size_t)slot];
    if (p0 == -1 && p1 == -1) {
        span.reset();
    } else if (span) {
        const int32_t lo = p0 <= span->first ? p1 : span->first;
        const int32_t hi = (p1 >= span->second || p1 < 0) ? lo - 1 : span->second;
        if (lo > hi) span.reset();
        else span = std::make_pair(lo, hi);
    }
}

// fake.rs:372-400
void FakeBackend::seq_cp(int32_t src, int32_t dst, int32_t p0, int32_t p1) {
    if (src < 0 || src >= (int32_t)n_slots_ || dst < 0 || dst >= (int32_t)n_slots_)
        throw InferError::invalid("seq_cp slot out of range");
    const bool partial = !(p0 == -1 && p1 == -1);
    if (partial && !unified)
        throw InferError::invalid("seq_cp: a partial range between streams of a partitioned pool is unsupported");
    copies.push_back({src, dst, p0, p1});
    if (!slots_[(size_t)src]) throw InferError::invalid("seq_cp source slot is empty");
    const auto span = *slots_[(size_t)src];
    if (slots_[(size_t)dst]) throw InferError::invalid("seq_cp destination slot is not empty");
    if (!partial) {
        slots_[(size_t)dst] = span;
    } else {
        const int32_t lo = std::max(span.first, p0 < 0 ? 0 : p0);
        const int32_t hi = p1 < 0 ? span.second : std::min(span.second, p1 - 1);
        if (lo <= hi) slots_[(size_t)dst] = std::make_pair(lo, hi);
        else slots_[(size_t)dst].reset();
    }
}

std::pair<int32_t, int32_t> FakeBackend::seq_pos(int32_t slot) {
    if (slot < 0 || slot >= (int32_t)n_slots_) throw InferError::invalid("seq_pos slot out of range");
    return slots_[(size_t)slot] ? *slots_[(size_t)slot] : std::make_pair(-1, -1);
}

size_t FakeBackend::seq_save_len(int32_t slot, uint32_t flags) {
    if (slot < 0 || slot >= (int32_t)n_slots_) throw InferError::invalid("seq_save slot out of range");
    if (flags == kPartialOnly && recurrent) return 8;
    if (flags != 0 && flags != kPartialOnly) throw InferError::invalid("unknown snapshot flags");
    const auto buf = encode_snapshot(slot, flags);
    return buf ? buf->size() : 0;
}

size_t FakeBackend::seq_save_into(int32_t slot, uint32_t flags, uint8_t * buffer, size_t n) {
    std::vector<uint8_t> encoded;
    if (flags == kPartialOnly && recurrent) {
        put32(encoded, 0x5EED);
        put32(encoded, kPartialOnly);
    } else {
        const auto buf = encode_snapshot(slot, flags);
        if (!buf) throw InferError::invalid("seq_save slot is empty");
        encoded = *buf;
    }
    if (n < encoded.size()) throw InferError::invalid("save buffer too small");
    std::memcpy(buffer, encoded.data(), encoded.size());
    saves.push_back(StateLog{slot, flags, encoded.size()});
    return encoded.size();
}

size_t FakeBackend::seq_load(int32_t slot, uint32_t flags, const uint8_t * data, size_t n) {
    if (slot < 0 || slot >= (int32_t)n_slots_) throw InferError::invalid("seq_load slot out of range");
    loads.push_back(StateLog{slot, flags, n});
    if (flags == kPartialOnly && recurrent) return n;
    if (n < 16 || get32(data) != 0x5EED) throw InferError::invalid("corrupted snapshot");
    slots_[(size_t)slot] = std::make_pair((int32_t)get32(data + 8), (int32_t)get32(data + 12));
    return n;
}

EngineMemory FakeBackend::memory() {
    EngineMemory m;
    m.n_slots = n_slots_;
    m.cells_total = cells_total_;
    m.cells_used = cells_used();
    m.kv_bytes = m.cells_used * 16;
    m.recurrent_bytes = recurrent ? m.cells_used * 8 : 0;
    return m;
}

// fake.rs:509-529: the EOG token renders as text only when special tokens are unparsed.
std::string FakeBackend::detokenize_bytes(const int32_t * tokens, size_t n, bool unparse_special) {
    std::string out;
    for (size_t i = 0; i < n; ++i) {
        const int32_t token = tokens[i];
        if (token == eos_ && !unparse_special) continue;
        if (token >= 0 && (size_t)token < pieces_.size()) out += pieces_[(size_t)token];
        else out += "<" + std::to_string(token) + ">";
    }
    return out;
}

void FakeBackend::load_adapter(const std::string & name, const std::string & path) {
    if (name.empty()) throw InferError::invalid("adapter name must not be empty");
    register_adapter(name, path);
}

int32_t FakeBackend::load_row_adapter(const std::string & path, float) {
    if (!row_adapters_enabled) throw InferError::failed("per-row adapters are disabled");
    const int32_t id = next_row_adapter_;
    if (next_row_adapter_ == INT32_MAX) throw InferError::overflow("per-row adapter ids are exhausted");
    next_row_adapter_ += 1;
    row_adapters_[id] = path;
    adapter_ops.emplace_back("load_row", std::to_string(id));
    return id;
}

void FakeBackend::unload_row_adapter(int32_t id) {
    if (!row_adapters_.erase(id)) throw InferError::invalid("no per-row adapter " + std::to_string(id));
    adapter_ops.emplace_back("unload_row", std::to_string(id));
}

}  // namespace sched
