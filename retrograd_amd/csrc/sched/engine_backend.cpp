// The decode engine as a scheduler backend, through the library's own C ABI
// (reference `impl DecodeBackend for Engine`, crates/retrograd-infer/src/backend.rs:266-371).
#include "engine_backend.hpp"

#include <cstring>

namespace sched {

namespace {
[[noreturn]] void fail() { throw InferError::backend(retro_last_error()); }
void ok(int status) { if (status != 0) fail(); }
}  // namespace

// step.rs:150-203, 412-505: staging into reused buffers; the same checks the
// reference makes before the call.
void EngineBackend::step(const std::vector<StepRow> & rows, StepOutput & out) {
    if (rows.empty()) throw InferError::backend("a step requires at least one row");
    ffi_rows_.assign(rows.size(), retro_step_row_v2{});
    bias_ids_.clear();
    bias_values_.clear();
    size_t n_bias = 0;
    for (const StepRow & row : rows) n_bias += row.sampling ? row.sampling->logit_bias.size() : 0;
    bias_ids_.reserve(n_bias);
    bias_values_.reserve(n_bias);
    size_t stride = 0;
    struct Grammars {
        std::vector<std::pair<std::string, retro_grammar *>> held;
        ~Grammars() { for (auto & g : held) retro_grammar_free(g.second); }
    } grammars;
    for (size_t i = 0; i < rows.size(); ++i) {
        const StepRow & row = rows[i];
        if (row.n == 0) throw InferError::backend("a step row requires at least one token");
        if (row.pos0 < 0) throw InferError::backend("a step row's pos0 must be >= 0");
        if ((int64_t)row.pos0 + (int64_t)row.n - 1 > INT32_MAX) throw InferError::backend("a step row's positions overflow i32");
        if (row.sample && row.request < 0) throw InferError::backend("a sampling step row requires a request id >= 0");
        retro_step_row_v2 & f = ffi_rows_[i];
        f.struct_size = sizeof(retro_step_row_v2);
        f.request = row.request;
        f.slot = row.slot;
        f.tokens = row.tokens;
        f.n = row.n;
        f.pos0 = row.pos0;
        f.sample = row.sample;
        f.n_top_logprobs = row.n_top_logprobs;
        f.want_logprob = row.want_logprob ? 1 : 0;
        f.adapter = row.adapter;
        const SamplingParamsV2 & p = *row.sampling;
        if (p.logit_bias.size() > 4096) throw InferError::backend("logit_bias takes at most 4096 entries");
        retro_sampling_params_v2 & s = f.sampling;
        if (p.grammar_gbnf && row.sample) {
            // one handle per distinct text of the call (step.rs:440-470), freed when the call is over
            const retro_grammar * h = nullptr;
            for (const auto & g : grammars.held) if (g.first == *p.grammar_gbnf) h = g.second;
            if (!h) {
                retro_grammar * made = retro_grammar_from_gbnf(p.grammar_gbnf->c_str());
                if (!made) fail();
                grammars.held.push_back({*p.grammar_gbnf, made});
                h = made;
            }
            s.grammar = h;
        }
        s.struct_size = sizeof(retro_sampling_params_v2);
        s.temperature = p.temperature; s.top_p = p.top_p; s.max_new_tokens = p.max_new_tokens; s.seed = p.seed;
        s.top_k = p.top_k; s.min_p = p.min_p; s.repeat_penalty = p.repeat_penalty;
        s.frequency_penalty = p.frequency_penalty; s.presence_penalty = p.presence_penalty;
        s.penalty_window = p.penalty_window;
        s.n_logit_bias = (uint32_t)p.logit_bias.size();
        if (!p.logit_bias.empty()) {
            s.logit_bias_ids = bias_ids_.data() + bias_ids_.size();
            s.logit_bias_values = bias_values_.data() + bias_values_.size();
            for (const auto & b : p.logit_bias) { bias_ids_.push_back(b.first); bias_values_.push_back(b.second); }
        }
        stride = std::max<size_t>(stride, row.n_top_logprobs);
    }
    ffi_out_.assign(rows.size(), retro_step_out_row_v2{});
    for (auto & o : ffi_out_) o.struct_size = sizeof(retro_step_out_row_v2);
    out.n_top_stride = stride;
    out.top_ids.assign(rows.size() * stride, 0);
    out.top_logprobs.assign(rows.size() * stride, 0.0f);
    ok(retro_engine_step_v2(engine_, ffi_rows_.data(), ffi_rows_.size(), ffi_out_.data(),
                            stride ? out.top_ids.data() : nullptr, stride ? out.top_logprobs.data() : nullptr, stride));
    out.rows.assign(rows.size(), StepOutRow());
    for (size_t i = 0; i < rows.size(); ++i) {
        StepOutRow & o = out.rows[i];
        o.token = ffi_out_[i].token;
        o.logprob = ffi_out_[i].logprob;
        o.forced = ffi_out_[i].forced != 0;
        o.sampled = ffi_out_[i].sampled != 0;
        o.n_top = ffi_out_[i].n_top;
        o.sampled_logprob = ffi_out_[i].sampled_logprob;
    }
}

void EngineBackend::seq_rm(int32_t slot, int32_t p0, int32_t p1) { ok(retro_engine_seq_rm(engine_, slot, p0, p1)); }
void EngineBackend::seq_cp(int32_t src, int32_t dst, int32_t p0, int32_t p1) { ok(retro_engine_seq_cp(engine_, src, dst, p0, p1)); }
std::pair<int32_t, int32_t> EngineBackend::seq_pos(int32_t slot) {
    int32_t lo = -1, hi = -1;
    ok(retro_engine_seq_pos(engine_, slot, &lo, &hi));
    return {lo, hi};
}
size_t EngineBackend::seq_save_len(int32_t slot, uint32_t flags) {
    size_t n = 0;
    ok(retro_engine_seq_save(engine_, slot, flags, nullptr, 0, &n));
    return n;
}
size_t EngineBackend::seq_save_into(int32_t slot, uint32_t flags, uint8_t * buffer, size_t n) {
    size_t written = 0;
    ok(retro_engine_seq_save(engine_, slot, flags, buffer, n, &written));
    return written;
}
size_t EngineBackend::seq_load(int32_t slot, uint32_t flags, const uint8_t * data, size_t n) {
    size_t read = 0;
    ok(retro_engine_seq_load(engine_, slot, flags, data, n, &read));
    return read;
}
bool EngineBackend::kv_unified() { bool v = false; ok(retro_engine_kv_unified(engine_, &v)); return v; }
uint64_t EngineBackend::weights_version() { uint64_t v = 0; ok(retro_engine_weights_version(engine_, &v)); return v; }
uint64_t EngineBackend::model_fingerprint() { uint64_t v = 0; ok(retro_engine_model_fingerprint(engine_, &v)); return v; }
bool EngineBackend::is_hybrid() { bool v = false; ok(retro_engine_is_hybrid(engine_, &v)); return v; }
EngineMemory EngineBackend::memory() {
    retro_engine_memory_info info{};
    info.struct_size = sizeof(info);
    ok(retro_engine_memory(engine_, &info));
    EngineMemory m;
    m.n_slots = info.n_slots; m.cells_total = info.cells_total; m.cells_used = info.cells_used;
    m.kv_bytes = info.kv_bytes; m.recurrent_bytes = info.recurrent_bytes;
    return m;
}
void EngineBackend::request_free(int32_t request) { ok(retro_engine_request_free(engine_, request)); }
bool EngineBackend::is_eog_token(int32_t token) { bool v = false; ok(retro_engine_is_eog_token(engine_, token, &v)); return v; }
std::string EngineBackend::detokenize_bytes(const int32_t * tokens, size_t n, bool unparse_special) {
    size_t need = 0;
    ok(retro_engine_detokenize(engine_, tokens, n, unparse_special, nullptr, 0, &need));
    std::string out(need + 1, '\0');
    ok(retro_engine_detokenize(engine_, tokens, n, unparse_special, out.data(), out.size(), &need));
    out.resize(need);
    return out;
}
uint32_t EngineBackend::context_size() { uint32_t v = 0; ok(retro_engine_context_size(engine_, &v)); return v; }
uint32_t EngineBackend::vocab_size() { uint32_t v = 0; ok(retro_engine_vocab_size(engine_, &v)); return v; }
void EngineBackend::load_adapter(const std::string & name, const std::string & path) {
    ok(retro_engine_load_lora_named(engine_, name.c_str(), path.c_str()));
}
void EngineBackend::activate_adapter(const std::optional<std::string> & name) {
    ok(retro_engine_activate_lora(engine_, name ? name->c_str() : nullptr));
}
std::optional<std::string> EngineBackend::active_adapter() {
    size_t need = 0;
    ok(retro_engine_active_adapter(engine_, nullptr, 0, &need));
    if (need == 0) return std::nullopt;
    std::string out(need + 1, '\0');
    ok(retro_engine_active_adapter(engine_, out.data(), out.size(), &need));
    out.resize(need);
    return out;
}
int32_t EngineBackend::load_row_adapter(const std::string & path, float scale) {
    int32_t id = 0;
    ok(retro_engine_adapter_load(engine_, path.c_str(), scale, &id));
    return id;
}
void EngineBackend::unload_row_adapter(int32_t id) { ok(retro_engine_adapter_unload(engine_, id)); }
AdapterRowsInfo EngineBackend::adapter_rows_info() {
    retro_adapter_rows_info info{};
    info.struct_size = sizeof(info);
    ok(retro_engine_adapter_rows_info(engine_, &info));
    AdapterRowsInfo a;
    a.n_adapters = info.n_adapters; a.max_rank = info.max_rank;
    a.stacked_bytes = info.stacked_bytes; a.unpadded_bytes = info.unpadded_bytes;
    return a;
}

}  // namespace sched
