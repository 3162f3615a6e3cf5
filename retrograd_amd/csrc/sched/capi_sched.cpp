// C ABI of the step scheduler (include/retro_scheduler.h).
#include "../../../include/retro_scheduler.h"

#include <cstring>

#include "../engine.hpp"
#include "engine_backend.hpp"
#include "fake_backend.hpp"
#include "scheduler.hpp"

// defined with the trainer handle (capi_trainer.cpp)
struct retro_trainer;
namespace retro { retro_engine * generation_engine_of(retro_trainer * trainer); }

using namespace sched;

struct retro_scheduler {
    std::unique_ptr<Scheduler> impl;
    FakeBackend * fake = nullptr;      // owned by impl when set
};

struct retro_sched_stream {
    StreamRef stream;
    Event current;                     // storage behind the pointers of the last polled event
    std::vector<int32_t> top_ids;
    std::vector<float> top_logprobs;
    std::vector<const char *> top_pieces;
    std::vector<size_t> top_piece_lens;
};

namespace {

thread_local uint64_t g_needed = 0, g_available = 0, g_capacity = 0;

template <typename Fn> int guarded(Fn && fn) {
    try {
        return fn();
    } catch (const InferError & e) {
        retro::set_error(e.what());
        g_needed = e.needed; g_available = e.available; g_capacity = e.capacity;
        return -(int)e.kind;
    } catch (const std::exception & e) {
        retro::set_error(e.what());
        return -(int)ErrKind::Failed;
    } catch (...) {
        retro::set_error("unknown C++ exception");
        return -(int)ErrKind::Failed;
    }
}

Scheduler & sched_of(retro_scheduler * s) {
    if (!s || !s->impl) throw InferError::invalid("scheduler is required");
    return *s->impl;
}
FakeBackend & fake_of(retro_scheduler * s) {
    sched_of(s);
    if (!s->fake) throw InferError::invalid("this scheduler does not run on the fake backend");
    return *s->fake;
}

SchedulerOptions options_from(const retro_sched_options * o) {
    SchedulerOptions out;
    if (!o) return out;
    if (o->struct_size < sizeof(retro_sched_options)) throw InferError::invalid("retro_sched_options.struct_size is too small");
    if (o->mode != RETRO_SCHED_LOCKSTEP && o->mode != RETRO_SCHED_CONTINUOUS) throw InferError::invalid("unknown admission mode");
    out.mode = o->mode == RETRO_SCHED_LOCKSTEP ? AdmissionMode::Lockstep : AdmissionMode::Continuous;
    out.n_batch = o->n_batch;
    out.queue_capacity = o->queue_capacity;
    out.event_capacity = o->event_capacity;
    out.slow_client_timeout = std::chrono::nanoseconds(o->slow_client_timeout_ns);
    out.prefix_cache = o->prefix_cache != 0;
    out.min_prefix_len = o->min_prefix_len;
    out.max_snapshot_bytes = o->max_snapshot_bytes;
    out.swap_min_tokens = o->swap_min_tokens;
    out.max_retained = o->max_retained;
    out.retain_ttl = std::chrono::nanoseconds(o->retain_ttl_ns);
    return out;
}

}  // namespace

extern "C" {

void retro_sched_options_default(retro_sched_options * out) {
    if (!out) return;
    const SchedulerOptions d;
    std::memset(out, 0, sizeof(*out));
    out->struct_size = sizeof(*out);
    out->mode = RETRO_SCHED_LOCKSTEP;
    out->n_batch = d.n_batch;
    out->queue_capacity = d.queue_capacity;
    out->event_capacity = d.event_capacity;
    out->slow_client_timeout_ns = (uint64_t)d.slow_client_timeout.count();
    out->prefix_cache = d.prefix_cache ? 1 : 0;
    out->min_prefix_len = d.min_prefix_len;
    out->max_snapshot_bytes = d.max_snapshot_bytes;
    out->swap_min_tokens = d.swap_min_tokens;
    out->max_retained = d.max_retained;
    out->retain_ttl_ns = (uint64_t)d.retain_ttl.count();
}

retro_scheduler * retro_scheduler_new(retro_engine * engine, const retro_sched_options * options) {
    retro_scheduler * out = nullptr;
    guarded([&]() -> int {
        if (!engine) throw InferError::invalid("engine is required");
        auto s = std::make_unique<retro_scheduler>();
        s->impl = std::make_unique<Scheduler>(std::make_unique<EngineBackend>(engine), options_from(options));
        out = s.release();
        return 0;
    });
    return out;
}

retro_scheduler * retro_scheduler_new_trainer(retro_trainer * trainer, const retro_sched_options * options) {
    retro_scheduler * out = nullptr;
    guarded([&]() -> int {
        retro_engine * engine = retro::generation_engine_of(trainer);
        if (!engine) throw InferError::invalid("trainer is required");
        auto s = std::make_unique<retro_scheduler>();
        s->impl = std::make_unique<Scheduler>(std::make_unique<EngineBackend>(engine), options_from(options));
        out = s.release();
        return 0;
    });
    return out;
}

retro_scheduler * retro_scheduler_new_fake(uint32_t n_slots, uint32_t n_ctx_seq, uint64_t cells_total, uint32_t vocab,
                                           int32_t eos, const char * const * pieces, size_t n_pieces,
                                           const retro_sched_options * options) {
    retro_scheduler * out = nullptr;
    guarded([&]() -> int {
        std::vector<std::string> table;
        for (size_t i = 0; i < n_pieces; ++i) table.emplace_back(pieces && pieces[i] ? pieces[i] : "");
        auto fake = std::make_unique<FakeBackend>(n_slots, n_ctx_seq, cells_total, vocab, eos, std::move(table));
        auto s = std::make_unique<retro_scheduler>();
        s->fake = fake.get();
        s->impl = std::make_unique<Scheduler>(std::move(fake), options_from(options));
        out = s.release();
        return 0;
    });
    return out;
}

void retro_scheduler_free(retro_scheduler * s) { delete s; }

int retro_scheduler_initialize(retro_scheduler * s) {
    return guarded([&]() -> int { sched_of(s).initialize(); return 0; });
}

int retro_scheduler_submit(retro_scheduler * s, const retro_sched_request * r, retro_sched_stream ** out_stream) {
    return guarded([&]() -> int {
        Scheduler & sc = sched_of(s);
        if (!r || !out_stream) throw InferError::invalid("request and out_stream are required");
        if (r->struct_size < sizeof(retro_sched_request)) throw InferError::invalid("retro_sched_request.struct_size is too small");
        Request req;
        if (r->n_prompt > 0 && !r->prompt) throw InferError::invalid("prompt is required");
        req.prompt.assign(r->prompt, r->prompt + r->n_prompt);
        if (r->n_sampling > 0 && !r->sampling) throw InferError::invalid("sampling is required");
        for (size_t i = 0; i < r->n_sampling; ++i) {
            const retro_sampling_params_v2 & p = r->sampling[i];
            if (p.struct_size < sizeof(retro_sampling_params_v2)) throw InferError::invalid("retro_sampling_params_v2.struct_size is too small");
            if (p.grammar) throw InferError::invalid("pass grammars as text through grammar_gbnf");
            SamplingParamsV2 q;
            q.temperature = p.temperature; q.top_p = p.top_p; q.max_new_tokens = p.max_new_tokens; q.seed = p.seed;
            q.top_k = p.top_k; q.min_p = p.min_p; q.repeat_penalty = p.repeat_penalty;
            q.frequency_penalty = p.frequency_penalty; q.presence_penalty = p.presence_penalty;
            q.penalty_window = p.penalty_window;
            if (p.n_logit_bias > 0 && (!p.logit_bias_ids || !p.logit_bias_values)) throw InferError::invalid("logit_bias arrays are required");
            for (uint32_t b = 0; b < p.n_logit_bias; ++b) q.logit_bias.emplace_back(p.logit_bias_ids[b], p.logit_bias_values[b]);
            if (r->grammar_gbnf && r->grammar_gbnf[i]) q.grammar_gbnf = std::string(r->grammar_gbnf[i]);
            req.sampling.push_back(std::move(q));
        }
        for (size_t i = 0; i < r->n_stop; ++i) req.stop.emplace_back(r->stop[i] ? r->stop[i] : "");
        req.n_top_logprobs = r->n_top_logprobs;
        req.logprobs = r->logprobs != 0;
        if (r->adapter) req.adapter = std::string(r->adapter);
        req.unparse_special = r->unparse_special != 0;
        if (r->retention_key) {
            Retention ret;
            ret.key = r->retention_key;
            if (r->retention_release) ret.release = std::string(r->retention_release);
            req.retention = std::move(ret);
        }
        StreamRef stream = sc.submit(std::move(req));
        auto handle = std::make_unique<retro_sched_stream>();
        handle->stream = std::move(stream);
        *out_stream = handle.release();
        return 0;
    });
}

int retro_scheduler_pump(retro_scheduler * s, uint8_t * out_progressed) {
    return guarded([&]() -> int {
        const bool progressed = sched_of(s).pump();
        if (out_progressed) *out_progressed = progressed ? 1 : 0;
        return 0;
    });
}

int retro_scheduler_run_until_idle(retro_scheduler * s) {
    return guarded([&]() -> int { sched_of(s).run_until_idle(); return 0; });
}

int retro_scheduler_counts(retro_scheduler * s, uint64_t * out_queued, uint64_t * out_live) {
    return guarded([&]() -> int {
        Scheduler & sc = sched_of(s);
        if (out_queued) *out_queued = sc.queued_len();
        if (out_live) *out_live = sc.live_len();
        return 0;
    });
}

int retro_scheduler_fail_queued(retro_scheduler * s) {
    return guarded([&]() -> int { sched_of(s).fail_queued(); return 0; });
}

int retro_scheduler_kv_stats(retro_scheduler * s, retro_sched_kv_stats * out) {
    return guarded([&]() -> int {
        if (!out) throw InferError::invalid("out is required");
        const KvStats k = sched_of(s).kv_stats();
        out->struct_size = sizeof(*out);
        out->hits = k.hits; out->misses = k.misses; out->prefilled_cells = k.prefilled_cells;
        out->prompt_cells = k.prompt_cells; out->evictions = k.evictions; out->swaps = k.swaps;
        out->nodes = k.nodes; out->resident_slots = k.resident_slots; out->snapshot_bytes = k.snapshot_bytes;
        return 0;
    });
}

int retro_scheduler_pin_prefix(retro_scheduler * s, const int32_t * prefix, size_t n, uint64_t * out_pin) {
    return guarded([&]() -> int {
        if (!out_pin || (n > 0 && !prefix)) throw InferError::invalid("prefix and out_pin are required");
        *out_pin = sched_of(s).pin_prefix(std::vector<int32_t>(prefix, prefix + n));
        return 0;
    });
}

int retro_scheduler_lend_slot(retro_scheduler * s, uint64_t cells, int32_t * out_slot) {
    return guarded([&]() -> int {
        if (!out_slot) throw InferError::invalid("out_slot is required");
        *out_slot = sched_of(s).lend_slot(cells);
        return 0;
    });
}

int retro_scheduler_queue_capacity(retro_scheduler * s, size_t * out_capacity) {
    return guarded([&]() -> int {
        if (!out_capacity) throw InferError::invalid("out_capacity is required");
        *out_capacity = sched_of(s).queue_capacity();
        return 0;
    });
}

int retro_scheduler_unpin(retro_scheduler * s, uint64_t pin, uint8_t * out_released) {
    return guarded([&]() -> int {
        const bool released = sched_of(s).unpin(pin);
        if (out_released) *out_released = released ? 1 : 0;
        return 0;
    });
}

int retro_scheduler_load_adapter(retro_scheduler * s, const char * name, const char * path) {
    return guarded([&]() -> int { sched_of(s).load_adapter(name ? name : "", path ? path : ""); return 0; });
}

int retro_scheduler_unload_adapter(retro_scheduler * s, const char * name) {
    return guarded([&]() -> int { sched_of(s).unload_adapter(name ? name : ""); return 0; });
}

int retro_scheduler_set_mode(retro_scheduler * s, int32_t mode) {
    return guarded([&]() -> int {
        if (mode != RETRO_SCHED_LOCKSTEP && mode != RETRO_SCHED_CONTINUOUS) throw InferError::invalid("unknown admission mode");
        sched_of(s).set_mode(mode == RETRO_SCHED_LOCKSTEP ? AdmissionMode::Lockstep : AdmissionMode::Continuous);
        return 0;
    });
}

void retro_sched_last_error_detail(uint64_t * out_needed, uint64_t * out_available, uint64_t * out_capacity) {
    if (out_needed) *out_needed = g_needed;
    if (out_available) *out_available = g_available;
    if (out_capacity) *out_capacity = g_capacity;
}

int retro_sched_stream_poll(retro_sched_stream * h, retro_sched_event * out) {
    if (!h || !out) return 2;
    Stream & st = *h->stream;
    if (st.queue.empty()) return st.senders > 0 ? 1 : 2;
    h->current = std::move(st.queue.front());
    st.queue.pop_front();
    const Event & e = h->current;
    std::memset(out, 0, sizeof(*out));
    out->struct_size = sizeof(*out);
    out->type = (int32_t)e.type;
    out->index = e.index;
    out->token = e.token;
    out->logprob = e.logprob;
    out->has_sampled_logprob = e.has_sampled_logprob ? 1 : 0;
    out->sampled_logprob = e.sampled_logprob;
    out->forced = e.forced ? 1 : 0;
    out->text = e.text.data(); out->n_text = e.text.size();
    out->piece = e.piece.data(); out->n_piece = e.piece.size();
    h->top_ids.clear(); h->top_logprobs.clear(); h->top_pieces.clear(); h->top_piece_lens.clear();
    for (const TopLogprob & t : e.top_logprobs) {
        h->top_ids.push_back(t.token);
        h->top_logprobs.push_back(t.logprob);
        h->top_pieces.push_back(t.piece.data());
        h->top_piece_lens.push_back(t.piece.size());
    }
    out->n_top = e.top_logprobs.size();
    out->top_ids = h->top_ids.data();
    out->top_logprobs = h->top_logprobs.data();
    out->top_pieces = h->top_pieces.data();
    out->top_piece_lens = h->top_piece_lens.data();
    out->reason = (int32_t)e.reason;
    out->cached_tokens = e.cached_tokens;
    out->error_kind = (int32_t)e.error_kind;
    out->error_message = e.error_message.c_str();
    out->error_needed = e.error_needed;
    out->error_available = e.error_available;
    return 0;
}

void retro_sched_stream_free(retro_sched_stream * h) {
    if (!h) return;
    h->stream->receiver_alive = false;
    h->stream->cancelled = true;
    delete h;
}

int retro_sched_fake_set(retro_scheduler * s, const char * key, int64_t value) {
    return guarded([&]() -> int {
        FakeBackend & f = fake_of(s);
        const std::string k = key ? key : "";
        if (k == "eog_after") { if (value < 0) f.eog_after.reset(); else f.eog_after = (size_t)value; }
        else if (k == "kv_unified") f.unified = value != 0;
        else if (k == "recurrent") f.recurrent = value != 0;
        else if (k == "row_adapters") f.row_adapters_enabled = value != 0;
        else if (k == "fail_after_steps") f.fail_after_steps = (int)value;
        else if (k == "bump_weights_version") f.bump_weights_version();
        else throw InferError::invalid("unknown fake backend setting '" + k + "'");
        return 0;
    });
}

int retro_sched_fake_script(retro_scheduler * s, const int32_t * tokens, size_t n) {
    return guarded([&]() -> int {
        FakeBackend & f = fake_of(s);
        f.script.assign(tokens, tokens + n);
        return 0;
    });
}

int retro_sched_fake_register_adapter(retro_scheduler * s, const char * name, const char * path) {
    return guarded([&]() -> int { fake_of(s).register_adapter(name ? name : "", path ? path : ""); return 0; });
}

int retro_sched_fake_cells_used(retro_scheduler * s, uint64_t * out) {
    return guarded([&]() -> int {
        if (!out) throw InferError::invalid("out is required");
        *out = fake_of(s).memory().cells_used;
        return 0;
    });
}

int retro_sched_fake_log(retro_scheduler * s, const char * what, int64_t * buffer, size_t n_buffer, size_t * out_n) {
    return guarded([&]() -> int {
        FakeBackend & f = fake_of(s);
        if (!out_n) throw InferError::invalid("out_n is required");
        const std::string w = what ? what : "";
        std::vector<int64_t> flat;
        if (w == "steps") {
            for (size_t i = 0; i < f.steps.size(); ++i)
                for (size_t r = 0; r < f.steps[i].size(); ++r) {
                    flat.push_back((int64_t)i);
                    flat.push_back(f.steps[i][r].slot);
                    flat.push_back(f.steps[i][r].n);
                    flat.push_back(f.steps[i][r].request);
                    flat.push_back(f.step_adapters[i][r]);
                }
        } else if (w == "copies") {
            for (const auto & c : f.copies) for (int32_t v : c) flat.push_back(v);
        } else if (w == "removed") {
            for (int32_t v : f.removed) flat.push_back(v);
        } else if (w == "request_order") {
            for (int32_t v : f.request_order) flat.push_back(v);
        } else if (w == "saves" || w == "loads") {
            for (const auto & e : (w == "saves" ? f.saves : f.loads)) {
                flat.push_back(e.slot);
                flat.push_back(e.flags);
                flat.push_back((int64_t)e.len);
            }
        } else if (w == "seq_pos") {
            const uint32_t n = f.memory().n_slots;
            for (uint32_t slot = 0; slot < n; ++slot) {
                const auto range = f.seq_pos((int32_t)slot);
                flat.push_back(slot);
                flat.push_back(range.first);
                flat.push_back(range.second);
            }
        } else {
            throw InferError::invalid("unknown fake backend log '" + w + "'");
        }
        *out_n = flat.size();
        if (buffer) std::memcpy(buffer, flat.data(), std::min(n_buffer, flat.size()) * sizeof(int64_t));
        return 0;
    });
}

int retro_sched_fake_adapter_ops(retro_scheduler * s, char * buffer, size_t n_buffer, size_t * out_n_bytes) {
    return guarded([&]() -> int {
        FakeBackend & f = fake_of(s);
        if (!out_n_bytes) throw InferError::invalid("out_n_bytes is required");
        std::string text;
        for (const auto & op : f.adapter_ops) text += op.first + ":" + op.second + "\n";
        *out_n_bytes = text.size();
        if (buffer && n_buffer > 0) {
            if (text.size() > n_buffer - 1) throw InferError::invalid("output buffer is too small");
            std::memcpy(buffer, text.data(), text.size());
            buffer[text.size()] = '\0';
        }
        return 0;
    });
}

}  // extern "C"
