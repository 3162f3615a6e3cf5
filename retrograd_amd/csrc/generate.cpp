// Batched generators on top of the step: the whole generation loop of
// retro_engine_generate_batch and retro_engine_generate_continuous_batch
// (reference crates/retrograd-ffi/runtime/src/retro_gen_core.cpp:317-707,
// 1696-2049). Host logic only: every decode is Engine::step over v1 rows, so
// the tokens, log-probabilities and KV contents are those a caller-side loop
// over retro_engine_step produces when it composes the same steps.
#include "engine.hpp"

#include <cmath>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <sstream>

namespace retro {

namespace {

// Request ids of the generators' own rows: the per-request sampler state of
// the step is keyed by request id, and a caller's ids are non-negative ints it
// chooses itself, so the generators take theirs from the top of the range and
// free them before they return.
constexpr int32_t kGenRequestBase = 0x7f000000;

bool prefix_cache_enabled() {      // retro_gen_core.cpp:397-400
    const char * value = std::getenv("RETRO_GENERATION_PREFIX_CACHE");
    return !(value && (std::strcmp(value, "0") == 0 || std::strcmp(value, "false") == 0));
}

bool same_prompt(const retro_generation_sequence & a, const retro_generation_sequence & b) {
    return a.n_prompt == b.n_prompt && std::equal(a.prompt_tokens, a.prompt_tokens + a.n_prompt, b.prompt_tokens);
}

// retro_gen_core.cpp:333-358: prompt length, prompt tokens, then seed,
// max_new_tokens, temperature, top_p; stable, so equal rows keep caller order.
std::vector<size_t> canonical_order(const retro_generation_sequence * sequences, size_t n) {
    std::vector<size_t> order(n);
    std::iota(order.begin(), order.end(), size_t{0});
    std::stable_sort(order.begin(), order.end(), [&](size_t l, size_t r) {
        const retro_generation_sequence & a = sequences[l];
        const retro_generation_sequence & b = sequences[r];
        if (a.n_prompt != b.n_prompt) return a.n_prompt < b.n_prompt;
        for (size_t i = 0; i < a.n_prompt; ++i)
            if (a.prompt_tokens[i] != b.prompt_tokens[i]) return a.prompt_tokens[i] < b.prompt_tokens[i];
        if (a.sampling.seed != b.sampling.seed) return a.sampling.seed < b.sampling.seed;
        if (a.sampling.max_new_tokens != b.sampling.max_new_tokens) return a.sampling.max_new_tokens < b.sampling.max_new_tokens;
        if (a.sampling.temperature != b.sampling.temperature) return a.sampling.temperature < b.sampling.temperature;
        return a.sampling.top_p < b.sampling.top_p;
    });
    return order;
}

// retro_gen_core.cpp:411-423: a hit is an exact extension; a resident block as
// long as the prompt would leave the terminal position already decoded.
size_t resident_prefix(const std::vector<int32_t> & resident, const retro_generation_sequence & item) {
    if (resident.empty() || resident.size() >= item.n_prompt) return 0;
    return std::equal(resident.begin(), resident.end(), item.prompt_tokens) ? resident.size() : 0;
}

retro_step_row v1_row(int32_t request, int32_t slot, const int32_t * tokens, uint32_t n, int32_t pos0, bool sample,
                      const retro_sampling_params & sampling) {
    retro_step_row row {};
    row.struct_size = (uint32_t)sizeof(retro_step_row);
    row.request = request;
    row.slot = slot;
    row.tokens = tokens;
    row.n = n;
    row.pos0 = pos0;
    row.sample = sample;
    row.sampling = sampling;
    row.n_top_logprobs = 0;
    row.adapter = 0;     // the context adapter, as the batched generators decode
    return row;
}

}  // namespace

void Engine::GenCache::forget() {
    for (auto & resident : slots) resident.clear();
    std::fill(used_at.begin(), used_at.end(), 0);
}

void Engine::clear_generation_memory() {     // retro_gen_core.cpp:1483-1495
    for (int32_t slot = 0; slot < (int32_t)cfg_.n_seq_max; ++slot) (void)seq_rm(slot, -1, -1);
    gen_cache_.forget();
}

bool Engine::gen_validate_sampling(const retro_sampling_params & s) {      // retro_gen_core.cpp:1523-1537
    if (!(s.temperature > 0.0f) || !std::isfinite(s.temperature)) {
        set_error("sampling temperature must be finite and greater than zero");
        return false;
    }
    if (!(s.top_p > 0.0f && s.top_p <= 1.0f)) {
        set_error("sampling top_p must be in (0, 1]");
        return false;
    }
    if (s.max_new_tokens == 0) {
        set_error("sampling max_new_tokens must be greater than zero");
        return false;
    }
    return true;
}

bool Engine::gen_validate_tokens(const int32_t * tokens, size_t n) {       // retro_gen_core.cpp:1509-1521
    for (size_t i = 0; i < n; ++i) {
        if (tokens[i] < 0 || tokens[i] >= hp_.n_vocab) {
            std::ostringstream m;
            m << "token " << tokens[i] << " at index " << i << " is outside the vocabulary of size " << hp_.n_vocab;
            set_error(m.str());
            return false;
        }
    }
    return true;
}

// Decodes positions [p0, p1) of `tokens` into `slot` without sampling, n_batch at a time.
bool Engine::gen_prefill(int32_t slot, const int32_t * tokens, size_t p0, size_t p1) {
    const size_t n_batch = cfg_.n_batch;
    const retro_sampling_params none {};
    for (size_t at = p0; at < p1; at += n_batch) {
        const size_t n = std::min(n_batch, p1 - at);
        const retro_step_row row = v1_row(-1, slot, tokens + at, (uint32_t)n, (int32_t)at, false, none);
        retro_step_out_row out {};
        if (step(nullptr, &row, 1, nullptr, &out, nullptr, nullptr, 0) != 0) return false;
    }
    return true;
}

// One step of sampling rows for the generators' own requests, one token span per row. A row samples with the v1 or
// the v2 parameters of its sequence (all rows of a call alike); what comes back is the part both versions share.
int Engine::gen_sample_rows(const std::vector<GenRow> & specs, const std::vector<GenSampling> & sampling,
                            std::vector<retro_step_out_row> & outs) {
    outs.assign(specs.size(), retro_step_out_row{});
    if (specs.empty()) return 0;
    if (!sampling[specs[0].seq].v2) {
        std::vector<retro_step_row> rows;
        for (const GenRow & g : specs)
            rows.push_back(v1_row(kGenRequestBase + (int32_t)g.seq, g.slot, g.tokens, g.n, g.pos0, g.sample, *sampling[g.seq].v1));
        return step(nullptr, rows.data(), rows.size(), nullptr, outs.data(), nullptr, nullptr, 0);
    }
    std::vector<retro_step_row_v2> rows(specs.size());
    std::vector<retro_step_out_row_v2> outs2(specs.size());
    for (size_t i = 0; i < specs.size(); ++i) {
        const GenRow & g = specs[i];
        retro_step_row_v2 & row = rows[i];
        row = retro_step_row_v2{};
        row.struct_size = (uint32_t)sizeof(retro_step_row_v2);
        row.request = kGenRequestBase + (int32_t)g.seq;
        row.slot = g.slot;
        row.tokens = g.tokens;
        row.n = g.n;
        row.pos0 = g.pos0;
        row.sample = g.sample;
        row.sampling = *sampling[g.seq].v2;
        row.adapter = 0;     // the context adapter, as the batched generators decode
        outs2[i].struct_size = (uint32_t)sizeof(retro_step_out_row_v2);
    }
    const int status = step(rows.data(), nullptr, rows.size(), outs2.data(), nullptr, nullptr, nullptr, 0);
    if (status != 0) return status;
    for (size_t i = 0; i < specs.size(); ++i) {
        outs[i].struct_size = (uint32_t)sizeof(retro_step_out_row);
        outs[i].token = outs2[i].token;
        outs[i].logprob = outs2[i].logprob;      // the temperature-1 policy log-probability, as a v1 row reports it
        outs[i].forced = outs2[i].forced;
        outs[i].sampled = outs2[i].sampled;
    }
    return 0;
}

// The decode loop both generators share (retro_gen_core.cpp:1798-1875, 1982-2041):
// `first` holds what the terminal prompt rows sampled; every pass records one
// token per live row, in `order`, and decodes the rows that go on.
int Engine::gen_decode_loop(const std::vector<size_t> & order, const std::vector<int32_t> & slot_of,
                            const std::vector<size_t> & n_prompt_of, const std::vector<GenSampling> & sampling,
                            const std::vector<size_t> & limits, std::vector<retro_step_out_row> produced,
                            int32_t * out_tokens, float * out_logprobs, size_t n_out_max, size_t * out_n_tokens,
                            uint8_t * out_forced) {
    const size_t n = order.size();
    std::vector<bool> live(n, true);
    size_t n_live = n;
    std::vector<size_t> active;
    std::vector<GenRow> rows;
    std::vector<retro_step_out_row> outs;
    while (n_live > 0) {
        active.clear();
        for (const size_t seq : order) {
            if (!live[seq]) continue;
            const retro_step_out_row & got = produced[seq];
            const size_t count = out_n_tokens[seq];
            const size_t at = seq * n_out_max + count;
            out_tokens[at] = got.token;
            if (out_forced) out_forced[at] = got.forced ? 1 : 0;
            if (out_logprobs) out_logprobs[at] = got.logprob;
            out_n_tokens[seq] = count + 1;
            const bool eog = (vocab_.eos >= 0 && got.token == vocab_.eos) || (vocab_.eot >= 0 && got.token == vocab_.eot);
            if (eog || out_n_tokens[seq] == limits[seq]) {
                live[seq] = false;
                --n_live;
            } else {
                active.push_back(seq);
            }
        }
        if (active.empty()) break;
        rows.clear();
        for (const size_t seq : active) {
            const size_t count = out_n_tokens[seq];
            rows.push_back({seq, slot_of[seq], out_tokens + seq * n_out_max + count - 1, 1, (int32_t)(n_prompt_of[seq] + count - 1), true});
        }
        if (gen_sample_rows(rows, sampling, outs) != 0) return -1;
        for (size_t r = 0; r < active.size(); ++r) produced[active[r]] = outs[r];
    }
    return 0;
}

int Engine::generate_batch(const int32_t * prompt_tokens, size_t n_prompt, const retro_sampling_params * sampling,
                           size_t n_sequences, int32_t * out_tokens, float * out_logprobs, size_t n_out_max,
                           size_t * out_n_tokens, uint8_t * out_forced) {
    // validation in the reference's order, with its messages (retro_gen_core.cpp:1710-1750)
    if (!prompt_tokens || n_prompt == 0) {
        set_error("prompt tokens are required");
        return -1;
    }
    if (!sampling || n_sequences == 0 || !out_tokens || !out_n_tokens || n_out_max == 0) {
        set_error("sampling params and output buffers are required");
        return -1;
    }
    if (n_sequences > cfg_.n_seq_max) {
        std::ostringstream m;
        m << "generation batch has " << n_sequences << " sequences but the context supports " << cfg_.n_seq_max;
        set_error(m.str());
        return -1;
    }
    if (n_sequences > cfg_.n_batch) {
        set_error("generation batch exceeds the configured batch capacity");
        return -1;
    }
    if (n_sequences > SIZE_MAX / n_out_max) {
        set_error("generation batch output shape overflows size_t");
        return -1;
    }
    for (size_t i = 0; i < n_sequences; ++i)
        if (!gen_validate_sampling(sampling[i])) return -1;
    if (!gen_validate_tokens(prompt_tokens, n_prompt)) return -1;
    const size_t n_ctx = (size_t)n_ctx_seq_;
    if (n_prompt >= n_ctx) {
        std::ostringstream m;
        m << "prompt of " << n_prompt << " tokens leaves no room to generate in context " << n_ctx;
        set_error(m.str());
        return -1;
    }

    clear_generation_memory();
    struct Cleanup {
        Engine * e; size_t n;
        ~Cleanup() {
            for (size_t i = 0; i < n; ++i) e->request_free(kGenRequestBase + (int32_t)i);
            e->clear_generation_memory();
        }
    } cleanup{this, n_sequences};

    // The prompt is decoded once: its prefix into slot 0, copied whole to every
    // member, and the terminal position per member, since each member's first
    // token is drawn from the terminal logits with the member's own generator.
    if (!gen_prefill(0, prompt_tokens, 0, n_prompt - 1)) return -1;
    for (size_t i = 1; i < n_sequences; ++i)
        if (!seq_cp(0, (int32_t)i, -1, -1)) return -1;

    std::vector<size_t> order(n_sequences);
    std::iota(order.begin(), order.end(), size_t{0});
    std::vector<int32_t> slot_of(n_sequences);
    std::iota(slot_of.begin(), slot_of.end(), 0);
    std::vector<size_t> n_prompt_of(n_sequences, n_prompt), limits(n_sequences);
    std::vector<GenSampling> params(n_sequences);
    for (size_t i = 0; i < n_sequences; ++i) {
        params[i].v1 = &sampling[i];
        limits[i] = std::min<size_t>(std::min<size_t>(n_out_max, sampling[i].max_new_tokens), n_ctx - n_prompt);
        out_n_tokens[i] = 0;
    }
    std::vector<retro_step_row> rows;
    for (size_t i = 0; i < n_sequences; ++i)
        rows.push_back(v1_row(kGenRequestBase + (int32_t)i, (int32_t)i, prompt_tokens + n_prompt - 1, 1, (int32_t)(n_prompt - 1),
                              true, sampling[i]));
    std::vector<retro_step_out_row> produced(n_sequences);
    if (step(nullptr, rows.data(), rows.size(), nullptr, produced.data(), nullptr, nullptr, 0) != 0) return -1;
    return gen_decode_loop(order, slot_of, n_prompt_of, params, limits, std::move(produced), out_tokens, out_logprobs,
                           n_out_max, out_n_tokens, out_forced);
}

int Engine::generate_continuous_batch(const retro_generation_sequence * sequences, size_t n_sequences,
                                      int32_t * out_tokens, float * out_logprobs, size_t n_out_max,
                                      size_t * out_n_tokens, uint8_t * out_forced) {
    // retro_gen_core.cpp:1890-1913
    if (!sequences || n_sequences == 0 || !out_tokens || !out_n_tokens || n_out_max == 0) {
        set_error("continuous generation inputs and output buffers are required");
        return -1;
    }
    if (n_sequences > cfg_.n_seq_max || n_sequences > cfg_.n_batch) {
        set_error("continuous generation batch exceeds the configured sequence or batch capacity");
        return -1;
    }
    if (n_sequences > SIZE_MAX / n_out_max) {
        set_error("continuous generation output shape overflows size_t");
        return -1;
    }
    const size_t n_ctx_seq = (size_t)n_ctx_seq_;
    std::vector<GenSampling> sampling(n_sequences);
    std::vector<uint32_t> max_new(n_sequences);
    for (size_t i = 0; i < n_sequences; ++i) {
        const retro_generation_sequence & item = sequences[i];
        clear_error();
        if (!item.prompt_tokens || item.n_prompt == 0 || item.n_prompt >= n_ctx_seq || !gen_validate_sampling(item.sampling)
                || !gen_validate_tokens(item.prompt_tokens, item.n_prompt)) {
            if (last_error().empty()) set_error("invalid continuous generation prompt");
            return -1;
        }
        out_n_tokens[i] = 0;
        sampling[i].v1 = &item.sampling;
        max_new[i] = item.sampling.max_new_tokens;
    }
    return generate_continuous_impl(sequences, sampling, max_new, n_sequences, out_tokens, out_logprobs, n_out_max, out_n_tokens,
                                    out_forced);
}

// The v2 rows of retro_trainer_generate_continuous_batch_v2 (reference retro_gen_core.cpp:2051-2254): the same
// placement, prefill and bookkeeping over a view of the rows that holds their prompts only (so the canonical order and
// the cell budget do not see the sampling parameters, as in the reference), every token sampled through the v2 chain
// with the row's own generator, history and grammar.
int Engine::generate_continuous_batch_v2(const retro_generation_sequence_v2 * sequences, size_t n_sequences,
                                         int32_t * out_tokens, float * out_logprobs, size_t n_out_max,
                                         size_t * out_n_tokens, uint8_t * out_forced) {
    if (!sequences || n_sequences == 0 || !out_tokens || !out_n_tokens || n_out_max == 0) {
        set_error("continuous v2 generation inputs and output buffers are required");
        return -1;
    }
    if (n_sequences > cfg_.n_seq_max || n_sequences > cfg_.n_batch) {
        set_error("continuous v2 generation batch exceeds the configured sequence or batch capacity");
        return -1;
    }
    if (n_sequences > SIZE_MAX / n_out_max) {
        set_error("continuous v2 generation output shape overflows size_t");
        return -1;
    }
    const size_t n_ctx_seq = (size_t)n_ctx_seq_;
    std::vector<retro_generation_sequence> view(n_sequences);
    std::vector<GenSampling> sampling(n_sequences);
    std::vector<uint32_t> max_new(n_sequences);
    for (size_t i = 0; i < n_sequences; ++i) {
        const retro_generation_sequence_v2 & item = sequences[i];
        clear_error();
        if (!item.prompt_tokens || item.n_prompt == 0 || item.n_prompt >= n_ctx_seq || !valid_sampling_v2(item.sampling, hp_.n_vocab)
                || item.sampling.max_new_tokens == 0 || !gen_validate_tokens(item.prompt_tokens, item.n_prompt)) {
            if (last_error().empty()) set_error("invalid continuous v2 generation prompt");
            return -1;
        }
        if (item.sampling.grammar) {
            try {
                Grammar check(item.sampling.grammar->gbnf);
            } catch (const std::exception & e) {
                set_error(std::string("failed to compile the row's grammar (invalid GBNF): ") + e.what());
                clear_generation_memory();
                return -1;
            }
        }
        out_n_tokens[i] = 0;
        view[i] = retro_generation_sequence{};
        view[i].prompt_tokens = item.prompt_tokens;
        view[i].n_prompt = item.n_prompt;
        sampling[i].v2 = &item.sampling;
        max_new[i] = item.sampling.max_new_tokens;
    }
    return generate_continuous_impl(view.data(), sampling, max_new, n_sequences, out_tokens, out_logprobs, n_out_max, out_n_tokens,
                                    out_forced);
}

int Engine::generate_continuous_impl(const retro_generation_sequence * sequences, const std::vector<GenSampling> & sampling,
                                     const std::vector<uint32_t> & max_new, size_t n_sequences,
                                     int32_t * out_tokens, float * out_logprobs, size_t n_out_max,
                                     size_t * out_n_tokens, uint8_t * out_forced) {
    const size_t n_ctx_seq = (size_t)n_ctx_seq_;
    const bool cache = prefix_cache_enabled();
    if (!cache) clear_generation_memory();
    gen_cache_.stats.calls++;

    struct FreeRequests {
        Engine * e; size_t n;
        ~FreeRequests() { for (size_t i = 0; i < n; ++i) e->request_free(kGenRequestBase + (int32_t)i); }
    } free_requests{this, n_sequences};

    const std::vector<size_t> order = canonical_order(sequences, n_sequences);

    // ---- placement: the decisions of place_generation_sequences (reference retro_gen_core.cpp:430-546), stated as
    // a ranking. In canonical order every sequence takes, of the slots no earlier sequence of the call took, the
    // one ranked first by (longest resident prefix of its prompt; among slots that hold nothing of it the one
    // extended longest ago; lowest slot number). Then the slots nobody took give way, least recently extended
    // first, until what they hold fits beside the cells this call can come to occupy.
    const size_t n_slots = cfg_.n_seq_max;
    std::vector<int32_t> slot_of(n_sequences);
    std::vector<size_t> reuse_of(n_sequences, 0);
    if (!cache) {
        for (size_t i = 0; i < n_sequences; ++i) slot_of[i] = (int32_t)i;
    } else {
        GenCache & ledger = gen_cache_;
        ledger.slots.resize(n_slots);
        ledger.used_at.resize(n_slots, 0);
        std::vector<bool> taken(n_slots, false);
        struct Offer { size_t slot, kept; uint64_t age; };
        auto outranks = [](const Offer & a, const Offer & b) {
            if (a.kept != b.kept) return a.kept > b.kept;
            if (a.kept == 0 && a.age != b.age) return a.age < b.age;
            return a.slot < b.slot;
        };
        for (const size_t seq : order) {
            const retro_generation_sequence & item = sequences[seq];
            Offer pick{n_slots, 0, 0};
            for (size_t slot = 0; slot < n_slots; ++slot) {
                if (taken[slot]) continue;
                const Offer offer{slot, resident_prefix(ledger.slots[slot], item), ledger.used_at[slot]};
                if (pick.slot == n_slots || outranks(offer, pick)) pick = offer;
            }
            taken[pick.slot] = true;
            slot_of[seq] = (int32_t)pick.slot;
            reuse_of[seq] = pick.kept;
            if (pick.kept > 0) {
                ledger.stats.hits++;
            } else {
                // a cold start: whatever the slot held is given up
                if (!ledger.slots[pick.slot].empty()) ledger.stats.evictions++;
                (void)seq_rm((int32_t)pick.slot, -1, -1);
                ledger.slots[pick.slot].clear();
            }
            ledger.stats.sequences++;
            ledger.stats.prompt_tokens += item.n_prompt;
            ledger.stats.reused_tokens += pick.kept;
        }
        // cells this call may occupy: every prompt and all but the last of the tokens it can emit
        size_t room = cfg_.n_ctx;
        for (size_t i = 0; i < n_sequences; ++i) {
            const retro_generation_sequence & item = sequences[i];
            const size_t new_tokens = std::min<size_t>(std::min<size_t>(n_out_max, item.sampling.max_new_tokens),
                                                       n_ctx_seq - item.n_prompt);
            room -= std::min(room, item.n_prompt + new_tokens - 1);
        }
        // idle slots by the time they were last extended (slot number breaking ties), oldest first
        std::vector<size_t> idle;
        uint64_t idle_cells = 0;
        for (size_t slot = 0; slot < n_slots; ++slot)
            if (!taken[slot] && !ledger.slots[slot].empty()) {
                idle.push_back(slot);
                idle_cells += ledger.slots[slot].size();
            }
        std::stable_sort(idle.begin(), idle.end(), [&](size_t a, size_t b) { return ledger.used_at[a] < ledger.used_at[b]; });
        for (size_t i = 0; i < idle.size() && idle_cells > room; ++i) {
            const size_t slot = idle[i];
            (void)seq_rm((int32_t)slot, -1, -1);
            idle_cells -= ledger.slots[slot].size();
            ledger.slots[slot].clear();
            ledger.used_at[slot] = 0;
            ledger.stats.evictions++;
        }
    }

    // ---- prefill, group by group (retro_gen_core.cpp:585-705): a group is a run of cold
    // sequences with the same prompt; each group gets its own launches
    std::vector<retro_step_out_row> produced(n_sequences);
    auto fail = [&]() { clear_generation_memory(); return -1; };
    size_t group_start = 0;
    while (group_start < order.size()) {
        const size_t leader = order[group_start];
        const retro_generation_sequence & item = sequences[leader];
        const size_t reuse = reuse_of[leader];
        size_t group_end = group_start + 1;
        if (reuse == 0)
            while (group_end < order.size() && reuse_of[order[group_end]] == 0 && same_prompt(sequences[order[group_end]], item))
                ++group_end;
        const size_t members = group_end - group_start;
        const size_t terminal = item.n_prompt - 1;
        gen_cache_.stats.prefilled_tokens += (terminal - reuse) + members;
        std::vector<GenRow> rows;
        std::vector<retro_step_out_row> outs;
        if (members > 1) {
            // the prefix has to be resident before it can be copied
            if (!gen_prefill(slot_of[leader], item.prompt_tokens, reuse, terminal)) return fail();
            for (size_t m = group_start + 1; m < group_end; ++m)
                if (!seq_cp(slot_of[leader], slot_of[order[m]], -1, -1)) return fail();
            // the terminal rows of the members, n_batch per launch
            for (size_t m = group_start; m < group_end; m += cfg_.n_batch) {
                const size_t stop = std::min(group_end, m + cfg_.n_batch);
                rows.clear();
                for (size_t k = m; k < stop; ++k)
                    rows.push_back({order[k], slot_of[order[k]], item.prompt_tokens + terminal, 1, (int32_t)terminal, true});
                if (gen_sample_rows(rows, sampling, outs) != 0) return fail();
                for (size_t k = m; k < stop; ++k) produced[order[k]] = outs[k - m];
            }
        } else {
            // a group of one decodes its prefix and its terminal together: full launches of
            // n_batch positions, the terminal position closing the last one
            const size_t n_batch = cfg_.n_batch;
            size_t at = reuse;
            while (at < item.n_prompt) {
                const size_t n = std::min(n_batch, item.n_prompt - at);
                const bool last = at + n == item.n_prompt;
                rows.assign(1, GenRow{leader, slot_of[leader], item.prompt_tokens + at, (uint32_t)n, (int32_t)at, last});
                if (gen_sample_rows(rows, sampling, outs) != 0) return fail();
                if (last) produced[leader] = outs[0];
                at += n;
            }
        }
        group_start = group_end;
    }

    // ---- decode
    std::vector<size_t> n_prompt_of(n_sequences), limits(n_sequences);
    for (size_t i = 0; i < n_sequences; ++i) {
        n_prompt_of[i] = sequences[i].n_prompt;
        limits[i] = std::min<size_t>(std::min<size_t>(n_out_max, max_new[i]), n_ctx_seq - sequences[i].n_prompt);
    }
    if (gen_decode_loop(order, slot_of, n_prompt_of, sampling, limits, std::move(produced), out_tokens, out_logprobs, n_out_max,
                        out_n_tokens, out_forced) != 0)
        return fail();

    if (cache) {
        // what each slot holds now: the prompt and every sampled token but the last,
        // which was emitted and never fed back (retro_gen_core.cpp:548-582)
        GenCache & bk = gen_cache_;
        ++bk.clock;
        for (size_t i = 0; i < n_sequences; ++i) {
            std::vector<int32_t> & resident = bk.slots[(size_t)slot_of[i]];
            const size_t decoded = out_n_tokens[i] > 0 ? out_n_tokens[i] - 1 : 0;
            resident.assign(sequences[i].prompt_tokens, sequences[i].prompt_tokens + sequences[i].n_prompt);
            resident.insert(resident.end(), out_tokens + i * n_out_max, out_tokens + i * n_out_max + decoded);
            bk.used_at[(size_t)slot_of[i]] = bk.clock;
        }
    } else {
        clear_generation_memory();
    }
    return 0;
}

}  // namespace retro
