// extern "C" surface of libretro_hip.so: the entry points include/retro_step.h
// declares, each a thin boundary over retro::Engine. Every body runs inside
// boundary(), which clears the thread's error string and turns any C++
// exception into -1 (reference retro_runtime.hpp:1255-1267).
#include "engine.hpp"
#include "json_grammar.hpp"
#include "json_schema.hpp"

#include <cmath>
#include <cstring>

using namespace retro;

namespace {

template <typename Fn> int boundary(Fn && fn) {
    try {
        clear_error();
        return fn();
    } catch (const std::exception & e) {
        set_error(e.what());
        return -1;
    } catch (...) {
        set_error("unknown C++ exception");
        return -1;
    }
}

Engine * checked(retro_engine * e) {
    if (!e) {
        set_error("engine is required");
        return nullptr;
    }
    return &e->impl;
}

bool blank(const char * s) { return s == nullptr || s[0] == '\0'; }

// Defaults and validation of the reference (retro_engine.cpp:93-153), plus the
// refusals of what this library does not contain.
retro_engine_config default_config() {
    retro_engine_config c {};
    c.struct_size = sizeof(retro_engine_config);
    c.n_ctx = 4096;
    c.n_seq_max = 8;
    c.n_batch = 512;
    c.n_ubatch = 512;
    c.kv_dtype = RETRO_ENGINE_KV_DTYPE_F16;
    c.flash_attn = true;
    c.device = RETRO_DEVICE_AUTO;
    c.threads = 0;
    c.verbose = false;
    c.kv_unified = 1;
    c.expert_placement = RETRO_EXPERT_PLACEMENT_DEVICE;
    c.expert_host_layers = 0;
    c.expert_device_cache_bytes = 0;
    return c;
}

bool validate_config(const retro_engine_config & c, bool * invalid_placement) {
    if (c.n_ctx == 0 || c.n_seq_max == 0) {
        set_error("engine n_ctx and n_seq_max must be greater than zero");
        return false;
    }
    if (c.n_batch == 0 || c.n_ubatch == 0 || c.n_ubatch > c.n_batch) {
        set_error("engine n_ubatch must be in (0, n_batch]");
        return false;
    }
    if (c.n_ctx > INT32_MAX || c.n_batch > INT32_MAX || c.n_ubatch > INT32_MAX || c.threads > INT32_MAX) {
        set_error("engine context, batch and thread counts must fit in int32_t");
        return false;
    }
    if (c.n_seq_max > RETRO_MAX_SEQ || c.n_seq_max > std::min(c.n_batch, c.n_ctx)) {
        set_error("engine n_seq_max must not exceed LLAMA_MAX_SEQ, n_batch or n_ctx");
        return false;
    }
    if (c.kv_dtype < RETRO_ENGINE_KV_DTYPE_F32 || c.kv_dtype > RETRO_ENGINE_KV_DTYPE_Q4_0) {
        set_error("engine kv_dtype must be one of retro_engine_kv_dtype");
        return false;
    }
    if ((c.kv_dtype == RETRO_ENGINE_KV_DTYPE_Q8_0 || c.kv_dtype == RETRO_ENGINE_KV_DTYPE_Q4_0) && !c.flash_attn) {
        set_error("a quantized engine kv_dtype requires flash_attn");
        return false;
    }
    if (c.device < RETRO_DEVICE_AUTO || c.device > RETRO_DEVICE_GPU) {
        set_error("engine device must be one of retro_device");
        return false;
    }
    if (c.expert_placement != RETRO_EXPERT_PLACEMENT_DEVICE && c.expert_placement != RETRO_EXPERT_PLACEMENT_HOST) {
        set_error("engine expert_placement must be one of retro_expert_placement");
        return false;
    }
    if (c.device == RETRO_DEVICE_CPU) {
        set_error("device=cpu requested, but this library only executes on an MI355X GPU");
        return false;
    }
    if (c.kv_dtype == RETRO_ENGINE_KV_DTYPE_F32) {
        set_error("the f32 KV cache is not implemented by this library (f16, q8_0 and q4_0 are)");
        return false;
    }
    if (c.expert_placement == RETRO_EXPERT_PLACEMENT_HOST || c.expert_device_cache_bytes != 0) {
        if (invalid_placement) *invalid_placement = true;
        set_error("host expert placement is not supported: every tensor lives in device memory");
        return false;
    }
    return true;
}

// Two-call string contract of the reference (retro_runtime.hpp:551-576).
int string_out(const std::string & s, char * buffer, size_t n_buffer, size_t * out_n_bytes) {
    *out_n_bytes = s.size();
    if (!buffer || n_buffer == 0) return 0;
    if (s.size() > n_buffer - 1) {
        set_error("output buffer is too small");
        return -2;
    }
    std::memcpy(buffer, s.data(), s.size());
    buffer[s.size()] = '\0';
    return 0;
}

}  // namespace

extern "C" {

const char * retro_last_error(void) {
    return last_error().empty() ? "no runtime error" : last_error().c_str();
}

retro_engine * retro_engine_new(const char * model_path, const retro_engine_config * config) {
    return retro_engine_new_checked(model_path, config, nullptr);
}

retro_engine * retro_engine_new_checked(const char * model_path, const retro_engine_config * config,
                                        bool * out_invalid_placement) {
    if (out_invalid_placement) *out_invalid_placement = false;
    try {
        clear_error();
        if (blank(model_path)) {
            set_error("model_path is required");
            return nullptr;
        }
        retro_engine_config resolved = default_config();
        if (config) {
            // Read the evolution key before any other field; copy only the
            // prefix the caller owns (retro_engine.cpp:474-494).
            uint32_t size = 0;
            std::memcpy(&size, config, sizeof(size));
            constexpr size_t required = offsetof(retro_engine_config, verbose) + sizeof(bool);
            if (size < required) {
                set_error("retro_engine_config.struct_size is too small for this build");
                return nullptr;
            }
            std::memcpy(&resolved, config, std::min<size_t>(size, sizeof(resolved)));
        }
        if (!validate_config(resolved, out_invalid_placement)) return nullptr;
        return new retro_engine(model_path, resolved);
    } catch (const std::exception & e) {
        set_error(e.what());
        return nullptr;
    } catch (...) {
        set_error("unknown C++ exception");
        return nullptr;
    }
}

void retro_engine_free(retro_engine * engine) { delete engine; }

int retro_engine_step(retro_engine * engine, const retro_step_row * rows, size_t n_rows,
                      retro_step_out_row * out_rows, int32_t * out_top_ids, float * out_top_logprobs,
                      size_t n_top_stride) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        if (!rows || n_rows == 0 || !out_rows) {
            set_error("step rows and output rows are required");
            return -3;
        }
        e->forget_generation_bookkeeping();
        return e->step(nullptr, rows, n_rows, nullptr, out_rows, out_top_ids, out_top_logprobs, n_top_stride);
    });
}

int retro_engine_step_v2(retro_engine * engine, const retro_step_row_v2 * rows, size_t n_rows,
                         retro_step_out_row_v2 * out_rows, int32_t * out_top_ids, float * out_top_logprobs,
                         size_t n_top_stride) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        if (!rows || n_rows == 0 || !out_rows) {
            set_error("step rows and output rows are required");
            return -3;
        }
        e->forget_generation_bookkeeping();
        return e->step(rows, nullptr, n_rows, out_rows, nullptr, out_top_ids, out_top_logprobs, n_top_stride);
    });
}

int retro_engine_seq_rm(retro_engine * engine, int32_t slot, int32_t p0, int32_t p1) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        e->forget_generation_bookkeeping();
        return e->seq_rm(slot, p0, p1) ? 0 : -1;
    });
}

int retro_engine_seq_cp(retro_engine * engine, int32_t src, int32_t dst, int32_t p0, int32_t p1) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        e->forget_generation_bookkeeping();
        return e->seq_cp(src, dst, p0, p1) ? 0 : -1;
    });
}

int retro_engine_seq_save(retro_engine * engine, int32_t slot, uint32_t flags, uint8_t * buffer, size_t n_buffer,
                          size_t * out_n_bytes) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        return e->seq_save(slot, flags, buffer, n_buffer, out_n_bytes);
    });
}

int retro_engine_seq_load(retro_engine * engine, int32_t slot, uint32_t flags, const uint8_t * buffer,
                          size_t n_bytes, size_t * out_n_read) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        e->forget_generation_bookkeeping();
        return e->seq_load(slot, flags, buffer, n_bytes, out_n_read);
    });
}

int retro_engine_seq_pos(retro_engine * engine, int32_t slot, int32_t * out_pos_min, int32_t * out_pos_max) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        return e->seq_pos(slot, out_pos_min, out_pos_max);
    });
}

int retro_engine_memory(retro_engine * engine, retro_engine_memory_info * out) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        return e->memory(out);
    });
}

int retro_engine_request_free(retro_engine * engine, int32_t request) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        e->request_free(request);
        return 0;
    });
}

int retro_engine_generate_batch(retro_engine * engine, const int32_t * prompt_tokens, size_t n_prompt,
                                const retro_sampling_params * sampling, size_t n_sequences, int32_t * out_tokens,
                                float * out_logprobs, size_t n_out_max, size_t * out_n_tokens, uint8_t * out_forced) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        return e->generate_batch(prompt_tokens, n_prompt, sampling, n_sequences, out_tokens, out_logprobs, n_out_max,
                                 out_n_tokens, out_forced);
    });
}

int retro_engine_generate_continuous_batch(retro_engine * engine, const retro_generation_sequence * sequences,
                                           size_t n_sequences, int32_t * out_tokens, float * out_logprobs,
                                           size_t n_out_max, size_t * out_n_tokens, uint8_t * out_forced) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        return e->generate_continuous_batch(sequences, n_sequences, out_tokens, out_logprobs, n_out_max, out_n_tokens,
                                            out_forced);
    });
}

int retro_engine_generation_stats(retro_engine * engine, retro_generation_stats * out_stats) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e || !out_stats) {
            if (e) set_error("out_stats is required");
            return -1;
        }
        *out_stats = e->generation_stats();
        return 0;
    });
}

int retro_engine_kv_unified(retro_engine * engine, bool * out_unified) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e || !out_unified) {
            if (e) set_error("out_unified is required");
            return -1;
        }
        *out_unified = e->config().kv_unified != 0;
        return 0;
    });
}

int retro_engine_weights_version(retro_engine * engine, uint64_t * out_version) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e || !out_version) {
            if (e) set_error("out_version is required");
            return -1;
        }
        *out_version = e->weights_version();
        return 0;
    });
}

int retro_engine_model_fingerprint(retro_engine * engine, uint64_t * out_fingerprint) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e || !out_fingerprint) {
            if (e) set_error("out_fingerprint is required");
            return -1;
        }
        *out_fingerprint = e->fingerprint();
        return 0;
    });
}

int retro_engine_is_hybrid(retro_engine * engine, bool * out_is_hybrid) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e || !out_is_hybrid) {
            if (e) set_error("out_is_hybrid is required");
            return -1;
        }
        *out_is_hybrid = false;   // attention-only architectures
        return 0;
    });
}

// Two-call contract of the reference's tokenize_into (retro_engine.cpp:331-378): with no buffer (or no room at all)
// the count is reported and the call succeeds; a buffer that is too small is -2 with the count.
static int tokenize_into(Engine & e, const char * text, bool add_special, bool parse_special, int32_t * tokens,
                         size_t n_tokens_max, size_t * out_n_tokens) {
    if (!text || text[0] == '\0') {
        set_error("text is required");
        return -1;
    }
    if (!out_n_tokens) {
        set_error("out_n_tokens is required");
        return -1;
    }
    if (std::strlen(text) > (size_t)INT32_MAX) {
        set_error("text is too large to tokenize");
        return -1;
    }
    const Vocab & v = e.vocab();
    if (!v.tokenizer_error.empty()) {
        set_error("this model's vocabulary cannot tokenize: " + v.tokenizer_error);
        return -1;
    }
    const std::vector<int32_t> ids = v.tokenizer.tokenize(text, add_special, parse_special);     // throws for a vocabulary kind that is not built
    *out_n_tokens = ids.size();
    if (!tokens || n_tokens_max == 0) return 0;
    if (ids.size() > n_tokens_max) return -2;
    std::copy(ids.begin(), ids.end(), tokens);
    return 0;
}

/* text with BOS / EOS as the model asks, special-token texts read as tokens (ref retro_engine.cpp:594-607) */
int retro_engine_tokenize_text(retro_engine * engine, const char * text, int32_t * tokens, size_t n_tokens_max, size_t * out_n_tokens) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        return tokenize_into(*e, text, true, true, tokens, n_tokens_max, out_n_tokens);
    });
}

/* the same without BOS / EOS (ref retro_engine.cpp:609-622) */
int retro_engine_tokenize_fragment(retro_engine * engine, const char * text, int32_t * tokens, size_t n_tokens_max, size_t * out_n_tokens) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        return tokenize_into(*e, text, false, true, tokens, n_tokens_max, out_n_tokens);
    });
}

/* both flags explicit (ref retro_lora_train.h:2879-2889) */
int retro_engine_tokenize(retro_engine * engine, const char * text, bool add_special, bool parse_special, int32_t * tokens,
                          size_t n_tokens_max, size_t * out_n_tokens) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        return tokenize_into(*e, text, add_special, parse_special, tokens, n_tokens_max, out_n_tokens);
    });
}

int retro_engine_eos_token(retro_engine * engine, int32_t * out_token) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e || !out_token) {
            if (e) set_error("out_token is required");
            return -1;
        }
        *out_token = e->vocab().eos;
        return 0;
    });
}

int retro_engine_vocab_size(retro_engine * engine, uint32_t * out_n_vocab) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e || !out_n_vocab) {
            if (e) set_error("out_n_vocab is required");
            return -1;
        }
        *out_n_vocab = (uint32_t)e->hparams().n_vocab;
        return 0;
    });
}

int retro_engine_is_eog_token(retro_engine * engine, int32_t token, bool * out_is_eog) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e || !out_is_eog) {
            if (e) set_error("out_is_eog is required");
            return -1;
        }
        if (token < 0 || token >= e->hparams().n_vocab) {
            set_error("token is outside the vocabulary");
            return -1;
        }
        const Vocab & v = e->vocab();
        *out_is_eog = v.is_eog(token);
        return 0;
    });
}

int retro_engine_context_size(retro_engine * engine, uint32_t * out_n_ctx) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e || !out_n_ctx) {
            if (e) set_error("out_n_ctx is required");
            return -1;
        }
        *out_n_ctx = e->context_size();
        return 0;
    });
}

// Concatenates what the tokens stand for (Vocab::append_text); control tokens are skipped unless unparse_special.
int retro_engine_detokenize(retro_engine * engine, const int32_t * tokens, size_t n_tokens, bool unparse_special,
                            char * buffer, size_t n_buffer, size_t * out_n_bytes) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        if (!out_n_bytes) {
            set_error("out_n_bytes is required");
            return -1;
        }
        if (n_tokens > 0 && !tokens) {
            set_error("tokens are required");
            return -1;
        }
        if (n_tokens > (size_t)INT32_MAX) {
            set_error("too many tokens to detokenize");
            return -1;
        }
        const Vocab & v = e->vocab();
        const int32_t n_vocab = e->hparams().n_vocab;
        std::string text;
        for (size_t i = 0; i < n_tokens; ++i) {
            const int32_t t = tokens[i];
            if (t < 0 || t >= n_vocab) {
                set_error("token " + std::to_string(t) + " at index " + std::to_string(i)
                          + " is outside the vocabulary of size " + std::to_string(n_vocab));
                return -1;
            }
            v.append_text(t, unparse_special, text);
        }
        return string_out(text, buffer, n_buffer, out_n_bytes);
    });
}

int retro_engine_token_piece(retro_engine * engine, int32_t token, bool special, char * buffer, size_t n_buffer, size_t * out_n_bytes) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        if (!out_n_bytes) {
            set_error("out_n_bytes is required");
            return -1;
        }
        if (token < 0 || token >= e->hparams().n_vocab) {
            set_error("token is outside the vocabulary");
            return -1;
        }
        std::string text;
        e->vocab().append_text(token, special, text);
        return string_out(text, buffer, n_buffer, out_n_bytes);
    });
}

int retro_engine_graphs_reused(retro_engine * engine, uint64_t * out_n_reused) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        if (!out_n_reused) {
            set_error("out_n_reused is required");
            return -1;
        }
        *out_n_reused = 0;   // every step launches its kernels directly; nothing is cached between steps
        return 0;
    });
}

// ---- adapters ---------------------------------------------------------------------------

int retro_engine_load_lora(retro_engine * engine, const char * adapter_path) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        if (blank(adapter_path)) {
            set_error("adapter_path is required");
            return -1;
        }
        return e->load_lora(adapter_path);
    });
}

int retro_engine_set_lora_enabled(retro_engine * engine, bool enabled) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        return e->set_lora_enabled(enabled);
    });
}

int retro_engine_load_lora_named(retro_engine * engine, const char * name, const char * adapter_path) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        if (blank(name)) {
            set_error("name is required");
            return -1;
        }
        if (blank(adapter_path)) {
            set_error("adapter_path is required");
            return -1;
        }
        return e->load_lora_named(name, adapter_path);
    });
}

int retro_engine_activate_lora(retro_engine * engine, const char * name) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        return e->activate_lora(name ? name : "");
    });
}

int retro_engine_active_adapter(retro_engine * engine, char * buffer, size_t n_buffer, size_t * out_n_bytes) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        if (!out_n_bytes) {
            set_error("out_n_bytes is required");
            return -1;
        }
        return string_out(e->active_adapter(), buffer, n_buffer, out_n_bytes);
    });
}

int retro_engine_adapter_load(retro_engine * engine, const char * adapter_path, float scale, int32_t * out_id) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        if (blank(adapter_path)) {
            set_error("adapter_path is required");
            return -1;
        }
        if (!out_id) {
            set_error("out_id is required");
            return -1;
        }
        if (!std::isfinite(scale)) {
            set_error("the adapter scale must be finite");
            return -1;
        }
        return e->adapter_load(adapter_path, scale, out_id);
    });
}

int retro_engine_adapter_unload(retro_engine * engine, int32_t id) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        return e->adapter_unload(id);
    });
}

int retro_engine_adapter_rows_info(retro_engine * engine, retro_adapter_rows_info * out_info) {
    return boundary([&]() -> int {
        Engine * e = checked(engine);
        if (!e) return -1;
        if (!out_info) {
            set_error("out_info is required");
            return -1;
        }
        e->adapter_rows_info(out_info);
        return 0;
    });
}

// ---- grammar handles -------------------------------------------------------------------

retro_grammar * retro_grammar_from_json_schema(const char * json_schema) {
    clear_error();
    if (blank(json_schema)) {
        set_error("json_schema is required");
        return nullptr;
    }
    try {
        return new retro_grammar{SchemaToGbnf::convert(json_schema)};
    } catch (const std::exception & e) {
        set_error(std::string("failed to convert the JSON schema to a grammar: ") + e.what());
        return nullptr;
    }
}

retro_grammar * retro_grammar_from_gbnf(const char * gbnf) {
    clear_error();
    if (blank(gbnf)) {
        set_error("gbnf is required");
        return nullptr;
    }
    return new retro_grammar{gbnf};
}

retro_grammar * retro_grammar_json_object(void) {
    clear_error();
    return new retro_grammar{kJsonObjectGbnf};
}

const char * retro_grammar_gbnf(const retro_grammar * grammar) { return grammar ? grammar->gbnf.c_str() : nullptr; }

void retro_grammar_free(retro_grammar * grammar) { delete grammar; }

}  // extern "C"
