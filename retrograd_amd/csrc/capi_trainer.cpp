// extern "C" surface of include/retro_trainer.h: the generation side of the
// reference's trainer handle. A trainer here is an engine built with the
// geometry of the reference's dedicated generation context
// (retro_backend.cpp:1218-1287) whose rows with adapter 0 decode under the
// trained LoRA adapter; every twin forwards to the engine entry point it mirrors
// (reference retro_lora_train.cpp:1148-1290, retro_rollout.cpp:150-340).
#include "engine.hpp"
#include "../../include/retro_trainer.h"

#include <algorithm>
#include <climits>

using namespace retro;

struct retro_trainer {
    retro_train_config config;
    retro_engine * engine = nullptr;
    ~retro_trainer() { if (engine) retro_engine_free(engine); }
};

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

retro_engine * checked(retro_trainer * t) {
    if (!t) {
        set_error("trainer is required");
        return nullptr;
    }
    return t->engine;
}

// The checks of the reference's validate_train_config (retro_runtime.cpp:158-262)
// on the fields this library reads, with its messages.
bool validate(const retro_train_config & c) {
    if (c.n_ctx > INT32_MAX || c.n_batch > INT32_MAX || c.n_ubatch > INT32_MAX) {
        set_error("training dimensions exceed signed native counters");
        return false;
    }
    if (c.n_ctx == 0) { set_error("n_ctx must be greater than zero"); return false; }
    if (c.n_batch == 0) { set_error("n_batch must be greater than zero"); return false; }
    if (c.generation_concurrency == 0 || c.generation_concurrency > 256) {
        set_error("generation_concurrency must be between 1 and 256");
        return false;
    }
    if (c.generation_concurrency > c.n_batch) {
        set_error("generation_concurrency must not exceed n_batch");
        return false;
    }
    if (c.n_ctx > INT32_MAX / c.generation_concurrency) {
        set_error("n_ctx * generation_concurrency exceeds signed native counters");
        return false;
    }
    if (c.generation_kv_dtype < 0 || c.generation_kv_dtype > 2) {
        set_error("generation_kv_dtype must be f16, q8_0, or q4_0");
        return false;
    }
    if (c.generation_kv_dtype != 0 && !c.fast_generation_context) {
        set_error("a quantized generation_kv_dtype requires fast_generation_context");
        return false;
    }
    if (c.device < RETRO_DEVICE_AUTO || c.device > RETRO_DEVICE_GPU) {
        set_error("device must be one of retro_device");
        return false;
    }
    if (c.device == RETRO_DEVICE_CPU) {
        set_error("device=cpu requested, but this library only executes on an MI355X GPU");
        return false;
    }
    return true;
}

}  // namespace

// The engine behind a trainer's generation context, for the scheduler (capi_sched.cpp).
namespace retro {
retro_engine * generation_engine_of(retro_trainer * trainer) { return trainer ? trainer->engine : nullptr; }
}

extern "C" {

retro_trainer * retro_trainer_new(const char * model_path, const retro_train_config * train_config) {
    retro_trainer * out = nullptr;
    boundary([&]() -> int {
        if (!model_path || !model_path[0]) { set_error("model_path is required"); return -1; }
        if (!train_config) { set_error("train_config is required"); return -1; }
        if (!validate(*train_config)) return -1;
        std::unique_ptr<retro_trainer> t(new retro_trainer());
        t->config = *train_config;
        // the dedicated generation context (retro_backend.cpp:1244-1266); its batch needs the vocabulary
        // size, so the engine is opened once to read it when generation_batch is left to the default
        retro_engine_config ec {};
        ec.struct_size = sizeof(retro_engine_config);
        ec.n_ctx = train_config->n_ctx * train_config->generation_concurrency;
        ec.n_seq_max = train_config->generation_concurrency;
        uint32_t batch = train_config->generation_batch;
        if (batch == 0) {
            const uint64_t n_vocab = Engine::vocab_size_of(model_path);
            const uint64_t affordable = std::max<uint64_t>(1, ((uint64_t)64 << 20) / std::max<uint64_t>(1, n_vocab * 4));
            batch = (uint32_t)std::min<uint64_t>(std::min<uint32_t>(train_config->n_ctx, 512), affordable);
        }
        batch = std::max(batch, train_config->generation_concurrency);
        ec.n_batch = batch;
        ec.n_ubatch = batch;
        ec.kv_dtype = train_config->generation_kv_dtype == 1 ? RETRO_ENGINE_KV_DTYPE_Q8_0
                    : train_config->generation_kv_dtype == 2 ? RETRO_ENGINE_KV_DTYPE_Q4_0 : RETRO_ENGINE_KV_DTYPE_F16;
        ec.flash_attn = true;
        ec.device = train_config->device;
        ec.threads = train_config->threads;
        ec.verbose = train_config->verbose;
        ec.kv_unified = 1;
        ec.expert_placement = RETRO_EXPERT_PLACEMENT_DEVICE;
        t->engine = retro_engine_new(model_path, &ec);
        if (!t->engine) return -1;          // the engine's message stands
        out = t.release();
        return 0;
    });
    return out;
}

void retro_trainer_free(retro_trainer * trainer) { delete trainer; }

int retro_trainer_load_lora(retro_trainer * trainer, const char * adapter_path) {
    return boundary([&]() -> int {
        retro_engine * e = checked(trainer);
        if (!e) return -1;
        if (!adapter_path || !adapter_path[0]) { set_error("adapter_path is required"); return -1; }
        if (e->impl.policy_adapter_load(adapter_path) != 0) return -1;
        e->impl.forget_generation_kv();
        return 0;
    });
}

#define TWIN(call) do { retro_engine * e = checked(trainer); if (!e) return -1; return call; } while (0)

int retro_trainer_eos_token(retro_trainer * trainer, int32_t * out_token) { TWIN(retro_engine_eos_token(e, out_token)); }
int retro_trainer_vocab_size(retro_trainer * trainer, uint32_t * out_n_vocab) { TWIN(retro_engine_vocab_size(e, out_n_vocab)); }
int retro_trainer_is_eog_token(retro_trainer * trainer, int32_t token, bool * out_is_eog) {
    TWIN(retro_engine_is_eog_token(e, token, out_is_eog));
}
int retro_trainer_context_size(retro_trainer * trainer, uint32_t * out_n_ctx) {
    return boundary([&]() -> int {
        if (!checked(trainer)) return -1;
        if (!out_n_ctx) { set_error("out_n_ctx is required"); return -1; }
        *out_n_ctx = trainer->config.n_ctx;
        return 0;
    });
}
int retro_trainer_tokenize_text(retro_trainer * trainer, const char * text, int32_t * tokens, size_t n_tokens_max, size_t * out_n_tokens) {
    TWIN(retro_engine_tokenize_text(e, text, tokens, n_tokens_max, out_n_tokens));
}
int retro_trainer_tokenize_fragment(retro_trainer * trainer, const char * text, int32_t * tokens, size_t n_tokens_max, size_t * out_n_tokens) {
    TWIN(retro_engine_tokenize_fragment(e, text, tokens, n_tokens_max, out_n_tokens));
}
int retro_trainer_tokenize_with(retro_trainer * trainer, const char * text, bool add_special, bool parse_special, int32_t * tokens,
                                size_t n_tokens_max, size_t * out_n_tokens) {
    TWIN(retro_engine_tokenize(e, text, add_special, parse_special, tokens, n_tokens_max, out_n_tokens));
}
int retro_trainer_detokenize(retro_trainer * trainer, const int32_t * tokens, size_t n_tokens, bool unparse_special,
                             char * buffer, size_t n_buffer, size_t * out_n_bytes) {
    TWIN(retro_engine_detokenize(e, tokens, n_tokens, unparse_special, buffer, n_buffer, out_n_bytes));
}

int retro_trainer_generation_step(retro_trainer * trainer, const retro_step_row * rows, size_t n_rows,
                                  retro_step_out_row * out_rows, int32_t * out_top_ids, float * out_top_logprobs,
                                  size_t n_top_stride) {
    TWIN(retro_engine_step(e, rows, n_rows, out_rows, out_top_ids, out_top_logprobs, n_top_stride));
}
int retro_trainer_generation_step_v2(retro_trainer * trainer, const retro_step_row_v2 * rows, size_t n_rows,
                                     retro_step_out_row_v2 * out_rows, int32_t * out_top_ids, float * out_top_logprobs,
                                     size_t n_top_stride) {
    TWIN(retro_engine_step_v2(e, rows, n_rows, out_rows, out_top_ids, out_top_logprobs, n_top_stride));
}

int retro_trainer_generation_seq_rm(retro_trainer * trainer, int32_t slot, int32_t p0, int32_t p1) {
    TWIN(retro_engine_seq_rm(e, slot, p0, p1));
}
int retro_trainer_generation_seq_cp(retro_trainer * trainer, int32_t src, int32_t dst, int32_t p0, int32_t p1) {
    TWIN(retro_engine_seq_cp(e, src, dst, p0, p1));
}
int retro_trainer_generation_seq_save(retro_trainer * trainer, int32_t slot, uint32_t flags, uint8_t * buffer,
                                      size_t n_buffer, size_t * out_n_bytes) {
    TWIN(retro_engine_seq_save(e, slot, flags, buffer, n_buffer, out_n_bytes));
}
int retro_trainer_generation_seq_load(retro_trainer * trainer, int32_t slot, uint32_t flags, const uint8_t * buffer,
                                      size_t n_bytes, size_t * out_n_read) {
    TWIN(retro_engine_seq_load(e, slot, flags, buffer, n_bytes, out_n_read));
}
int retro_trainer_generation_seq_pos(retro_trainer * trainer, int32_t slot, int32_t * out_pos_min, int32_t * out_pos_max) {
    TWIN(retro_engine_seq_pos(e, slot, out_pos_min, out_pos_max));
}
int retro_trainer_generation_memory(retro_trainer * trainer, retro_engine_memory_info * out) {
    TWIN(retro_engine_memory(e, out));
}
int retro_trainer_generation_request_free(retro_trainer * trainer, int32_t request) {
    TWIN(retro_engine_request_free(e, request));
}

int retro_trainer_generation_kv_unified(retro_trainer * trainer, bool * out_unified) {
    TWIN(retro_engine_kv_unified(e, out_unified));
}
int retro_trainer_generation_weights_version(retro_trainer * trainer, uint64_t * out_version) {
    TWIN(retro_engine_weights_version(e, out_version));
}
int retro_trainer_model_fingerprint(retro_trainer * trainer, uint64_t * out_fingerprint) {
    TWIN(retro_engine_model_fingerprint(e, out_fingerprint));
}
int retro_trainer_is_hybrid(retro_trainer * trainer, bool * out_is_hybrid) { TWIN(retro_engine_is_hybrid(e, out_is_hybrid)); }

int retro_trainer_generate_batch(retro_trainer * trainer, const int32_t * prompt_tokens, size_t n_prompt,
                                 const retro_sampling_params * sampling, size_t n_sequences, int32_t * out_tokens,
                                 float * out_logprobs, size_t n_out_max, size_t * out_n_tokens, uint8_t * out_forced) {
    TWIN(retro_engine_generate_batch(e, prompt_tokens, n_prompt, sampling, n_sequences, out_tokens, out_logprobs,
                                     n_out_max, out_n_tokens, out_forced));
}
int retro_trainer_generate_continuous_batch(retro_trainer * trainer, const retro_generation_sequence * sequences,
                                            size_t n_sequences, int32_t * out_tokens, float * out_logprobs,
                                            size_t n_out_max, size_t * out_n_tokens, uint8_t * out_forced) {
    TWIN(retro_engine_generate_continuous_batch(e, sequences, n_sequences, out_tokens, out_logprobs, n_out_max,
                                                out_n_tokens, out_forced));
}
int retro_trainer_generate_continuous_batch_v2(retro_trainer * trainer, const retro_generation_sequence_v2 * sequences,
                                               size_t n_sequences, int32_t * out_tokens, float * out_logprobs,
                                               size_t n_out_max, size_t * out_n_tokens, uint8_t * out_forced) {
    retro_engine * e = checked(trainer);
    if (!e) return -1;
    try {
        clear_error();
        return e->impl.generate_continuous_batch_v2(sequences, n_sequences, out_tokens, out_logprobs, n_out_max, out_n_tokens, out_forced);
    } catch (const std::exception & ex) {
        set_error(ex.what());
        return -1;
    }
}
int retro_trainer_generation_stats(retro_trainer * trainer, retro_generation_stats * out_stats) {
    TWIN(retro_engine_generation_stats(e, out_stats));
}

int retro_trainer_generation_adapter_snapshot(retro_trainer * trainer, int32_t replace, float scale, int32_t * out_id) {
    return boundary([&]() -> int {
        retro_engine * e = checked(trainer);
        if (!e) return -1;
        if (!out_id) { set_error("out_id is required"); return -1; }
        return e->impl.adapter_snapshot(replace, scale, out_id);
    });
}
int retro_trainer_generation_adapter_unload(retro_trainer * trainer, int32_t id) {
    TWIN(retro_engine_adapter_unload(e, id));
}
int retro_trainer_get_generation_adapter(retro_trainer * trainer, int32_t * out_adapter) {
    return boundary([&]() -> int {
        retro_engine * e = checked(trainer);
        if (!e) return -1;
        if (!out_adapter) { set_error("out_adapter is required"); return -1; }
        *out_adapter = e->impl.default_adapter();
        return 0;
    });
}
int retro_trainer_set_generation_adapter(retro_trainer * trainer, int32_t adapter) {
    return boundary([&]() -> int {
        retro_engine * e = checked(trainer);
        if (!e) return -1;
        return e->impl.set_default_adapter(adapter);
    });
}
int retro_trainer_generation_adapter_rows_info(retro_trainer * trainer, retro_adapter_rows_info * out_info) {
    TWIN(retro_engine_adapter_rows_info(e, out_info));
}

#undef TWIN

}  // extern "C"
