/* The generation side of the reference's trainer handle: the twins of the step
 * surface that GRPO / PPO rollouts call on a `retro_trainer`, so that rollouts,
 * not only serving, go through the HIP decode step.
 *
 * Reference: crates/retrograd-ffi/runtime/include/retro_lora_train.h (line
 * numbers below are that file's), bound by crates/retrograd-ffi/src/lib.rs and
 * driven by crates/retrograd-infer/src/backend.rs:376-461 (TrainerBackend).
 *
 * What this library's trainer handle is: the dedicated generation context of
 * the reference's trainer (retro_backend.cpp:1218-1287: n_ctx x
 * generation_concurrency cells, generation_concurrency sequence slots, its own
 * batch geometry, unified f16 KV) plus the trained LoRA adapter that rows with
 * adapter 0 decode under. The optimizer, the training context and everything
 * that differentiates are not part of it: the train_*, score_*, save_* and
 * optimizer entry points of the reference header are not exported. New weights
 * arrive through retro_trainer_load_lora(), which does what the reference does
 * after every optimizer step: drops every resident cell and the generators'
 * bookkeeping, and bumps the weights version (retro_runtime.hpp:515-523).
 *
 * All functions return 0 on success and a negative status with
 * retro_last_error() set otherwise, as the engine entry points do. */
#ifndef RETRO_TRAINER_H
#define RETRO_TRAINER_H

#include "retro_step.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct retro_trainer retro_trainer;

/* retro_lora_train.h:944-1059. The layout is the reference's, field for field,
 * so that a caller's struct is read correctly; this library reads n_ctx,
 * n_batch, generation_concurrency, fast_generation_context, device,
 * generation_batch and generation_kv_dtype, validates what it reads as
 * retro_runtime.cpp:158-262 does, and ignores the optimizer's fields. */
typedef struct retro_train_config {
    uint32_t n_ctx;
    uint32_t n_batch;
    uint32_t n_ubatch;
    uint32_t n_seq_max;
    uint32_t generation_concurrency;   /* rollout sequences decoded together: slots of the generation context */
    bool fast_generation_context;      /* f16 KV for generation; the only KV this library has, so either value gives it */
    int32_t kv_dtype;
    uint32_t threads;
    uint32_t epochs;
    float learning_rate;
    float weight_decay;
    float max_grad_norm;
    int32_t lr_scheduler;
    uint64_t warmup_steps;
    bool verbose;
    int32_t device;                    /* retro_device; CPU is refused */
    bool chunked_cross_entropy;
    uint32_t chunked_ce_tiles;
    uint32_t chunked_ce_seq_chunk;
    bool chunked_ce_offload_logsoftmax;
    bool gradient_checkpointing;
    uint32_t checkpoint_every_n_layers;
    int32_t checkpoint_dtype;
    bool require_gpu_resident;
    uint32_t generation_batch;         /* n_batch of the generation context; 0 derives min(n_ctx, 512, 64 MiB of logits) */
    bool shuffle_dataset;
    int32_t optimizer;
    uint64_t shuffle_seed;
    int32_t trainable;
    float muon_momentum;
    float muon_ns_epsilon;
    float muon_fallback_learning_rate;
    uint32_t muon_ns_steps;
    bool muon_nesterov;
    int32_t gefen_variant;
    uint32_t gefen_block_size;
    float gefen_beta1;
    float gefen_beta2;
    float gefen_eps;
    int32_t master_weights;
    int32_t generation_kv_dtype;       /* retro_generation_kv_dtype: f16 (0), q8_0 (1), q4_0 (2) */
} retro_train_config;

/* :1532 / :2456. */
retro_trainer * retro_trainer_new(const char * model_path, const retro_train_config * train_config);
void retro_trainer_free(retro_trainer * trainer);

/* :1571. Loads a LoRA adapter file as the trained adapter (targets attn_q,
 * attn_k, attn_v, attn_output; rank <= 64). Every call is a weight change: the
 * generation KV and the generators' bookkeeping are dropped and the weights
 * version moves on. */
int retro_trainer_load_lora(retro_trainer * trainer, const char * adapter_path);

/* :1633-1639, :2037. context_size is the training context's n_ctx, as in the
 * reference; the generation context's pool is reported by generation_memory. */
int retro_trainer_eos_token(retro_trainer * trainer, int32_t * out_token);
int retro_trainer_vocab_size(retro_trainer * trainer, uint32_t * out_n_vocab);
int retro_trainer_is_eog_token(retro_trainer * trainer, int32_t token, bool * out_is_eog);
int retro_trainer_context_size(retro_trainer * trainer, uint32_t * out_n_ctx);
/* :1604-1632: text -> token ids on the generation engine's vocabulary, the twins of retro_engine_tokenize_text,
 * retro_engine_tokenize_fragment and retro_engine_tokenize (same two-call contract and return codes). */
int retro_trainer_tokenize_text(retro_trainer * trainer, const char * text, int32_t * tokens, size_t n_tokens_max, size_t * out_n_tokens);
int retro_trainer_tokenize_fragment(retro_trainer * trainer, const char * text, int32_t * tokens, size_t n_tokens_max, size_t * out_n_tokens);
int retro_trainer_tokenize_with(retro_trainer * trainer, const char * text, bool add_special, bool parse_special, int32_t * tokens,
                                size_t n_tokens_max, size_t * out_n_tokens);
int retro_trainer_detokenize(retro_trainer * trainer, const int32_t * tokens, size_t n_tokens, bool unparse_special,
                             char * buffer, size_t n_buffer, size_t * out_n_bytes);

/* :1906 and :1418: retro_engine_step / retro_engine_step_v2 on the generation
 * context. Rows with adapter 0 decode under the generation default (below):
 * the trained adapter unless told otherwise. */
int retro_trainer_generation_step(retro_trainer * trainer, const retro_step_row * rows, size_t n_rows,
                                  retro_step_out_row * out_rows, int32_t * out_top_ids, float * out_top_logprobs,
                                  size_t n_top_stride);
int retro_trainer_generation_step_v2(retro_trainer * trainer, const retro_step_row_v2 * rows, size_t n_rows,
                                     retro_step_out_row_v2 * out_rows, int32_t * out_top_ids, float * out_top_logprobs,
                                     size_t n_top_stride);

/* :1914-1936: the sequence operations, occupancy and request bookkeeping of the
 * generation context, same contracts as the engine's. */
int retro_trainer_generation_seq_rm(retro_trainer * trainer, int32_t slot, int32_t p0, int32_t p1);
int retro_trainer_generation_seq_cp(retro_trainer * trainer, int32_t src, int32_t dst, int32_t p0, int32_t p1);
int retro_trainer_generation_seq_save(retro_trainer * trainer, int32_t slot, uint32_t flags, uint8_t * buffer,
                                      size_t n_buffer, size_t * out_n_bytes);
int retro_trainer_generation_seq_load(retro_trainer * trainer, int32_t slot, uint32_t flags, const uint8_t * buffer,
                                      size_t n_bytes, size_t * out_n_read);
int retro_trainer_generation_seq_pos(retro_trainer * trainer, int32_t slot, int32_t * out_pos_min, int32_t * out_pos_max);
int retro_trainer_generation_memory(retro_trainer * trainer, retro_engine_memory_info * out);
int retro_trainer_generation_request_free(retro_trainer * trainer, int32_t request);

/* :1942-1945. The weights version counts the weight changes since creation. */
int retro_trainer_generation_kv_unified(retro_trainer * trainer, bool * out_unified);
int retro_trainer_generation_weights_version(retro_trainer * trainer, uint64_t * out_version);
int retro_trainer_model_fingerprint(retro_trainer * trainer, uint64_t * out_fingerprint);
int retro_trainer_is_hybrid(retro_trainer * trainer, bool * out_is_hybrid);

/* :1855, :1871, :2136: the batched generators and their reuse counters on the
 * generation context, under the generation default adapter. */
int retro_trainer_generate_batch(retro_trainer * trainer, const int32_t * prompt_tokens, size_t n_prompt,
                                 const retro_sampling_params * sampling, size_t n_sequences, int32_t * out_tokens,
                                 float * out_logprobs, size_t n_out_max, size_t * out_n_tokens, uint8_t * out_forced);
int retro_trainer_generate_continuous_batch(retro_trainer * trainer, const retro_generation_sequence * sequences,
                                            size_t n_sequences, int32_t * out_tokens, float * out_logprobs,
                                            size_t n_out_max, size_t * out_n_tokens, uint8_t * out_forced);
/* :1880-1897: the same over v2 rows (extended sampling, an optional grammar per row); every token is sampled through
 * the v2 chain with the row's own generator, history and grammar. out_logprobs holds the temperature-1 policy
 * log-probability of each emitted token, as the v1 entry point's does. Only on the trainer handle, as in the reference. */
int retro_trainer_generate_continuous_batch_v2(retro_trainer * trainer, const retro_generation_sequence_v2 * sequences,
                                               size_t n_sequences, int32_t * out_tokens, float * out_logprobs,
                                               size_t n_out_max, size_t * out_n_tokens, uint8_t * out_forced);
int retro_trainer_generation_stats(retro_trainer * trainer, retro_generation_stats * out_stats);

/* :1438-1453: per-row adapters of the generation context. A snapshot is a
 * frozen device-to-device copy of the trained adapter, selected per step row by
 * its id like an engine's per-row adapter, so a judge can decode under an older
 * policy in the same batch as the current one. `replace`, when not 0, is
 * unloaded first. The generation default is what rows with adapter 0 and the
 * batched generators decode under: 0 the trained adapter,
 * RETRO_STEP_ADAPTER_BASE the base model, or a snapshot id; changing it forgets
 * the generators' bookkeeping, the KV stays. */
int retro_trainer_generation_adapter_snapshot(retro_trainer * trainer, int32_t replace, float scale, int32_t * out_id);
int retro_trainer_generation_adapter_unload(retro_trainer * trainer, int32_t id);
int retro_trainer_get_generation_adapter(retro_trainer * trainer, int32_t * out_adapter);
int retro_trainer_set_generation_adapter(retro_trainer * trainer, int32_t adapter);
int retro_trainer_generation_adapter_rows_info(retro_trainer * trainer, retro_adapter_rows_info * out_info);

#ifdef __cplusplus
}
#endif

#endif /* RETRO_TRAINER_H */
