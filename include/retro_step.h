/*
 * retro_step.h - C ABI of the MI355X decode-step library (libretro_hip.so).
 *
 * Every declaration here carries the name, argument meaning, struct layout and
 * error convention of the declaration it replaces in the reference header
 * crates/retrograd-ffi/runtime/include/retro_lora_train.h (cited per item as
 * "ref h:LINE"), so the reference's Rust FFI crate (crates/retrograd-ffi/src/lib.rs,
 * `unsafe extern "C"` block from :1175) binds to this library unchanged for the
 * step path: what `impl DecodeBackend for Engine`
 * (crates/retrograd-infer/src/backend.rs:266-371) reaches.
 *
 * Conventions (ref h:2676-2711, retro_runtime.hpp:1255-1267):
 *   0  success
 *  -1  runtime failure            (retro_last_error() holds the message)
 *  -2  output buffer too small    (required size written to the out-param)
 *  -3  invalid argument, reported before anything is decoded
 * Every entry point clears the calling thread's error string on entry and turns
 * any C++ exception into -1. A handle is used from one thread at a time.
 * Pointers passed in are borrowed for the duration of the call only.
 */
#ifndef RETRO_STEP_H
#define RETRO_STEP_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ref h:15-23 */
typedef enum retro_device {
    RETRO_DEVICE_AUTO = 0,
    RETRO_DEVICE_CPU  = 1, /* refused by this library: there is no CPU path */
    RETRO_DEVICE_GPU  = 2,
} retro_device;

/* ref h:88-93. Only F16 is implemented; the others are refused at creation. */
typedef enum retro_engine_kv_dtype {
    RETRO_ENGINE_KV_DTYPE_F32  = 0,
    RETRO_ENGINE_KV_DTYPE_F16  = 1,
    RETRO_ENGINE_KV_DTYPE_Q8_0 = 2,
    RETRO_ENGINE_KV_DTYPE_Q4_0 = 3,
} retro_engine_kv_dtype;

/* ref h:819-822 */
enum retro_expert_placement {
    RETRO_EXPERT_PLACEMENT_DEVICE = 0,
    RETRO_EXPERT_PLACEMENT_HOST   = 1, /* refused: every tensor lives in HBM */
};

/* ref h:1260-1262 */
#define RETRO_STATE_SEQ_FLAGS_NONE         0u
#define RETRO_STATE_SEQ_FLAGS_PARTIAL_ONLY 1u
#define RETRO_STATE_SEQ_FLAGS_ON_DEVICE    2u

/* ref h:1296 */
#define RETRO_STEP_ADAPTER_BASE (-1)

/* The most sequence slots a context may have (llama.cpp's LLAMA_MAX_SEQ,
 * enforced at retro_engine.cpp:129-133). */
#define RETRO_MAX_SEQ 256

typedef struct retro_engine  retro_engine;
typedef struct retro_grammar retro_grammar;

/* ref h:1218-1223 (16 bytes) */
typedef struct retro_sampling_params {
    float    temperature;    /* finite, > 0 */
    float    top_p;          /* (0, 1] */
    uint32_t max_new_tokens; /* > 0 */
    uint32_t seed;
} retro_sampling_params;

/* ref h:1266-1292 (64 bytes, align 8) */
typedef struct retro_step_row {
    uint32_t        struct_size;
    int32_t         request;
    int32_t         slot;
    const int32_t * tokens;
    uint32_t        n;
    int32_t         pos0;
    bool            sample;
    retro_sampling_params sampling;
    uint32_t        n_top_logprobs;
    int32_t         adapter;
} retro_step_row;

/* ref h:1310-1318 (20 bytes, align 4) */
typedef struct retro_step_out_row {
    uint32_t struct_size;
    int32_t  token;
    float    logprob;
    uint32_t n_top;
    uint8_t  forced;
    uint8_t  sampled;
} retro_step_out_row;

/* ref h:1334-1350 (72 bytes, align 8) */
typedef struct retro_sampling_params_v2 {
    uint32_t struct_size;
    float    temperature;
    float    top_p;
    uint32_t max_new_tokens;
    uint32_t seed;
    int32_t  top_k;
    float    min_p;
    float    repeat_penalty;
    float    frequency_penalty;
    float    presence_penalty;
    uint32_t penalty_window;
    uint32_t n_logit_bias;
    const int32_t * logit_bias_ids;
    const float   * logit_bias_values;
    const retro_grammar * grammar;
} retro_sampling_params_v2;

/* ref h:1371-1383 (128 bytes, align 8) */
typedef struct retro_step_row_v2 {
    uint32_t        struct_size;
    int32_t         request;
    int32_t         slot;
    const int32_t * tokens;
    uint32_t        n;
    int32_t         pos0;
    bool            sample;
    retro_sampling_params_v2 sampling;
    uint32_t        n_top_logprobs;
    uint8_t         want_logprob;
    int32_t         adapter;
} retro_step_row_v2;

/* ref h:1385-1393 (24 bytes, align 4) */
typedef struct retro_step_out_row_v2 {
    uint32_t struct_size;
    int32_t  token;
    float    logprob;
    uint32_t n_top;
    uint8_t  forced;
    uint8_t  sampled;
    float    sampled_logprob;
} retro_step_out_row_v2;

/* ref h:1300-1306 (32 bytes, align 8) */
typedef struct retro_adapter_rows_info {
    uint32_t struct_size;
    uint32_t n_adapters;
    uint32_t max_rank;
    uint64_t stacked_bytes;
    uint64_t unpadded_bytes;
} retro_adapter_rows_info;

/* ref h:1472-1482 (40 bytes, align 8) */
typedef struct retro_engine_memory_info {
    uint32_t struct_size;
    uint32_t n_slots;
    uint64_t cells_total;
    uint64_t cells_used;
    uint64_t kv_bytes;
    uint64_t recurrent_bytes;
} retro_engine_memory_info;

/* ref h:2470-2494 (64 bytes, align 8). Versioned by struct_size: only the
 * prefix the caller's struct_size covers is read (retro_engine.cpp:474-494). */
typedef struct retro_engine_config {
    uint32_t struct_size;
    uint32_t n_ctx;
    uint32_t n_seq_max;
    uint32_t n_batch;
    uint32_t n_ubatch;
    int32_t  kv_dtype;
    bool     flash_attn;
    int32_t  device;
    uint32_t threads;
    bool     verbose;
    uint32_t kv_unified;
    int32_t  expert_placement;
    uint32_t expert_host_layers;
    uint64_t expert_device_cache_bytes;
} retro_engine_config;

/* ---- lifetime: ref h:2498, h:2504, h:2509 ------------------------------- */
retro_engine * retro_engine_new(const char * model_path, const retro_engine_config * config);
retro_engine * retro_engine_new_checked(
    const char * model_path, const retro_engine_config * config, bool * out_invalid_placement);
void retro_engine_free(retro_engine * engine);

/* ---- the step: ref h:2712-2719 (v1), h:1410-1417 (v2) -------------------- */
int retro_engine_step(
    retro_engine * engine, const retro_step_row * rows, size_t n_rows,
    retro_step_out_row * out_rows, int32_t * out_top_ids, float * out_top_logprobs,
    size_t n_top_stride);
int retro_engine_step_v2(
    retro_engine * engine, const retro_step_row_v2 * rows, size_t n_rows,
    retro_step_out_row_v2 * out_rows, int32_t * out_top_ids, float * out_top_logprobs,
    size_t n_top_stride);

/* ---- sequence operations: ref h:2724, 2728, 2738, 2751, 2761, 2765, 2769 - */
int retro_engine_seq_rm(retro_engine * engine, int32_t slot, int32_t p0, int32_t p1);
int retro_engine_seq_cp(retro_engine * engine, int32_t src, int32_t dst, int32_t p0, int32_t p1);
int retro_engine_seq_save(
    retro_engine * engine, int32_t slot, uint32_t flags,
    uint8_t * buffer, size_t n_buffer, size_t * out_n_bytes);
int retro_engine_seq_load(
    retro_engine * engine, int32_t slot, uint32_t flags,
    const uint8_t * buffer, size_t n_bytes, size_t * out_n_read);
int retro_engine_seq_pos(
    retro_engine * engine, int32_t slot, int32_t * out_pos_min, int32_t * out_pos_max);
int retro_engine_memory(retro_engine * engine, retro_engine_memory_info * out);
int retro_engine_request_free(retro_engine * engine, int32_t request);

/* ---- batched generators on top of the step: ref h:1238-1242, 1123-1131,
 * 2511-2534, 2672-2674 (contract text h:1844-1879) --------------------------
 * The whole generation loop inside one call, over the same step and the same
 * sampling oracle (mt19937 seeded once per sequence), so a caller-side loop of
 * retro_engine_step calls composed in the canonical order reproduces them bit
 * for bit (h:2696-2698).
 * Outputs are row-major with a stride of n_out_max. A row stops at
 * max_new_tokens, at an end-of-generation token (included), or when its
 * sequence context is full. out_logprobs may be NULL; otherwise it receives the
 * temperature-1 policy log-probability of every emitted token. out_n_tokens
 * holds n_sequences counts. out_forced may be NULL; otherwise all zeros (no
 * reasoning budget in this build). Returns 0, or -1 with retro_last_error(). */

/* ref h:1238-1242 */
typedef struct retro_generation_sequence {
    const int32_t * prompt_tokens;
    size_t          n_prompt;
    retro_sampling_params sampling;
} retro_generation_sequence;

/* ref h:1352-1362: a row of the v2 continuous generator - the prompt and the extended sampling parameters, an
 * optional grammar handle among them, which constrains every token the row samples. */
typedef struct retro_generation_sequence_v2 {
    const int32_t * prompt_tokens;
    size_t          n_prompt;
    retro_sampling_params_v2 sampling;
} retro_generation_sequence_v2;

/* ref h:1123-1131: lifetime counters of the continuous generator's slot-level
 * prefix reuse; a caller attributes one call by differencing two snapshots. */
typedef struct retro_generation_stats {
    uint64_t calls;
    uint64_t sequences;
    uint64_t prompt_tokens;      /* what the callers asked to be resident before sampling */
    uint64_t prefilled_tokens;   /* what was decoded to get there */
    uint64_t reused_tokens;
    uint64_t hits;
    uint64_t evictions;
} retro_generation_stats;

/* ref h:2514-2524 (retro_gen_core.cpp:1696-1876): n_sequences completions of
 * one prompt. The prompt is decoded once, its KV copied to one slot per member
 * (slot i for member i), and all live members advance in one step per token.
 * Starts from, and leaves, an empty KV. */
int retro_engine_generate_batch(
    retro_engine * engine, const int32_t * prompt_tokens, size_t n_prompt,
    const retro_sampling_params * sampling, size_t n_sequences,
    int32_t * out_tokens, float * out_logprobs, size_t n_out_max, size_t * out_n_tokens,
    uint8_t * out_forced);

/* ref h:2526-2534 (retro_gen_core.cpp:317-707, 1878-2049): one completion per
 * input, heterogeneous prompts. Every launch is built in the canonical order
 * of the contents (prompt length, prompt tokens, seed, max_new_tokens,
 * temperature, top_p), equal prompts are prefilled once and copied, and the
 * slots keep what they decoded between calls: a later call whose prompt
 * strictly extends a slot's resident tokens decodes only the extension.
 * RETRO_GENERATION_PREFIX_CACHE=0 (or "false") in the environment turns the
 * reuse off: every call then starts and ends with an empty KV. A step or a raw
 * sequence operation through this ABI forgets what the slots hold. */
int retro_engine_generate_continuous_batch(
    retro_engine * engine, const retro_generation_sequence * sequences, size_t n_sequences,
    int32_t * out_tokens, float * out_logprobs, size_t n_out_max, size_t * out_n_tokens,
    uint8_t * out_forced);

/* ref h:2672-2674 */
int retro_engine_generation_stats(retro_engine * engine, retro_generation_stats * out_stats);

/* ---- introspection: ref h:2775, 2799, 2803, 2808, 2550-2561, 2612 -------- */
int retro_engine_kv_unified(retro_engine * engine, bool * out_unified);
int retro_engine_weights_version(retro_engine * engine, uint64_t * out_version);
int retro_engine_model_fingerprint(retro_engine * engine, uint64_t * out_fingerprint);
int retro_engine_is_hybrid(retro_engine * engine, bool * out_is_hybrid);
/* ref h:2890-2899: the text of one token (what detokenize appends for it); `special` renders a control token as its
 * text instead of nothing. Two calls: with no buffer the byte count is reported, a buffer that is too small returns -2. */
int retro_engine_token_piece(retro_engine * engine, int32_t token, bool special, char * buffer, size_t n_buffer, size_t * out_n_bytes);

/* ref h:2538-2549, 2879-2889 (retro_engine.cpp:331-378, 594-622): text -> token ids. tokenize_text adds the model's
 * BOS / EOS and reads the text of a special token as that token; tokenize_fragment adds nothing; tokenize takes both
 * flags. Two calls: with tokens == NULL or n_tokens_max == 0 the count is reported; a buffer that is too small returns
 * -2 with the count. Built for sentencepiece-kind vocabularies (tokenizer.ggml.model = "llama") and for byte-level
 * byte-pair ones ("gpt2") whose tokenizer.ggml.pre names the Llama 3, Qwen 2 or GPT-2 pattern; any other returns -1. */
int retro_engine_tokenize_text(retro_engine * engine, const char * text, int32_t * tokens, size_t n_tokens_max, size_t * out_n_tokens);
int retro_engine_tokenize_fragment(retro_engine * engine, const char * text, int32_t * tokens, size_t n_tokens_max, size_t * out_n_tokens);
int retro_engine_tokenize(retro_engine * engine, const char * text, bool add_special, bool parse_special, int32_t * tokens,
                          size_t n_tokens_max, size_t * out_n_tokens);
int retro_engine_eos_token(retro_engine * engine, int32_t * out_token);
int retro_engine_vocab_size(retro_engine * engine, uint32_t * out_n_vocab);
int retro_engine_is_eog_token(retro_engine * engine, int32_t token, bool * out_is_eog);
int retro_engine_context_size(retro_engine * engine, uint32_t * out_n_ctx);
int retro_engine_detokenize(
    retro_engine * engine, const int32_t * tokens, size_t n_tokens, bool unparse_special,
    char * buffer, size_t n_buffer, size_t * out_n_bytes);
int retro_engine_graphs_reused(retro_engine * engine, uint64_t * out_n_reused);

/* ---- adapters: ref h:2566-2567 (the one context-wide adapter), h:2574, 2584, 2616 (named), h:2597-2605 (per row).
 * The active context-wide adapter is what rows with adapter 0 decode under. Every change of what is active
 * is a weight change: all cells and the generators' bookkeeping are dropped, the weights version moves on. */
int retro_engine_load_lora(retro_engine * engine, const char * adapter_path);
int retro_engine_set_lora_enabled(retro_engine * engine, bool enabled);
int retro_engine_load_lora_named(retro_engine * engine, const char * name, const char * adapter_path);
int retro_engine_activate_lora(retro_engine * engine, const char * name);
int retro_engine_active_adapter(
    retro_engine * engine, char * buffer, size_t n_buffer, size_t * out_n_bytes);
int retro_engine_adapter_load(
    retro_engine * engine, const char * adapter_path, float scale, int32_t * out_id);
int retro_engine_adapter_unload(retro_engine * engine, int32_t id);
int retro_engine_adapter_rows_info(retro_engine * engine, retro_adapter_rows_info * out_info);

/* ---- grammar handles: ref h:1395-1408 ------------------------------------
 * A handle owns a GBNF string; all three constructors return NULL with the error set on failure. from_gbnf takes the
 * text as it is (it is compiled by the step that carries it: -3 there when it is invalid); json_object is a grammar
 * for one JSON object; from_json_schema converts a subset of JSON Schema and names the keyword it cannot convert.
 * The handle may be freed as soon as the step call that carried it returns. */
retro_grammar * retro_grammar_from_json_schema(const char * json_schema);
retro_grammar * retro_grammar_from_gbnf(const char * gbnf);
retro_grammar * retro_grammar_json_object(void);
const char *    retro_grammar_gbnf(const retro_grammar * grammar);
void            retro_grammar_free(retro_grammar * grammar);

/* ref h:3038. Thread-local; "no runtime error" when empty. */
const char * retro_last_error(void);

#ifdef __cplusplus
}
#endif

#endif /* RETRO_STEP_H */
