/* C ABI of the step scheduler (the policy that composes every decode step).
 *
 * The reference implements this layer in Rust (crates/retrograd-infer) and
 * exposes it as a crate API, not as C functions, so these entry points have no
 * C counterpart there: each one names the Rust item it mirrors. A Rust
 * maintainer would bind them with an `unsafe extern "C"` block and implement
 * `retrograd_infer`'s public types on top.
 *
 * Every function returns 0 on success and a negative code otherwise:
 * -(retro_sched_error_kind) of the failure, with the message available from
 * retro_last_error() on the calling thread and the structured fields from
 * retro_sched_last_error_detail(). A scheduler and its streams belong to one
 * thread at a time (the synchronous driver of the reference). */
#ifndef RETRO_SCHEDULER_H
#define RETRO_SCHEDULER_H

#include "retro_step.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct retro_scheduler    retro_scheduler;
typedef struct retro_sched_stream retro_sched_stream;

/* InferError (crates/retrograd-infer/src/error.rs:8-27) */
typedef enum retro_sched_error_kind {
    RETRO_SCHED_ERR_INVALID    = 1,
    RETRO_SCHED_ERR_FAILED     = 2,
    RETRO_SCHED_ERR_OVERFLOW   = 3,
    RETRO_SCHED_ERR_QUEUE_FULL = 4,
    RETRO_SCHED_ERR_KV_FULL    = 5,
    RETRO_SCHED_ERR_CANCELLED  = 6,
    RETRO_SCHED_ERR_BACKEND    = 7,
} retro_sched_error_kind;

/* AdmissionMode (scheduler.rs:69-77) */
enum { RETRO_SCHED_LOCKSTEP = 0, RETRO_SCHED_CONTINUOUS = 1 };

/* SchedulerOptions (scheduler.rs:86-135); the defaults of the reference are
 * written by retro_sched_options_default. Durations are nanoseconds. */
typedef struct retro_sched_options {
    uint32_t struct_size;
    int32_t  mode;
    uint64_t n_batch;
    uint64_t queue_capacity;
    uint64_t event_capacity;
    uint64_t slow_client_timeout_ns;
    uint8_t  prefix_cache;
    uint64_t min_prefix_len;
    uint64_t max_snapshot_bytes;
    uint64_t swap_min_tokens;
    uint64_t max_retained;
    uint64_t retain_ttl_ns;
} retro_sched_options;
void retro_sched_options_default(retro_sched_options * out);

/* Request (request.rs:16-47). sampling[i].grammar must be NULL; grammar_gbnf,
 * when given, holds one GBNF text (or NULL) per sampling entry. */
typedef struct retro_sched_request {
    uint32_t struct_size;
    const int32_t * prompt;
    size_t   n_prompt;
    const retro_sampling_params_v2 * sampling;
    size_t   n_sampling;
    const char * const * grammar_gbnf;
    const char * const * stop;
    size_t   n_stop;
    uint32_t n_top_logprobs;
    uint8_t  logprobs;
    const char * adapter;            /* NULL = base model */
    uint8_t  unparse_special;
    const char * retention_key;      /* NULL = no retention */
    const char * retention_release;  /* NULL = releases nothing */
} retro_sched_request;

/* Event (request.rs:227-257), TokenEvent (:172-198), FinishReason (:211-224) */
enum { RETRO_SCHED_EVENT_TOKEN = 0, RETRO_SCHED_EVENT_END = 1, RETRO_SCHED_EVENT_ERROR = 2 };
enum { RETRO_SCHED_FINISH_EOG = 0, RETRO_SCHED_FINISH_STOP = 1, RETRO_SCHED_FINISH_MAX_TOKENS = 2,
       RETRO_SCHED_FINISH_CONTEXT_FULL = 3, RETRO_SCHED_FINISH_CANCELLED = 4 };
typedef struct retro_sched_event {
    uint32_t struct_size;
    int32_t  type;
    uint64_t index;
    int32_t  token;
    float    logprob;
    uint8_t  has_sampled_logprob;
    float    sampled_logprob;
    uint8_t  forced;
    const char * text;  size_t n_text;     /* Token: newly emittable text; End: the flushed tail */
    const char * piece; size_t n_piece;
    size_t   n_top;
    const int32_t * top_ids;
    const float *   top_logprobs;
    const char * const * top_pieces;
    const size_t *  top_piece_lens;
    int32_t  reason;
    uint64_t cached_tokens;
    int32_t  error_kind;
    const char * error_message;
    uint64_t error_needed, error_available;
} retro_sched_event;

/* KvStats (kv.rs:100-118) */
typedef struct retro_sched_kv_stats {
    uint32_t struct_size;
    uint64_t hits, misses, prefilled_cells, prompt_cells, evictions, swaps;
    uint64_t nodes, resident_slots, snapshot_bytes;
} retro_sched_kv_stats;

/* Scheduler::new over an engine (`impl DecodeBackend for Engine`, backend.rs:266-371). The engine is
 * borrowed: it must outlive the scheduler and is freed by the caller. */
retro_scheduler * retro_scheduler_new(retro_engine * engine, const retro_sched_options * options);
/* Scheduler::new over a trainer's generation context (`impl DecodeBackend for TrainerBackend`,
 * backend.rs:376-461): rollouts admitted, batched and prefix-cached like serving requests. Rows decode
 * under the trainer's generation default adapter; the per-sequence context is the whole generation pool
 * (backend.rs:446-453); a weight change moves weights_version on, which makes the scheduler drop every
 * cached prefix (scheduler.rs, refresh_key). The trainer is borrowed like the engine above. */
struct retro_trainer;
retro_scheduler * retro_scheduler_new_trainer(struct retro_trainer * trainer, const retro_sched_options * options);
/* Scheduler::new over FakeBackend::new(n_slots, n_ctx_seq, cells_total, vocab, eos, pieces) (fake.rs:77-118):
 * the in-memory backend the reference tests its policy with. */
retro_scheduler * retro_scheduler_new_fake(uint32_t n_slots, uint32_t n_ctx_seq, uint64_t cells_total, uint32_t vocab,
                                           int32_t eos, const char * const * pieces, size_t n_pieces,
                                           const retro_sched_options * options);
void retro_scheduler_free(retro_scheduler * s);

int retro_scheduler_initialize(retro_scheduler * s);                                       /* scheduler.rs:665 */
int retro_scheduler_submit(retro_scheduler * s, const retro_sched_request * request,
                           retro_sched_stream ** out_stream);                              /* scheduler.rs:687 */
int retro_scheduler_pump(retro_scheduler * s, uint8_t * out_progressed);                   /* scheduler.rs:736 */
int retro_scheduler_run_until_idle(retro_scheduler * s);                                   /* scheduler.rs:783 */
int retro_scheduler_counts(retro_scheduler * s, uint64_t * out_queued, uint64_t * out_live);  /* queued_len, live_len */
int retro_scheduler_fail_queued(retro_scheduler * s);                                      /* scheduler.rs:631 */
int retro_scheduler_kv_stats(retro_scheduler * s, retro_sched_kv_stats * out);             /* scheduler.rs:427 */
int retro_scheduler_pin_prefix(retro_scheduler * s, const int32_t * prefix, size_t n, uint64_t * out_pin);  /* :534 */
int retro_scheduler_unpin(retro_scheduler * s, uint64_t pin, uint8_t * out_released);      /* scheduler.rs:542 */
/* lend_slot (scheduler.rs:746-777): a slot that no live sequence and no dormant prefix holds, with `cells` of the
 * pool free beside the dormant prefixes, evicting least recently used prefix nodes until both fit; *out_slot = -1
 * when nothing more can be evicted. Fails while a sequence is live. The caller empties the slot before the next pump. */
int retro_scheduler_lend_slot(retro_scheduler * s, uint64_t cells, int32_t * out_slot);
int retro_scheduler_queue_capacity(retro_scheduler * s, size_t * out_capacity);            /* scheduler.rs, queue_capacity */
int retro_scheduler_load_adapter(retro_scheduler * s, const char * name, const char * path);   /* scheduler.rs:454 */
int retro_scheduler_unload_adapter(retro_scheduler * s, const char * name);                /* scheduler.rs:488 */
int retro_scheduler_set_mode(retro_scheduler * s, int32_t mode);
void retro_sched_last_error_detail(uint64_t * out_needed, uint64_t * out_available, uint64_t * out_capacity);

/* EventStream (request.rs:259-308). poll: 0 = an event was written to *out (its pointers stay valid until the
 * next call on this stream), 1 = empty but open, 2 = closed. Freeing a stream is dropping it: the request is
 * cancelled at the next step. */
int  retro_sched_stream_poll(retro_sched_stream * stream, retro_sched_event * out);
void retro_sched_stream_free(retro_sched_stream * stream);

/* FakeBackend script and log (fake.rs:22-75), only on a scheduler made by retro_scheduler_new_fake.
 * set: "eog_after" (-1 = never), "kv_unified", "recurrent", "row_adapters", "fail_after_steps" (-1 = never),
 *      "bump_weights_version" (value ignored). */
int retro_sched_fake_set(retro_scheduler * s, const char * key, int64_t value);
int retro_sched_fake_script(retro_scheduler * s, const int32_t * tokens, size_t n);
int retro_sched_fake_register_adapter(retro_scheduler * s, const char * name, const char * path);
int retro_sched_fake_cells_used(retro_scheduler * s, uint64_t * out);
/* Log read-out: `what` is "steps" (5 ints per row: step, slot, n, request or -1, adapter), "copies" (4 ints),
 * "removed" (1), "request_order" (1), "saves" / "loads" (3: slot, flags, len). Returns the number of ints
 * through *out_n and copies up to n_buffer of them. */
int retro_sched_fake_log(retro_scheduler * s, const char * what, int64_t * buffer, size_t n_buffer, size_t * out_n);
/* adapter operations as "op:name" lines joined by '\n' (two-call string contract). */
int retro_sched_fake_adapter_ops(retro_scheduler * s, char * buffer, size_t n_buffer, size_t * out_n_bytes);

#ifdef __cplusplus
}
#endif

#endif /* RETRO_SCHEDULER_H */
