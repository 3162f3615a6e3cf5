/*
 * retro_kernels.h - kernel-level and state-inspection entry points of
 * libretro_hip.so. None of these has a counterpart in the reference's C ABI
 * (crates/retrograd-ffi/runtime/include/retro_lora_train.h): they exist so the
 * parity tests and micro-benchmarks can drive single gfx950 kernels, and read
 * back device state, through plain C calls. Same error convention as
 * retro_step.h (0 / -1 / -2, message in retro_last_error()).
 */
#ifndef RETRO_KERNELS_H
#define RETRO_KERNELS_H

#include "retro_step.h"

#ifdef __cplusplus
extern "C" {
#endif

/* y[t][n] (=|+=) sum_k W[n][k] * a[t][k] (+ bias[n]) with W given as n_rows raw
 * GGUF rows of `type`. The low byte of use_tiles picks the kernel: 0 the generic
 * one, 1 the register-only MFMA tile kernel, 2 the LDS-staged MFMA tile kernel
 * (tiles need K % 256 == 0, n_rows % 16 == 0, Q4_K or Q8_0). a is x (carried as
 * f16 hi/lo pairs) or, with bit 8 (0x100) of use_tiles set, x as ggml's CPU
 * matmul converts it for this weight type: Q8_K codes times their scale for
 * Q4_K, Q8_0 ones for Q8_0 and MXFP4, f16 / bf16 rounding for F16 / BF16.
 * With bit 9 (0x200) as well (Q4_K or Q8_0 tiles, at most two tokens) the conversion
 * leaves the converted blocks themselves and the integer matrix-vector kernel of very
 * small steps multiplies the codes; anything else with that bit is refused.
 * y is [n_tokens][n_rows] and is read first when accumulate is set. */
int retro_kernel_matmul(int32_t type, const uint8_t * raw, int64_t n_rows, int64_t k, const float * x,
                        int32_t n_tokens, int32_t use_tiles, const float * bias, int32_t accumulate, float * y);

/* The integer matrix-vector kernel with the producer of its rows fused into its staging, beside the same product
 * as two launches. kind 1: x is [n_tokens][k] residual rows, the rows multiplied are their RMSNorm (norm_w, eps)
 * converted as ggml converts them for the weight type; kind 2: x is [n_tokens][2 k] gate and up values in alternating
 * groups of `group` columns (0: side by side), the rows are silu(gate) * up converted likewise. raw: n_rows rows of
 * k, Q4_K (the rows become Q8_K blocks) or Q8_0 (Q8_0 blocks). Both results are [n_tokens][n_rows]; at most two
 * tokens. kinds 11 and 12: the same two producers for the exact arithmetic's matrix-vector kernel (one token): the row
 * stays f32 when the kernel makes it itself (y_fused) and is read back from the hi / lo f16 planes the producer's launch
 * leaves otherwise (y_unfused). */
int retro_kernel_gemv_fused(int32_t kind, int32_t type, const uint8_t * raw, int64_t n_rows, int64_t k, const float * x, const float * norm_w,
                            float eps, int32_t n_tokens, int32_t group, float * y_fused, float * y_unfused);

/* Per logits row: argmax (lowest id on ties), max, sum exp(double(l) - max),
 * and the k[r] best (id, logit) pairs in (logit desc, id asc) order, written
 * to out_top_*[r * retro_kernel_max_topk() + j]. */
int retro_kernel_sample_prepare(const float * logits, int32_t n_rows, int32_t n_vocab, const int32_t * k,
                                int32_t * out_argmax, float * out_max, double * out_sum_exp,
                                int32_t * out_top_ids, float * out_top_logits);

/* No counterpart in the reference. For callers that cannot allocate device
 * memory - code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc: the greedy scan of retro_kernel_sample_prepare (every row
 * with k = 1: argmax with the lowest id on ties, max, sum exp(double(l) - max))
 * over DEVICE buffers the caller owns, launched on the caller's stream
 * (a hipStream_t; NULL = the default stream), not waited for. The per-slice
 * partial results, which retro_kernel_sample_prepare keeps in a buffer it
 * allocates, live in a static device array of the library (64 KiB per GPU,
 * held until the process ends); the call allocates and frees nothing.
 * d_logits is [n_rows][n_vocab] f32; the three outputs hold n_rows entries.
 * At most retro_kernel_sample_greedy_noalloc_max_rows() (4096) rows per call:
 * more is refused with -1 and a message, nothing launched. Every call on one
 * GPU shares that GPU's array: calls that overlap there (two streams, two
 * threads) race; calls on one stream are ordered and need no clearing between
 * them. The array's address on a device is looked up once, by engine creation
 * or else by the first call on that device: in a process that creates no
 * engine, make the first call outside stream capture. */
int retro_kernel_sample_greedy_noalloc(const float * d_logits, int32_t n_rows, int32_t n_vocab,
                                       int32_t * d_out_argmax, float * d_out_max, double * d_out_sum_exp,
                                       void * stream);
int32_t retro_kernel_sample_greedy_noalloc_max_rows(void);

/* Micro-benchmark: microseconds per launch of one tile matmul (mode 1 register
 * tiles, 2 LDS-staged tiles, 3 the same with the K-slices left to the
 * consumer) over `iters` back-to-back launches on device-only data: weight
 * codes and activations are pseudo-random (constant operands let the pipes
 * clock higher and flatter the kernel by 15-20 %). Adding 16 to the mode gives
 * every launch another copy of the weights (1 GiB of copies in turn; adding 32,
 * 6 GiB), so that they are read from HBM as in a decode step instead of from
 * the last-level cache. debug must be 0 (the library carries no switches that
 * change results); force_ksplit > 0 overrides the number of K-slices for this
 * call. type is Q4_K, Q5_K, Q6_K or Q8_0 (Q5_K and Q6_K in modes 2 and
 * 3 only), n_rows a multiple of 16 and k of 256: anything else is refused
 * before a buffer is allocated. Mode 4 times the integer matrix-vector kernel
 * of very small steps under the ggml arithmetic instead (Q4_K or Q8_0, at most
 * two tokens, pseudo-random activation blocks), mode 5 the exact arithmetic's
 * matrix-vector kernel over the hi / lo planes (one token). */
int retro_kernel_matmul_time(int32_t type, int64_t n_rows, int64_t k, int32_t n_tokens, int32_t mode,
                             int32_t iters, int32_t debug, int32_t force_ksplit, double * out_us);

/* MXFP4 rows (GGUF block_mxfp4: an E8M0 byte and 16 nibble bytes per 32
 * values) times at most 16 tokens on the block-scaled FP4 x FP8 matrix
 * instruction. y is [n_tokens][n_rows].
 * exact == 0: ggml's arithmetic for this type - the activations become Q8_0
 * blocks (quantize_row_q8_0_ref), the integer code products of a block are
 * summed and scaled by both block scales (ggml_vec_dot_mxfp4_q8_0 of
 * ggml-org/llama.cpp@cd8427d0, the base of the fork pinned in reference
 * crates/retrograd-ffi/runtime/llama.cpp.lock:6-7). n_rows in 16s, k in 256s
 * and at most 4608 (the activation operands stay in LDS).
 * exact != 0: the f32 activations themselves, to f32-accumulation accuracy
 * (each written as a power of two times six signed hexadecimal digits, which
 * are exact FP8 values with power-of-two block scales). n_rows in 32s, k in
 * 256s.
 * Kernel-level entries for measurement and parity; the engine's expert block
 * runs the exact variant's mixture-of-experts form only under
 * RETRO_MOE_SCALED=1 (measured slower there than its default kernels). */
int retro_kernel_mxfp4_scaled(const uint8_t * raw, int64_t n_rows, int64_t k, const float * x, int32_t n_tokens, int32_t exact, float * y);
/* Microseconds per launch of the same product over pseudo-random device data;
 * cold != 0 gives every launch another copy of the weights (1 GiB of copies in
 * turn), so that they come from HBM. */
int retro_kernel_mxfp4_scaled_time(int64_t n_rows, int64_t k, int32_t n_tokens, int32_t exact, int32_t cold, int32_t iters, double * out_us);

/* Microseconds per launch of a plain streaming kernel over `bytes` of device
 * memory: a copy (reads and writes `bytes` each) or, read_only, a pure read.
 * Known traffic: the yardstick the memory counters and bandwidth figures of the
 * real kernels are scaled by. */
int retro_kernel_stream_time(int64_t bytes, int32_t read_only, int32_t iters, double * out_us);

int32_t retro_kernel_page_size(void);   /* positions per KV page */
int32_t retro_kernel_max_topk(void);    /* candidates sample_prepare can return */

/* Logits of the last step's sampling rows, [rows][n_vocab], in row order.
 * out == NULL only reports the row count. */
int retro_engine_debug_logits(retro_engine * engine, float * out, size_t n_floats, size_t * out_rows);
/* The stored K (want_v = 0) or V row of (layer, slot, pos) in natural element order: n_head_kv * head_dim
 * halves (an f16 cache), or - a Q8_0 cache - per kv head head_dim code bytes (code + 128) followed by
 * head_dim / 32 f16 block scales, n_head_kv * (head_dim / 2 + head_dim / 32) 16-bit units in all. */
int retro_engine_debug_kv(retro_engine * engine, int32_t layer, int32_t slot, int32_t pos, int32_t want_v,
                          uint16_t * out);
/* The device-side packing of the last step: per-token arrays and
 * counts[4] = tokens, outputs, attention tiles, attention work items. */
int retro_engine_debug_pack(retro_engine * engine, int32_t * tok, int32_t * pos, int32_t * seq, int32_t * cell,
                            int32_t * out_index, int32_t * last_index, size_t cap_tokens, size_t cap_rows,
                            int32_t * counts);
/* Page id per page index of a slot (-1 = none); out == NULL reports the length. */
int retro_engine_debug_pages(retro_engine * engine, int32_t slot, int32_t * out, size_t cap, size_t * out_n);

/* HIP-event timing of the step's kernel categories on the engine's own stream:
 * level 0 off, 1 attention only, 2 every category. Categories, in order: pack,
 * embed, norm, qkv, rope, attention, combine, o_proj, gate_up, swiglu, down,
 * head, sample. read() returns accumulated milliseconds and span counts. */
int retro_engine_debug_profile(retro_engine * engine, int32_t level);
int32_t retro_engine_debug_profile_categories(void);
int retro_engine_debug_profile_read(retro_engine * engine, double * out_ms, uint64_t * out_launches, int32_t reset);

/* Timeline of the decode attention launch (the one launch of a pure decode step that rotates, stores the KV cell,
 * attends and merges; one workgroup per row and kv head). While enabled, the launch of the model's middle layer
 * leaves six values per workgroup, in launch order of the workgroups: the GPU's constant 100 MHz clock at the
 * workgroup's start, after the prologue's barrier, when its first wave has attended its pages, after the barrier
 * behind all its waves, at its end, and the number of KV pages of its row. read() copies those of the last such
 * launch ([workgroups][6]; out == NULL reports the count; 0 workgroups when no step took that launch). */
int retro_engine_debug_attention_timeline(retro_engine * engine, int32_t enable);
int retro_engine_debug_attention_timeline_read(retro_engine * engine, uint64_t * out, size_t cap_workgroups, size_t * out_workgroups);

/* Single-token steps of the exact arithmetic on the matrix-vector kernel with f32 rows (RMSNorm and SwiGLU made in its
 * staging, the attention output read from the planes the attention launch leaves) instead of the tile kernels: what
 * RETRO_GEMV_EXACT=1 selects when the engine is created. Off by default: a sequence decoded alone then no longer gives
 * bit for bit the logprobs it gives inside a batch, which the tile kernels do for steps of up to 16 tokens and the
 * reference's tests hold (tests/engine_runtime.rs:713-722). */
int retro_engine_debug_single_token_matvec(retro_engine * engine, int32_t enable);

#ifdef __cplusplus
}
#endif

#endif /* RETRO_KERNELS_H */
