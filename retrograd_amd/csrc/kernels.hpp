// Host-side launch interface of the gfx950 kernels behind the decode step.
// Everything here is plain C++ over HIP pointers; the C ABI lives in capi.cpp.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstddef>
#include <cstdint>

namespace rk {

// ggml tensor type ids as stored in GGUF.
enum : int { WT_F32 = 0, WT_F16 = 1, WT_Q4_1 = 3, WT_Q5_1 = 7, WT_Q8_0 = 8, WT_Q2_K = 10, WT_Q4_K = 12, WT_Q5_K = 13, WT_Q6_K = 14,
              WT_IQ4_XS = 23, WT_BF16 = 30, WT_MXFP4 = 39 };

// One KV page holds PAGE consecutive positions of one sequence.
constexpr int PAGE = 32;
// One attention work item scans at most split_pages pages of one sequence;
// count_attention_work picks the step's split, at most MAX_SPLIT_PAGES.
constexpr int MAX_SPLIT_PAGES = 16;
// Candidates the sampling kernel can return per row.
constexpr int MAX_TOPK = 64;

struct BlockGeom { int elements; int bytes; };
BlockGeom geom_of(int type);                 // throws on an unknown type
size_t row_bytes(int type, int64_t k);       // throws when k is not block aligned

// A weight matrix [N rows][K] in HBM. Exactly one of raw/packed is set:
// `raw` keeps the GGUF row-major block layout (generic kernel, row gathers);
// `packed` is the MFMA tile layout of the same bytes (K % 256 == 0, N % 16 == 0).
struct Weight {
    int type = 0;
    int K = 0;
    int N = 0;
    const uint8_t * raw = nullptr;
    const uint8_t * packed = nullptr;
    size_t bytes = 0;
    const uint8_t * records = nullptr;      // MXFP4 expert rows again, in the records of the block-scaled kernels (mxs_repack)
};

// Activations handed to a matmul. An f32 value v travels as two f16 numbers,
// hi = f16(v) and lo = f16(v - hi), which together carry about 22 significant
// bits. For every 32-wide block of a row the f32 sum of hi + lo is kept as
// well, split the same way; the sums are what the Q4_K min term multiplies.
//
// ggml's CPU matmul does not multiply a quantised weight with the f32
// activations themselves: it first converts the row to the weight type's
// companion format (Q8_K blocks of 256 for Q4_K; Q8_0 blocks of 32 for Q8_0 and
// MXFP4; f16 / bf16 rounding for F16 / BF16 weights) and multiplies the codes.
// An engine can run either arithmetic. In the ggml one (`faithful`) a producer
// writes up to two versions of a row: the values as they are (x, sums: what
// F32 / F16 / BF16 weights, the expert router and LoRA factors read, the latter
// rounding on the way) and the values after the conversion, scale times code
// (qx, qsums, with `quant` the block rule), which the quantised weights read.
// In the exact one only x and sums exist and every consumer reads them.
//
// All buffers are stored in MFMA operand order, so that a matmul stages them
// with contiguous 1 KiB loads. Tokens are grouped in chunks of 64 (4 tiles of
// 16); with Kp = K rounded up to 32:
//   x:    [chunk][k / 32][hi, lo][tile][lane = 16 * ((k % 32) / 8) + token % 16][k % 8]
//   sums: [chunk][k / 256][tile][lane = 16 * (hi: 0, lo: 1) + token % 16][(k % 256) / 32]
// The sums blocks also have lanes 32-63, which stay zero from allocation: they
// pad the operand of the min-term MFMA.
enum : int { AQ_NONE = 0, AQ_Q8_0 = 32, AQ_Q8_K = 256 };
// The conversion ggml's CPU matmul applies for a weight of this storage type.
inline int act_quant_of(int ggml_type) {
    switch (ggml_type) {
        case 10: case 12: case 13: case 14: case 23: return AQ_Q8_K;   // Q2_K, Q4_K, Q5_K, Q6_K, IQ4_XS
        case 3: case 7: case 8: case 39: return AQ_Q8_0;    // Q4_1, Q5_1 (Q8_1 has Q8_0's codes and scale), Q8_0, MXFP4
        default: return AQ_NONE;
    }
}
struct Act {
    __half * x = nullptr;       // act_halves(T, K) halves
    __half * sums = nullptr;    // act_sum_halves(T, K) halves, zero-initialised; null when K % 32 != 0
    int K = 0;
    __half * qx = nullptr;      // the converted row, same layouts
    __half * qsums = nullptr;
    int quant = AQ_NONE;
    int faithful = 0;           // ggml's arithmetic: F16 / BF16 operands are rounded as well
    // A producer can leave the blocks of the conversion themselves as well, for the integer matrix-vector
    // kernel that multiplies very small steps (gemv). Q8_K: the int8 codes [token][K], the eight codes of a
    // group k / 8 in the order 0 4 1 5 2 6 3 7 (act_code_pos; the order in which a Q4_K tile's nibbles unpack
    // into bytes); the block scales 1 / iscale, f32 [token][K / 256]; and the sums of the codes of every 16,
    // int16 [token][K / 16] (ggml's bsums). Q8_0: the codes in element order, the scales (f16 values) as f32 [token][K / 32],
    // no sums.
    int8_t * qc = nullptr;
    float * qd = nullptr;
    int16_t * qbs = nullptr;
    // What a weight of this type multiplies: the converted row for the quantised
    // types under ggml's arithmetic, the values themselves otherwise.
    Act operand(int ggml_type) const {
        Act a;
        a.K = K;
        a.faithful = faithful;
        if (faithful && act_quant_of(ggml_type) != AQ_NONE) {
            a.x = qx; a.sums = qsums;
            if (act_quant_of(ggml_type) == quant) { a.qc = qc; a.qd = qd; a.qbs = qbs; a.quant = quant; }
        } else { a.x = x; a.sums = sums; }
        return a;
    }
};
constexpr int act_code_pos(int i) { return (i & 3) * 2 + (i >> 2); }    // byte of code i within its group of eight
inline size_t act_halves(int T, int K) { return (size_t)((T + 63) / 64) * (size_t)((K + 31) / 32 * 32) * 128; }
inline size_t act_sum_halves(int T, int K) { return (size_t)((T + 63) / 64) * (size_t)((K + 255) / 256) * 2048; }

// dst = src (16-byte words, grid-stride) or, read_only, a pure read of src
// (dst needs 64 KiB): plain streaming kernels of known traffic.
void stream_copy(hipStream_t s, const void * src, void * dst, size_t bytes, int read_only);

bool can_pack(int type, int64_t K, int64_t N);
// raw (device, GGUF layout) -> packed (device). Both hold `bytes` bytes.
void repack(hipStream_t s, int type, const uint8_t * raw, uint8_t * packed, int K, int N);

enum : int { MM_STORE = 0, MM_ADD = 1, MM_SWIGLU = 2 };
// A matmul result left as n K-slices in the workspace instead of in y: element
// (t, c) of the product (bias included) is the sum over s < n, in that order,
// of data[s * stride + t * N + c]. n == 0: there are no slices, y holds the result.
struct Slices {
    const float * data = nullptr;
    int n = 0;
    size_t stride = 0;
    int N = 0;
    // or (weight != null) a weighted sum of n rows per row: term j of row t is weight[t n + j] * data[t n + j][:] - or
    // data[gather[t n + j]][:] with a gather list - the terms added with fused multiply-adds in order j, their sum added
    // to the row (what k_moe_combine computes)
    const float * weight = nullptr;
    const int32_t * gather = nullptr;
};
// y[t][col0 + n] (=|+=) sum_k W[n][k] * x[t][k] (+ bias[n]); y has row stride ldy.
// `ws` is a device workspace of matmul_workspace_bytes() that selects the
// LDS-staged tile kernels; without it the register-only tile kernels run.
void matmul(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0,
            int mode, const float * bias, void * ws = nullptr);
// The same product, but a decode-sized matmul with few output rows may return
// it as K-slices in ws and leave y untouched: the caller hands the slices to
// the kernel that consumes the result (rmsnorm_act, rope_store) or to
// reduce_slices. The slices live until the next matmul that uses ws.
Slices matmul_deferred(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0,
                       int mode, const float * bias, void * ws);
// y[t][col0 + c] (=|+=) sum of the slices.
void reduce_slices(hipStream_t s, const Slices & sl, int T, float * y, int ldy, int col0, int mode);
size_t matmul_workspace_bytes();
// The integer matrix-vector kernel: a Q4_K (Q8_0) tile matrix times the Q8_K (Q8_0) blocks of one or two
// tokens, as ggml's CPU dot products multiply them (integer sums of code products per block, Q4_K: times
// the integer sub-block scale, one float multiply per super-block). One workgroup per 16-row tile, the
// waves of a workgroup share the tile's super-blocks; no K-slices. x is the operand (Act::operand) of the weight.
constexpr int GEMV_MAX_T = 2;     // beyond two tokens the tile kernels are as fast
bool gemv_can(const Weight & w, const Act & x, int T);
void gemv(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0, int mode, const float * bias);
// MXFP4 weights times the Q8_0 blocks of at most MXS_MAX_TOKENS tokens on the block-scaled FP4 x FP8 matrix
// instruction (ggml's arithmetic for MXFP4: integer code products per block of 32, times both block scales).
// mxs_repack lays the GGUF rows out in the kernel's records (mxs_packed_bytes), mxs_quantise converts f32 rows to
// the kernel's activation operands (mxs_operand_bytes) and block scales (mxs_scale_bytes), mxs_matmul writes
// y [n_tokens][N]. Columns in 128s, rows in 16s; K is bounded by the operands having to fit LDS (mxs_lds_bytes).
constexpr int MXS_MAX_TOKENS = 16;
bool mxs_can(int64_t K, int64_t N, int n_tokens);
size_t mxs_packed_bytes(int64_t K, int64_t N);
size_t mxs_operand_bytes(int K);
size_t mxs_scale_bytes(int K);
size_t mxs_lds_bytes(int K);
void mxs_repack(hipStream_t s, const uint8_t * raw, uint8_t * packed, int K, int64_t N);
void mxs_quantise(hipStream_t s, const float * x, int n_tokens, int K, uint8_t * operands, float * scales);
void mxs_matmul(hipStream_t s, const uint8_t * packed, const uint8_t * operands, const float * scales, int K, int64_t N,
                int n_tokens, float * y);
// The same product on f32 activations to f32-accumulation accuracy: mxe_pieces writes every activation as a power of
// two times six signed hexadecimal digits (operands mxe_operand_bytes, scales mxe_scale_bytes), mxe_matmul multiplies
// them with the records mxs_repack made (rows in 32s, columns in 256s of any length).
bool mxe_can(int64_t K, int64_t N, int n_tokens);
size_t mxe_operand_bytes(int K);
size_t mxe_scale_bytes(int K);
void mxe_pieces(hipStream_t s, const float * x, int n_tokens, int K, uint8_t * operands, uint8_t * scales);
void mxe_matmul(hipStream_t s, const uint8_t * packed, const uint8_t * operands, const uint8_t * scales, int K, int64_t N,
                int n_tokens, float * y);
// The expert products of a mixture-of-experts step on the same instruction (MXFP4 experts whose rows are also held as
// records, f32-accumulation accuracy): per group of 16 pair slots the activation rows are written as digits
// (operands mxe_moe_operand_bytes, scales mxe_moe_scale_bytes for `slots` slots of width K), then gate and up with
// SwiGLU leave f32 rows h [slot][F], and down leaves out_pair [slot][E]. Widths in 256s.
bool mxe_moe_can(int E, int F);
size_t mxe_moe_operand_bytes(int K, size_t slots);
size_t mxe_moe_scale_bytes(int K, size_t slots);
void mxe_moe_gate_up(hipStream_t s, const uint8_t * gate, const uint8_t * up, const Act & x, int E, int F, int n_expert,
                     const int32_t * off_pad, const int32_t * tok_of_q, size_t slots, uint8_t * ops, uint8_t * scales, float * h);
void mxe_moe_down(hipStream_t s, const uint8_t * down, const float * h, int E, int F, int n_expert, const int32_t * off_pad,
                  const int32_t * tok_of_q, size_t slots, uint8_t * ops, uint8_t * scales, float * out_pair);
// The weight's side of gemv_can. With it the same product can take its rows as f32 and make the Q8_K blocks while
// it stages them, one launch instead of two: gemv_norm from the residual rows (x row rows[t], or t; RMSNorm with
// norm_w and eps as rmsnorm_act computes it, then the conversion), gemv_swiglu from the f32 rows of a gate/up product
// (gu rows of 2 K floats laid out as swiglu_act reads them with `group`).
bool gemv_can_weight(const Weight & w, int T);
void gemv_norm(hipStream_t s, const Weight & w, const float * x, const float * norm_w, float eps, const int32_t * rows, int T,
               float * y, int ldy, int col0, int mode, const float * bias);
void gemv_swiglu(hipStream_t s, const Weight & w, const float * gu, int group, int T, float * y, int ldy, int col0, int mode);
// ... and gemv_combine from the split partials of a single-token step's attention (the token's work items start at
// item0, n_split per kv head, at most GEMV_COMBINE_MAX_SPLITS: every workgroup merges all heads itself, which pays
// while the partials are few): the product of the output projection without attention_combine's launch.
constexpr int GEMV_COMBINE_MAX_SPLITS = 16;
void gemv_combine(hipStream_t s, const Weight & w, const float * partial, int item0, int n_split, int n_head, int G, int head_dim,
                  float * y, int ldy, int col0, int mode);
// The same kernel in the exact arithmetic (f32 rows, every code converted and multiplied by a fused multiply-add):
// from the hi / lo planes a producer left (x.x), from residual rows through RMSNorm, from a gate/up product through SwiGLU.
bool gemv_f32_can_weight(const Weight & w, int T);
void gemv_f32(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0, int mode, const float * bias);
void gemv_f32_norm(hipStream_t s, const Weight & w, const float * x, const float * norm_w, float eps, const int32_t * rows, int T,
                   float * y, int ldy, int col0, int mode, const float * bias);
void gemv_f32_swiglu(hipStream_t s, const Weight & w, const float * gu, int group, int T, float * y, int ldy, int col0, int mode);
extern thread_local int g_gemv_max_t;   // steps of at most this many tokens take the kernel (default GEMV_MAX_T; 0 switches it off);
                                        // an engine sets it from its own configuration at the start of every forward pass
extern thread_local int g_mm_force_ksplit;  // > 0 overrides the split-K heuristic for the calling thread (kernel-level timing entry point)
// Fused gate/up matmul and SwiGLU: w holds, for every 64 columns of the hidden
// layer, their 64 gate rows followed by their 64 up rows (w.N = 2 F, F % 64 == 0,
// a tile storage type); out (K = F) receives silu(gate) * up as activations.
// When out asks for the Q8_K conversion, whose blocks are wider than the 64
// columns a workgroup holds, the products leave as f32 rows in h_f32 ([T][F])
// and a second launch converts them. h_f32 has room for [T][2 F]: a very small step whose rows came with
// Q8_K code buffers is multiplied by the integer kernel (gemv) into gate and up rows there.
void matmul_swiglu(hipStream_t s, const Weight & w, const Act & x, int T, const Act & out, void * ws, float * h_f32);
// Several tile-packed matrices over the same activations, outputs side by side in y from column 0 (bias likewise):
// one launch each, all leaving the same number of K-slices in one set of slices of the full row width.
Slices matmul_deferred_parts(hipStream_t s, const Weight * const * parts, int n_parts, const Act & x, int T, float * y,
                             int ldy, const float * bias, void * ws);
Slices matmul_lds(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0,
                  int mode, const float * bias, void * ws, bool may_slice);
// Forces the generic (raw layout) kernel; used to cross-check the tile kernels.
void matmul_generic(hipStream_t s, const Weight & w, const Act & x, int T, float * y, int ldy, int col0,
                    int mode, const float * bias);

struct RowDesc;
// Per-row LoRA. One loaded adapter's pair for one target matrix: A [rank][K] and
// B [N][rank] as f32, scale = adapter scale * alpha / rank.
struct LoraEntry {
    const float * A = nullptr;
    const float * B = nullptr;
    int32_t rank = 0;
    float scale = 0.0f;
    // storage types of the factors in the adapter file: an F16 (BF16) factor multiplies
    // its operand rounded to f16 (bf16), as ggml's CPU dot products do
    int32_t a_type = WT_F32;
    int32_t b_type = WT_F32;
};
constexpr int LORA_MAX_RANK = 64;
// For every token whose row routes to an adapter (rows[tok_row[t]].route > 0,
// entry table[route - 1], skipped when the entry has no pair for this target):
//   y[t][col0 + n] += scale * sum_r B[n][r] * (sum_k A[r][k] * x[t][k]).
// mid is scratch of T * LORA_MAX_RANK floats.
// The same for up to three targets that read the same activations (tables[i], widths[i], cols[i]), in one
// pair of launches; mid is scratch of n_targets * T * LORA_MAX_RANK floats. group > 0: output n of a target
// lands in column cols[i] + (n / group) * 2 group + n % group (gate and up outputs interleaved by `group`).
void lora_apply_targets(hipStream_t s, int n_targets, const LoraEntry * const * tables, const int * widths, const int * cols,
                        const RowDesc * rows, const int32_t * tok_row, const Act & x, int T, float * y, int ldy, float * mid,
                        int group = 0);
void lora_apply(hipStream_t s, const LoraEntry * table, const RowDesc * rows, const int32_t * tok_row,
                const Act & x, int T, int N, float * y, int ldy, int col0, float * mid);
// out[r][k] = decode(raw row r)[k] as f32: any tensor to f32, row by row.
void decode_rows(hipStream_t s, int type, const uint8_t * raw, int K, int n_rows, float * out);

// Mixture-of-experts feed-forward (qwen3moe). Expert tensors are tiled by
// moe_repack as one matrix of n_expert * N rows; router is raw F32 [n_expert][E].
bool moe_can_pack(int type, int64_t K, int64_t N);
void moe_repack(hipStream_t s, int type, const uint8_t * raw, uint8_t * packed, int K, int64_t n_rows);
struct MoeLayer { Weight router, gate, up, down; };
struct MoeShape { int E, F, n_expert, k_used; };
struct MoeBuffers {            // device scratch of one step, sized with moe_slots(n_batch, ...)
    float * logits;            // [T][n_expert]
    int32_t * sel;             // [T][k_used] chosen experts, by descending probability
    float * wgt;               // [T][k_used] renormalised weights
    int32_t * expert_n;        // [n_expert]
    int32_t * off_pad;         // [n_expert + 1]
    int32_t * tok_of_q;        // [slots]
    int32_t * q_of_pair;       // [T * k_used]
    Act h;                     // [slots] x F
    float * out_pair;          // [slots][E]
    // the block-scaled path of MXFP4 experts (decode-sized steps of the exact arithmetic), or null: activation operands
    // and scales for mx_slots pair slots of the wider of the two products, and the hidden rows as f32 [mx_slots][F]
    uint8_t * mx_ops = nullptr;
    uint8_t * mx_scales = nullptr;
    float * mx_h = nullptr;
    size_t mx_slots = 0;
    int32_t * pair_of_q = nullptr;   // [slots] the pair (token * k_used + choice) of a slot, -1 for padding; or null: then the
                                     // down projection leaves its rows in slot order instead of pair order
};
size_t moe_slots(int n_tokens, int k_used, int n_expert);
// x[t] += sum over the token's k_used experts of w * down_e(silu(gate_e xn) * (up_e xn))
// With defer_combine the weighted sum is not added to x: it is returned as gathered slices for the next rmsnorm_act.
Slices moe_ffn(hipStream_t s, const MoeLayer & L, const MoeShape & sh, const Act & xn, int T, float * x, const MoeBuffers & b,
               bool defer_combine = false);

// x[t][:] = decode(raw row tok[t]) as f32.
void embed(hipStream_t s, const Weight & emb, const int32_t * tok, int T, float * x);

// act = f16(x * rsqrt(mean(x^2) + eps) * w) (+ block sums). `rows` selects the
// input rows (null: identity), n_rows outputs. With slices, x[row] += their sum
// first (written back), which completes a deferred matmul into the residual.
void rmsnorm_act(hipStream_t s, float * x, const float * w, int E, float eps,
                 const int32_t * rows, int n_rows, const Act & out, const Slices & add = Slices());

// act = f16(x) (+ block sums): the plain conversion every producer fuses.
void to_act(hipStream_t s, const float * x, int T, int K, const Act & out);
// The T rows stored as hi/lo planes at `src` (layout of Act::x, width out.K), converted by
// out.quant into out.qx / out.qsums; src may be out.qx itself. out.x must be null.
void requant_act(hipStream_t s, const __half * src, int T, const Act & out);

// act = f16(silu(gu[t][i]) * gu[t][F + i]) (+ block sums).
// group: gate c at column (c / group) * 2 group + c % group, up c `group` columns further (0: group = F, side by side)
void swiglu_act(hipStream_t s, const float * gu, int T, int F, const Act & out, int group = 0);
// silu(gate) * up of a gate/up product left as K-slices (groups of 128 columns: 64 gate, 64 up) into columns col0 .. of out
void swiglu_slices(hipStream_t s, const Slices & sl, int T, const Act & out, int col0);

// ---- step packing -----------------------------------------------------------
struct RowDesc {           // one per step row, written by the host
    int32_t slot;
    int32_t pos0;
    int32_t n;
    int32_t tok_off;       // flat index of the row's first token
    int32_t sample;
    int32_t kv_begin;      // first resident position of the slot
    int32_t route;         // adapter route (0 = none)
    int32_t pad;
};
struct TableUpdate { int32_t slot; int32_t index; int32_t page; int32_t pad; };

struct PackBuffers {       // device arrays, sized for n_batch tokens / rows
    int32_t * tok;         // [T] token id
    int32_t * pos;         // [T] absolute position
    int32_t * seq;         // [T] slot
    int32_t * row;         // [T] owning row
    int32_t * cell;        // [T] page_id * PAGE + pos % PAGE
    int32_t * out_index;   // [T] index among the output rows, or -1
    int32_t * out_tok;     // [n_out] flat token index of each output row
    int32_t * last_index;  // [n_rows] flat index of the row's last token
    int32_t * row_offset;  // [n_rows + 1]
    int32_t * counts;      // [4]: n_tokens, n_outputs, n_tiles, n_items
    // attention query tiles: up to `qt` consecutive tokens of one row
    int32_t * tile_t0;     // first flat token
    int32_t * tile_nq;     // tokens in the tile
    int32_t * tile_item0;  // first work item of the tile
    int32_t * tile_nsplit; // KV splits per kv head
    int32_t * tile_page0;  // first page index (within the slot) the tile reads
    int32_t * tile_kv_begin;
    int32_t * tok_tile;    // [T] tile of each token
    int4 * tok_merge;      // [T] first work item of the token's tile, its KV splits, the token's index in the tile
    // attention work items (one wave each), everything a wave needs in two 16-byte loads:
    int4 * item_a;         // [n_items, longest first] first flat token of the tile, tokens in the tile | kv head << 8, the item's number, slot
    int4 * item_b;         // [n_items] position of the first token, first resident position of the slot,
                           //           first page index of this split, pages in this split
    int32_t * dec_order;   // [n_rows] rows by resident length, longest first (the order the decode-step attention starts its workgroups in)
    int4 * dec_desc;       // [n_rows] in that order: {the row's token index, its position, the first resident position, the slot}
    int32_t * dec_pid;     // [n_rows][8] in that order: with the row's pages dealt evenly to eight waves, the id of each wave's first page
    float * rope_cos;      // [T][rope_dim/2]
    float * rope_sin;
    int split_pages = MAX_SPLIT_PAGES;   // pages per attention work item in this step (set from count_attention_work)
};
// Applies the block-table updates, then derives every per-token / per-tile
// array of the step from the row descriptors. One workgroup. inv_freq holds rope_pairs angles per position and
// one more value, the factor on the rotation's cosines and sines (1 for a plain rotation).
void pack_step(hipStream_t s, const RowDesc * rows, int n_rows, const int32_t * tokens_concat,
               const TableUpdate * updates, int n_updates, int32_t * table, int max_pages,
               int qt, int n_kv_heads, const double * inv_freq, int rope_pairs, const PackBuffers & out);

// Query tokens per attention tile for G query heads per kv head: 8 / G when the hi and lo halves of a query
// share a matrix instruction (G <= 8), else 16 / G.
inline int attention_tile_tokens(int G) { return G <= 8 ? 8 / G : (16 / G > 0 ? 16 / G : 1); }
// Host mirror of the tile/item count (same formula as the kernel).
void count_attention_work(const RowDesc * rows, int n_rows, int qt, int n_kv_heads,
                          int * n_tiles, int * n_items, int * split_pages);

// ---- attention ----------------------------------------------------------------
struct AttnShape {
    int n_head, n_head_kv, head_dim;
    int rope_dim;
    bool rope_neox;
    float eps;
    // element strides of a KV pool between pages and between the kv heads of a page (see kv_strides)
    size_t page_stride = 0, head_stride = 0;
    int kv_quant = 0;          // 0: f16 pools; 8 / 4: the pools hold Q8_0 / Q4_0 blocks (see kv_block_halves)
    bool q_q8 = false;         // over such blocks: the query rows are converted to Q8_0 too (ggml's CPU attention)
};
// A pool holds one block per page and kv head, PAGE positions of one head. f16: PAGE x head_dim halves in the
// operand orders of the attention kernel. Q8_0 (blocks of 32 along the head's row, one f16 scale each, as the
// reference's kv_dtype Q8_0 stores a row): head_dim / 32 loads of 1 KiB of codes, a code as the byte code + 128,
// then head_dim / 32 groups of 32 f16 scales; 17/32 of the f16 block.
//   K codes  [j = dim / 32][lane = g * 16 + t][16 B]: bytes 0-7 dims 32 j + 8 g + (0..7) of token t, bytes 8-15 of token 16 + t
//   V codes  [p = dim / 32][lane = g * 16 + d][16 B]: bytes 0-7 dim 32 p + d, bytes 8-15 dim 32 p + 16 + d, byte i of
//            either the token 4 g + i (i < 4) or 16 + 4 g + (i - 4)
//   scales   [j or p][g][8]: the scale of block j (p) of token 4 g + i (i < 4) or 16 + 4 g + (i - 4)
// Q4_0 (kv_dtype Q4_0: the same blocks with four-bit codes q, value d (q - 8)): the same arrangement with 8 bytes
// per lane, i.e. two 32-bit words where Q8_0 has two groups of eight bytes; the code of index i among a word's eight
// is the nibble at bits 4 p(i) with p(i) = i / 2 + 4 (i % 2), the order in which one mask and shift pair widens
// them to f16 (kv_nibble). head_dim / 32 loads of 512 bytes of codes, then the scales as above; 9/32 of the f16 block.
// All strides and sizes are in halves (2 bytes), also for the quantised pools.
enum : int { KV_F16 = 0, KV_Q8 = 8, KV_Q4 = 4 };
constexpr int kv_nibble(int i) { return (i >> 1) + 4 * (i & 1); }
inline size_t kv_block_halves(int head_dim, int kvq) {
    return kvq == KV_Q8 ? (size_t)(head_dim / 32) * 544 : kvq == KV_Q4 ? (size_t)(head_dim / 32) * 288 : (size_t)PAGE * head_dim;
}
// head_major: [kv head][page], else [page][kv head].
struct KvStrides { size_t page, head; };
inline KvStrides kv_strides(int n_pages, int n_kv_heads, int head_dim, bool head_major, int kvq = KV_F16) {
    const size_t unit = kv_block_halves(head_dim, kvq);
    return head_major ? KvStrides{unit, (size_t)n_pages * unit} : KvStrides{(size_t)n_kv_heads * unit, unit};
}
// Halves of one cell's K (or V) row over all kv heads in the natural order kv_gather writes: f16 values, or per
// head the codes in element order (Q8_0: head_dim bytes, code + 128; Q4_0: head_dim / 2 bytes, element 2 k in the
// low nibble of byte k) followed by head_dim / 32 f16 scales.
inline size_t kv_row_halves(int n_kv_heads, int head_dim, int kvq) {
    return kvq == KV_Q8 ? (size_t)n_kv_heads * (head_dim / 2 + head_dim / 32)
         : kvq == KV_Q4 ? (size_t)n_kv_heads * (head_dim / 4 + head_dim / 32) : (size_t)n_kv_heads * head_dim;
}
// qkv f32 [T][QD + 2*KD] (+ optional per-head RMSNorm weights) -> q as an f16
// hi/lo pair [T][QD] each (rotated, pre-scaled by log2(e)/sqrt(head_dim)) and
// the K/V pages of the layer (f16, the KV cache precision).
// With slices (of a [T][QD + 2*KD] product) the values are their sum and qkv is not read.
void rope_store(hipStream_t s, const float * qkv, int T, const AttnShape & sh, const PackBuffers & pk,
                const float * q_norm, const float * k_norm, __half * q_out, __half * q_out_lo,
                __half * k_pool, __half * v_pool, const Slices & from = Slices());

// Split-KV paged attention over the step's query tiles (one_token_rows: every
// row of the step has a single token, so every tile has a single query). partial holds, per
// (item, column), m (log2 domain), l and head_dim unnormalised outputs.
void attention(hipStream_t s, const __half * q, const __half * q_lo, const AttnShape & sh, const PackBuffers & pk,
               const int32_t * table, int max_pages, const __half * k_pool, const __half * v_pool,
               int n_items, int n_tiles, float * partial, bool one_token_rows = false);
// Merges the splits: out act [T][QD] (+ block sums).
// The three launches above in one, for a step in which every row decodes one token over an f16 cache (see
// k_attention_decode): reads the q, k, v product (its K-slices or the buffer), stores the new K and V rows, writes the
// output projection's activations. attention_decode_can: whether the shape allows it (head dims 64 / 128 rotated
// over their whole width, at most eight query heads per kv head, sequences of at most 16384 positions; q_norm / k_norm: the per-head RMSNorm weights of architectures that have them, or null; stamps: null, or six
// clock values per workgroup (n_rows * n_head_kv of them) for a timeline of the launch).
bool attention_decode_can(const AttnShape & sh, int max_positions);
void attention_decode(hipStream_t s, const float * qkv, const Slices & from, int n_rows, const AttnShape & sh,
                      const PackBuffers & pk, const int32_t * table, int max_pages, __half * k_pool, __half * v_pool,
                      const float * q_norm, const float * k_norm, const Act & out, unsigned long long * stamps = nullptr);
void attention_combine(hipStream_t s, const float * partial, int T, const AttnShape & sh,
                       const PackBuffers & pk, const Act & out);
size_t attention_partial_floats(int n_items, int head_dim);

// Gathers the K or V row of one (layer pool, cell) into natural order, and the
// inverse; used by sequence snapshots and by tests.
void kv_gather(hipStream_t s, const __half * pool, KvStrides st, int n_kv_heads, int head_dim, bool is_v,
               const int32_t * cells, int n, __half * out, int kvq = KV_F16);
void kv_scatter(hipStream_t s, __half * pool, KvStrides st, int n_kv_heads, int head_dim, bool is_v,
                const int32_t * cells, int n, const __half * in, int kvq = KV_F16);
// Copies page src to page dst in one layer's pools.
void kv_copy_page(hipStream_t s, __half * k_pool, __half * v_pool, KvStrides st, int n_kv_heads, int head_dim,
                  int src_page, int dst_page, int kvq = KV_F16);

// ---- sampling -------------------------------------------------------------------
struct SampleOut {          // one per output row, read back by the host
    int32_t argmax;
    float max;
    double sum_exp;         // sum exp(double(logit) - max)
    int32_t edge_tie;       // k > 1 and the entry right behind the k-th candidate has the k-th's logit
    int32_t pad;
    int32_t top_id[MAX_TOPK];
    float top_logit[MAX_TOPK];
};
// k[r] candidates per row by (logit desc, id asc); k = 0 rows only get argmax/max/sum. max_k is the
// largest k[r] (known to the host): when no row asks for more than one candidate and scratch
// (sample_scratch_bytes(n_rows) bytes) is given, a large vocabulary is scanned in slices by many workgroups.
size_t sample_scratch_bytes(int n_rows);
void sample_prepare(hipStream_t s, const float * logits, int n_rows, int n_vocab, const int32_t * k,
                    SampleOut * out, int max_k, void * scratch);

// The greedy scan (argmax with the lowest id on ties, max, sum exp(double(logit) - max) per row) over device
// buffers of the caller, on the caller's stream, with its slice partials in a static device array: allocates
// nothing and waits for nothing. At most sample_static_max_rows() rows per call.
int sample_static_max_rows();
// Looks the static array's address up for the current device (a host-side call that may load the code object), so
// that later calls of sample_greedy_static do nothing but launch; engine creation calls it.
void sample_static_prepare();
void sample_greedy_static(hipStream_t s, const float * logits, int n_rows, int n_vocab, int32_t * out_argmax,
                          float * out_max, double * out_sum);

}  // namespace rk
