// Kernel-level and state-inspection entry points declared in
// include/retro_kernels.h. They have no counterpart in the reference ABI: they
// exist so parity tests can compare single kernels and device state with the
// CPU oracle through plain C calls.
#include <algorithm>
#include "../../include/retro_kernels.h"
#include "engine.hpp"
#include <vector>

#include <cstring>

using namespace retro;


namespace {
template <typename Fn> int guarded(Fn && fn) {
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
void ok(hipError_t e, const char * what) {
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}
}  // namespace

extern "C" {

int retro_kernel_matmul(int32_t type, const uint8_t * raw, int64_t n_rows, int64_t k, const float * x,
                        int32_t n_tokens, int32_t use_tiles, const float * bias, int32_t accumulate, float * y) {
    return guarded([&]() -> int {
        const size_t bytes = rk::row_bytes(type, k) * (size_t)n_rows;
        DevBuf d_raw, d_packed, d_x, d_xh, d_sums, d_y, d_bias;
        d_raw.alloc(bytes);
        ok(hipMemcpy(d_raw.ptr, raw, bytes, hipMemcpyHostToDevice), "upload weights");
        rk::Weight w;
        w.type = type; w.K = (int)k; w.N = (int)n_rows; w.bytes = bytes;
        if (use_tiles & 0xff) {
            if (!rk::can_pack(type, k, n_rows)) throw std::runtime_error("this shape or type has no tile layout");
            d_packed.alloc(bytes);
            rk::repack(nullptr, type, d_raw.as<uint8_t>(), d_packed.as<uint8_t>(), (int)k, (int)n_rows);
            w.packed = d_packed.as<uint8_t>();
        } else {
            w.raw = d_raw.as<uint8_t>();
        }
        d_x.alloc((size_t)n_tokens * k * 4);
        ok(hipMemcpy(d_x.ptr, x, d_x.bytes, hipMemcpyHostToDevice), "upload activations");
        d_xh.alloc(rk::act_halves(n_tokens, (int)k) * 2);
        d_sums.alloc(rk::act_sum_halves(n_tokens, (int)k) * 2);
        ok(hipMemset(d_xh.ptr, 0, d_xh.bytes), "clear activations");
        ok(hipMemset(d_sums.ptr, 0, d_sums.bytes), "clear block sums");
        // use_tiles bit 8: ggml's arithmetic - the rows are converted (quantised types) or rounded (F16 / BF16)
        // before the product; otherwise the f32 values are multiplied
        // bit 9 (with bit 8, Q8_K conversions, at most GEMV_MAX_T = 2 tokens): the producer leaves the Q8_K blocks as
        // well and the integer matrix-vector kernel multiplies them
        const bool faithful = (use_tiles & 0x100) != 0, integer = (use_tiles & 0x200) != 0;
        use_tiles &= 0xff;
        rk::Act act;
        act.K = (int)k;
        act.faithful = faithful ? 1 : 0;
        if (!faithful || rk::act_quant_of(type) == rk::AQ_NONE) {
            act.x = d_xh.as<__half>(); act.sums = k % 32 == 0 ? d_sums.as<__half>() : nullptr;
        } else {
            act.qx = d_xh.as<__half>(); act.qsums = d_sums.as<__half>(); act.quant = rk::act_quant_of(type);
        }
        DevBuf d_codes, d_scales, d_bsums;
        // the switch an engine's configuration may have left off is on for the call
        struct Restore { int was; ~Restore() { rk::g_gemv_max_t = was; } } restore{rk::g_gemv_max_t};
        if (integer) rk::g_gemv_max_t = rk::GEMV_MAX_T;
        if (integer) {
            if (!faithful || act.quant == rk::AQ_NONE || n_tokens > rk::GEMV_MAX_T)
                throw std::runtime_error("the integer kernel takes Q8_K or Q8_0 conversions of at most " + std::to_string(rk::GEMV_MAX_T) + " tokens");
            d_codes.alloc((size_t)n_tokens * k);
            d_scales.alloc((size_t)n_tokens * (k / 32) * 4);
            d_bsums.alloc((size_t)n_tokens * (k / 16) * 2);
            act.qc = d_codes.as<int8_t>(); act.qd = d_scales.as<float>(); act.qbs = d_bsums.as<int16_t>();
            if (!rk::gemv_can(w, act.operand(type), n_tokens)) throw std::runtime_error("the integer kernel does not take this matrix");
        }
        rk::to_act(nullptr, d_x.as<float>(), n_tokens, (int)k, act);
        d_y.alloc((size_t)n_tokens * n_rows * 4);
        ok(hipMemcpy(d_y.ptr, y, d_y.bytes, hipMemcpyHostToDevice), "upload outputs");
        if (bias) {
            d_bias.alloc((size_t)n_rows * 4);
            ok(hipMemcpy(d_bias.ptr, bias, d_bias.bytes, hipMemcpyHostToDevice), "upload bias");
        }
        DevBuf d_ws;
        if (use_tiles == 2) {
            d_ws.alloc(rk::matmul_workspace_bytes());
            ok(hipMemset(d_ws.ptr, 0, d_ws.bytes), "clear workspace");
        }
        rk::matmul(nullptr, w, act, n_tokens, d_y.as<float>(), (int)n_rows, 0, accumulate ? rk::MM_ADD : rk::MM_STORE,
                   d_bias.as<float>(), d_ws.ptr);
        ok(hipDeviceSynchronize(), "matmul");
        ok(hipMemcpy(y, d_y.ptr, d_y.bytes, hipMemcpyDeviceToHost), "download outputs");
        return 0;
    });
}

int retro_kernel_gemv_fused(int32_t kind, int32_t type, const uint8_t * raw, int64_t n_rows, int64_t k, const float * x, const float * norm_w,
                            float eps, int32_t n_tokens, int32_t group, float * y_fused, float * y_unfused) {
    return guarded([&]() -> int {
        // kinds 11 and 12: the exact arithmetic's kernel (f32 rows, a single token) for the same two producers
        const bool exact = kind == 11 || kind == 12;
        if (exact) kind -= 10;
        if ((kind != 1 && kind != 2) || n_tokens < 1 || n_tokens > (exact ? 1 : rk::GEMV_MAX_T) || k <= 0 || k % 256 != 0 || n_rows <= 0 || n_rows % 16 != 0)
            throw std::runtime_error("gemv_fused: kind 1 / 11 (RMSNorm) or 2 / 12 (SwiGLU), whole tiles and super-blocks, at most " + std::to_string(rk::GEMV_MAX_T)
                                     + " tokens (kinds 11 and 12: one)");
        if (kind == 1 && !norm_w) throw std::runtime_error("gemv_fused: the RMSNorm needs its weights");
        if (type != rk::WT_Q4_K && type != rk::WT_Q5_K && type != rk::WT_Q6_K && type != rk::WT_Q8_0) throw std::runtime_error("gemv_fused: Q4_K, Q5_K, Q6_K or Q8_0 rows");
        struct Restore { int was; ~Restore() { rk::g_gemv_max_t = was; } } restore{rk::g_gemv_max_t};
        rk::g_gemv_max_t = rk::GEMV_MAX_T;      // whatever an engine's configuration left
        const size_t bytes = rk::row_bytes(type, k) * (size_t)n_rows;
        const size_t in_floats = (size_t)n_tokens * k * (kind == 2 ? 2 : 1);
        DevBuf d_raw, d_packed, d_x, d_w, d_xh, d_sums, d_codes, d_scales, d_bsums, d_y;
        d_raw.alloc(bytes); d_packed.alloc(bytes);
        ok(hipMemcpy(d_raw.ptr, raw, bytes, hipMemcpyHostToDevice), "upload weights");
        rk::repack(nullptr, type, d_raw.as<uint8_t>(), d_packed.as<uint8_t>(), (int)k, (int)n_rows);
        rk::Weight w;
        w.type = type; w.K = (int)k; w.N = (int)n_rows; w.bytes = bytes; w.packed = d_packed.as<uint8_t>();
        d_x.alloc(in_floats * 4);
        ok(hipMemcpy(d_x.ptr, x, d_x.bytes, hipMemcpyHostToDevice), "upload rows");
        if (kind == 1) {
            d_w.alloc((size_t)k * 4);
            ok(hipMemcpy(d_w.ptr, norm_w, d_w.bytes, hipMemcpyHostToDevice), "upload norm weights");
        }
        d_xh.alloc(rk::act_halves(n_tokens, (int)k) * 2);
        d_sums.alloc(rk::act_sum_halves(n_tokens, (int)k) * 2);
        ok(hipMemset(d_xh.ptr, 0, d_xh.bytes), "clear"); ok(hipMemset(d_sums.ptr, 0, d_sums.bytes), "clear");
        d_codes.alloc((size_t)n_tokens * k); d_scales.alloc((size_t)n_tokens * (k / 32) * 4); d_bsums.alloc((size_t)n_tokens * (k / 16) * 2);
        rk::Act act;
        act.K = (int)k;
        if (exact) {
            if (!rk::gemv_f32_can_weight(w, n_tokens)) throw std::runtime_error("gemv_fused: the exact kernel does not take this matrix");
            act.x = d_xh.as<__half>(); act.sums = d_sums.as<__half>();
        } else {
            act.faithful = 1; act.quant = rk::act_quant_of(type);
            act.qx = d_xh.as<__half>(); act.qsums = d_sums.as<__half>();
            act.qc = d_codes.as<int8_t>(); act.qd = d_scales.as<float>(); act.qbs = d_bsums.as<int16_t>();
        }
        d_y.alloc((size_t)n_tokens * n_rows * 4);
        // the two launches: the producer leaves the blocks (exact: the hi / lo planes), the kernel multiplies them
        if (kind == 1) rk::rmsnorm_act(nullptr, d_x.as<float>(), d_w.as<float>(), (int)k, eps, nullptr, n_tokens, act);
        else rk::swiglu_act(nullptr, d_x.as<float>(), n_tokens, (int)k, act, group);
        if (exact) rk::gemv_f32(nullptr, w, act, n_tokens, d_y.as<float>(), (int)n_rows, 0, rk::MM_STORE, nullptr);
        else rk::gemv(nullptr, w, act.operand(type), n_tokens, d_y.as<float>(), (int)n_rows, 0, rk::MM_STORE, nullptr);
        ok(hipDeviceSynchronize(), "gemv");
        ok(hipMemcpy(y_unfused, d_y.ptr, d_y.bytes, hipMemcpyDeviceToHost), "download");
        ok(hipMemset(d_y.ptr, 0, d_y.bytes), "clear");
        // one launch: the kernel makes the rows while it stages them
        if (exact) {
            if (kind == 1) rk::gemv_f32_norm(nullptr, w, d_x.as<float>(), d_w.as<float>(), eps, nullptr, n_tokens, d_y.as<float>(), (int)n_rows, 0, rk::MM_STORE, nullptr);
            else rk::gemv_f32_swiglu(nullptr, w, d_x.as<float>(), group, n_tokens, d_y.as<float>(), (int)n_rows, 0, rk::MM_STORE);
        } else {
            if (kind == 1) rk::gemv_norm(nullptr, w, d_x.as<float>(), d_w.as<float>(), eps, nullptr, n_tokens, d_y.as<float>(), (int)n_rows, 0, rk::MM_STORE, nullptr);
            else rk::gemv_swiglu(nullptr, w, d_x.as<float>(), group, n_tokens, d_y.as<float>(), (int)n_rows, 0, rk::MM_STORE);
        }
        ok(hipDeviceSynchronize(), "gemv fused");
        ok(hipMemcpy(y_fused, d_y.ptr, d_y.bytes, hipMemcpyDeviceToHost), "download");
        return 0;
    });
}

int retro_kernel_sample_prepare(const float * logits, int32_t n_rows, int32_t n_vocab, const int32_t * k,
                                int32_t * out_argmax, float * out_max, double * out_sum_exp,
                                int32_t * out_top_ids, float * out_top_logits) {
    return guarded([&]() -> int {
        DevBuf d_l, d_k, d_o;
        d_l.alloc((size_t)n_rows * n_vocab * 4);
        d_k.alloc((size_t)n_rows * 4);
        d_o.alloc((size_t)n_rows * sizeof(rk::SampleOut));
        ok(hipMemcpy(d_l.ptr, logits, d_l.bytes, hipMemcpyHostToDevice), "upload logits");
        ok(hipMemcpy(d_k.ptr, k, d_k.bytes, hipMemcpyHostToDevice), "upload k");
        int max_k = 0;
        for (int r = 0; r < n_rows; ++r) max_k = std::max(max_k, k[r]);
        DevBuf d_scratch;
        d_scratch.alloc(rk::sample_scratch_bytes(n_rows));
        rk::sample_prepare(nullptr, d_l.as<float>(), n_rows, n_vocab, d_k.as<int32_t>(), d_o.as<rk::SampleOut>(), max_k,
                           d_scratch.ptr);
        ok(hipDeviceSynchronize(), "sample_prepare");
        std::vector<rk::SampleOut> h((size_t)n_rows);
        ok(hipMemcpy(h.data(), d_o.ptr, d_o.bytes, hipMemcpyDeviceToHost), "download");
        for (int r = 0; r < n_rows; ++r) {
            out_argmax[r] = h[(size_t)r].argmax;
            out_max[r] = h[(size_t)r].max;
            out_sum_exp[r] = h[(size_t)r].sum_exp;
            for (int j = 0; j < rk::MAX_TOPK; ++j) {
                out_top_ids[r * rk::MAX_TOPK + j] = j < k[r] ? h[(size_t)r].top_id[j] : -1;
                out_top_logits[r * rk::MAX_TOPK + j] = j < k[r] ? h[(size_t)r].top_logit[j] : 0.0f;
            }
        }
        return 0;
    });
}

int32_t retro_kernel_sample_greedy_noalloc_max_rows(void) { return rk::sample_static_max_rows(); }

int retro_kernel_sample_greedy_noalloc(const float * d_logits, int32_t n_rows, int32_t n_vocab, int32_t * d_out_argmax,
                                       float * d_out_max, double * d_out_sum_exp, void * stream) {
    return guarded([&]() -> int {
        rk::sample_greedy_static((hipStream_t)stream, d_logits, n_rows, n_vocab, d_out_argmax, d_out_max, d_out_sum_exp);
        return 0;
    });
}

// Times `iters` launches of one tile matmul on random device data with HIP
// events; returns microseconds per launch through out_us.
int retro_kernel_matmul_time(int32_t type, int64_t n_rows, int64_t k, int32_t n_tokens, int32_t mode,
                             int32_t iters, int32_t debug, int32_t force_ksplit, double * out_us) {
    return guarded([&]() -> int {
        if (type != rk::WT_Q4_K && type != rk::WT_Q8_0 && type != rk::WT_Q6_K && type != rk::WT_Q5_K)
            throw std::runtime_error("matmul_time: the tile kernels take Q4_K, Q5_K, Q6_K and Q8_0");
        if (n_rows <= 0 || k <= 0 || n_rows % 16 != 0 || k % 256 != 0 || n_tokens <= 0 || iters <= 0)
            throw std::runtime_error("matmul_time: whole 16-row tiles and super-blocks of 256, at least one token and one launch");
        const size_t bytes = rk::row_bytes(type, k) * (size_t)n_rows;
        // mode bit 4: every launch reads another copy of the weights, 1 GiB of them in turn,
        // so that they come from HBM as in a decode step and not from the last-level cache
        // mode bit 5: 6 GiB of copies instead (more address space than a decode step's weights)
        const bool cold = (mode & 48) != 0;
        const size_t span = (mode & 32) ? (size_t)6 << 30 : (size_t)1 << 30;
        mode &= 15;
        const size_t copies = cold ? std::max<size_t>(2, span / bytes) : 1;
        DevBuf d_w, d_xh, d_sums, d_y, d_ws;
        d_w.alloc(bytes * copies);
        d_xh.alloc(rk::act_halves(n_tokens, (int)k) * 2);
        d_sums.alloc(rk::act_sum_halves(n_tokens, (int)k) * 2);
        {
            // Pseudo-random codes and activations: how fast the matrix pipes may clock depends on how many
            // bits toggle, so constant operands would flatter the kernel. Every fourth byte pair that could
            // be a block scale is kept a small finite f16.
            std::vector<uint8_t> host(bytes);
            uint32_t state = 0x9e3779b9u;
            for (size_t i = 0; i < bytes; ++i) { state = state * 1664525u + 1013904223u; host[i] = (uint8_t)(state >> 24); }
            if (type == rk::WT_Q6_K) {        // the buffer is read as tiles: the sixteen d of a tile sit at 256..287 of its 3360 bytes
                for (size_t t = 0; t + 3360 <= bytes; t += 3360)
                    for (size_t i = 256; i < 288; i += 2) { host[t + i] = 0x1f; host[t + i + 1] = 0x21; }
            } else {
                const size_t blk = type == rk::WT_Q4_K ? 144 : (type == rk::WT_Q5_K ? 176 : 34);
                for (size_t i = 0; i + 4 <= bytes; i += blk) { host[i] = 0x1f; host[i + 1] = 0x21; host[i + 2] = 0x1f; host[i + 3] = 0x21; }
            }
            for (size_t c = 0; c < copies; ++c) ok(hipMemcpy(d_w.as<uint8_t>() + c * bytes, host.data(), bytes, hipMemcpyHostToDevice), "fill");
            std::vector<uint16_t> xs(d_xh.bytes / 2);
            for (size_t i = 0; i < xs.size(); ++i) {
                state = state * 1664525u + 1013904223u;
                xs[i] = (uint16_t)(((state >> 16) & 0x83ffu) | 0x3800u);       // +-[0.5, 1)
            }
            ok(hipMemcpy(d_xh.ptr, xs.data(), d_xh.bytes, hipMemcpyHostToDevice), "fill");
            ok(hipMemset(d_sums.ptr, 0, d_sums.bytes), "fill");
        }
        d_y.alloc((size_t)n_tokens * n_rows * 4);
        d_ws.alloc(rk::matmul_workspace_bytes());
        ok(hipMemset(d_ws.ptr, 0, d_ws.bytes), "fill");
        rk::Weight w;
        w.type = type; w.K = (int)k; w.N = (int)n_rows; w.bytes = bytes; w.packed = d_w.as<uint8_t>();
        rk::Act act;
        act.K = (int)k;
        act.x = act.qx = d_xh.as<__half>(); act.sums = act.qsums = d_sums.as<__half>(); act.quant = rk::act_quant_of(type);
        struct Restore { int was; ~Restore() { rk::g_gemv_max_t = was; } } restore{rk::g_gemv_max_t};
        if (mode == 4) rk::g_gemv_max_t = rk::GEMV_MAX_T;      // whatever an engine's configuration left
        // mode 4: the integer matrix-vector kernel over pseudo-random activation blocks (Q4_K, Q5_K, Q6_K, Q8_0; at most GEMV_MAX_T tokens)
        DevBuf d_codes, d_scales, d_bsums;
        if (mode == 4) {
            if ((type != rk::WT_Q4_K && type != rk::WT_Q5_K && type != rk::WT_Q6_K && type != rk::WT_Q8_0) || n_tokens > rk::GEMV_MAX_T)
                throw std::runtime_error("matmul_time: the integer kernel takes Q4_K, Q5_K, Q6_K or Q8_0 and at most " + std::to_string(rk::GEMV_MAX_T) + " tokens");
            std::vector<uint8_t> codes((size_t)n_tokens * k);
            uint32_t state = 0x85ebca6bu;
            for (uint8_t & c : codes) { state = state * 1664525u + 1013904223u; c = (uint8_t)(state >> 24); }
            std::vector<float> scales((size_t)n_tokens * (k / 32), 0.01f);
            std::vector<int16_t> bsums((size_t)n_tokens * (k / 16));
            for (int16_t & b : bsums) { state = state * 1664525u + 1013904223u; b = (int16_t)((int)(state >> 21) - 1024); }
            d_codes.alloc(codes.size()); d_scales.alloc(scales.size() * 4); d_bsums.alloc(bsums.size() * 2);
            ok(hipMemcpy(d_codes.ptr, codes.data(), d_codes.bytes, hipMemcpyHostToDevice), "fill");
            ok(hipMemcpy(d_scales.ptr, scales.data(), d_scales.bytes, hipMemcpyHostToDevice), "fill");
            ok(hipMemcpy(d_bsums.ptr, bsums.data(), d_bsums.bytes, hipMemcpyHostToDevice), "fill");
            act.faithful = 1;
            act.qc = d_codes.as<int8_t>(); act.qd = d_scales.as<float>(); act.qbs = d_bsums.as<int16_t>();
            if (!rk::gemv_can(w, act.operand(type), n_tokens)) throw std::runtime_error("matmul_time: the integer kernel does not take this shape");
        }
        if (debug != 0) throw std::runtime_error("matmul_time: the library has no timing switches; debug must be 0");
        rk::g_mm_force_ksplit = force_ksplit;
        hipEvent_t e0, e1;
        ok(hipEventCreate(&e0), "event"); ok(hipEventCreate(&e1), "event");
        size_t turn = 0;
        auto run = [&]() {
            w.packed = d_w.as<uint8_t>() + (turn++ % copies) * bytes;
            // mode 1: register-only tiles, 2: LDS-staged tiles, 3: the same with the K-slices left unreduced
            // mode 5: the exact arithmetic's matrix-vector kernel over the hi / lo planes (one token)
            if (mode == 5) rk::gemv_f32(nullptr, w, act, n_tokens, d_y.as<float>(), (int)n_rows, 0, rk::MM_STORE, nullptr);
            else if (mode == 3) rk::matmul_deferred(nullptr, w, act, n_tokens, d_y.as<float>(), (int)n_rows, 0, rk::MM_STORE, nullptr, d_ws.ptr);
            else rk::matmul(nullptr, w, act, n_tokens, d_y.as<float>(), (int)n_rows, 0, rk::MM_STORE, nullptr, mode == 2 || mode == 4 ? d_ws.ptr : nullptr);
        };
        for (int i = 0; i < 3; ++i) run();
        ok(hipEventRecord(e0, nullptr), "record");
        for (int i = 0; i < iters; ++i) run();
        ok(hipEventRecord(e1, nullptr), "record");
        ok(hipEventSynchronize(e1), "sync");
        float ms = 0;
        ok(hipEventElapsedTime(&ms, e0, e1), "elapsed");
        rk::g_mm_force_ksplit = 0;
        (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
        *out_us = (double)ms * 1e3 / iters;
        return 0;
    });
}

int retro_kernel_mxfp4_scaled(const uint8_t * raw, int64_t n_rows, int64_t k, const float * x, int32_t n_tokens, int32_t exact, float * y) {
    return guarded([&]() -> int {
        if (exact ? !rk::mxe_can(k, n_rows, n_tokens) : !rk::mxs_can(k, n_rows, n_tokens))
            throw std::runtime_error(exact ? "mxfp4_scaled, exact: rows in 32s, columns in 256s, 1..16 tokens"
                                           : "mxfp4_scaled: rows in 16s, columns in 256s (at most 4608), 1..16 tokens");
        const size_t bytes = (size_t)n_rows * (size_t)(k / 32) * 17;
        DevBuf d_raw, d_packed, d_x, d_ops, d_dx, d_y;
        d_raw.alloc(bytes);
        ok(hipMemcpy(d_raw.ptr, raw, bytes, hipMemcpyHostToDevice), "upload weights");
        d_packed.alloc(rk::mxs_packed_bytes(k, n_rows));
        rk::mxs_repack(nullptr, d_raw.as<uint8_t>(), d_packed.as<uint8_t>(), (int)k, n_rows);
        d_x.alloc((size_t)n_tokens * k * 4);
        ok(hipMemcpy(d_x.ptr, x, d_x.bytes, hipMemcpyHostToDevice), "upload activations");
        d_y.alloc((size_t)n_tokens * n_rows * 4);
        if (exact) {
            d_ops.alloc(rk::mxe_operand_bytes((int)k));
            d_dx.alloc(rk::mxe_scale_bytes((int)k));
            rk::mxe_pieces(nullptr, d_x.as<float>(), n_tokens, (int)k, d_ops.as<uint8_t>(), d_dx.as<uint8_t>());
            rk::mxe_matmul(nullptr, d_packed.as<uint8_t>(), d_ops.as<uint8_t>(), d_dx.as<uint8_t>(), (int)k, n_rows, n_tokens, d_y.as<float>());
        } else {
            d_ops.alloc(rk::mxs_operand_bytes((int)k));
            d_dx.alloc(rk::mxs_scale_bytes((int)k));
            rk::mxs_quantise(nullptr, d_x.as<float>(), n_tokens, (int)k, d_ops.as<uint8_t>(), d_dx.as<float>());
            rk::mxs_matmul(nullptr, d_packed.as<uint8_t>(), d_ops.as<uint8_t>(), d_dx.as<float>(), (int)k, n_rows, n_tokens, d_y.as<float>());
        }
        ok(hipMemcpy(y, d_y.ptr, d_y.bytes, hipMemcpyDeviceToHost), "download");
        return 0;
    });
}

int retro_kernel_mxfp4_scaled_time(int64_t n_rows, int64_t k, int32_t n_tokens, int32_t exact, int32_t cold, int32_t iters, double * out_us) {
    return guarded([&]() -> int {
        if ((exact ? !rk::mxe_can(k, n_rows, n_tokens) : !rk::mxs_can(k, n_rows, n_tokens)) || iters <= 0)
            throw std::runtime_error("mxfp4_scaled_time: rows in 16s, columns in 256s (at most 4608), 1..16 tokens, at least one launch");
        const size_t bytes = rk::mxs_packed_bytes(k, n_rows);
        const size_t copies = cold ? std::max<size_t>(2, ((size_t)1 << 30) / bytes) : 1;
        DevBuf d_w, d_x, d_ops, d_dx, d_y;
        d_w.alloc(bytes * copies);
        {
            // pseudo-random nibbles; the exponent bytes (the last 128 of every 2176) between 2^-8 and 2^7
            std::vector<uint8_t> host(bytes);
            uint32_t state = 0x9e3779b9u;
            for (size_t i = 0; i < bytes; ++i) {
                state = state * 1664525u + 1013904223u;
                host[i] = (i % 2176 >= 2048) ? (uint8_t)(119 + ((state >> 24) & 15)) : (uint8_t)(state >> 24);
            }
            for (size_t c = 0; c < copies; ++c) ok(hipMemcpy(d_w.as<uint8_t>() + c * bytes, host.data(), bytes, hipMemcpyHostToDevice), "fill");
            std::vector<float> xs((size_t)n_tokens * k);
            for (float & v : xs) { state = state * 1664525u + 1013904223u; v = (float)((int)(state >> 16) - 32768) / 32768.0f; }
            d_x.alloc(xs.size() * 4);
            ok(hipMemcpy(d_x.ptr, xs.data(), d_x.bytes, hipMemcpyHostToDevice), "fill");
        }
        if (exact) {
            d_ops.alloc(rk::mxe_operand_bytes((int)k));
            d_dx.alloc(rk::mxe_scale_bytes((int)k));
            rk::mxe_pieces(nullptr, d_x.as<float>(), n_tokens, (int)k, d_ops.as<uint8_t>(), d_dx.as<uint8_t>());
        } else {
            d_ops.alloc(rk::mxs_operand_bytes((int)k));
            d_dx.alloc(rk::mxs_scale_bytes((int)k));
            rk::mxs_quantise(nullptr, d_x.as<float>(), n_tokens, (int)k, d_ops.as<uint8_t>(), d_dx.as<float>());
        }
        d_y.alloc((size_t)n_tokens * n_rows * 4);
        hipEvent_t e0, e1;
        ok(hipEventCreate(&e0), "event"); ok(hipEventCreate(&e1), "event");
        size_t turn = 0;
        auto run = [&]() {
            const uint8_t * w = d_w.as<uint8_t>() + (turn++ % copies) * bytes;
            if (exact) rk::mxe_matmul(nullptr, w, d_ops.as<uint8_t>(), d_dx.as<uint8_t>(), (int)k, n_rows, n_tokens, d_y.as<float>());
            else rk::mxs_matmul(nullptr, w, d_ops.as<uint8_t>(), d_dx.as<float>(), (int)k, n_rows, n_tokens, d_y.as<float>());
        };
        for (int i = 0; i < 3; ++i) run();
        ok(hipEventRecord(e0, nullptr), "record");
        for (int i = 0; i < iters; ++i) run();
        ok(hipEventRecord(e1, nullptr), "record");
        ok(hipEventSynchronize(e1), "sync");
        float ms = 0;
        ok(hipEventElapsedTime(&ms, e0, e1), "elapsed");
        (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
        *out_us = (double)ms * 1e3 / iters;
        return 0;
    });
}

int retro_kernel_stream_time(int64_t bytes, int32_t read_only, int32_t iters, double * out_us) {
    return guarded([&]() -> int {
        DevBuf src, dst;
        src.alloc((size_t)bytes);
        dst.alloc(read_only ? (size_t)1 << 16 : (size_t)bytes);
        ok(hipMemset(src.ptr, 0x5a, src.bytes), "fill");
        hipEvent_t e0, e1;
        ok(hipEventCreate(&e0), "event"); ok(hipEventCreate(&e1), "event");
        for (int i = 0; i < 2; ++i) rk::stream_copy(nullptr, src.ptr, dst.ptr, (size_t)bytes, read_only);
        ok(hipEventRecord(e0, nullptr), "record");
        for (int i = 0; i < iters; ++i) rk::stream_copy(nullptr, src.ptr, dst.ptr, (size_t)bytes, read_only);
        ok(hipEventRecord(e1, nullptr), "record");
        ok(hipEventSynchronize(e1), "sync");
        float ms = 0;
        ok(hipEventElapsedTime(&ms, e0, e1), "elapsed");
        (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
        *out_us = (double)ms * 1e3 / iters;
        return 0;
    });
}

int32_t retro_kernel_page_size(void) { return rk::PAGE; }
int32_t retro_kernel_max_topk(void) { return rk::MAX_TOPK; }

int retro_engine_debug_logits(retro_engine * engine, float * out, size_t n_floats, size_t * out_rows) {
    return guarded([&]() -> int {
        if (!engine) { set_error("engine is required"); return -1; }
        return engine->impl.debug_last_logits(out, n_floats, out_rows);
    });
}

int retro_engine_debug_kv(retro_engine * engine, int32_t layer, int32_t slot, int32_t pos, int32_t want_v,
                          uint16_t * out) {
    return guarded([&]() -> int {
        if (!engine) { set_error("engine is required"); return -1; }
        return engine->impl.debug_read_kv(layer, slot, pos, want_v, out);
    });
}

int retro_engine_debug_pack(retro_engine * engine, int32_t * tok, int32_t * pos, int32_t * seq, int32_t * cell,
                            int32_t * out_index, int32_t * last_index, size_t cap_tokens, size_t cap_rows,
                            int32_t * counts) {
    return guarded([&]() -> int {
        if (!engine) { set_error("engine is required"); return -1; }
        return engine->impl.debug_pack(tok, pos, seq, cell, out_index, last_index, cap_tokens, cap_rows, counts);
    });
}

int retro_engine_debug_profile(retro_engine * engine, int32_t level) {
    return guarded([&]() -> int {
        if (!engine) { set_error("engine is required"); return -1; }
        engine->impl.profile_level(level);
        return 0;
    });
}

int32_t retro_engine_debug_profile_categories(void) { return retro::PC_COUNT; }

int retro_engine_debug_profile_read(retro_engine * engine, double * out_ms, uint64_t * out_launches, int32_t reset) {
    return guarded([&]() -> int {
        if (!engine) { set_error("engine is required"); return -1; }
        engine->impl.profile_read(out_ms, out_launches, reset != 0);
        return 0;
    });
}

int retro_engine_debug_attention_timeline(retro_engine * engine, int32_t enable) {
    return guarded([&]() -> int {
        if (!engine) { set_error("engine is required"); return -1; }
        engine->impl.attention_timeline(enable != 0);
        return 0;
    });
}

int retro_engine_debug_single_token_matvec(retro_engine * engine, int32_t enable) {
    return guarded([&]() -> int {
        if (!engine) { set_error("engine is required"); return -1; }
        engine->impl.single_token_matvec(enable != 0);
        return 0;
    });
}

int retro_engine_debug_attention_timeline_read(retro_engine * engine, uint64_t * out, size_t cap_workgroups, size_t * out_workgroups) {
    return guarded([&]() -> int {
        if (!engine) { set_error("engine is required"); return -1; }
        static_assert(sizeof(uint64_t) == sizeof(unsigned long long), "clock values are 64 bits");
        return engine->impl.attention_timeline_read((unsigned long long *)out, cap_workgroups, out_workgroups);
    });
}

int retro_engine_debug_pages(retro_engine * engine, int32_t slot, int32_t * out, size_t cap, size_t * out_n) {
    return guarded([&]() -> int {
        if (!engine) { set_error("engine is required"); return -1; }
        return engine->impl.debug_page_table(slot, out, cap, out_n);
    });
}

}  // extern "C"
