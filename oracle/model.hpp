// TEST INFRASTRUCTURE - CPU oracle, never linked into or called by the product.
//
// The transformer forward the decode step runs: exact f32 dequantisation of the
// stored blocks, every reduction accumulated in double, K/V rounded to f16 when
// stored (the configs' "f16 KV cache"), and one of two treatments of the
// activations that enter a matmul (context::exact):
//   ggml  - converted, as ggml's CPU matmul does before every dot product, to
//           the companion format of the weight type (Q8_K blocks of 256 for
//           Q4_K, Q8_0 blocks of 32 for Q8_0 and MXFP4, f16 / bf16 rounding for
//           F16 / BF16, nothing for F32): the reference's CPU arithmetic;
//   exact - taken as they are: the plain mathematical product, which is what the
//           2e-2 max-abs / 1e-3 mean-abs logit tolerances are demonstrated on.
// The two differ by a few percent of the logit scale, and two implementations
// of the ggml treatment drift as far apart as soon as one activation lands on
// the other side of a rounding boundary (tests/test_oracle_model.py measures
// both), so no tolerance of 1e-3 can hold between independent implementations
// of it.
//
// The arithmetic of the reference's forward lives in its llama.cpp fork
// (.gitmodules:1-4; upstream base ggml-org/llama.cpp@cd8427d0, recorded at
// crates/retrograd-ffi/runtime/llama.cpp.lock:6-7), which is absent from the
// reference checkout, so this file follows the published architectures the
// reference's fixtures name (scripts/gen-tiny-fixture.py:245-261 qwen2 tensor
// names and metadata keys; scripts/gen-tiny-moe-fixture.py:221-244 MoE names):
//   llama    : RMSNorm, GQA attention, RoPE on adjacent pairs (2i, 2i+1), SwiGLU
//   qwen2    : the same with q/k/v biases and RoPE on split halves (i, i+d/2)
//   qwen3moe : per-head RMSNorm on q and k, split-half RoPE, softmax router,
//              top-k experts with renormalised weights, SwiGLU experts
// RMSNorm is x / sqrt(mean(x^2) + eps) with the weight multiply a separate op
// (generated/rir/rms_norm/kernel.shared_reduce.cu:27-55).
//
// What pins this file (tests/test_oracle_model.py): logits of Hugging Face
// transformers' LlamaForCausalLM, Qwen2ForCausalLM and Qwen3MoeForCausalLM in
// float64 over the dequantised weights of synthetic files, committed as a
// fixture (tests/golden/hf_reference_logits.npz: adjacent-pair and split-half
// rotation, rope_freqs / linear scaling, biases, q/k-norm, the expert router,
// LoRA pairs on all seven layer matrices merged into the dense weights); a
// numpy float64 transformer written independently from the formulas;
// permutation invariance over batch rows, chunked prefill == token-by-token
// decode, seq_cp copy == source.
// PARITY UNPINNED against the reference's own ggml build at float level: the
// fork is absent and no reference test or fixture records absolute logits of
// a causal model.
#pragma once

#include "gguf.hpp"
#include "quant.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <memory>
#include <numeric>

namespace oracle {

struct hparams {
    std::string arch;
    int n_layer = 0, n_embd = 0, n_head = 0, n_head_kv = 0, head_dim = 0, n_ff = 0, n_vocab = 0;
    int n_expert = 0, n_expert_used = 0, n_ff_exp = 0;
    int rope_dim = 0;
    bool rope_neox = false;
    double eps = 1e-5, rope_base = 10000.0;
};

struct lora_pair {
    const gguf_tensor * a = nullptr;  // ne = [n_in, r]
    const gguf_tensor * b = nullptr;  // ne = [r, n_out]
};

struct adapter {
    std::unique_ptr<gguf_file> file;
    double alpha = 0.0;
    float scale = 1.0f;
    std::map<std::string, lora_pair> pairs;  // keyed by base weight name
};

struct model {
    explicit model(const std::string & path) : file(path) {
        hparams & h = hp;
        h.arch = file.s("general.architecture");
        const std::string p = h.arch + ".";
        h.n_layer = (int)file.u(p + "block_count");
        h.n_embd = (int)file.u(p + "embedding_length");
        h.n_head = (int)file.u(p + "attention.head_count");
        h.n_head_kv = (int)file.u_or(p + "attention.head_count_kv", h.n_head);
        h.head_dim = (int)file.u_or(p + "attention.key_length", h.n_embd / h.n_head);
        h.n_ff = (int)file.u_or(p + "feed_forward_length", 0);
        h.eps = file.f_or(p + "attention.layer_norm_rms_epsilon", 1e-5);
        h.rope_base = file.f_or(p + "rope.freq_base", 10000.0);
        h.rope_dim = (int)file.u_or(p + "rope.dimension_count", h.head_dim);
        h.n_expert = (int)file.u_or(p + "expert_count", 0);
        h.n_expert_used = (int)file.u_or(p + "expert_used_count", 0);
        h.n_ff_exp = (int)file.u_or(p + "expert_feed_forward_length", h.n_ff);
        if (h.arch == "llama") h.rope_neox = false;
        else if (h.arch == "qwen2" || h.arch == "qwen3moe" || h.arch == "qwen3") h.rope_neox = true;
        else throw std::runtime_error("oracle: unsupported architecture " + h.arch);
        h.n_vocab = (int)file.need("token_embd.weight").ne[1];
    }
    gguf_file file;
    hparams hp;
    std::map<int, adapter> adapters;
    int next_adapter = 1;
};

// ---------------------------------------------------------------------------

// When set, matmuls take their activations as given (the plain mathematical
// product). Only for measuring what the conversion below changes.
inline bool & exact_activations() {
    static bool flag = false;
    return flag;
}

// Round to nearest, ties to even: ggml's nearest_int() (the 12582912.f trick of
// ggml-quants.c), valid for |v| < 2^22.
inline int nearest_int(float v) { return (int)std::nearbyint(v); }

// What ggml's CPU matmul multiplies a weight row with. ggml_compute_forward_mul_mat
// (ggml-cpu.c of ggml-org/llama.cpp@cd8427d0, the base the reference's fork pins in
// crates/retrograd-ffi/runtime/llama.cpp.lock:6-7; the submodule itself is absent)
// converts every f32 activation row to the weight type's vec_dot_type and the
// dot product runs on that: Q4_K and Q6_K -> Q8_K, Q8_0 and MXFP4 -> Q8_0, F16 -> F16,
// BF16 -> BF16, F32 -> F32 (type_traits_cpu). This writes the converted row back
// as the f32 values it stands for (scale times code).
//   Q8_K (quantize_row_q8_K_ref): per 256 values, `max` is the first value of
//   largest magnitude, iscale = -127 / max, code = min(127, nearest_int(iscale * x)),
//   d = 1 / iscale; an all-zero block has d = 0.
//   Q8_0 (quantize_row_q8_0_ref): per 32 values, d = amax / 127, code =
//   roundf(x / d) (half away from zero) with the unrounded d, the value uses d
//   rounded to f16.
// A row as Q8_0 blocks hold it (quantize_row_q8_0_ref), written back as scale times code.
inline void q8_0_row_values(const float * x, size_t K, float * out) {
    if (K % 32) throw std::runtime_error("oracle: Q8_0 rows need whole blocks of 32");
    for (size_t b = 0; b < K; b += 32) {
        float amax = 0.0f;
        for (int j = 0; j < 32; ++j) amax = std::fmax(amax, std::fabs(x[b + j]));
        const float d = amax / 127.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        const float dh = half_to_float(float_to_half(d));
        for (int j = 0; j < 32; ++j) out[b + j] = dh * std::round(x[b + j] * id);
    }
}

// A row as Q4_0 blocks hold it (ggml's quantize_row_q4_0_ref: per 32 values the element m of largest magnitude, the
// first of equals; d = m / -8; code = min(15, (int8)(x / d + 8.5)) with the unrounded d), written back as
// (code - 8) times d rounded to f16 (quant.rs:236-245 decodes such a block the same way).
inline void q4_0_row_values(const float * x, size_t K, float * out) {
    if (K % 32) throw std::runtime_error("oracle: Q4_0 rows need whole blocks of 32");
    for (size_t b = 0; b < K; b += 32) {
        float amax = 0.0f, mx = 0.0f;
        for (int j = 0; j < 32; ++j) {
            const float v = x[b + j];
            if (amax < std::fabs(v)) { amax = std::fabs(v); mx = v; }
        }
        const float d = mx / -8.0f;
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        const float dh = half_to_float(float_to_half(d));
        for (int j = 0; j < 32; ++j) {
            const int q = std::min(15, (int)(int8_t)(x[b + j] * id + 8.5f));
            out[b + j] = dh * (float)(q - 8);
        }
    }
}

inline void ggml_activation_row(uint32_t wtype, const float * x, size_t K, float * out) {
    if (exact_activations()) { std::copy(x, x + K, out); return; }
    switch (wtype) {
        case T_Q2_K:
        case T_Q3_K:
        case T_IQ4_XS:
        case T_Q4_K:
        case T_Q5_K:
        case T_Q6_K: {
            if (K % 256) throw std::runtime_error("oracle: Q8_K activations need K % 256 == 0");
            for (size_t b = 0; b < K; b += 256) {
                float amax = 0.0f, max = 0.0f;
                for (int j = 0; j < 256; ++j) {
                    const float ax = std::fabs(x[b + j]);
                    if (ax > amax) { amax = ax; max = x[b + j]; }
                }
                if (amax == 0.0f) { std::fill(out + b, out + b + 256, 0.0f); continue; }
                const float iscale = -127.0f / max;
                const float d = 1.0f / iscale;
                for (int j = 0; j < 256; ++j) {
                    const int code = std::min(127, nearest_int(iscale * x[b + j]));
                    out[b + j] = d * (float)code;
                }
            }
            return;
        }
        case T_Q4_0:
        case T_Q5_0:
        case T_IQ4_NL:
        case T_Q4_1:      // ggml pairs these two with Q8_1, whose codes and scale are Q8_0's
        case T_Q5_1:
        case T_Q8_0:
        case T_MXFP4: {
            q8_0_row_values(x, K, out);
            return;
        }
        case T_F16:
            for (size_t k = 0; k < K; ++k) out[k] = half_to_float(float_to_half(x[k]));
            return;
        case T_BF16:
            for (size_t k = 0; k < K; ++k) {
                uint32_t u;
                std::memcpy(&u, &x[k], 4);
                if ((u & 0x7fffffffu) > 0x7f800000u) u |= 0x00400000u;          // quiet NaN, as ggml
                else u += 0x7fffu + ((u >> 16) & 1u);                            // round to nearest even
                u &= 0xffff0000u;
                std::memcpy(&out[k], &u, 4);
            }
            return;
        default:
            std::copy(x, x + K, out);
            return;
    }
}

// y[t][n] = sum_k W[n][k] a[t][k], a = the activations as ggml's CPU path would
// see them (see above). W is stored row by row (ne = [K, N]) in any supported
// block format; one thread owns an output feature, so the result does not
// depend on the thread count.
inline void matmul(const gguf_tensor & w, const float * x_in, int T, float * y, int ldy = -1) {
    const size_t K = w.ne[0];
    const size_t N = w.ne[1];
    const size_t rb = row_bytes(w.type, K);
    if (ldy < 0) ldy = (int)N;
    std::vector<float> converted((size_t)T * K);
    for (int t = 0; t < T; ++t) ggml_activation_row(w.type, x_in + (size_t)t * K, K, converted.data() + (size_t)t * K);
    const float * x = converted.data();
#pragma omp parallel
    {
        std::vector<float> row(K);
#pragma omp for schedule(static)
        for (long n = 0; n < (long)N; ++n) {
            decode_row(w.type, w.data + (size_t)n * rb, K, row.data());
            for (int t = 0; t < T; ++t) {
                const float * xt = x + (size_t)t * K;
                double a0 = 0, a1 = 0, a2 = 0, a3 = 0;
                size_t k = 0;
                for (; k + 4 <= K; k += 4) {
                    a0 += (double)row[k] * xt[k];
                    a1 += (double)row[k + 1] * xt[k + 1];
                    a2 += (double)row[k + 2] * xt[k + 2];
                    a3 += (double)row[k + 3] * xt[k + 3];
                }
                for (; k < K; ++k) a0 += (double)row[k] * xt[k];
                y[(size_t)t * ldy + n] = (float)((a0 + a1) + (a2 + a3));
            }
        }
    }
}

inline void rmsnorm(const float * x, const float * w, int n, double eps, float * y) {
    double ss = 0.0;
    for (int i = 0; i < n; ++i) ss += (double)x[i] * x[i];
    const float scale = (float)(1.0 / std::sqrt(ss / n + eps));
    for (int i = 0; i < n; ++i) y[i] = (x[i] * scale) * (w ? w[i] : 1.0f);
}

inline const float * f32_data(const gguf_tensor & t) {
    if (t.type != T_F32) throw std::runtime_error("oracle: expected an F32 vector: " + t.name);
    return (const float *)t.data;
}

// Rotates one head in place; angle = pos * base^(-2i/d) / factor_i evaluated in double. The factors are the
// model's rope_freqs.weight (ggml's rope divides theta by them: ggml_rope_cache_init, theta / ff) times the linear
// scaling factor, null for none; under yarn scaling (ggml's rope_yarn: theta = theta_interp (1 - mix) + theta_extrap mix
// with mix = the ramp 1 - clamp((i - low) / (high - low), 0, 1) over the pair index between the correction
// dimensions of beta_fast = 32 and beta_slow = 1 rotations within the original context) the divisor is
// 1 / ((1 - mix) / factor + mix) and cosine and sine are multiplied by `magnitude` = attn_factor (1 + 0.1 ln factor).
inline void rope(float * v, int head_dim, int rope_dim, int pos, double base, bool neox, const double * factors = nullptr,
                 double magnitude = 1.0) {
    const int half = rope_dim / 2;
    for (int i = 0; i < half; ++i) {
        const double angle = (double)pos * std::pow(base, -2.0 * i / rope_dim) / (factors ? factors[i] : 1.0);
        const double c = std::cos(angle) * magnitude, s = std::sin(angle) * magnitude;
        const int i0 = neox ? i : 2 * i;
        const int i1 = neox ? i + half : 2 * i + 1;
        const double a = v[i0], b = v[i1];
        v[i0] = (float)(a * c - b * s);
        v[i1] = (float)(a * s + b * c);
    }
    (void)head_dim;
}

struct slot_state {
    int begin = 0, end = 0;              // resident positions [begin, end)
    // per layer: pos * kv_dim values, indexed by absolute pos; the values the cache's storage type holds for what
    // was written (f16 rounding, or scale times code of Q8_0 blocks), as floats
    std::vector<std::vector<float>> k, v;
};

struct context {
    context(model * m, int n_seq_max) : mdl(m), slots((size_t)n_seq_max) {
        for (auto & s : slots) {
            s.k.resize((size_t)m->hp.n_layer);
            s.v.resize((size_t)m->hp.n_layer);
        }
    }
    model * mdl;
    std::vector<slot_state> slots;
    // Which arithmetic step() runs: the activations as they are (what the product computes unless
    // told otherwise, and what the logit tolerances are demonstrated on) or as ggml's CPU matmul
    // converts them (see ggml_activation_row).
    bool exact = true;
    // Storage of the K and V cache: f16, or Q8_0 blocks of 32 along a head's row (the reference's kv_dtype;
    // retro_engine.cpp:84-91 maps it to ggml's type_k / type_v). A row is quantised as quantize_row_q8_0_ref does
    // (quant.hpp) when it is stored; attention then reads scale times code. Under the ggml arithmetic ggml's CPU
    // flash attention would also convert the query row to Q8_0 for the K product (the vec_dot_type of Q8_0): done
    // here when `exact` is off.
    int kv_q8 = 0;          // 0: an f16 cache; 8 / 4: Q8_0 / Q4_0 blocks

    int kv_dim() const { return mdl->hp.n_head_kv * mdl->hp.head_dim; }

    void seq_rm(int slot, int p0, int p1) {
        slot_state & s = slots.at((size_t)slot);
        if (p0 < 0) p0 = 0;
        if (p1 < 0) p1 = 1 << 30;
        if (s.end <= s.begin) return;
        if (p0 <= s.begin && p1 >= s.end) { s.begin = s.end = 0; return; }
        if (p1 >= s.end) { s.end = std::max(s.begin, p0); return; }
        if (p0 <= s.begin) { s.begin = std::min(s.end, p1); return; }
        throw std::runtime_error("oracle: seq_rm would leave a hole");
    }
    void seq_cp(int src, int dst, int p0, int p1) {
        const slot_state & a = slots.at((size_t)src);
        slot_state & b = slots.at((size_t)dst);
        if (p0 < 0) p0 = 0;
        if (p1 < 0) p1 = 1 << 30;
        p0 = std::max(p0, a.begin);
        p1 = std::min(p1, a.end);
        if (p1 <= p0 || src == dst) return;
        const size_t kd = (size_t)kv_dim();
        if (b.end <= b.begin) { b.begin = p0; b.end = p0; }
        if (p0 != b.end && p1 != b.begin) throw std::runtime_error("oracle: seq_cp range is not adjacent to dst");
        for (size_t l = 0; l < b.k.size(); ++l) {
            if (b.k[l].size() < (size_t)p1 * kd) { b.k[l].resize((size_t)p1 * kd); b.v[l].resize((size_t)p1 * kd); }
            std::copy(a.k[l].begin() + (size_t)p0 * kd, a.k[l].begin() + (size_t)p1 * kd, b.k[l].begin() + (size_t)p0 * kd);
            std::copy(a.v[l].begin() + (size_t)p0 * kd, a.v[l].begin() + (size_t)p1 * kd, b.v[l].begin() + (size_t)p0 * kd);
        }
        b.begin = std::min(b.begin, p0);
        b.end = std::max(b.end, p1);
    }

    // y += scale * alpha/r * B (A x) for the adapter each token decodes under.
    void add_lora(const std::string & wname, const float * x, int T, const int32_t * adapter_of,
                  float * y, int N) const {
        if (!adapter_of) return;
        for (int t = 0; t < T; ++t) {
            if (adapter_of[t] <= 0) continue;
            auto ai = mdl->adapters.find(adapter_of[t]);
            if (ai == mdl->adapters.end()) throw std::runtime_error("oracle: adapter not loaded");
            auto pi = ai->second.pairs.find(wname);
            if (pi == ai->second.pairs.end()) continue;
            const gguf_tensor & A = *pi->second.a;
            const gguf_tensor & B = *pi->second.b;
            const int r = (int)A.ne[1];
            const int K = (int)A.ne[0];
            std::vector<float> mid((size_t)r), delta((size_t)N);
            matmul(A, x + (size_t)t * K, 1, mid.data());
            matmul(B, mid.data(), 1, delta.data());
            const float s = (float)((double)ai->second.scale * ai->second.alpha / r);
            for (int n = 0; n < N; ++n) y[(size_t)t * N + n] += s * delta[n];
        }
    }

    // One decode over a packed batch. logits_out: n_outputs rows of n_vocab.
    void step(int T, const int32_t * tok, const int32_t * pos, const int32_t * slot,
              const int32_t * adapter_of, const uint8_t * want, float * logits_out) {
        struct restore {
            bool saved;
            ~restore() { exact_activations() = saved; }
        } keep{exact_activations()};
        exact_activations() = exact;
        const hparams & h = mdl->hp;
        const gguf_file & g = mdl->file;
        const int E = h.n_embd, HD = h.head_dim, NH = h.n_head, NKV = h.n_head_kv;
        const int QD = NH * HD, KD = NKV * HD;
        const size_t kd = (size_t)KD;
        // per-frequency divisors of the rotation angle: rope_freqs.weight and linear scaling (see rope())
        std::vector<double> rope_div;
        double rope_magnitude = 1.0;
        {
            const std::string p = h.arch + ".rope.scaling.type";
            const std::string scaling = g.has(p) ? g.s(p) : std::string("none");
            double lin = 1.0;
            if (scaling == "linear") lin = g.f_or(h.arch + ".rope.scaling.factor", 1.0);
            else if (scaling != "none" && !scaling.empty() && scaling != "yarn") throw std::runtime_error("oracle: rope scaling type " + scaling + " is not modelled");
            const gguf_tensor * rf = g.find("rope_freqs.weight");
            if (rf || lin != 1.0 || scaling == "yarn") {
                rope_div.assign((size_t)(h.rope_dim / 2), lin);
                if (rf) {
                    if (rf->type != T_F32 || (int)rf->ne[0] != h.rope_dim / 2) throw std::runtime_error("oracle: rope_freqs.weight has an unexpected shape");
                    for (size_t i = 0; i < rope_div.size(); ++i) rope_div[i] *= (double)f32_data(*rf)[i];
                }
            }
            if (scaling == "yarn") {
                const double factor = g.f_or(h.arch + ".rope.scaling.factor", 1.0);
                const double n_orig = (double)g.u_or(h.arch + ".rope.scaling.original_context_length", 0);
                if (!(factor > 0.0) || !(n_orig > 0.0)) throw std::runtime_error("oracle: yarn scaling needs a factor and the original context length");
                const double n_dims = (double)h.rope_dim;
                auto corr_dim = [&](double n_rot) { return n_dims * std::log(n_orig / (n_rot * 2.0 * M_PI)) / (2.0 * std::log(h.rope_base)); };
                const double low = std::max(0.0, std::floor(corr_dim(g.f_or(h.arch + ".rope.scaling.yarn_beta_fast", 32.0))));
                const double high = std::min(n_dims - 1.0, std::ceil(corr_dim(g.f_or(h.arch + ".rope.scaling.yarn_beta_slow", 1.0))));
                for (size_t i = 0; i < rope_div.size(); ++i) {
                    const double mix = 1.0 - std::min(1.0, std::max(0.0, ((double)i - low) / std::max(0.001, high - low)));
                    rope_div[i] /= (1.0 - mix) / factor + mix;
                }
                rope_magnitude = g.f_or(h.arch + ".rope.scaling.attn_factor", 1.0) * (1.0 + 0.1 * std::log(factor));
            }
        }
        const double * rope_factors = rope_div.empty() ? nullptr : rope_div.data();
        std::vector<float> x((size_t)T * E), xn((size_t)T * E);
        {
            const gguf_tensor & emb = g.need("token_embd.weight");
            const size_t rb = row_bytes(emb.type, (size_t)E);
            for (int t = 0; t < T; ++t) decode_row(emb.type, emb.data + (size_t)tok[t] * rb, (size_t)E, &x[(size_t)t * E]);
        }
        // Make the positions this step writes resident before attention reads them.
        for (int t = 0; t < T; ++t) {
            slot_state & s = slots.at((size_t)slot[t]);
            if (s.end <= s.begin) { s.begin = pos[t]; s.end = pos[t] + 1; }
            if (pos[t] < s.begin) throw std::runtime_error("oracle: position before the resident range");
            s.end = std::max(s.end, pos[t] + 1);
            const size_t need = ((size_t)pos[t] + 1) * kd;
            for (int l = 0; l < h.n_layer; ++l) {
                if (s.k[(size_t)l].size() < need) { s.k[(size_t)l].resize(need); s.v[(size_t)l].resize(need); }
            }
        }
        std::vector<float> q((size_t)T * QD), k((size_t)T * KD), v((size_t)T * KD), att((size_t)T * QD), proj((size_t)T * E);
        for (int l = 0; l < h.n_layer; ++l) {
            const std::string b = "blk." + std::to_string(l) + ".";
            const float * wn = f32_data(g.need(b + "attn_norm.weight"));
            for (int t = 0; t < T; ++t) rmsnorm(&x[(size_t)t * E], wn, E, h.eps, &xn[(size_t)t * E]);
            matmul(g.need(b + "attn_q.weight"), xn.data(), T, q.data());
            matmul(g.need(b + "attn_k.weight"), xn.data(), T, k.data());
            matmul(g.need(b + "attn_v.weight"), xn.data(), T, v.data());
            add_lora(b + "attn_q.weight", xn.data(), T, adapter_of, q.data(), QD);
            add_lora(b + "attn_k.weight", xn.data(), T, adapter_of, k.data(), KD);
            add_lora(b + "attn_v.weight", xn.data(), T, adapter_of, v.data(), KD);
            if (const gguf_tensor * bq = g.find(b + "attn_q.bias")) {
                const float * bk = f32_data(g.need(b + "attn_k.bias"));
                const float * bv = f32_data(g.need(b + "attn_v.bias"));
                const float * bqd = f32_data(*bq);
                for (int t = 0; t < T; ++t) {
                    for (int i = 0; i < QD; ++i) q[(size_t)t * QD + i] += bqd[i];
                    for (int i = 0; i < KD; ++i) { k[(size_t)t * KD + i] += bk[i]; v[(size_t)t * KD + i] += bv[i]; }
                }
            }
            const gguf_tensor * qn = g.find(b + "attn_q_norm.weight");
            const gguf_tensor * kn = g.find(b + "attn_k_norm.weight");
            for (int t = 0; t < T; ++t) {
                for (int hh = 0; hh < NH; ++hh) {
                    float * qh = &q[(size_t)t * QD + (size_t)hh * HD];
                    if (qn) rmsnorm(qh, f32_data(*qn), HD, h.eps, qh);
                    rope(qh, HD, h.rope_dim, pos[t], h.rope_base, h.rope_neox, rope_factors, rope_magnitude);
                }
                slot_state & s = slots[(size_t)slot[t]];
                for (int hh = 0; hh < NKV; ++hh) {
                    float * kh = &k[(size_t)t * KD + (size_t)hh * HD];
                    if (kn) rmsnorm(kh, f32_data(*kn), HD, h.eps, kh);
                    rope(kh, HD, h.rope_dim, pos[t], h.rope_base, h.rope_neox, rope_factors, rope_magnitude);
                }
                float * kc = &s.k[(size_t)l][(size_t)pos[t] * kd];
                float * vc = &s.v[(size_t)l][(size_t)pos[t] * kd];
                if (kv_q8) {
                    if (HD % 32 != 0) throw std::runtime_error("oracle: a quantised cache needs heads of whole 32-blocks");
                    (kv_q8 == 4 ? q4_0_row_values : q8_0_row_values)(&k[(size_t)t * KD], (size_t)KD, kc);
                    (kv_q8 == 4 ? q4_0_row_values : q8_0_row_values)(&v[(size_t)t * KD], (size_t)KD, vc);
                } else {
                    for (int i = 0; i < KD; ++i) {
                        kc[i] = half_to_float(float_to_half(k[(size_t)t * KD + i]));
                        vc[i] = half_to_float(float_to_half(v[(size_t)t * KD + i]));
                    }
                }
                s.end = std::max(s.end, pos[t] + 1);
            }
            const int G = NH / NKV;
            const double inv_sqrt = 1.0 / std::sqrt((double)HD);
#pragma omp parallel for collapse(2) schedule(dynamic)
            for (int t = 0; t < T; ++t) {
                for (int hh = 0; hh < NH; ++hh) {
                    const slot_state & s = slots[(size_t)slot[t]];
                    const int p0 = s.begin, p1 = pos[t] + 1;
                    const int kvh = hh / G;
                    const float * qh = &q[(size_t)t * QD + (size_t)hh * HD];
                    std::vector<float> qconv;
                    if (kv_q8 && !exact) {      // ggml: the query row as Q8_0, the companion format of a Q8_0 or Q4_0 K row
                        qconv.resize((size_t)HD);
                        q8_0_row_values(qh, (size_t)HD, qconv.data());
                        qh = qconv.data();
                    }
                    std::vector<double> sc((size_t)(p1 - p0));
                    double mx = -INFINITY;
                    for (int p = p0; p < p1; ++p) {
                        const float * kc = &s.k[(size_t)l][(size_t)p * kd + (size_t)kvh * HD];
                        double d = 0.0;
                        for (int i = 0; i < HD; ++i) d += (double)qh[i] * kc[i];
                        d *= inv_sqrt;
                        sc[(size_t)(p - p0)] = d;
                        mx = std::max(mx, d);
                    }
                    double den = 0.0;
                    for (auto & e : sc) { e = std::exp(e - mx); den += e; }
                    std::vector<double> acc((size_t)HD, 0.0);
                    for (int p = p0; p < p1; ++p) {
                        const float * vc = &s.v[(size_t)l][(size_t)p * kd + (size_t)kvh * HD];
                        const double w = sc[(size_t)(p - p0)];
                        for (int i = 0; i < HD; ++i) acc[(size_t)i] += w * vc[i];
                    }
                    float * o = &att[(size_t)t * QD + (size_t)hh * HD];
                    for (int i = 0; i < HD; ++i) o[i] = (float)(acc[(size_t)i] / den);
                }
            }
            matmul(g.need(b + "attn_output.weight"), att.data(), T, proj.data());
            add_lora(b + "attn_output.weight", att.data(), T, adapter_of, proj.data(), E);
            for (size_t i = 0; i < x.size(); ++i) x[i] += proj[i];

            const float * wf = f32_data(g.need(b + "ffn_norm.weight"));
            for (int t = 0; t < T; ++t) rmsnorm(&x[(size_t)t * E], wf, E, h.eps, &xn[(size_t)t * E]);
            if (h.n_expert > 0) {
                moe_ffn(b, xn.data(), T, proj.data());
            } else {
                const int F = h.n_ff;
                std::vector<float> gate((size_t)T * F), up((size_t)T * F);
                matmul(g.need(b + "ffn_gate.weight"), xn.data(), T, gate.data());
                matmul(g.need(b + "ffn_up.weight"), xn.data(), T, up.data());
                // adapters may target every true matrix of a layer (retro_lora.cpp:165-169)
                add_lora(b + "ffn_gate.weight", xn.data(), T, adapter_of, gate.data(), F);
                add_lora(b + "ffn_up.weight", xn.data(), T, adapter_of, up.data(), F);
                for (size_t i = 0; i < gate.size(); ++i) gate[i] = silu(gate[i]) * up[i];
                matmul(g.need(b + "ffn_down.weight"), gate.data(), T, proj.data());
                add_lora(b + "ffn_down.weight", gate.data(), T, adapter_of, proj.data(), E);
            }
            for (size_t i = 0; i < x.size(); ++i) x[i] += proj[i];
        }
        // Output rows only.
        std::vector<int> outs;
        for (int t = 0; t < T; ++t) if (want[t]) outs.push_back(t);
        if (outs.empty()) return;
        const float * wo = f32_data(g.need("output_norm.weight"));
        std::vector<float> xo(outs.size() * (size_t)E);
        for (size_t i = 0; i < outs.size(); ++i) rmsnorm(&x[(size_t)outs[i] * E], wo, E, h.eps, &xo[i * (size_t)E]);
        const gguf_tensor * head = g.find("output.weight");
        if (!head) head = &g.need("token_embd.weight");
        matmul(*head, xo.data(), (int)outs.size(), logits_out);
        if (const gguf_tensor * ob = g.find("output.bias")) {
            const float * bd = f32_data(*ob);
            for (size_t i = 0; i < outs.size(); ++i)
                for (int n = 0; n < h.n_vocab; ++n) logits_out[i * (size_t)h.n_vocab + n] += bd[n];
        }
    }

    static float silu(float g) { return (float)((double)g / (1.0 + std::exp(-(double)g))); }

    // Softmax router over all experts, top-k by probability (ties to the lower
    // index), weights renormalised over the selected experts, SwiGLU experts.
    void moe_ffn(const std::string & b, const float * xn, int T, float * out) const {
        const hparams & h = mdl->hp;
        const gguf_file & g = mdl->file;
        const int E = h.n_embd, NE = h.n_expert, KU = h.n_expert_used, F = h.n_ff_exp;
        std::vector<float> rl((size_t)T * NE);
        matmul(g.need(b + "ffn_gate_inp.weight"), xn, T, rl.data());
        const gguf_tensor & wg = g.need(b + "ffn_gate_exps.weight");
        const gguf_tensor & wu = g.need(b + "ffn_up_exps.weight");
        const gguf_tensor & wd = g.need(b + "ffn_down_exps.weight");
        const size_t g_bytes = row_bytes(wg.type, (size_t)E) * (size_t)F;
        const size_t d_bytes = row_bytes(wd.type, (size_t)F) * (size_t)E;
        std::vector<float> gate((size_t)F), up((size_t)F), down((size_t)E);
        for (int t = 0; t < T; ++t) {
            const float * r = &rl[(size_t)t * NE];
            double mx = -INFINITY;
            for (int e = 0; e < NE; ++e) mx = std::max(mx, (double)r[e]);
            std::vector<double> p((size_t)NE);
            double den = 0.0;
            for (int e = 0; e < NE; ++e) { p[(size_t)e] = std::exp((double)r[e] - mx); den += p[(size_t)e]; }
            for (auto & e : p) e /= den;
            std::vector<int> order((size_t)NE);
            std::iota(order.begin(), order.end(), 0);
            std::stable_sort(order.begin(), order.end(), [&](int a, int c) { return p[(size_t)a] > p[(size_t)c]; });
            double wsum = 0.0;
            for (int j = 0; j < KU; ++j) wsum += p[(size_t)order[(size_t)j]];
            std::vector<double> acc((size_t)E, 0.0);
            for (int j = 0; j < KU; ++j) {
                const int e = order[(size_t)j];
                gguf_tensor eg = wg, eu = wu, ed = wd;
                eg.ne = {(uint64_t)E, (uint64_t)F}; eg.data = wg.data + (size_t)e * g_bytes;
                eu.ne = {(uint64_t)E, (uint64_t)F}; eu.data = wu.data + (size_t)e * g_bytes;
                ed.ne = {(uint64_t)F, (uint64_t)E}; ed.data = wd.data + (size_t)e * d_bytes;
                matmul(eg, xn + (size_t)t * E, 1, gate.data());
                matmul(eu, xn + (size_t)t * E, 1, up.data());
                for (int i = 0; i < F; ++i) gate[(size_t)i] = silu(gate[(size_t)i]) * up[(size_t)i];
                matmul(ed, gate.data(), 1, down.data());
                const double w = p[(size_t)e] / wsum;
                for (int i = 0; i < E; ++i) acc[(size_t)i] += w * down[(size_t)i];
            }
            for (int i = 0; i < E; ++i) out[(size_t)t * E + i] = (float)acc[(size_t)i];
        }
    }
};

// LoRA adapter file as the reference writes it (retro_lora.cpp:1004-1043,
// 1143-1153): general.type = "adapter", adapter.type = "lora",
// adapter.lora.alpha (f32), tensors "<weight>.lora_a" / "<weight>.lora_b".
inline int load_adapter(model & m, const std::string & path, float scale) {
    adapter a;
    a.file.reset(new gguf_file(path));
    if (a.file->s("general.type") != "adapter" || a.file->s("adapter.type") != "lora")
        throw std::runtime_error("oracle: not a LoRA adapter file");
    a.alpha = a.file->f("adapter.lora.alpha");
    a.scale = scale;
    for (const gguf_tensor & t : a.file->tensors) {
        const std::string suffix_a = ".lora_a";
        if (t.name.size() > suffix_a.size() && t.name.compare(t.name.size() - suffix_a.size(), suffix_a.size(), suffix_a) == 0) {
            const std::string base = t.name.substr(0, t.name.size() - suffix_a.size());
            lora_pair p;
            p.a = &t;
            p.b = &a.file->need(base + ".lora_b");
            a.pairs.emplace(base, p);
        }
    }
    const int id = m.next_adapter++;
    m.adapters.emplace(id, std::move(a));
    return id;
}

}  // namespace oracle
