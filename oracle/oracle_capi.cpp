// TEST INFRASTRUCTURE - CPU oracle, never linked into or called by the product.
//
// Plain-C entry points over the oracle headers so tests, smoke() and the
// bench's cpu_baseline leg can drive it through ctypes. Every function returns
// 0 on success and -1 with orc_last_error() set otherwise.
#include "model.hpp"
#include "sampler.hpp"

#include <chrono>

namespace {
thread_local std::string g_err;

template <typename Fn> int guard(Fn && fn) {
    try {
        g_err.clear();
        return fn();
    } catch (const std::exception & e) {
        g_err = e.what();
        return -1;
    } catch (...) {
        g_err = "unknown exception";
        return -1;
    }
}
}  // namespace

using namespace oracle;

extern "C" {

const char * orc_last_error(void) { return g_err.c_str(); }

// ---- block formats ---------------------------------------------------------
int orc_decode_row(uint32_t type, const uint8_t * src, size_t n, float * out) {
    return guard([&] { decode_row(type, src, n, out); return 0; });
}
int orc_row_bytes(uint32_t type, size_t n, size_t * out) {
    return guard([&] { *out = row_bytes(type, n); return 0; });
}
int orc_quantize_q8_0(const float * x, size_t n, uint8_t * dst) {
    return guard([&] {
        if (n % 32) throw std::runtime_error("oracle: q8_0 needs a multiple of 32");
        quantize_q8_0(x, n, dst);
        return 0;
    });
}
void orc_half_to_float(const uint16_t * h, size_t n, float * out) {
    for (size_t i = 0; i < n; ++i) out[i] = half_to_float(h[i]);
}
void orc_float_to_half(const float * f, size_t n, uint16_t * out) {
    for (size_t i = 0; i < n; ++i) out[i] = float_to_half(f[i]);
}
void orc_double_to_half(const double * f, size_t n, uint16_t * out) {
    for (size_t i = 0; i < n; ++i) out[i] = double_to_half(f[i]);
}
float orc_e8m0_half(uint8_t x) { return e8m0_half(x); }

// The activations of one row as ggml's CPU matmul sees them for a weight of `wtype`.
int orc_activation_row(uint32_t wtype, const float * x, size_t n, float * out) {
    return guard([&] { ggml_activation_row(wtype, x, n, out); return 0; });
}
// y[T][N] = W x^T with W (N rows of K) in raw block format `type`, activations converted as above.
int orc_matmul(uint32_t type, const uint8_t * raw, size_t K, size_t N, const float * x, int T, float * y) {
    return guard([&] {
        gguf_tensor w;
        w.type = type;
        w.ne = {K, N};
        w.data = raw;
        matmul(w, x, T, y);
        return 0;
    });
}
void orc_set_exact_activations(int on) { exact_activations() = on != 0; }

// ---- packing ---------------------------------------------------------------
// The flat batch of one step (retro_gen_core.cpp:2578-2603): rows appended in
// order, flat index = running token count, pos = pos0 + i, seq id = slot, the
// output flag only on the last token of a sampling row; last_index[r] is the
// flat index of row r's last token. Returns the token count through *out_total.
int orc_pack_rows(size_t n_rows, const int32_t * slot, const int32_t * pos0, const uint32_t * n,
                  const uint8_t * sample, const int32_t * tokens_concat,
                  int32_t * out_token, int32_t * out_pos, int32_t * out_seq, uint8_t * out_output,
                  int32_t * out_row, int32_t * last_index, int32_t * row_offset, size_t * out_total) {
    return guard([&] {
        size_t at = 0;
        for (size_t r = 0; r < n_rows; ++r) {
            row_offset[r] = (int32_t)at;
            for (uint32_t i = 0; i < n[r]; ++i) {
                out_token[at] = tokens_concat[at];
                out_pos[at] = (int32_t)((int64_t)pos0[r] + i);
                out_seq[at] = slot[r];
                out_output[at] = (uint8_t)(sample[r] && i + 1 == n[r]);
                out_row[at] = (int32_t)r;
                if (i + 1 == n[r]) last_index[r] = (int32_t)at;
                ++at;
            }
        }
        row_offset[n_rows] = (int32_t)at;
        *out_total = at;
        return 0;
    });
}

// KV cell of every flat token under a paged block table: the page that holds
// position p of slot s is table[s * max_pages + p / page], the cell is
// page_id * page + p % page.
int orc_pack_cells(size_t n_tokens, const int32_t * pos, const int32_t * seq, const int32_t * table,
                   size_t max_pages, int32_t page, int64_t * out_cell) {
    return guard([&] {
        for (size_t t = 0; t < n_tokens; ++t) {
            const int32_t pid = table[(size_t)seq[t] * max_pages + (size_t)(pos[t] / page)];
            if (pid < 0) throw std::runtime_error("oracle: token position has no page");
            out_cell[t] = (int64_t)pid * page + pos[t] % page;
        }
        return 0;
    });
}

// ---- model + context -------------------------------------------------------
void * orc_model_load(const char * path) {
    void * out = nullptr;
    guard([&] { out = new model(path); return 0; });
    return out;
}
void orc_model_free(void * m) { delete (model *)m; }

// out[0..11] = n_layer, n_embd, n_head, n_head_kv, head_dim, n_ff, n_vocab,
//              n_expert, n_expert_used, n_ff_exp, rope_neox, rope_dim
int orc_model_info(void * m, int32_t * out) {
    return guard([&] {
        const hparams & h = ((model *)m)->hp;
        const int32_t v[12] = {h.n_layer, h.n_embd, h.n_head, h.n_head_kv, h.head_dim, h.n_ff, h.n_vocab,
                               h.n_expert, h.n_expert_used, h.n_ff_exp, h.rope_neox ? 1 : 0, h.rope_dim};
        std::memcpy(out, v, sizeof(v));
        return 0;
    });
}
int orc_adapter_load(void * m, const char * path, float scale, int32_t * out_id) {
    return guard([&] { *out_id = load_adapter(*(model *)m, path, scale); return 0; });
}

void * orc_ctx_new(void * m, int n_seq_max) {
    void * out = nullptr;
    guard([&] { out = new context((model *)m, n_seq_max); return 0; });
    return out;
}
void orc_ctx_free(void * c) { delete (context *)c; }
void orc_ctx_set_exact(void * c, int on) { ((context *)c)->exact = on != 0; }
void orc_ctx_set_kv_q8(void * c, int bits) { ((context *)c)->kv_q8 = bits == 8 || bits == 4 ? bits : 0; }
// The stored K or V row of (layer, slot, pos) as the kv_dim values the cache holds, f32.
int orc_ctx_read_kv_f32(void * c, int layer, int slot, int pos, int want_v, float * out) {
    return guard([&] {
        context * ctx = (context *)c;
        const slot_state & s = ctx->slots.at((size_t)slot);
        if (pos < s.begin || pos >= s.end) throw std::runtime_error("oracle: position not resident");
        const size_t kd = (size_t)ctx->kv_dim();
        const auto & src = want_v ? s.v.at((size_t)layer) : s.k.at((size_t)layer);
        std::copy(src.begin() + (size_t)pos * kd, src.begin() + ((size_t)pos + 1) * kd, out);
        return 0;
    });
}

// adapter_of may be NULL (base model for every token); entries <= 0 mean base.
int orc_ctx_step(void * c, int n_tokens, const int32_t * tok, const int32_t * pos, const int32_t * slot,
                 const int32_t * adapter_of, const uint8_t * want, float * logits_out) {
    return guard([&] { ((context *)c)->step(n_tokens, tok, pos, slot, adapter_of, want, logits_out); return 0; });
}
int orc_ctx_seq_rm(void * c, int slot, int p0, int p1) {
    return guard([&] { ((context *)c)->seq_rm(slot, p0, p1); return 0; });
}
int orc_ctx_seq_cp(void * c, int src, int dst, int p0, int p1) {
    return guard([&] { ((context *)c)->seq_cp(src, dst, p0, p1); return 0; });
}
int orc_ctx_seq_pos(void * c, int slot, int32_t * out_min, int32_t * out_max) {
    return guard([&] {
        const slot_state & s = ((context *)c)->slots.at((size_t)slot);
        if (s.end <= s.begin) { *out_min = -1; *out_max = -1; }
        else { *out_min = s.begin; *out_max = s.end - 1; }
        return 0;
    });
}
// Reads back the stored f16 K or V row of (layer, slot, pos) as kv_dim halves.
int orc_ctx_read_kv(void * c, int layer, int slot, int pos, int want_v, uint16_t * out) {
    return guard([&] {
        context * ctx = (context *)c;
        const slot_state & s = ctx->slots.at((size_t)slot);
        if (pos < s.begin || pos >= s.end) throw std::runtime_error("oracle: position not resident");
        const size_t kd = (size_t)ctx->kv_dim();
        const auto & src = want_v ? s.v.at((size_t)layer) : s.k.at((size_t)layer);
        for (size_t i = 0; i < kd; ++i) out[i] = float_to_half(src[(size_t)pos * kd + i]);      // exact for an f16 cache
        return 0;
    });
}

// Installs f16 K and V rows of positions [begin, end) of one layer of a slot
// (rows of kv_dim halves): lets a decode step be checked or timed at a long
// context without running the prefill on the CPU first.
int orc_ctx_import_kv(void * c, int layer, int slot, int begin, int end, const uint16_t * k_rows,
                      const uint16_t * v_rows) {
    return guard([&] {
        context * ctx = (context *)c;
        slot_state & s = ctx->slots.at((size_t)slot);
        const size_t kd = (size_t)ctx->kv_dim();
        auto & kk = s.k.at((size_t)layer);
        auto & vv = s.v.at((size_t)layer);
        if (kk.size() < (size_t)end * kd) { kk.resize((size_t)end * kd); vv.resize((size_t)end * kd); }
        for (size_t i = 0; i < (size_t)(end - begin) * kd; ++i) {
            kk[(size_t)begin * kd + i] = half_to_float(k_rows[i]);
            vv[(size_t)begin * kd + i] = half_to_float(v_rows[i]);
        }
        s.begin = begin;
        s.end = end;
        return 0;
    });
}

// The same with the rows given as the f32 values the cache holds (a Q8_0 cache's scale times code).
int orc_ctx_import_kv_f32(void * c, int layer, int slot, int begin, int end, const float * k_rows, const float * v_rows) {
    return guard([&] {
        context * ctx = (context *)c;
        slot_state & s = ctx->slots.at((size_t)slot);
        const size_t kd = (size_t)ctx->kv_dim();
        auto & kk = s.k.at((size_t)layer);
        auto & vv = s.v.at((size_t)layer);
        if (kk.size() < (size_t)end * kd) { kk.resize((size_t)end * kd); vv.resize((size_t)end * kd); }
        std::copy(k_rows, k_rows + (size_t)(end - begin) * kd, kk.begin() + (size_t)begin * kd);
        std::copy(v_rows, v_rows + (size_t)(end - begin) * kd, vv.begin() + (size_t)begin * kd);
        s.begin = begin;
        s.end = end;
        return 0;
    });
}

// ---- sampling --------------------------------------------------------------
void * orc_rng_new(uint32_t seed) { return new std::mt19937(seed); }
void orc_rng_free(void * r) { delete (std::mt19937 *)r; }
// One std::uniform_real_distribution<double>(0, hi) draw, for pinning the
// generator against the host's own library.
double orc_rng_uniform(void * r, double hi) {
    std::uniform_real_distribution<double> uni(0.0, hi);
    return uni(*(std::mt19937 *)r);
}
uint32_t orc_rng_u32(void * r) { return (*(std::mt19937 *)r)(); }

// v1 row (retro_gen_core.cpp:2751-2773): token, the logprob the step reports
// (temperature 1: logit - max - log(total) from the sampler's own terms;
// otherwise the temperature-1 log-softmax), optional raw top-k.
int orc_sample_v1(const float * logits, size_t n_vocab, float temperature, float top_p, void * rng,
                  int32_t * out_token, float * out_logprob, size_t k, int32_t * top_ids, float * top_lps) {
    return guard([&] {
        float mx;
        double total;
        sample_result r = sample_v1(logits, n_vocab, temperature, top_p, *(std::mt19937 *)rng, mx, total);
        *out_token = r.token;
        *out_logprob = temperature == 1.0f
            ? (float)((double)logits[r.token] - mx - std::log(total))
            : token_logprob(logits, n_vocab, r.token);
        if (k > 0) top_logprobs(logits, n_vocab, k, top_ids, top_lps);
        return 0;
    });
}

// v2 row (retro_gen_core.cpp:2682-2749): token, temperature-1 policy logprob,
// post-transformation sampled_logprob and top-k.
int orc_sample_v2(const float * logits, size_t n_vocab,
                  float temperature, float top_p, int32_t top_k, float min_p,
                  float repeat_penalty, float frequency_penalty, float presence_penalty,
                  uint32_t penalty_window, uint32_t n_bias, const int32_t * bias_ids, const float * bias_values,
                  void * rng, const int32_t * history, size_t n_history,
                  int32_t * out_token, float * out_logprob, float * out_sampled_logprob,
                  size_t k, int32_t * top_ids, float * top_lps, const uint8_t * allowed) {
    return guard([&] {
        params_v2 p;
        p.temperature = temperature; p.top_p = top_p; p.top_k = top_k; p.min_p = min_p;
        p.repeat_penalty = repeat_penalty; p.frequency_penalty = frequency_penalty;
        p.presence_penalty = presence_penalty; p.penalty_window = penalty_window;
        p.bias_ids.assign(bias_ids, bias_ids + n_bias);
        p.bias_values.assign(bias_values, bias_values + n_bias);
        std::vector<int32_t> hist(history, history + n_history);
        sample_result r = sample_v2(logits, n_vocab, p, *(std::mt19937 *)rng, hist, allowed);
        if (r.token < 0) throw std::runtime_error("oracle: no token");
        *out_token = r.token;
        *out_logprob = token_logprob(logits, n_vocab, r.token);
        if (out_sampled_logprob) *out_sampled_logprob = (float)std::log(r.probs[(size_t)r.token] / r.denom);
        if (k > 0) top_of_probs(r, k, top_ids, top_lps);
        return 0;
    });
}

float orc_token_logprob(const float * logits, size_t n_vocab, int32_t token) {
    return token_logprob(logits, n_vocab, token);
}
int orc_top_logprobs(const float * logits, size_t n_vocab, size_t k, int32_t * ids, float * lps) {
    return guard([&] { top_logprobs(logits, n_vocab, k, ids, lps); return 0; });
}

}  // extern "C"
