#include "engine.hpp"

#include <algorithm>
#include <array>
#include <climits>
#include <cmath>
#include <cstring>
#include <sstream>

namespace retro {

namespace {
thread_local std::string g_last_error;

void hip_check(hipError_t err, const char * what) {
    if (err != hipSuccess) {
        throw std::runtime_error(std::string("HIP error in ") + what + ": " + hipGetErrorString(err));
    }
}
}  // namespace

void set_error(std::string message) { g_last_error = std::move(message); }
void clear_error() { g_last_error.clear(); }
const std::string & last_error() { return g_last_error; }

// ---- buffers --------------------------------------------------------------------

DevBuf::~DevBuf() { release(); }
DevBuf & DevBuf::operator=(DevBuf && o) noexcept {
    if (this != &o) {
        release();
        ptr = o.ptr;
        bytes = o.bytes;
        o.ptr = nullptr;
        o.bytes = 0;
    }
    return *this;
}
void DevBuf::release() {
    if (ptr) (void)hipFree(ptr);
    ptr = nullptr;
    bytes = 0;
}
void DevBuf::alloc(size_t n) {
    release();
    if (n == 0) return;
    hip_check(hipMalloc(&ptr, n), "hipMalloc");
    bytes = n;
}
void DevBuf::ensure(size_t n) {
    if (n > bytes) alloc(n + n / 4);
}

HostPinned::~HostPinned() {
    if (ptr) (void)hipHostFree(ptr);
}
void HostPinned::ensure(size_t n) {
    if (n <= bytes) return;
    if (ptr) (void)hipHostFree(ptr);
    ptr = nullptr;
    bytes = 0;
    hip_check(hipHostMalloc(&ptr, n + n / 4, hipHostMallocDefault), "hipHostMalloc");
    bytes = n + n / 4;
}

// ---- construction -----------------------------------------------------------------

Engine::Engine(const std::string & path, const retro_engine_config & config) : cfg_(config) {
    int n_dev = 0;
    if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev == 0) {
        throw std::runtime_error("no HIP device is available: this library has no CPU path");
    }
    hip_check(hipSetDevice(0), "hipSetDevice");
    hip_check(hipStreamCreate(&stream_), "hipStreamCreate");
    rk::sample_static_prepare();       // the no-allocation greedy scan then only launches, also under stream capture
    if (const char * v = std::getenv("RETRO_FUSED_DECODE_ATTENTION")) fused_decode_attention_ = std::atoi(v) != 0;
    if (const char * v = std::getenv("RETRO_MOE_SCALED")) moe_scaled_ = std::atoi(v) != 0;
    {
        // RETRO_ACTIVATIONS=ggml: every matmul multiplies the activations as ggml's CPU path converts them
        // (Q8_K / Q8_0 codes, f16 / bf16 rounding); unset or "exact": the f32 values (as f16 hi/lo pairs).
        if (const char * f = std::getenv("RETRO_GEMV_FUSE")) gemv_fuse_ = std::atoi(f) != 0;
        if (const char * f = std::getenv("RETRO_GEMV_EXACT")) gemv_exact_ = std::atoi(f) != 0;
        // ... and the output projection merges at most this many attention splits per kv head itself (0: never)
        if (const char * f = std::getenv("RETRO_GEMV_MERGE_SPLITS")) merge_max_splits_ = std::max(0, std::min(std::atoi(f), rk::GEMV_COMBINE_MAX_SPLITS));      // 0: producers keep their own launches
        // steps of at most this many tokens go through the integer matrix-vector kernel under the ggml arithmetic (0: never)
        const char * g = std::getenv("RETRO_GEMV_MAX_T");
        gemv_max_t_ = g ? std::max(0, std::min(std::atoi(g), rk::GEMV_MAX_T)) : rk::GEMV_MAX_T;
        const char * v = std::getenv("RETRO_ACTIVATIONS");
        const std::string mode = v ? v : "exact";
        if (mode == "ggml") ggml_activations_ = true;
        else if (mode != "exact" && !mode.empty()) throw std::runtime_error("RETRO_ACTIVATIONS must be \"exact\" or \"ggml\"");
    }
    load_model(path);

    // Per-sequence context: the whole pool when unified, an equal share otherwise.
    n_ctx_seq_ = cfg_.kv_unified ? (int)cfg_.n_ctx : (int)(cfg_.n_ctx / cfg_.n_seq_max);
    if (n_ctx_seq_ <= 0) throw std::runtime_error("engine n_ctx is too small for n_seq_max sequences");
    max_pages_ = (n_ctx_seq_ + rk::PAGE - 1) / rk::PAGE;
    // What paging can waste against a cache that shares single cells: per slot the partially filled last
    // page, and the page in which the slot left a range it shares with another (its private copy of that
    // page repeats up to PAGE - 1 shared cells). Two spare pages per slot cover both, so a step that fits
    // n_ctx distinct cells always finds its pages.
    n_pages_ = (int)((cfg_.n_ctx + rk::PAGE - 1) / rk::PAGE + 2 * cfg_.n_seq_max);
    // [page][kv head]: the other order (a head's pages side by side) was measured 3 % slower in the attention kernel
    kv_q8_ = cfg_.kv_dtype == RETRO_ENGINE_KV_DTYPE_Q8_0 ? rk::KV_Q8 : cfg_.kv_dtype == RETRO_ENGINE_KV_DTYPE_Q4_0 ? rk::KV_Q4 : rk::KV_F16;
    if (kv_q8_ != rk::KV_F16 && hp_.head_dim % 32 != 0) throw std::runtime_error("a Q8_0 or Q4_0 KV cache needs head_dim to be a multiple of 32");
    kv_strides_ = rk::kv_strides(n_pages_, hp_.n_head_kv, hp_.head_dim, false, kv_q8_);
    const int G = hp_.n_head / hp_.n_head_kv;
    if (hp_.n_head % hp_.n_head_kv != 0 || G > 16) throw std::runtime_error("unsupported attention head grouping");
    qt_ = rk::attention_tile_tokens(G);

    const size_t pool_halves = (size_t)n_pages_ * hp_.n_head_kv * rk::kv_block_halves(hp_.head_dim, kv_q8_);
    k_pool_.resize((size_t)hp_.n_layer);
    v_pool_.resize((size_t)hp_.n_layer);
    const size_t pool_bytes = (pool_halves * 2 + 255) / 256 * 256;
    kv_slab_.alloc(pool_bytes * 2 * (size_t)hp_.n_layer);
    // Pages must never hold non-finite bit patterns: a masked score times a
    // NaN value would poison the output.
    hip_check(hipMemsetAsync(kv_slab_.ptr, 0, kv_slab_.bytes, stream_), "hipMemsetAsync");
    for (int l = 0; l < hp_.n_layer; ++l) {
        k_pool_[(size_t)l] = PoolView{(uint8_t *)kv_slab_.ptr + pool_bytes * (2 * (size_t)l), pool_halves * 2};
        v_pool_[(size_t)l] = PoolView{(uint8_t *)kv_slab_.ptr + pool_bytes * (2 * (size_t)l + 1), pool_halves * 2};
    }
    table_.alloc((size_t)cfg_.n_seq_max * max_pages_ * sizeof(int32_t));
    hip_check(hipMemsetAsync(table_.ptr, 0xff, table_.bytes, stream_), "hipMemsetAsync");
    slots_.resize(cfg_.n_seq_max);
    for (auto & s : slots_) s.pages.assign((size_t)max_pages_, -1);
    page_ref_.assign((size_t)n_pages_, 0);
    for (int p = 0; p < n_pages_; ++p) free_pages_.push(p);

    build_buffers();
    hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
}

Engine::~Engine() {
    for (hipEvent_t e : prof_events_) (void)hipEventDestroy(e);
    if (stream_) {
        (void)hipStreamSynchronize(stream_);
        (void)hipStreamDestroy(stream_);
    }
}

void Engine::upload_f32(const TensorInfo * t, DevBuf & out, size_t expect) {
    if (!t) return;
    if (t->type != rk::WT_F32) throw std::runtime_error("tensor " + t->name + " must be F32");
    if (t->nbytes != expect * 4) throw std::runtime_error("tensor " + t->name + " has an unexpected size");
    out.alloc(t->nbytes);
    hip_check(hipMemcpy(out.ptr, t->data, t->nbytes, hipMemcpyHostToDevice), "hipMemcpy");
}

void Engine::upload_weight(const TensorInfo & t, int64_t K, int64_t N, const uint8_t * data, size_t bytes,
                           bool keep_raw, DevWeight & out) {
    rk::geom_of(t.type);   // refuses unsupported storage
    if (rk::row_bytes(t.type, K) * (size_t)N != bytes) throw std::runtime_error("tensor " + t.name + " has an unexpected size");
    out.w.type = t.type;
    out.w.K = (int)K;
    out.w.N = (int)N;
    out.w.bytes = bytes;
    DevBuf raw;
    raw.alloc(bytes);
    hip_check(hipMemcpy(raw.ptr, data, bytes, hipMemcpyHostToDevice), "hipMemcpy");
    if (!keep_raw && rk::can_pack(t.type, K, N)) {
        out.buf.alloc(bytes);
        rk::repack(stream_, t.type, raw.as<uint8_t>(), out.buf.as<uint8_t>(), (int)K, (int)N);
        hip_check(hipStreamSynchronize(stream_), "repack");
        out.w.packed = out.buf.as<uint8_t>();
        out.w.raw = nullptr;
    } else {
        out.buf = std::move(raw);
        out.w.raw = out.buf.as<uint8_t>();
        out.w.packed = nullptr;
    }
}

// An expert tensor [K][N][n_expert]: n_expert * N rows of K, tiled per expert.
void Engine::upload_experts(const TensorInfo & t, int64_t K, int64_t N, DevWeight & out) {
    const int64_t rows = N * hp_.n_expert;
    if (!rk::moe_can_pack(t.type, K, N)) throw std::runtime_error("expert tensor " + t.name + " must be MXFP4, Q8_0, Q4_K, Q5_K, Q6_K or a type rewritten as Q8_0 (Q4_0, Q5_0, IQ4_NL, Q3_K), with widths that are multiples of 256 and 16");
    if (rk::row_bytes(t.type, K) * (size_t)rows != t.nbytes) throw std::runtime_error("tensor " + t.name + " has an unexpected size");
    out.w.type = t.type;
    out.w.K = (int)K;
    out.w.N = (int)N;              // rows per expert
    out.w.bytes = t.nbytes;
    DevBuf raw;
    raw.alloc(t.nbytes);
    hip_check(hipMemcpy(raw.ptr, t.data, t.nbytes, hipMemcpyHostToDevice), "hipMemcpy");
    out.buf.alloc(t.nbytes);
    rk::moe_repack(stream_, t.type, raw.as<uint8_t>(), out.buf.as<uint8_t>(), (int)K, rows);
    hip_check(hipStreamSynchronize(stream_), "repack");
    out.w.packed = out.buf.as<uint8_t>();
    out.w.raw = nullptr;
    // MXFP4 experts of the exact arithmetic also in the records of the block-scaled kernels (decode-sized steps take them)
    if (t.type == rk::WT_MXFP4 && moe_scaled_ && !ggml_activations_ && rk::mxe_moe_can((int)K, (int)N)) {
        out.records.alloc(rk::mxs_packed_bytes(K, rows));
        rk::mxs_repack(stream_, raw.as<uint8_t>(), out.records.as<uint8_t>(), (int)K, rows);
        hip_check(hipStreamSynchronize(stream_), "repack");
        out.w.records = out.records.as<uint8_t>();
    }
}

// Row-wise concatenation of matrices that share K and storage type: one matmul
// instead of several. Neighbours that differ stay separate matrices (a Q4_K_M
// file keeps attn_v in Q6_K: q and k are joined, v follows on its own).
void Engine::upload_fused(const std::vector<const TensorInfo *> & parts, std::vector<DevWeight> & out) {
    out.clear();
    size_t i = 0;
    while (i < parts.size()) {
        size_t j = i + 1;
        while (j < parts.size() && parts[j]->type == parts[i]->type && parts[j]->ne[0] == parts[i]->ne[0]) ++j;
        out.emplace_back();
        if (j == i + 1) {
            upload_weight(*parts[i], parts[i]->ne[0], parts[i]->ne[1], parts[i]->data, parts[i]->nbytes, false, out.back());
        } else {
            std::vector<uint8_t> joined;
            int64_t N = 0;
            for (size_t p = i; p < j; ++p) {
                joined.insert(joined.end(), parts[p]->data, parts[p]->data + parts[p]->nbytes);
                N += parts[p]->ne[1];
            }
            upload_weight(*parts[i], parts[i]->ne[0], N, joined.data(), joined.size(), false, out.back());
        }
        i = j;
    }
}

// Gate and up projections as one matrix whose rows alternate in groups of 64:
// the 64 gate rows of hidden columns [64 b, 64 b + 64), then their 64 up rows.
// A matmul workgroup owns 128 consecutive rows, so it holds both factors of
// its 64 hidden columns and applies SwiGLU in its epilogue. Returns false (and
// uploads nothing) when the pair does not qualify.
bool Engine::upload_gate_up_interleaved(const TensorInfo & g, const TensorInfo & u, std::vector<DevWeight> & out) {
    const int64_t K = g.ne[0], F = g.ne[1];
    if (g.type != u.type || u.ne[0] != K || u.ne[1] != F || F % 64 != 0) return false;
    if (!rk::can_pack(g.type, K, 2 * F)) return false;
    const size_t rb = g.nbytes / (size_t)F;
    std::vector<uint8_t> joined(2 * g.nbytes);
    for (int64_t b = 0; b < F / 64; ++b) {
        std::memcpy(joined.data() + (size_t)(2 * b) * 64 * rb, g.data + (size_t)b * 64 * rb, 64 * rb);
        std::memcpy(joined.data() + (size_t)(2 * b + 1) * 64 * rb, u.data + (size_t)b * 64 * rb, 64 * rb);
    }
    out.clear();
    out.emplace_back();
    upload_weight(g, K, 2 * F, joined.data(), joined.size(), false, out.back());
    if (!out.back().w.packed) { out.clear(); return false; }
    return true;
}

void Engine::load_model(const std::string & path) {
    GgufFile g(path);
    g.rewrite_as_q8_0();      // Q4_0, Q5_0, IQ4_NL and Q3_K tensors become the Q8_0 rows that hold the same values
    HParams & h = hp_;
    h.arch = g.get_string("general.architecture");
    if (h.arch == "llama") h.rope_neox = false;
    else if (h.arch == "qwen2" || h.arch == "qwen3" || h.arch == "qwen3moe") h.rope_neox = true;
    else throw std::runtime_error("unsupported model architecture: " + h.arch);
    const std::string a = h.arch + ".";
    h.n_layer = (int)g.need_int(a + "block_count");
    h.n_embd = (int)g.need_int(a + "embedding_length");
    h.n_head = (int)g.need_int(a + "attention.head_count");
    h.n_head_kv = (int)g.get_int(a + "attention.head_count_kv", h.n_head);
    h.head_dim = (int)g.get_int(a + "attention.key_length", h.n_embd / h.n_head);
    h.n_ff = (int)g.get_int(a + "feed_forward_length", 0);
    h.eps = (float)g.get_float(a + "attention.layer_norm_rms_epsilon", 1e-5);
    h.rope_base = g.get_float(a + "rope.freq_base", 10000.0);
    h.rope_dim = (int)g.get_int(a + "rope.dimension_count", h.head_dim);
    h.n_expert = (int)g.get_int(a + "expert_count", 0);
    h.n_expert_used = (int)g.get_int(a + "expert_used_count", 0);
    h.n_ff_exp = (int)g.get_int(a + "expert_feed_forward_length", h.n_ff);
    if (h.n_layer < 1 || h.n_embd < 1 || h.n_head < 1 || h.n_head_kv < 1 || h.n_layer > 4096 || h.n_embd > (1 << 20) || h.n_head > 4096)
        throw std::runtime_error("the model's block_count, embedding_length and head counts must be positive");
    if (h.n_expert > 0 && (h.n_expert > 256 || h.n_expert_used < 1 || h.n_expert_used > 16 || h.n_expert_used > h.n_expert))
        throw std::runtime_error("unsupported expert configuration (at most 256 experts, 1 to 16 used per token)");
    if (h.head_dim != 32 && h.head_dim != 64 && h.head_dim != 128) throw std::runtime_error("head_dim must be 32, 64 or 128");
    if (h.rope_dim > h.head_dim || h.rope_dim % 2 != 0) throw std::runtime_error("unsupported rotary width");

    const TensorInfo & emb = g.require("token_embd.weight");
    h.n_vocab = (int)emb.ne[1];
    const int E = h.n_embd, QD = h.n_head * h.head_dim, KD = h.n_head_kv * h.head_dim;
    if (emb.ne[0] != E) throw std::runtime_error("token_embd.weight does not match embedding_length");

    upload_weight(emb, E, h.n_vocab, emb.data, emb.nbytes, true, tok_embd_);
    const TensorInfo * head = g.find("output.weight");
    if (!head) head = &emb;   // tied
    upload_weight(*head, E, h.n_vocab, head->data, head->nbytes, false, lm_head_);
    upload_f32(&g.require("output_norm.weight"), out_norm_, (size_t)E);
    upload_f32(g.find("output.bias"), out_bias_, (size_t)h.n_vocab);

    layers_.resize((size_t)h.n_layer);
    for (int l = 0; l < h.n_layer; ++l) {
        LayerWeights & L = layers_[(size_t)l];
        const std::string b = "blk." + std::to_string(l) + ".";
        upload_f32(&g.require(b + "attn_norm.weight"), L.attn_norm, (size_t)E);
        upload_f32(&g.require(b + "ffn_norm.weight"), L.ffn_norm, (size_t)E);
        upload_f32(g.find(b + "attn_q_norm.weight"), L.q_norm, (size_t)h.head_dim);
        upload_f32(g.find(b + "attn_k_norm.weight"), L.k_norm, (size_t)h.head_dim);
        const TensorInfo & wq = g.require(b + "attn_q.weight");
        const TensorInfo & wk = g.require(b + "attn_k.weight");
        const TensorInfo & wv = g.require(b + "attn_v.weight");
        if (wq.ne[0] != E || wq.ne[1] != QD || wk.ne[0] != E || wk.ne[1] != KD || wv.ne[0] != E || wv.ne[1] != KD) throw std::runtime_error("attention weights of layer " + std::to_string(l) + " have unexpected shapes");
        upload_fused({&wq, &wk, &wv}, L.qkv);
        const TensorInfo * bq = g.find(b + "attn_q.bias");
        if (bq) {
            const TensorInfo & bk = g.require(b + "attn_k.bias");
            const TensorInfo & bv = g.require(b + "attn_v.bias");
            if (bq->type != rk::WT_F32 || bk.type != rk::WT_F32 || bv.type != rk::WT_F32) throw std::runtime_error("attention biases must be F32");
            if (bq->nbytes != (size_t)QD * 4 || bk.nbytes != (size_t)KD * 4 || bv.nbytes != (size_t)KD * 4)
                throw std::runtime_error("attention biases of layer " + std::to_string(l) + " have unexpected lengths");
            std::vector<float> joined((size_t)(QD + 2 * KD));
            std::memcpy(joined.data(), bq->data, (size_t)QD * 4);
            std::memcpy(joined.data() + QD, bk.data, (size_t)KD * 4);
            std::memcpy(joined.data() + QD + KD, bv.data, (size_t)KD * 4);
            L.qkv_bias.alloc(joined.size() * 4);
            hip_check(hipMemcpy(L.qkv_bias.ptr, joined.data(), joined.size() * 4, hipMemcpyHostToDevice), "hipMemcpy");
        }
        const TensorInfo & wo = g.require(b + "attn_output.weight");
        upload_weight(wo, QD, E, wo.data, wo.nbytes, false, L.wo);
        if (h.n_expert > 0) {
            const int F = h.n_ff_exp;
            const TensorInfo & wr = g.require(b + "ffn_gate_inp.weight");
            if (wr.type != rk::WT_F32 || wr.ne[0] != E || wr.ne[1] != h.n_expert) throw std::runtime_error("the router of layer " + std::to_string(l) + " must be F32 [n_embd][n_expert]");
            upload_weight(wr, E, h.n_expert, wr.data, wr.nbytes, true, L.router);
            const TensorInfo & eg = g.require(b + "ffn_gate_exps.weight");
            const TensorInfo & eu = g.require(b + "ffn_up_exps.weight");
            const TensorInfo & ed = g.require(b + "ffn_down_exps.weight");
            for (const TensorInfo * t : {&eg, &eu})
                if (t->ne[0] != E || t->ne[1] != F || t->ne[2] != h.n_expert) throw std::runtime_error("expert weights of layer " + std::to_string(l) + " have unexpected shapes");
            if (ed.ne[0] != F || ed.ne[1] != E || ed.ne[2] != h.n_expert) throw std::runtime_error("expert weights of layer " + std::to_string(l) + " have unexpected shapes");
            upload_experts(eg, E, F, L.gate_exps);
            upload_experts(eu, E, F, L.up_exps);
            upload_experts(ed, F, E, L.down_exps);
            continue;
        }
        const TensorInfo & wg = g.require(b + "ffn_gate.weight");
        const TensorInfo & wu = g.require(b + "ffn_up.weight");
        const TensorInfo & wd = g.require(b + "ffn_down.weight");
        if (wg.ne[0] != E || wu.ne[0] != E || wg.ne[1] != wu.ne[1] || wd.ne[0] != wg.ne[1] || wd.ne[1] != E) throw std::runtime_error("feed-forward weights of layer " + std::to_string(l) + " have unexpected shapes");
        h.n_ff = (int)wg.ne[1];
        L.gate_up_interleaved = upload_gate_up_interleaved(wg, wu, L.gate_up);
        if (!L.gate_up_interleaved) upload_fused({&wg, &wu}, L.gate_up);
        upload_weight(wd, h.n_ff, E, wd.data, wd.nbytes, false, L.down);
    }

    // rotary frequencies in double: angle = pos * base^(-2i/d), divided by the model's per-frequency factors
    // (rope_freqs.weight, the long-context rule of Llama 3.1 and later: ggml's rope divides theta by them) and
    // multiplied by 1 / factor under linear scaling. Under yarn scaling (ggml's rope_yarn) the frequencies below the
    // correction range are interpolated (1 / factor), those above it kept, those inside mixed along a linear ramp
    // over the pair index, and cosines and sines are multiplied by attn_factor (1 + 0.1 ln factor). Another rule
    // (longrope) is not implemented: a model that declares one is refused rather than rotated wrongly.
    std::vector<double> inv((size_t)(h.rope_dim / 2));
    for (size_t i = 0; i < inv.size(); ++i) inv[i] = std::pow(h.rope_base, -2.0 * (double)i / h.rope_dim);
    double magnitude = 1.0;
    {
        const std::string scaling = g.get_string(a + "rope.scaling.type", "none");
        const TensorInfo * rf = g.find("rope_freqs.weight");
        if (rf) {
            if (rf->type != rk::WT_F32 || rf->ne[0] != (int64_t)inv.size() || rf->nbytes != inv.size() * sizeof(float))
                throw std::runtime_error("rope_freqs.weight must hold rope_dim / 2 f32 factors");
            const float * ff = (const float *)rf->data;
            for (size_t i = 0; i < inv.size(); ++i) {
                if (!(ff[i] > 0.0f)) throw std::runtime_error("rope_freqs.weight holds a factor that is not positive");
                inv[i] /= (double)ff[i];
            }
        }
        if (scaling == "linear" || scaling == "yarn") {
            const double factor = g.get_float(a + "rope.scaling.factor", 1.0);
            if (!(factor > 0.0)) throw std::runtime_error("rope.scaling.factor must be positive");
            if (scaling == "linear") {
                for (double & f : inv) f /= factor;
            } else {
                const double n_orig = (double)g.get_int(a + "rope.scaling.original_context_length", 0);
                if (!(n_orig > 0.0)) throw std::runtime_error("yarn scaling needs rope.scaling.original_context_length");
                const double beta_fast = g.get_float(a + "rope.scaling.yarn_beta_fast", 32.0);
                const double beta_slow = g.get_float(a + "rope.scaling.yarn_beta_slow", 1.0);
                const double n_dims = (double)h.rope_dim;
                auto corr = [&](double n_rot) { return n_dims * std::log(n_orig / (n_rot * 2.0 * M_PI)) / (2.0 * std::log(h.rope_base)); };
                const double low = std::max(0.0, std::floor(corr(beta_fast)));
                const double high = std::min(n_dims - 1.0, std::ceil(corr(beta_slow)));
                for (size_t i = 0; i < inv.size(); ++i) {
                    const double y = ((double)i - low) / std::max(0.001, high - low);
                    const double keep = 1.0 - std::min(1.0, std::max(0.0, y));      // 1: the frequency as it is, 0: interpolated
                    inv[i] *= (1.0 - keep) / factor + keep;
                }
                magnitude = g.get_float(a + "rope.scaling.attn_factor", 1.0) * (1.0 + 0.1 * std::log(factor));
            }
        } else if (scaling != "none" && !scaling.empty()) {
            throw std::runtime_error("rope scaling type '" + scaling + "' is not implemented");
        }
    }
    inv.push_back(magnitude);
    inv_freq_.alloc(inv.size() * sizeof(double));
    hip_check(hipMemcpy(inv_freq_.ptr, inv.data(), inv.size() * sizeof(double), hipMemcpyHostToDevice), "hipMemcpy");

    // vocabulary
    if (const MetaValue * toks = g.meta("tokenizer.ggml.tokens")) vocab_.pieces = toks->sa;
    if (const MetaValue * types = g.meta("tokenizer.ggml.token_type")) {
        vocab_.types.assign(types->ia.begin(), types->ia.end());
    }
    vocab_.eos = (int32_t)g.get_int("tokenizer.ggml.eos_token_id", -1);
    vocab_.eot = (int32_t)g.get_int("tokenizer.ggml.eot_token_id", -1);
    {
        Tokenizer & tk = vocab_.tokenizer;
        tk.model = g.get_string("tokenizer.ggml.model");
        tk.pieces = vocab_.pieces;
        tk.types = vocab_.types;
        if (const MetaValue * sc = g.meta("tokenizer.ggml.scores")) tk.scores.assign(sc->fa.begin(), sc->fa.end());
        tk.bos = (int32_t)g.get_int("tokenizer.ggml.bos_token_id", -1);
        tk.eos = vocab_.eos;
        tk.unk = (int32_t)g.get_int("tokenizer.ggml.unknown_token_id", -1);
        tk.pre = g.get_string("tokenizer.ggml.pre");
        if (const MetaValue * mg = g.meta("tokenizer.ggml.merges")) tk.merges = mg->sa;
        tk.set_kind_defaults();
        tk.add_bos = g.get_int("tokenizer.ggml.add_bos_token", tk.add_bos) != 0;
        tk.add_eos = g.get_int("tokenizer.ggml.add_eos_token", tk.add_eos) != 0;
        tk.add_space_prefix = g.get_int("tokenizer.ggml.add_space_prefix", tk.add_space_prefix) != 0;
        try {
            tk.prepare();
        } catch (const std::exception & e) {
            vocab_.tokenizer_error = e.what();      // the model still decodes token ids
        }
    }

    // FNV-1a over the path bytes then the u64 weight size
    // (reference retro_runtime.hpp:856-868).
    uint64_t hash = UINT64_C(14695981039346656037);
    auto mix = [&hash](const void * data, size_t n) {
        const unsigned char * p = (const unsigned char *)data;
        for (size_t i = 0; i < n; ++i) { hash ^= p[i]; hash *= UINT64_C(1099511628211); }
    };
    mix(path.data(), path.size());
    const uint64_t size = g.tensor_bytes();
    mix(&size, sizeof(size));
    fingerprint_ = hash;
}

void Engine::build_buffers() {
    const int B = (int)cfg_.n_batch;
    const int E = hp_.n_embd, QD = hp_.n_head * hp_.head_dim, KD = hp_.n_head_kv * hp_.head_dim, F = hp_.n_ff;
    auto i32 = [&](size_t n) {
        pk_store_.emplace_back();
        pk_store_.back().alloc(n * 4);
        return pk_store_.back().as<int32_t>();
    };
    pk_.tok = i32((size_t)B); pk_.pos = i32((size_t)B); pk_.seq = i32((size_t)B); pk_.row = i32((size_t)B);
    pk_.cell = i32((size_t)B); pk_.out_index = i32((size_t)B); pk_.out_tok = i32((size_t)B);
    pk_.last_index = i32((size_t)B); pk_.row_offset = i32((size_t)B + 1); pk_.counts = i32(4);
    pk_.tile_t0 = i32((size_t)B); pk_.tile_nq = i32((size_t)B); pk_.tile_item0 = i32((size_t)B);
    pk_.tile_nsplit = i32((size_t)B); pk_.tile_page0 = i32((size_t)B); pk_.tile_kv_begin = i32((size_t)B);
    pk_.tok_tile = i32((size_t)B);
    pk_.dec_order = i32((size_t)B);
    pk_.dec_desc = (int4 *)i32((size_t)B * 4);
    pk_.dec_pid = i32((size_t)B * 8);
    pk_.tok_merge = (int4 *)i32((size_t)B * 4);
    pk_.rope_cos = (float *)i32((size_t)B * (hp_.rope_dim / 2));
    pk_.rope_sin = (float *)i32((size_t)B * (hp_.rope_dim / 2));

    x_.alloc((size_t)B * E * 4);
    qkv_.alloc((size_t)B * (QD + 2 * KD) * 4);
    gu_.alloc((size_t)B * 2 * std::max(F, 1) * 4);
    if (hp_.n_expert > 0) {
        const int NE = hp_.n_expert, KU = hp_.n_expert_used, FE = hp_.n_ff_exp;
        const size_t slots = rk::moe_slots(B, KU, NE);
        moe_logits_.alloc((size_t)B * NE * 4);
        moe_sel_.alloc((size_t)B * KU * 4);
        moe_wgt_.alloc((size_t)B * KU * 4);
        moe_n_.alloc((size_t)NE * 4);
        moe_off_.alloc((size_t)(NE + 1) * 4);
        moe_tok_.alloc(slots * 4);
        moe_pair_.alloc(slots * 4);
        moe_q_.alloc((size_t)B * KU * 4);
        moe_h_.alloc(rk::act_halves((int)slots, FE) * 2);
        hip_check(hipMemsetAsync(moe_h_.ptr, 0, moe_h_.bytes, stream_), "hipMemsetAsync");
        moe_out_.alloc(slots * (size_t)E * 4);
        if (moe_scaled_ && !ggml_activations_ && rk::mxe_moe_can(E, FE)) {
            // the block-scaled expert path serves steps of at most 12 pairs per expert on average
            const int t_small = std::min(B, 12 * NE / KU);
            moe_mx_slots_ = rk::moe_slots(t_small, KU, NE);
            const int wide = std::max(E, FE);
            moe_mx_ops_.alloc(rk::mxe_moe_operand_bytes(wide, moe_mx_slots_));
            moe_mx_scales_.alloc(rk::mxe_moe_scale_bytes(wide, moe_mx_slots_));
            moe_mx_h_.alloc(moe_mx_slots_ * (size_t)FE * 4);
        }
    }
    q_half_.alloc((size_t)B * QD * 2);
    // operand-order activations; the sums keep zero padding lanes, so they are cleared once
    auto act = [&](DevBuf & x, DevBuf & sums, int K) {
        x.alloc(rk::act_halves(B, K) * 2);
        sums.alloc(rk::act_sum_halves(B, K) * 2);
        hip_check(hipMemsetAsync(x.ptr, 0, x.bytes, stream_), "hipMemsetAsync");
        hip_check(hipMemsetAsync(sums.ptr, 0, sums.bytes, stream_), "hipMemsetAsync");
    };
    act(act_e_x_, act_e_sums_, E);
    act(act_q_x_, act_q_sums_, QD);
    act(act_f_x_, act_f_sums_, F);
    act(act_o_x_, act_o_sums_, E);
    if (ggml_activations_) {
        act(act_e_qx_, act_e_qsums_, E);
        act(act_q_qx_, act_q_qsums_, QD);
        act(act_f_qx_, act_f_qsums_, F);
        act(act_o_qx_, act_o_qsums_, E);
        auto codes = [&](ActCodes & c, int K) {
            if (K % 256 != 0) return;          // no Q8_K conversion of such rows
            c.codes.alloc((size_t)rk::GEMV_MAX_T * K);
            c.d.alloc((size_t)rk::GEMV_MAX_T * (K / 32) * 4);          // one scale per 32 (Q8_0) or per 256 (Q8_K)
            c.bsums.alloc((size_t)rk::GEMV_MAX_T * (K / 16) * 2);
        };
        codes(act_e_codes_, E);
        codes(act_q_codes_, QD);
        codes(act_f_codes_, F);
        codes(act_o_codes_, E);
    }
    q_half_lo_.alloc((size_t)B * QD * 2);
    mm_ws_.alloc(rk::matmul_workspace_bytes());
    hip_check(hipMemsetAsync(mm_ws_.ptr, 0, mm_ws_.bytes, stream_), "hipMemsetAsync");
    sample_k_.alloc((size_t)B * 4);
    sample_out_.alloc((size_t)B * sizeof(rk::SampleOut));
    sample_scratch_.alloc(rk::sample_scratch_bytes(B));
    const size_t stage = (size_t)B * (sizeof(rk::RowDesc) + 4) + 65536;
    d_stage_.alloc(stage);
    h_stage_.ensure(stage);
    h_sample_.ensure((size_t)B * sizeof(rk::SampleOut));
}

// ---- pages ---------------------------------------------------------------------------

int32_t Engine::alloc_page() {
    if (free_pages_.empty()) return -1;
    const int32_t p = free_pages_.top();
    free_pages_.pop();
    page_ref_[(size_t)p] = 1;
    return p;
}

void Engine::release_page(int32_t page) {
    if (page < 0) return;
    if (--page_ref_[(size_t)page] == 0) free_pages_.push(page);
}

void Engine::copy_page(int32_t src, int32_t dst) {
    for (int l = 0; l < hp_.n_layer; ++l) {
        rk::kv_copy_page(stream_, k_pool_[(size_t)l].as<__half>(), v_pool_[(size_t)l].as<__half>(), kv_strides_,
                         hp_.n_head_kv, hp_.head_dim, src, dst, kv_q8_);
    }
}

void Engine::set_page(int32_t slot, int idx, int32_t page) {
    slots_[(size_t)slot].pages[(size_t)idx] = page;
    pending_updates_[(int64_t)slot * max_pages_ + idx] = page;
}

void Engine::clear_slot(Slot & s, int32_t slot) {
    if (s.end > s.begin) {
        for (int idx = s.begin / rk::PAGE; idx <= (s.end - 1) / rk::PAGE; ++idx) {
            release_page(s.pages[(size_t)idx]);
            set_page(slot, idx, -1);
        }
    }
    s.begin = s.end = 0;
}

bool Engine::seq_rm(int32_t slot, int32_t p0, int32_t p1) {
    if (slot < 0 || slot >= (int32_t)cfg_.n_seq_max) {
        set_error("slot is outside the context's sequence range");
        return false;
    }
    Slot & s = slots_[(size_t)slot];
    if (p0 < 0) p0 = 0;
    if (p1 < 0) p1 = INT_MAX;
    if (s.end <= s.begin || p0 >= s.end || p1 <= s.begin || p0 >= p1) return true;
    if (p0 <= s.begin && p1 >= s.end) {
        clear_slot(s, slot);
        return true;
    }
    if (p1 >= s.end) {                       // drop a suffix: keep [begin, p0)
        const int keep_last = (p0 - 1) / rk::PAGE;
        for (int idx = keep_last + 1; idx <= (s.end - 1) / rk::PAGE; ++idx) {
            release_page(s.pages[(size_t)idx]);
            set_page(slot, idx, -1);
        }
        s.end = p0;
        return true;
    }
    if (p0 <= s.begin) {                     // drop a prefix: keep [p1, end)
        const int keep_first = p1 / rk::PAGE;
        for (int idx = s.begin / rk::PAGE; idx < keep_first; ++idx) {
            release_page(s.pages[(size_t)idx]);
            set_page(slot, idx, -1);
        }
        s.begin = p1;
        return true;
    }
    set_error("the memory cannot remove that partial range; remove the whole sequence instead");
    return false;
}

bool Engine::seq_cp(int32_t src, int32_t dst, int32_t p0, int32_t p1) {
    const int32_t n = (int32_t)cfg_.n_seq_max;
    if (src < 0 || src >= n || dst < 0 || dst >= n) {
        set_error("seq_cp slots are outside the context's sequence range");
        return false;
    }
    if (src == dst) return true;
    const Slot & a = slots_[(size_t)src];
    Slot & b = slots_[(size_t)dst];
    const bool whole = p0 <= 0 && p1 < 0;
    if (p0 < 0) p0 = 0;
    if (p1 < 0) p1 = INT_MAX;
    const int lo = std::max(p0, a.begin), hi = std::min(p1, a.end);
    if (a.end <= a.begin || hi <= lo) return true;
    if (!cfg_.kv_unified && !(whole || (lo == a.begin && hi == a.end))) {
        set_error("a partitioned KV pool only supports whole-sequence copies");
        return false;
    }
    if (b.end > b.begin) {
        if (lo < b.end && b.begin < hi) {
            set_error("seq_cp: the copied range of the destination is not empty");
            return false;
        }
        if (lo != b.end && hi != b.begin) {
            set_error("seq_cp: the copied range is not adjacent to the destination's resident range");
            return false;
        }
    }
    // Pages are shared by reference; a page either side later writes into is
    // copied first (see the step), so a partially used last page costs nothing here.
    for (int idx = lo / rk::PAGE; idx <= (hi - 1) / rk::PAGE; ++idx) {
        const int32_t sp = a.pages[(size_t)idx];
        const int32_t dp = b.pages[(size_t)idx];
        if (dp < 0) {
            ++page_ref_[(size_t)sp];
            set_page(dst, idx, sp);
        } else if (dp != sp) {
            // The destination already owns part of this page index (adjacent
            // ranges meeting inside one page): merge position by position.
            int32_t target = dp;
            if (page_ref_[(size_t)dp] > 1) {
                target = alloc_page();
                if (target < 0) {
                    set_error("the KV pool is full");
                    return false;
                }
                copy_page(dp, target);
                release_page(dp);
                set_page(dst, idx, target);
            }
            const int first = std::max(lo, idx * rk::PAGE), last = std::min(hi, (idx + 1) * rk::PAGE);
            std::vector<int32_t> cells_src, cells_dst;
            for (int p = first; p < last; ++p) {
                cells_src.push_back(sp * rk::PAGE + p % rk::PAGE);
                cells_dst.push_back(target * rk::PAGE + p % rk::PAGE);
            }
            const size_t kd = rk::kv_row_halves(hp_.n_head_kv, hp_.head_dim, kv_q8_);      // halves of a cell's row
            DevBuf cs, cd, tmp;
            cs.alloc(cells_src.size() * 4);
            cd.alloc(cells_dst.size() * 4);
            tmp.alloc(cells_src.size() * kd * 2);
            hip_check(hipMemcpyAsync(cs.ptr, cells_src.data(), cs.bytes, hipMemcpyHostToDevice, stream_), "hipMemcpyAsync");
            hip_check(hipMemcpyAsync(cd.ptr, cells_dst.data(), cd.bytes, hipMemcpyHostToDevice, stream_), "hipMemcpyAsync");
            for (int l = 0; l < hp_.n_layer; ++l) {
                for (int v = 0; v < 2; ++v) {
                    __half * pool = v ? v_pool_[(size_t)l].as<__half>() : k_pool_[(size_t)l].as<__half>();
                    rk::kv_gather(stream_, pool, kv_strides_, hp_.n_head_kv, hp_.head_dim, v != 0, cs.as<int32_t>(), (int)cells_src.size(), tmp.as<__half>(), kv_q8_);
                    rk::kv_scatter(stream_, pool, kv_strides_, hp_.n_head_kv, hp_.head_dim, v != 0, cd.as<int32_t>(), (int)cells_dst.size(), tmp.as<__half>(), kv_q8_);
                }
            }
            hip_check(hipStreamSynchronize(stream_), "seq_cp merge");
        }
    }
    if (b.end <= b.begin) { b.begin = lo; b.end = hi; }
    else { b.begin = std::min(b.begin, lo); b.end = std::max(b.end, hi); }
    return true;
}

int Engine::seq_pos(int32_t slot, int32_t * out_min, int32_t * out_max) {
    if (!out_min || !out_max) {
        set_error("the position outputs are required");
        return -1;
    }
    if (slot < 0 || slot >= (int32_t)cfg_.n_seq_max) {
        set_error("slot is outside the context's sequence range");
        return -1;
    }
    const Slot & s = slots_[(size_t)slot];
    if (s.end <= s.begin) { *out_min = -1; *out_max = -1; }
    else { *out_min = s.begin; *out_max = s.end - 1; }
    return 0;
}

int Engine::memory(retro_engine_memory_info * out) {
    if (!out) {
        set_error("out is required");
        return -1;
    }
    out->struct_size = sizeof(retro_engine_memory_info);
    out->n_slots = cfg_.n_seq_max;
    out->cells_total = cfg_.n_ctx;
    uint64_t used = 0;
    for (const Slot & s : slots_) if (s.end > s.begin) used += (uint64_t)(s.end - s.begin);
    out->cells_used = used;
    uint64_t kv = 0;
    for (const auto & b : k_pool_) kv += b.bytes;
    for (const auto & b : v_pool_) kv += b.bytes;
    out->kv_bytes = kv;
    out->recurrent_bytes = 0;
    return 0;
}

// ---- snapshots -------------------------------------------------------------------------
//
// Byte format (this library's own; only seq_load of the same build reads it):
//   u32 magic "RKV1" (an f16 cache), "RKV8" (Q8_0) or "RKV4" (Q4_0), u32 flags, i32 n_layer, i32 halves per row,
//   i32 begin, i32 end, then per layer the K rows [end-begin] and the V rows: kv_dim f16 values in
//   natural order, or per kv head the codes (Q8_0: head_dim bytes, code + 128; Q4_0: head_dim / 2 bytes, element
//   2 k in the low nibble of byte k) and head_dim / 32 f16 scales.
namespace {
struct SnapHeader { uint32_t magic, flags; int32_t n_layer, kv_dim, begin, end; };
constexpr uint32_t kSnapMagic = 0x31564b52u;
constexpr uint32_t kSnapMagicQ8 = 0x38564b52u;
constexpr uint32_t kSnapMagicQ4 = 0x34564b52u;        // "RKV4"
}

uint32_t Engine::snap_magic() const { return kv_q8_ == rk::KV_Q8 ? kSnapMagicQ8 : kv_q8_ == rk::KV_Q4 ? kSnapMagicQ4 : kSnapMagic; }

int Engine::seq_save(int32_t slot, uint32_t flags, uint8_t * buffer, size_t n_buffer, size_t * out_n_bytes) {
    if (!out_n_bytes) {
        set_error("out_n_bytes is required");
        return -1;
    }
    if (flags & ~RETRO_STATE_SEQ_FLAGS_PARTIAL_ONLY) {
        set_error("only host snapshots (flags 0 or PARTIAL_ONLY) are supported");
        return -1;
    }
    if (slot < 0 || slot >= (int32_t)cfg_.n_seq_max) {
        set_error("slot is outside the context's sequence range");
        return -1;
    }
    const Slot & s = slots_[(size_t)slot];
    const size_t kd = rk::kv_row_halves(hp_.n_head_kv, hp_.head_dim, kv_q8_);
    const bool partial_only = (flags & RETRO_STATE_SEQ_FLAGS_PARTIAL_ONLY) != 0;
    const int n_pos = partial_only ? 0 : std::max(0, s.end - s.begin);   // no recurrent or SWA state exists
    const size_t required = sizeof(SnapHeader) + (size_t)hp_.n_layer * 2 * (size_t)n_pos * kd * 2;
    *out_n_bytes = required;
    if (!buffer) return 0;
    if (n_buffer < required) {
        set_error("the save buffer is too small for this sequence's state");
        return -2;
    }
    SnapHeader h{snap_magic(), flags, hp_.n_layer, (int32_t)kd, partial_only ? 0 : s.begin, partial_only ? 0 : s.begin + n_pos};
    std::memcpy(buffer, &h, sizeof(h));
    if (n_pos > 0) {
        std::vector<int32_t> cells((size_t)n_pos);
        for (int p = s.begin; p < s.end; ++p) cells[(size_t)(p - s.begin)] = s.pages[(size_t)(p / rk::PAGE)] * rk::PAGE + p % rk::PAGE;
        DevBuf dc, tmp;
        dc.alloc(cells.size() * 4);
        tmp.alloc((size_t)n_pos * kd * 2);
        hip_check(hipMemcpyAsync(dc.ptr, cells.data(), dc.bytes, hipMemcpyHostToDevice, stream_), "hipMemcpyAsync");
        uint8_t * at = buffer + sizeof(h);
        for (int l = 0; l < hp_.n_layer; ++l) {
            for (int v = 0; v < 2; ++v) {
                const __half * pool = v ? v_pool_[(size_t)l].as<__half>() : k_pool_[(size_t)l].as<__half>();
                rk::kv_gather(stream_, pool, kv_strides_, hp_.n_head_kv, hp_.head_dim, v != 0, dc.as<int32_t>(), n_pos, tmp.as<__half>(), kv_q8_);
                hip_check(hipMemcpyAsync(at, tmp.ptr, tmp.bytes, hipMemcpyDeviceToHost, stream_), "hipMemcpyAsync");
                hip_check(hipStreamSynchronize(stream_), "seq_save");
                at += tmp.bytes;
            }
        }
    }
    return 0;
}

int Engine::seq_load(int32_t slot, uint32_t flags, const uint8_t * buffer, size_t n_bytes, size_t * out_n_read) {
    if (!out_n_read) {
        set_error("out_n_read is required");
        return -1;
    }
    if (flags & ~RETRO_STATE_SEQ_FLAGS_PARTIAL_ONLY) {
        set_error("only host snapshots (flags 0 or PARTIAL_ONLY) are supported");
        return -1;
    }
    if (slot < 0 || slot >= (int32_t)cfg_.n_seq_max) {
        set_error("slot is outside the context's sequence range");
        return -1;
    }
    if (!buffer || n_bytes == 0) {
        set_error("a snapshot buffer is required");
        return -1;
    }
    const char * refused = "the snapshot was refused (wrong size, flags or corrupted data)";
    SnapHeader h;
    if (n_bytes < sizeof(h)) { set_error(refused); return -1; }
    std::memcpy(&h, buffer, sizeof(h));
    const size_t kd = rk::kv_row_halves(hp_.n_head_kv, hp_.head_dim, kv_q8_);
    if (h.magic != snap_magic() || h.flags != flags || h.n_layer != hp_.n_layer || h.kv_dim != (int32_t)kd
            || h.begin < 0 || h.end < h.begin || h.end > n_ctx_seq_) {
        set_error(refused);
        return -1;
    }
    const int n_pos = h.end - h.begin;
    const size_t required = sizeof(h) + (size_t)hp_.n_layer * 2 * (size_t)n_pos * kd * 2;
    if (n_bytes < required) { set_error(refused); return -1; }
    if (flags & RETRO_STATE_SEQ_FLAGS_PARTIAL_ONLY) {
        *out_n_read = required;
        return 0;
    }
    Slot & s = slots_[(size_t)slot];
    clear_slot(s, slot);
    if (n_pos > 0) {
        const int first = h.begin / rk::PAGE, last = (h.end - 1) / rk::PAGE;
        if ((int)free_pages_.size() < last - first + 1) {
            set_error("the KV pool is full");
            return -1;
        }
        for (int idx = first; idx <= last; ++idx) set_page(slot, idx, alloc_page());
        s.begin = h.begin;
        s.end = h.end;
        std::vector<int32_t> cells((size_t)n_pos);
        for (int p = s.begin; p < s.end; ++p) cells[(size_t)(p - s.begin)] = s.pages[(size_t)(p / rk::PAGE)] * rk::PAGE + p % rk::PAGE;
        DevBuf dc, tmp;
        dc.alloc(cells.size() * 4);
        tmp.alloc((size_t)n_pos * kd * 2);
        hip_check(hipMemcpyAsync(dc.ptr, cells.data(), dc.bytes, hipMemcpyHostToDevice, stream_), "hipMemcpyAsync");
        const uint8_t * at = buffer + sizeof(h);
        for (int l = 0; l < hp_.n_layer; ++l) {
            for (int v = 0; v < 2; ++v) {
                __half * pool = v ? v_pool_[(size_t)l].as<__half>() : k_pool_[(size_t)l].as<__half>();
                hip_check(hipMemcpyAsync(tmp.ptr, at, tmp.bytes, hipMemcpyHostToDevice, stream_), "hipMemcpyAsync");
                rk::kv_scatter(stream_, pool, kv_strides_, hp_.n_head_kv, hp_.head_dim, v != 0, dc.as<int32_t>(), n_pos, tmp.as<__half>(), kv_q8_);
                hip_check(hipStreamSynchronize(stream_), "seq_load");
                at += tmp.bytes;
            }
        }
    }
    *out_n_read = required;
    return 0;
}

// ---- the step -------------------------------------------------------------------------

namespace {

bool valid_sampling_v1(const retro_sampling_params & s) {
    if (!(s.temperature > 0.0f) || !std::isfinite(s.temperature)) {
        set_error("sampling temperature must be finite and greater than zero");
        return false;
    }
    if (!(s.top_p > 0.0f && s.top_p <= 1.0f)) {
        set_error("sampling top_p must be in (0, 1]");
        return false;
    }
    if (s.max_new_tokens == 0) {
        set_error("sampling max_new_tokens must be greater than zero");
        return false;
    }
    return true;
}

bool valid_tokens(const int32_t * tokens, size_t n, int32_t n_vocab) {
    for (size_t i = 0; i < n; ++i) {
        if (tokens[i] < 0 || tokens[i] >= n_vocab) {
            std::ostringstream m;
            m << "token " << tokens[i] << " at index " << i << " is outside the vocabulary of size " << n_vocab;
            set_error(m.str());
            return false;
        }
    }
    return true;
}

}  // namespace

// Same checks, order and messages as the reference (retro_gen_core.cpp:1539-1589). Also read by the v2 generator.
bool valid_sampling_v2(const retro_sampling_params_v2 & s, int32_t n_vocab) {
    if (s.struct_size < sizeof(retro_sampling_params_v2)) {
        set_error("retro_sampling_params_v2.struct_size is too small for this build");
        return false;
    }
    if (!(s.temperature > 0.0f) || !std::isfinite(s.temperature)) {
        set_error("sampling temperature must be finite and greater than zero");
        return false;
    }
    if (!(s.top_p > 0.0f && s.top_p <= 1.0f)) {
        set_error("sampling top_p must be in (0, 1]");
        return false;
    }
    if (!(s.repeat_penalty > 0.0f) || !std::isfinite(s.repeat_penalty)) {
        set_error("sampling repeat_penalty must be finite and greater than zero");
        return false;
    }
    if (!(s.min_p >= 0.0f && s.min_p <= 1.0f) || !std::isfinite(s.min_p)) {
        set_error("sampling min_p must be in [0, 1]");
        return false;
    }
    if (!std::isfinite(s.frequency_penalty)) {
        set_error("sampling frequency_penalty must be finite");
        return false;
    }
    if (!std::isfinite(s.presence_penalty)) {
        set_error("sampling presence_penalty must be finite");
        return false;
    }
    if (s.n_logit_bias > 4096) {
        set_error("sampling n_logit_bias must not exceed 4096");
        return false;
    }
    if (s.n_logit_bias > 0) {
        if (!s.logit_bias_ids || !s.logit_bias_values) {
            set_error("logit_bias ids and values are required when n_logit_bias is nonzero");
            return false;
        }
        if (!valid_tokens(s.logit_bias_ids, s.n_logit_bias, n_vocab)) return false;
        for (uint32_t i = 0; i < s.n_logit_bias; ++i) {
            if (!std::isfinite(s.logit_bias_values[i])) {
                set_error("logit_bias values must be finite");
                return false;
            }
        }
    }
    return true;
}


int Engine::step(const retro_step_row_v2 * rows2, const retro_step_row * rows1, size_t n_rows,
                 retro_step_out_row_v2 * out2, retro_step_out_row * out1,
                 int32_t * out_top_ids, float * out_top_logprobs, size_t n_top_stride) {
    const bool is_v2 = rows2 != nullptr;
    if ((!rows2 && !rows1) || n_rows == 0 || (!out2 && !out1)) {
        set_error("step rows and output rows are required");
        return -3;
    }
    const int32_t n_seq_max = (int32_t)cfg_.n_seq_max;
    const int32_t n_batch = (int32_t)cfg_.n_batch;
    const int64_t n_ctx_seq = n_ctx_seq_;
    const int32_t n_vocab = hp_.n_vocab;

    // ---- validation: caller errors are reported before anything decodes
    // (order and messages follow retro_gen_core.cpp:2353-2516).
    std::vector<RowView> rows(n_rows);
    std::vector<std::shared_ptr<Grammar>> compiled(n_rows);
    if (is_v2) {
        for (size_t r = 0; r < n_rows; ++r) {
            const retro_step_row_v2 & in = rows2[r];
            if (in.struct_size < offsetof(retro_step_row_v2, adapter) + sizeof(int32_t)) {
                set_error("retro_step_row_v2.struct_size is too small for this build");
                return -3;
            }
            if (in.sampling.struct_size < sizeof(retro_sampling_params_v2)) {
                set_error("retro_sampling_params_v2.struct_size is too small for this build");
                return -3;
            }
            RowView & v = rows[r];
            v.request = in.request; v.slot = in.slot; v.tokens = in.tokens; v.n = in.n; v.pos0 = in.pos0;
            v.sample = in.sample; v.v2 = &in.sampling; v.v1 = retro_sampling_params{};
            v.n_top = in.n_top_logprobs; v.want_logprob = in.want_logprob != 0; v.adapter = in.adapter;
        }
    } else {
        for (size_t r = 0; r < n_rows; ++r) {
            const retro_step_row & in = rows1[r];
            // Read the evolution key before any other field.
            if (in.struct_size < offsetof(retro_step_row, adapter) + sizeof(int32_t)) {
                set_error("retro_step_row.struct_size is too small for this build");
                return -3;
            }
            RowView & v = rows[r];
            v.request = in.request; v.slot = in.slot; v.tokens = in.tokens; v.n = in.n; v.pos0 = in.pos0;
            v.sample = in.sample; v.v2 = nullptr; v.v1 = in.sampling;
            v.n_top = in.n_top_logprobs; v.want_logprob = false; v.adapter = in.adapter;
        }
    }
    if (n_rows > (size_t)n_batch || (n_top_stride != 0 && n_rows > SIZE_MAX / n_top_stride)) {
        set_error("the step row count or output shape exceeds capacity");
        return -3;
    }
    std::vector<int32_t> seen_requests;
    size_t total = 0;
    for (size_t r = 0; r < n_rows; ++r) {
        const RowView & row = rows[r];
        if (!row.tokens || row.n == 0) {
            set_error("a step row requires at least one token");
            return -3;
        }
        if (row.slot < 0 || row.slot >= n_seq_max) {
            set_error("step row slot is outside the context's sequence range");
            return -3;
        }
        if (row.adapter != 0 && row.adapter != RETRO_STEP_ADAPTER_BASE
                && (row.adapter == kPolicyAdapter || !row_adapters_.count(row.adapter))) {
            set_error("step row adapter " + std::to_string(row.adapter) + " is not a loaded per-row adapter");
            return -3;
        }
        if (row.pos0 < 0 || (int64_t)row.pos0 + row.n > n_ctx_seq) {
            set_error("step row positions exceed the per-sequence context");
            return -3;
        }
        for (size_t prev = 0; prev < r; ++prev) {
            const RowView & other = rows[prev];
            if (row.slot == other.slot && row.pos0 < (int64_t)other.pos0 + other.n
                    && other.pos0 < (int64_t)row.pos0 + row.n) {
                set_error("step rows overlap in the same sequence slot");
                return -3;
            }
            if (row.slot == other.slot && row.adapter != other.adapter) {
                set_error("step rows of one sequence slot select different adapters");
                return -3;
            }
        }
        if (!valid_tokens(row.tokens, row.n, n_vocab)) return -3;
        if (row.n > (uint32_t)n_batch || total + row.n > (size_t)n_batch) {
            set_error("the step's tokens exceed the context's physical batch (n_batch)");
            return -3;
        }
        total += row.n;
        if (row.n_top > 0 && (!out_top_ids || !out_top_logprobs)) {
            set_error("top logprobs requested but the output buffers are missing");
            return -3;
        }
        if (row.n_top > n_top_stride) {
            set_error("a step row's n_top_logprobs exceeds the output stride");
            return -3;
        }
        if (row.sample) {
            if (row.request < 0) {
                set_error("a sampling step row requires a request id");
                return -3;
            }
            if (row.v2) {
                if (!valid_sampling_v2(*row.v2, n_vocab)) return -3;
                if (row.v2->grammar) {
                    // compiled before anything decodes: an invalid grammar must not leave a prompt in the KV
                    const std::string & gbnf = row.v2->grammar->gbnf;
                    auto prev = requests_.find(row.request);
                    if (prev == requests_.end() || !prev->second.grammar || prev->second.grammar->gbnf() != gbnf) {
                        try {
                            compiled[r] = std::make_shared<Grammar>(gbnf);
                        } catch (const std::exception & e) {
                            set_error(std::string("failed to compile the request's grammar (invalid GBNF): ") + e.what());
                            return -3;
                        }
                    }
                }
            } else {
                retro_sampling_params s = row.v1;
                s.max_new_tokens = 1;   // the caller owns stopping
                if (!valid_sampling_v1(s)) return -3;
            }
        }
        if (row.request >= 0) {
            if (std::find(seen_requests.begin(), seen_requests.end(), row.request) != seen_requests.end()) {
                set_error("a request id appears twice in one step");
                return -3;
            }
            seen_requests.push_back(row.request);
        }
    }

    // ---- KV placement: positions must extend each slot's resident range.
    // Nothing is mutated until the whole plan is known to fit.
    {
        std::vector<std::pair<int, int>> span(slots_.size());
        for (size_t i = 0; i < slots_.size(); ++i) span[i] = {slots_[i].begin, slots_[i].end};
        std::vector<std::pair<int32_t, int>> touched;   // (slot, page index) already paid for
        size_t need = 0;
        for (const RowView & row : rows) {
            auto & sp = span[(size_t)row.slot];
            if (sp.second > sp.first && row.pos0 != sp.second) {
                set_error(row.pos0 < sp.second
                    ? "step row positions are already resident in the slot: remove them with seq_rm first"
                    : "step row positions leave a gap after the slot's resident range");
                return -1;
            }
            if (sp.second <= sp.first) sp.first = row.pos0;
            const int last = row.pos0 + (int)row.n;
            const Slot & s = slots_[(size_t)row.slot];
            for (int idx = row.pos0 / rk::PAGE; idx <= (last - 1) / rk::PAGE; ++idx) {
                const std::pair<int32_t, int> key{row.slot, idx};
                if (std::find(touched.begin(), touched.end(), key) != touched.end()) continue;
                const int32_t pg = s.pages[(size_t)idx];
                if (pg < 0 || page_ref_[(size_t)pg] > 1) {   // a fresh page, or a private copy of a shared one
                    ++need;
                    touched.push_back(key);
                }
            }
            sp.second = last;
        }
        if (need > free_pages_.size()) {
            set_error("the KV pool is full: the step needs " + std::to_string(need) + " pages, "
                      + std::to_string(free_pages_.size()) + " are free");
            return -1;
        }
    }
    for (const RowView & row : rows) {
        Slot & s = slots_[(size_t)row.slot];
        if (s.end <= s.begin) { s.begin = row.pos0; s.end = row.pos0; }
        const int last = row.pos0 + (int)row.n;
        for (int idx = row.pos0 / rk::PAGE; idx <= (last - 1) / rk::PAGE; ++idx) {
            const int32_t pg = s.pages[(size_t)idx];
            if (pg < 0) {
                set_page(row.slot, idx, alloc_page());
            } else if (page_ref_[(size_t)pg] > 1) {
                const int32_t fresh = alloc_page();
                copy_page(pg, fresh);
                release_page(pg);
                set_page(row.slot, idx, fresh);
            }
        }
        s.end = last;
    }

    // Every resident position of a slot the step reads must have a page: a
    // missing one would send a kernel outside the pool.
    for (const RowView & row : rows) {
        const Slot & s = slots_[(size_t)row.slot];
        for (int idx = s.begin / rk::PAGE; idx <= (s.end - 1) / rk::PAGE; ++idx) {
            const int32_t pg = s.pages[(size_t)idx];
            if (pg < 0 || pg >= n_pages_) throw std::runtime_error("internal error: a resident position has no KV page");
        }
    }

    // ---- upload the plan and pack it on the device
    const int T = (int)total;
    const size_t n_upd = pending_updates_.size();
    const size_t off_tok = n_rows * sizeof(rk::RowDesc);
    const size_t off_upd = off_tok + (size_t)T * 4;
    const size_t stage_bytes = off_upd + n_upd * sizeof(rk::TableUpdate);
    h_stage_.ensure(stage_bytes);
    d_stage_.ensure(stage_bytes);
    rk::RowDesc * hd = h_stage_.as<rk::RowDesc>();
    int32_t * ht = (int32_t *)((uint8_t *)h_stage_.ptr + off_tok);
    int n_out = 0;
    bool routed = false;
    step_max_resident_ = 0;
    {
        int at = 0;
        for (size_t r = 0; r < n_rows; ++r) {
            const RowView & row = rows[r];
            hd[r].slot = row.slot; hd[r].pos0 = row.pos0; hd[r].n = (int32_t)row.n; hd[r].tok_off = at;
            hd[r].sample = row.sample ? 1 : 0; hd[r].kv_begin = slots_[(size_t)row.slot].begin;
            step_max_resident_ = std::max(step_max_resident_, row.pos0 + (int32_t)row.n - hd[r].kv_begin);
            // route = 1-based index of the adapter in id order (0: the base model)
            hd[r].route = 0; hd[r].pad = 0;
            // adapter 0 follows the context: its default adapter, else the trained adapter when there is one
            int32_t eff = row.adapter;
            if (eff == 0) eff = default_adapter_ != 0 ? default_adapter_ : kPolicyAdapter;
            const auto found = eff > 0 ? row_adapters_.find(eff) : row_adapters_.end();
            if (found != row_adapters_.end()) {
                hd[r].route = 1 + (int32_t)std::distance(row_adapters_.begin(), found);
                routed = true;
            }
            std::memcpy(ht + at, row.tokens, (size_t)row.n * 4);
            at += (int)row.n;
            if (row.sample) ++n_out;
        }
    }
    {
        rk::TableUpdate * hu = (rk::TableUpdate *)((uint8_t *)h_stage_.ptr + off_upd);
        size_t i = 0;
        for (const auto & kv : pending_updates_) {
            hu[i++] = {(int32_t)(kv.first / max_pages_), (int32_t)(kv.first % max_pages_), kv.second, 0};
        }
        pending_updates_.clear();
    }
    int n_tiles = 0, n_items = 0;
    rk::count_attention_work(hd, (int)n_rows, qt_, hp_.n_head_kv, &n_tiles, &n_items, &pk_.split_pages);

    if ((size_t)n_items * 32 > item_meta_.bytes) item_meta_.ensure((size_t)n_items * 48);      // some room to grow into
    pk_.item_a = item_meta_.as<int4>();
    pk_.item_b = pk_.item_a + n_items;

    try {
        hip_check(hipMemcpyAsync(d_stage_.ptr, h_stage_.ptr, stage_bytes, hipMemcpyHostToDevice, stream_), "hipMemcpyAsync");
        const size_t pt_pack = prof_begin(PC_PACK);
        rk::pack_step(stream_, d_stage_.as<rk::RowDesc>(), (int)n_rows,
                      (const int32_t *)((const uint8_t *)d_stage_.ptr + off_tok),
                      (const rk::TableUpdate *)((const uint8_t *)d_stage_.ptr + off_upd), (int)n_upd,
                      table_.as<int32_t>(), max_pages_, qt_, hp_.n_head_kv, inv_freq_.as<double>(),
                      hp_.rope_dim / 2, pk_);
        prof_end(PC_PACK, pt_pack);
        forward(T, n_out, n_tiles, n_items, (size_t)T == n_rows, routed);

        // ---- sampling: the device scans the vocabulary, the host draws.
        std::vector<int32_t> kreq((size_t)std::max(n_out, 1), 0);
        std::vector<int> out_of_row(n_rows, -1);
        bool any_full = false;
        {
            int o = 0;
            for (size_t r = 0; r < n_rows; ++r) {
                const RowView & row = rows[r];
                if (!row.sample) continue;
                out_of_row[r] = o;
                const bool fast = row.v2 && sampling::neutral_extras(*row.v2) && row.v2->top_k > 0
                    && row.v2->top_k <= rk::MAX_TOPK && row.v2->top_k < n_vocab;
                kreq[(size_t)o] = fast ? row.v2->top_k : 0;
                any_full = any_full || !fast;
                ++o;
            }
        }
        if (n_out > 0) {
            hip_check(hipMemcpyAsync(sample_k_.ptr, kreq.data(), (size_t)n_out * 4, hipMemcpyHostToDevice, stream_), "hipMemcpyAsync");
            const size_t pt_s = prof_begin(PC_SAMPLE);
            rk::sample_prepare(stream_, logits_.as<float>(), n_out, n_vocab, sample_k_.as<int32_t>(), sample_out_.as<rk::SampleOut>(),
                               *std::max_element(kreq.begin(), kreq.end()), sample_scratch_.ptr);
            prof_end(PC_SAMPLE, pt_s);
            hip_check(hipMemcpyAsync(h_sample_.ptr, sample_out_.ptr, (size_t)n_out * sizeof(rk::SampleOut), hipMemcpyDeviceToHost, stream_), "hipMemcpyAsync");
            if (any_full) {
                h_logits_.ensure((size_t)n_out * n_vocab * 4);
                for (size_t r = 0; r < n_rows; ++r) {
                    const int o = out_of_row[r];
                    if (o < 0 || kreq[(size_t)o] != 0) continue;
                    hip_check(hipMemcpyAsync(h_logits_.as<float>() + (size_t)o * n_vocab, logits_.as<float>() + (size_t)o * n_vocab,
                                             (size_t)n_vocab * 4, hipMemcpyDeviceToHost, stream_), "hipMemcpyAsync");
                }
            }
        }
        hip_check(hipStreamSynchronize(stream_), "step");
        if (prof_level_) prof_resolve();
        last_n_out_ = n_out;
        ++steps_run_;

        const rk::SampleOut * so = h_sample_.as<rk::SampleOut>();
        for (size_t r = 0; r < n_rows; ++r) {
            const RowView & row = rows[r];
            int32_t token = 0;
            float logprob = 0.0f, sampled_logprob = 0.0f;
            uint32_t n_top = 0;
            uint8_t sampled = 0;
            if (row.sample) {
                const int o = out_of_row[r];
                const rk::SampleOut & s = so[o];
                RequestState & req = requests_[row.request];
                if (!req.seeded) {
                    req.rng.seed(row.v2 ? row.v2->seed : row.v1.seed);
                    req.seeded = true;
                }
                const uint32_t k = std::min<uint32_t>(row.n_top, (uint32_t)std::min<size_t>(n_top_stride, (size_t)n_vocab));
                int32_t * top_ids = k > 0 ? out_top_ids + r * n_top_stride : nullptr;
                float * top_lps = k > 0 ? out_top_logprobs + r * n_top_stride : nullptr;
                const double log_sum = std::log(s.sum_exp);
                if (row.v2) {
                    // the grammar of this row becomes (or stays) the request's; a row without one drops it
                    const GrammarVocab * gv = nullptr;
                    if (row.v2->grammar) {
                        if (compiled[r]) req.grammar = compiled[r];
                        if (!req.grammar || req.grammar->gbnf() != row.v2->grammar->gbnf) {      // the request was freed and reused inside one call
                            set_error("failed to compile the request's grammar (invalid GBNF)");
                            return -1;
                        }
                        gv = &vocab_.for_grammars(n_vocab);
                    } else {
                        req.grammar.reset();
                    }
                    RowSample got;
                    float token_logit = 0.0f;
                    // Equal logits where an unstable host algorithm of the reference decides which survive - the top_k cut
                    // (std::partial_sort) or, under top_p < 1, the nucleus order (std::sort): the candidates cannot
                    // say what those algorithms do with the whole row, so the row is fetched and takes the full path.
                    bool tied = kreq[(size_t)o] > 0 && s.edge_tie != 0;
                    if (kreq[(size_t)o] > 1 && row.v2->top_p != 1.0f)
                        for (int j = 1; j < kreq[(size_t)o] && !tied; ++j) tied = s.top_logit[j] == s.top_logit[j - 1];
                    if (tied) {
                        h_logits_.ensure((size_t)n_out * n_vocab * 4);
                        hip_check(hipMemcpy(h_logits_.as<float>() + (size_t)o * n_vocab, logits_.as<float>() + (size_t)o * n_vocab,
                                            (size_t)n_vocab * 4, hipMemcpyDeviceToHost), "hipMemcpy");
                    }
                    if (kreq[(size_t)o] > 0 && !tied) {
                        got = sampling::finish_from_candidates(*row.v2, s.top_id, s.top_logit, (size_t)kreq[(size_t)o],
                                                               (size_t)n_vocab, req.rng, row.want_logprob, k, top_ids, top_lps);
                        for (int j = 0; j < kreq[(size_t)o]; ++j) if (s.top_id[j] == got.token) token_logit = s.top_logit[j];
                    } else {
                        const float * host_row = h_logits_.as<float>() + (size_t)o * n_vocab;
                        std::string err;
                        got = sampling::sample_full_row_v2(host_row, (size_t)n_vocab, *row.v2, req.rng, req.history, scratch_,
                                                           row.want_logprob, k, top_ids, top_lps, err, gv ? req.grammar.get() : nullptr, gv);
                        if (got.token < 0) {
                            set_error(err);
                            return -1;
                        }
                        token_logit = host_row[got.token];
                    }
                    token = got.token;
                    sampled_logprob = row.want_logprob ? got.sampled_logprob : 0.0f;
                    n_top = k;
                    req.history.push_back(token);
                    if (gv && !req.grammar->accept(*gv, (uint32_t)token)) {
                        set_error("the grammar refused the token it had allowed");
                        return -1;
                    }
                    // temperature-1 policy logprob: logit - max - log(sum exp(logit - max))
                    logprob = (float)((double)token_logit - s.max - log_sum);
                } else {
                    const float * host_row = h_logits_.as<float>() + (size_t)o * n_vocab;
                    float smax = 0.0f;
                    double stotal = 0.0;
                    std::string err;
                    token = sampling::sample_full_row_v1(host_row, (size_t)n_vocab, row.v1.temperature, row.v1.top_p,
                                                         req.rng, scratch_, smax, stotal, err);
                    if (token < 0) {
                        set_error(err);
                        return -1;
                    }
                    logprob = row.v1.temperature == 1.0f
                        ? (float)((double)host_row[token] - smax - std::log(stotal))
                        : (float)((double)host_row[token] - s.max - log_sum);
                    if (k > 0) {
                        sampling::top_logprobs_dense(host_row, (size_t)n_vocab, k, s.max, log_sum, scratch_.order, top_ids, top_lps);
                        n_top = k;
                    }
                }
                sampled = 1;
            }
            if (out2) {
                retro_step_out_row_v2 & o = out2[r];
                o.struct_size = sizeof(retro_step_out_row_v2);
                o.token = token; o.logprob = logprob; o.n_top = n_top; o.forced = 0; o.sampled = sampled;
                o.sampled_logprob = sampled_logprob;
            } else {
                retro_step_out_row & o = out1[r];
                o.struct_size = sizeof(retro_step_out_row);
                o.token = token; o.logprob = logprob; o.n_top = n_top; o.forced = 0; o.sampled = sampled;
            }
        }
    } catch (const std::exception & e) {
        set_error(std::string("the step failed on the device: ") + e.what()
                  + " - the KV may hold a prefix of the submitted tokens (query it with the seq_pos entry point)");
        return -1;
    }
    return 0;
}

void Engine::forward(int T, int n_out, int n_tiles, int n_items, bool one_token_rows, bool routed) {
    const HParams & h = hp_;
    const int E = h.n_embd, QD = h.n_head * h.head_dim, KD = h.n_head_kv * h.head_dim, F = h.n_ff;
    rk::AttnShape sh{h.n_head, h.n_head_kv, h.head_dim, h.rope_dim, h.rope_neox, h.eps, kv_strides_.page, kv_strides_.head, kv_q8_, kv_q8_ != rk::KV_F16 && ggml_activations_};
    // The versions of a row its consumers need: the values themselves for F32 / F16 / BF16 weights, the
    // expert router and LoRA factors (`plain`); the converted row for the quantised weights.
    const bool faithful = ggml_activations_;
    const bool ffn_lora = routed && lora_has_ffn_ && h.n_expert == 0;      // some row may carry feed-forward deltas
    rk::g_gemv_max_t = gemv_max_t_;     // this engine's setting, for the matmul entry points called below
    const bool small_step = T <= rk::g_gemv_max_t;      // the producers leave the Q8_K blocks for the integer kernel as well
    // ... or, where every consumer of a row is that kernel and nothing else wants the row (no adapters), the kernel
    // makes the blocks itself while it stages them and the producer's launch is saved
    // (single-token steps only: the blocks of a second row cost every workgroup more than the launch saves)
    const bool fuse = faithful && small_step && T == 1 && !routed && gemv_fuse_;
    // The exact arithmetic's single-token steps: the same kernel with f32 rows (gemv_f32*), the same fusions, and the
    // output projection from the planes the attention launch leaves. One flag selects the flavour below.
    const bool fuse_x = !faithful && T == 1 && !routed && gemv_fuse_ && gemv_exact_;
    auto can_gemv = [&](const rk::Weight & w, int tokens) { return fuse_x ? rk::gemv_f32_can_weight(w, tokens) : rk::gemv_can_weight(w, tokens); };
    auto all_gemv = [&](const std::vector<DevWeight> & ws, int K, int room) {
        int total = 0;
        for (const DevWeight & w : ws) {
            if (!can_gemv(w.w, T) || w.w.K != K) return false;
            total += w.w.N;
        }
        return !ws.empty() && total <= room;
    };
    auto gemv_norm = [&](const rk::Weight & w, const float * rows, const float * norm_w, const int32_t * which, int tokens, float * y,
                         int ldy, int col, const float * bias) {
        if (fuse_x) rk::gemv_f32_norm(stream_, w, rows, norm_w, h.eps, which, tokens, y, ldy, col, rk::MM_STORE, bias);
        else rk::gemv_norm(stream_, w, rows, norm_w, h.eps, which, tokens, y, ldy, col, rk::MM_STORE, bias);
    };
    auto act_for = [faithful, small_step](DevBuf & x, DevBuf & sums, DevBuf & qx, DevBuf & qsums, int K, std::initializer_list<int> types,
                                          bool plain, ActCodes * codes = nullptr) {
        rk::Act a;
        a.K = K;
        a.faithful = faithful ? 1 : 0;
        if (!faithful) {
            a.x = x.as<__half>();
            a.sums = K % 32 == 0 ? sums.as<__half>() : nullptr;
            return a;
        }
        for (int t : types) {
            const int q = rk::act_quant_of(t);
            if (q == rk::AQ_NONE) { plain = true; continue; }
            if (a.quant != rk::AQ_NONE && a.quant != q)
                throw std::runtime_error("weights that share an input row mix Q8_0 / MXFP4 with Q4_K storage: unsupported");
            a.quant = q;
        }
        if (plain) { a.x = x.as<__half>(); a.sums = K % 32 == 0 ? sums.as<__half>() : nullptr; }
        if (a.quant != rk::AQ_NONE) { a.qx = qx.as<__half>(); a.qsums = qsums.as<__half>(); }
        if (a.quant != rk::AQ_NONE && small_step && codes && codes->codes.ptr) {
            a.qc = codes->codes.as<int8_t>(); a.qd = codes->d.as<float>(); a.qbs = codes->bsums.as<int16_t>();
        }
        return a;
    };
    auto types_of = [](const std::vector<DevWeight> & ws) {
        int t[3] = {-1, -1, -1};
        for (size_t i = 0; i < ws.size() && i < 3; ++i) t[i] = ws[i].w.type;
        for (size_t i = ws.size(); i < 3; ++i) t[i] = ws.empty() ? rk::WT_F32 : ws[0].w.type;
        return std::array<int, 3>{t[0], t[1], t[2]};
    };
    const rk::Act act_o = act_for(act_o_x_, act_o_sums_, act_o_qx_, act_o_qsums_, E, {lm_head_.w.type}, false, &act_o_codes_);
    partial_.ensure(rk::attention_partial_floats(n_items, h.head_dim) * 4);
    float * x = x_.as<float>();
    float * qkv = qkv_.as<float>();
    float * gu = gu_.as<float>();

    // A matmul into the residual stream may leave its result as K-slices; the
    // next norm adds them to x.
    rk::Slices pending;
    { const size_t pt_ = prof_begin(PC_EMBED); rk::embed(stream_, tok_embd_.w, pk_.tok, T, x); prof_end(PC_EMBED, pt_); }
    for (int l = 0; l < h.n_layer; ++l) {
        const LayerWeights & L = layers_[(size_t)l];
        const std::array<int, 3> qt = types_of(L.qkv), gt = types_of(L.gate_up);
        rk::Act act_e = act_for(act_e_x_, act_e_sums_, act_e_qx_, act_e_qsums_, E, {qt[0], qt[1], qt[2]}, routed, &act_e_codes_);
        const rk::Act act_q = act_for(act_q_x_, act_q_sums_, act_q_qx_, act_q_qsums_, QD, {L.wo.w.type}, routed, &act_q_codes_);
        const bool qkv_fused = (fuse || fuse_x) && pending.n == 0 && all_gemv(L.qkv, E, QD + 2 * KD);
        if (!qkv_fused) { const size_t pt_ = prof_begin(PC_NORM); rk::rmsnorm_act(stream_, x, L.attn_norm.as<float>(), E, h.eps, nullptr, T, act_e, pending); prof_end(PC_NORM, pt_); }
        rk::Slices qkv_slices;
        {
            const size_t pt_ = prof_begin(PC_QKV);
            if (qkv_fused) {
                int col = 0;
                for (const DevWeight & w : L.qkv) {
                    gemv_norm(w.w, x, L.attn_norm.as<float>(), nullptr, T, qkv, QD + 2 * KD, col,
                              L.qkv_bias.ptr ? L.qkv_bias.as<float>() + col : nullptr);
                    col += w.w.N;
                }
            } else if (L.qkv.size() == 1) {     // fused q, k, v: the rotation kernel can add the slices
                qkv_slices = rk::matmul_deferred(stream_, L.qkv[0].w, act_e, T, qkv, QD + 2 * KD, 0, rk::MM_STORE,
                                                 L.qkv_bias.as<float>(), mm_ws_.ptr);
            } else {
                bool tiled = L.qkv.size() <= 3;
                const rk::Weight * parts[3] = {nullptr, nullptr, nullptr};
                for (size_t i = 0; i < L.qkv.size() && tiled; ++i) {
                    parts[i] = &L.qkv[i].w;
                    tiled = L.qkv[i].w.packed != nullptr && L.qkv[i].w.K == L.qkv[0].w.K && L.qkv[i].w.N % 4 == 0;
                }
                if (tiled) {     // tile matrices of different types: their K-slices side by side, added by the rotation kernel
                    qkv_slices = rk::matmul_deferred_parts(stream_, parts, (int)L.qkv.size(), act_e, T, qkv, QD + 2 * KD,
                                                           L.qkv_bias.as<float>(), mm_ws_.ptr);
                } else {
                    int col = 0;
                    for (const DevWeight & w : L.qkv) {
                        rk::matmul(stream_, w.w, act_e, T, qkv, QD + 2 * KD, col, rk::MM_STORE,
                                   L.qkv_bias.ptr ? L.qkv_bias.as<float>() + col : nullptr, mm_ws_.ptr);
                        col += w.w.N;
                    }
                }
            }
            if (routed) {
                // the adapter deltas go where the rotation kernel reads q, k, v from: the first slice or the buffer
                float * dst = qkv_slices.n > 0 ? const_cast<float *>(qkv_slices.data) : qkv;
                const rk::RowDesc * rows_d = d_stage_.as<rk::RowDesc>();
                const int cols[3] = {0, QD, QD + KD}, widths[3] = {QD, KD, KD};
                const rk::LoraEntry * tables[3] = {lora_entries(l, 0), lora_entries(l, 1), lora_entries(l, 2)};
                rk::lora_apply_targets(stream_, 3, tables, widths, cols, rows_d, pk_.row, act_e, T, dst, QD + 2 * KD,
                                       lora_mid_.as<float>());
            }
            prof_end(PC_QKV, pt_);
        }
        // every row decodes one token over an f16 cache in the exact arithmetic: rotation, KV store, attention and
        // split merge are one launch (the output projection's plain activation planes are all it writes)
        const bool fused_decode = one_token_rows && fused_decode_attention_ && !faithful
                                  && rk::attention_decode_can(sh, step_max_resident_);
        size_t pt_;
        if (fused_decode) {
            unsigned long long * stamps = nullptr;
            if (attn_timeline_ && l == h.n_layer / 2) {
                attn_stamped_wgs_ = (size_t)T * (size_t)h.n_head_kv;
                attn_stamps_.ensure(attn_stamped_wgs_ * 6 * sizeof(unsigned long long));
                stamps = attn_stamps_.as<unsigned long long>();
            }
            pt_ = prof_begin(PC_ATTN);
            rk::attention_decode(stream_, qkv, qkv_slices, T, sh, pk_, table_.as<int32_t>(), max_pages_,
                                 k_pool_[(size_t)l].as<__half>(), v_pool_[(size_t)l].as<__half>(), L.q_norm.as<float>(),
                                 L.k_norm.as<float>(), act_q, stamps);
            prof_end(PC_ATTN, pt_);
            pt_ = prof_begin(PC_OPROJ);
            if (fuse_x && rk::gemv_f32_can_weight(L.wo.w, T) && L.wo.w.K == QD && L.wo.w.N == E) {
                rk::gemv_f32(stream_, L.wo.w, act_q, T, x, E, 0, rk::MM_ADD, nullptr);
                pending = rk::Slices();
            } else {
                pending = rk::matmul_deferred(stream_, L.wo.w, act_q, T, x, E, 0, rk::MM_ADD, nullptr, mm_ws_.ptr);
            }
            if (routed) {
                float * dst = pending.n > 0 ? const_cast<float *>(pending.data) : x;
                rk::lora_apply(stream_, lora_entries(l, 3), d_stage_.as<rk::RowDesc>(), pk_.row, act_q, T, E, dst, E, 0,
                               lora_mid_.as<float>());
            }
            prof_end(PC_OPROJ, pt_);
        } else {
        pt_ = prof_begin(PC_ROPE);
        rk::rope_store(stream_, qkv, T, sh, pk_, L.q_norm.as<float>(), L.k_norm.as<float>(), q_half_.as<__half>(),
                       q_half_lo_.as<__half>(), k_pool_[(size_t)l].as<__half>(), v_pool_[(size_t)l].as<__half>(),
                       qkv_slices);
        prof_end(PC_ROPE, pt_);
        pt_ = prof_begin(PC_ATTN);
        rk::attention(stream_, q_half_.as<__half>(), q_half_lo_.as<__half>(), sh, pk_, table_.as<int32_t>(), max_pages_,
                      k_pool_[(size_t)l].as<__half>(), v_pool_[(size_t)l].as<__half>(), n_items, n_tiles,
                      partial_.as<float>(), one_token_rows);
        prof_end(PC_ATTN, pt_);
        // a single token with few splits: the output projection merges them itself (n_items = kv heads x splits)
        const int n_split = T == 1 && n_tiles == 1 ? n_items / h.n_head_kv : 0;
        const bool merge_in_oproj = fuse && n_split >= 1 && n_split <= merge_max_splits_ && n_split * h.n_head_kv == n_items
                                    && rk::gemv_can_weight(L.wo.w, 1) && L.wo.w.K == QD && L.wo.w.N == E;
        if (merge_in_oproj) {
            pt_ = prof_begin(PC_OPROJ);
            rk::gemv_combine(stream_, L.wo.w, partial_.as<float>(), 0, n_split, h.n_head, h.n_head / h.n_head_kv, h.head_dim, x, E, 0,
                             rk::MM_ADD);
            pending = rk::Slices();
            prof_end(PC_OPROJ, pt_);
        } else {
        pt_ = prof_begin(PC_COMBINE);
        rk::attention_combine(stream_, partial_.as<float>(), T, sh, pk_, act_q);
        prof_end(PC_COMBINE, pt_);
        pt_ = prof_begin(PC_OPROJ);
        if (fuse_x && rk::gemv_f32_can_weight(L.wo.w, T) && L.wo.w.K == QD && L.wo.w.N == E) {
            rk::gemv_f32(stream_, L.wo.w, act_q, T, x, E, 0, rk::MM_ADD, nullptr);
            pending = rk::Slices();
        } else {
            pending = rk::matmul_deferred(stream_, L.wo.w, act_q, T, x, E, 0, rk::MM_ADD, nullptr, mm_ws_.ptr);
        }
        if (routed) {
            float * dst = pending.n > 0 ? const_cast<float *>(pending.data) : x;
            rk::lora_apply(stream_, lora_entries(l, 3), d_stage_.as<rk::RowDesc>(), pk_.row, act_q, T, E, dst, E, 0,
                           lora_mid_.as<float>());
        }
        prof_end(PC_OPROJ, pt_);
        }
        }
        if ((fuse || fuse_x) && h.n_expert == 0 && pending.n == 0 && all_gemv(L.gate_up, E, 2 * F)) {
            pt_ = prof_begin(PC_GATEUP);
            int col = 0;
            for (const DevWeight & w : L.gate_up) {
                gemv_norm(w.w, x, L.ffn_norm.as<float>(), nullptr, T, gu, 2 * F, col, nullptr);
                col += w.w.N;
            }
            prof_end(PC_GATEUP, pt_);
            const int group = L.gate_up_interleaved ? 64 : F;
            pt_ = prof_begin(PC_DOWN);
            if (can_gemv(L.down.w, T) && L.down.w.K == F && L.down.w.N == E) {
                if (fuse_x) rk::gemv_f32_swiglu(stream_, L.down.w, gu, group, T, x, E, 0, rk::MM_ADD);
                else rk::gemv_swiglu(stream_, L.down.w, gu, group, T, x, E, 0, rk::MM_ADD);
                pending = rk::Slices();
            } else {
                const rk::Act act_f = act_for(act_f_x_, act_f_sums_, act_f_qx_, act_f_qsums_, F, {L.down.w.type}, false, &act_f_codes_);
                rk::swiglu_act(stream_, gu, T, F, act_f, group);
                pending = rk::matmul_deferred(stream_, L.down.w, act_f, T, x, E, 0, rk::MM_ADD, nullptr, mm_ws_.ptr);
            }
            prof_end(PC_DOWN, pt_);
            continue;
        }
        pt_ = prof_begin(PC_NORM);
        if (h.n_expert > 0) act_e = act_for(act_e_x_, act_e_sums_, act_e_qx_, act_e_qsums_, E, {L.router.w.type, L.gate_exps.w.type}, false);
        else act_e = act_for(act_e_x_, act_e_sums_, act_e_qx_, act_e_qsums_, E, {gt[0], gt[1], gt[2]}, ffn_lora, &act_e_codes_);
        rk::rmsnorm_act(stream_, x, L.ffn_norm.as<float>(), E, h.eps, nullptr, T, act_e, pending);
        prof_end(PC_NORM, pt_);
        if (h.n_expert > 0) {
            pt_ = prof_begin(PC_GATEUP);
            rk::MoeLayer ml{L.router.w, L.gate_exps.w, L.up_exps.w, L.down_exps.w};
            rk::MoeShape ms{E, h.n_ff_exp, h.n_expert, h.n_expert_used};
            rk::MoeBuffers mb{moe_logits_.as<float>(), moe_sel_.as<int32_t>(), moe_wgt_.as<float>(), moe_n_.as<int32_t>(),
                              moe_off_.as<int32_t>(), moe_tok_.as<int32_t>(), moe_q_.as<int32_t>(),
                              rk::Act{moe_h_.as<__half>(), nullptr, h.n_ff_exp}, moe_out_.as<float>()};
            mb.mx_ops = moe_mx_ops_.as<uint8_t>(); mb.mx_scales = moe_mx_scales_.as<uint8_t>(); mb.mx_h = moe_mx_h_.as<float>();
            mb.mx_slots = moe_mx_slots_;
            mb.pair_of_q = moe_pair_.as<int32_t>();
            pending = rk::moe_ffn(stream_, ml, ms, act_e, T, x, mb, true);     // the next norm adds the experts' weighted sum
            prof_end(PC_GATEUP, pt_);
            continue;
        }
        pt_ = prof_begin(PC_GATEUP);
        const rk::Act act_f = act_for(act_f_x_, act_f_sums_, act_f_qx_, act_f_qsums_, F, {L.down.w.type}, ffn_lora, &act_f_codes_);
        if (L.gate_up_interleaved && !ffn_lora) {
            rk::matmul_swiglu(stream_, L.gate_up[0].w, act_e, T, act_f, mm_ws_.ptr, gu);
            prof_end(PC_GATEUP, pt_);
        } else {
            // gate and up as f32 rows: side by side, or - the interleaved matrix of the fused kernel multiplied
            // like any other - in alternating groups of 64 columns; the adapter deltas join them before the SiLU
            const int group = L.gate_up_interleaved ? 64 : F;
            int col = 0;
            for (const DevWeight & w : L.gate_up) {
                rk::matmul(stream_, w.w, act_e, T, gu, 2 * F, col, rk::MM_STORE, nullptr, mm_ws_.ptr);
                col += w.w.N;
            }
            if (ffn_lora) {
                const int cols[2] = {0, group}, widths[2] = {F, F};
                const rk::LoraEntry * tables[2] = {lora_entries(l, 4), lora_entries(l, 5)};
                rk::lora_apply_targets(stream_, 2, tables, widths, cols, d_stage_.as<rk::RowDesc>(), pk_.row, act_e, T, gu,
                                       2 * F, lora_mid_.as<float>(), L.gate_up_interleaved ? group : 0);
            }
            prof_end(PC_GATEUP, pt_);
            pt_ = prof_begin(PC_SWIGLU);
            rk::swiglu_act(stream_, gu, T, F, act_f, group);
            prof_end(PC_SWIGLU, pt_);
        }
        pt_ = prof_begin(PC_DOWN);
        pending = rk::matmul_deferred(stream_, L.down.w, act_f, T, x, E, 0, rk::MM_ADD, nullptr, mm_ws_.ptr);
        if (ffn_lora) {
            float * dst = pending.n > 0 ? const_cast<float *>(pending.data) : x;
            rk::lora_apply(stream_, lora_entries(l, 6), d_stage_.as<rk::RowDesc>(), pk_.row, act_f, T, E, dst, E, 0,
                           lora_mid_.as<float>());
        }
        prof_end(PC_DOWN, pt_);
    }
    if (n_out > 0) {
        logits_.ensure((size_t)n_out * h.n_vocab * 4);
        const size_t pt_ = prof_begin(PC_HEAD);
        if ((fuse || fuse_x) && pending.n == 0 && can_gemv(lm_head_.w, n_out) && lm_head_.w.K == E && lm_head_.w.N == h.n_vocab) {
            gemv_norm(lm_head_.w, x, out_norm_.as<float>(), pk_.out_tok, n_out, logits_.as<float>(), h.n_vocab, 0, out_bias_.as<float>());
        } else {
            rk::rmsnorm_act(stream_, x, out_norm_.as<float>(), E, h.eps, pk_.out_tok, n_out, act_o, pending);
            rk::matmul(stream_, lm_head_.w, act_o, n_out, logits_.as<float>(), h.n_vocab, 0, rk::MM_STORE,
                       out_bias_.as<float>(), mm_ws_.ptr);
        }
        prof_end(PC_HEAD, pt_);
    }
}

// ---- per-row adapters -----------------------------------------------------------------------

// A LoRA adapter file as the reference writes it (retro_lora.cpp:1004-1043,
// 1143-1153): general.type = "adapter", adapter.type = "lora",
// adapter.lora.alpha, tensors "<weight>.lora_a" ne = [n_in, r] and
// "<weight>.lora_b" ne = [r, n_out].
int Engine::adapter_load(const std::string & path, float scale, int32_t * out_id) {
    if (next_adapter_id_ == kPolicyAdapter) {
        set_error("per-row adapter ids are exhausted");
        return -1;
    }
    RowAdapterData data;
    if (read_adapter(path, scale, data) != 0) return -1;
    const int32_t id = next_adapter_id_++;
    row_adapters_.emplace(id, std::move(data));
    rebuild_lora_table();
    *out_id = id;
    return 0;
}

// The trained adapter of a trainer's generation context: what rows with adapter 0
// decode under until set_default_adapter() says otherwise. Replaces the one before.
int Engine::policy_adapter_load(const std::string & path) {
    RowAdapterData data;
    if (read_adapter(path, 1.0f, data) != 0) return -1;
    hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
    row_adapters_.erase(kPolicyAdapter);
    row_adapters_.emplace(kPolicyAdapter, std::move(data));
    rebuild_lora_table();
    return 0;
}

// A frozen device-to-device copy of the trained adapter as a per-row adapter
// (reference retro_rollout.cpp:184-244).
int Engine::adapter_snapshot(int32_t replace, float scale, int32_t * out_id) {
    if (!std::isfinite(scale)) {
        set_error("the adapter scale must be finite");
        return -1;
    }
    auto policy = row_adapters_.find(kPolicyAdapter);
    if (policy == row_adapters_.end()) {
        set_error("a snapshot copies the trained LoRA adapter, and the trainer has none");
        return -1;
    }
    if (replace != 0) {
        if (replace == kPolicyAdapter || !row_adapters_.count(replace)) {
            set_error("no per-row adapter is loaded under id " + std::to_string(replace));
            return -1;
        }
        if (default_adapter_ == replace) {
            default_adapter_ = 0;
            forget_generation_bookkeeping();
        }
        hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
        row_adapters_.erase(replace);       // freed before the copy is made: a refresh never holds two snapshots
    }
    if (next_adapter_id_ == kPolicyAdapter) {
        set_error("per-row adapter ids are exhausted");
        return -1;
    }
    RowAdapterData copy = clone_adapter(policy->second, scale);
    const int32_t id = next_adapter_id_++;
    row_adapters_.emplace(id, std::move(copy));
    rebuild_lora_table();
    *out_id = id;
    return 0;
}

Engine::RowAdapterData Engine::clone_adapter(const RowAdapterData & src, float scale) {
    RowAdapterData copy;
    copy.scale = scale;
    copy.alpha = src.alpha;
    copy.rank = src.rank;
    copy.elements = src.elements;
    copy.a_type = src.a_type;
    copy.b_type = src.b_type;
    copy.a.resize(src.a.size());
    copy.b.resize(src.b.size());
    for (size_t i = 0; i < src.a.size(); ++i) {
        if (!src.a[i].ptr) continue;
        copy.a[i].alloc(src.a[i].bytes);
        copy.b[i].alloc(src.b[i].bytes);
        hip_check(hipMemcpyAsync(copy.a[i].ptr, src.a[i].ptr, src.a[i].bytes, hipMemcpyDeviceToDevice, stream_), "hipMemcpyAsync");
        hip_check(hipMemcpyAsync(copy.b[i].ptr, src.b[i].ptr, src.b[i].bytes, hipMemcpyDeviceToDevice, stream_), "hipMemcpyAsync");
    }
    hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
    return copy;
}

// ---- context-wide adapters (reference retro_engine.cpp:756-870) ----------------------------
// Adapters registered under a name, one of them active: what rows with adapter 0 decode under.
// Every change of what is active is a change of the weights: all cells and the generators'
// bookkeeping go, the weights version moves on (forget_engine_kv, retro_engine.cpp:322-328).

void Engine::apply_active_adapter() {
    hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
    row_adapters_.erase(kPolicyAdapter);
    if (!active_adapter_.empty())
        row_adapters_.emplace(kPolicyAdapter, clone_adapter(named_adapters_.at(active_adapter_), 1.0f));
    rebuild_lora_table();
}

int Engine::load_lora_named(const std::string & name, const std::string & path) {
    RowAdapterData data;
    if (read_adapter(path, 1.0f, data) != 0) return -1;
    const bool was_active = active_adapter_ == name;
    named_adapters_.erase(name);
    named_adapters_.emplace(name, std::move(data));
    if (was_active) {              // registered beside the others, not applied - unless it replaces the active one
        apply_active_adapter();
        forget_generation_kv();
    }
    return 0;
}

int Engine::load_lora(const std::string & path) {
    RowAdapterData data;
    if (read_adapter(path, 1.0f, data) != 0) return -1;
    named_adapters_.clear();       // the single-adapter contract: every other adapter goes
    named_adapters_.emplace(path, std::move(data));
    active_adapter_ = path;
    apply_active_adapter();
    forget_generation_kv();
    return 0;
}

int Engine::activate_lora(const std::string & name) {
    if (!name.empty() && !named_adapters_.count(name)) {
        set_error("no LoRA adapter registered under '" + name + "'");
        return -1;
    }
    active_adapter_ = name;
    apply_active_adapter();
    forget_generation_kv();
    return 0;
}

int Engine::set_lora_enabled(bool enabled) {
    if (!enabled) {
        active_adapter_.clear();
    } else if (active_adapter_.empty()) {
        set_error("cannot enable LoRA: no adapter is active");
        return -1;
    }
    apply_active_adapter();
    forget_generation_kv();
    return 0;
}

// What rows with adapter 0 - and with them the batched generators - decode under:
// 0 the trained adapter (the base model when there is none), RETRO_STEP_ADAPTER_BASE
// the base model, or a per-row adapter id (reference retro_rollout.cpp:283-303).
int Engine::set_default_adapter(int32_t adapter) {
    if (adapter < RETRO_STEP_ADAPTER_BASE || adapter == kPolicyAdapter
            || (adapter > 0 && !row_adapters_.count(adapter))) {
        set_error("adapter " + std::to_string(adapter) + " is not a loaded per-row adapter");
        return -1;
    }
    if (default_adapter_ != adapter) {
        default_adapter_ = adapter;
        // the generators' prefix bookkeeping does not know which adapter a resident prefix was decoded under
        forget_generation_bookkeeping();
    }
    return 0;
}

// Every cell of the pool and the generators' bookkeeping: what a change of the
// weights leaves behind is no prefix of the new model (reference retro_runtime.hpp:515-523).
void Engine::forget_generation_kv() {
    clear_generation_memory();
    forget_generation_bookkeeping();
    weights_version_ += 1;
}

int Engine::read_adapter(const std::string & path, float scale, RowAdapterData & data) {
    std::unique_ptr<GgufFile> file;
    try {
        file.reset(new GgufFile(path));
    } catch (const std::exception &) {
        set_error("failed to load LoRA adapter: " + path);
        return -1;
    }
    if (file->get_string("general.type") != "adapter" || file->get_string("adapter.type") != "lora") {
        set_error("failed to load LoRA adapter: " + path);
        return -1;
    }
    const HParams & h = hp_;
    const int E = h.n_embd, QD = h.n_head * h.head_dim, KD = h.n_head_kv * h.head_dim;
    // every true matrix of a layer (reference retro_lora.cpp:165-169); a mixture-of-experts layer has no dense
    // feed-forward matrices, and its expert stacks are no per-row targets (retro_lora_train.h:2594-2596)
    static const char * kTargets[kLoraTargets] = {"attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down"};
    const int F = h.n_expert > 0 ? 0 : h.n_ff;
    const int n_in[kLoraTargets] = {E, E, E, QD, E, E, F}, n_out[kLoraTargets] = {QD, KD, KD, E, F, F, E};
    data = RowAdapterData();
    data.scale = scale;
    data.alpha = file->get_float("adapter.lora.alpha", 0.0);
    data.a.resize((size_t)h.n_layer * kLoraTargets);
    data.b.resize((size_t)h.n_layer * kLoraTargets);
    data.a_type.assign((size_t)h.n_layer * kLoraTargets, rk::WT_F32);
    data.b_type.assign((size_t)h.n_layer * kLoraTargets, rk::WT_F32);
    size_t claimed = 0;
    for (int l = 0; l < h.n_layer; ++l) {
        for (int tg = 0; tg < kLoraTargets; ++tg) {
            const std::string base = "blk." + std::to_string(l) + "." + kTargets[tg] + ".weight";
            const TensorInfo * ta = file->find(base + ".lora_a");
            const TensorInfo * tb = file->find(base + ".lora_b");
            if (!ta && !tb) continue;
            if (!ta || !tb) {
                set_error("LoRA adapter tensor " + base + " has no matching lora_a / lora_b pair");
                return -1;
            }
            if (n_in[tg] <= 0 || n_out[tg] <= 0) continue;       // not a matrix of this model: reported below as unclaimed
            const int r = (int)ta->ne[1];
            if (ta->ne[0] != n_in[tg] || tb->ne[1] != n_out[tg] || tb->ne[0] != r || r <= 0) {
                set_error("LoRA adapter tensor " + base + " does not match the base model's shape");
                return -1;
            }
            if (r > rk::LORA_MAX_RANK) {
                set_error("LoRA rank " + std::to_string(r) + " exceeds the supported maximum of " + std::to_string(rk::LORA_MAX_RANK));
                return -1;
            }
            if (data.rank != 0 && data.rank != r) {
                set_error("a per-row adapter must use one rank for all of its targets");
                return -1;
            }
            data.rank = r;
            auto to_f32 = [&](const TensorInfo & t, int K, int rows, DevBuf & out) {
                rk::geom_of(t.type);
                if (rk::row_bytes(t.type, K) * (size_t)rows != t.nbytes) throw std::runtime_error("tensor " + t.name + " has an unexpected size");
                DevBuf raw;
                raw.alloc(t.nbytes);
                hip_check(hipMemcpyAsync(raw.ptr, t.data, t.nbytes, hipMemcpyHostToDevice, stream_), "hipMemcpyAsync");
                out.alloc((size_t)rows * K * 4);
                rk::decode_rows(stream_, t.type, raw.as<uint8_t>(), K, rows, out.as<float>());
                hip_check(hipStreamSynchronize(stream_), "decode adapter tensor");
            };
            to_f32(*ta, n_in[tg], r, data.a[(size_t)l * kLoraTargets + tg]);      // A: r rows of n_in
            to_f32(*tb, r, n_out[tg], data.b[(size_t)l * kLoraTargets + tg]);     // B: n_out rows of r
            data.a_type[(size_t)l * kLoraTargets + tg] = (int32_t)ta->type;
            data.b_type[(size_t)l * kLoraTargets + tg] = (int32_t)tb->type;
            data.elements += (uint64_t)n_in[tg] + (uint64_t)n_out[tg];
            claimed += 2;
        }
    }
    // a target this engine does not route per row (embeddings, expert stacks) must not be dropped silently
    size_t lora_tensors = 0;
    for (const TensorInfo & t : file->tensors()) {
        const std::string & n = t.name;
        if (n.size() > 7 && (n.compare(n.size() - 7, 7, ".lora_a") == 0 || n.compare(n.size() - 7, 7, ".lora_b") == 0)) ++lora_tensors;
    }
    if (lora_tensors != claimed) {
        set_error("failed to stack the per-row adapters: only the attention and dense feed-forward matrices of a layer are routed per row");
        return -1;
    }
    if (data.rank == 0) {
        set_error("failed to load LoRA adapter: " + path + " holds no LoRA tensor pair");
        return -1;
    }
    return 0;
}

int Engine::adapter_unload(int32_t id) {
    auto it = row_adapters_.find(id);
    if (id == kPolicyAdapter || it == row_adapters_.end()) {
        set_error("no per-row adapter is loaded under id " + std::to_string(id));
        return -1;
    }
    if (default_adapter_ == id) {
        default_adapter_ = 0;
        forget_generation_bookkeeping();
    }
    hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
    row_adapters_.erase(it);
    rebuild_lora_table();
    return 0;
}

// Routes are the 1-based positions of the adapters in id order (reference
// lora_router_install, retro_gen_core.cpp:2987-3006).
void Engine::rebuild_lora_table() {
    lora_routes_ = (int)row_adapters_.size();
    lora_has_ffn_ = false;
    if (lora_routes_ == 0) return;
    std::vector<rk::LoraEntry> table((size_t)hp_.n_layer * kLoraTargets * (size_t)lora_routes_);
    int route = 0;
    for (const auto & kv : row_adapters_) {
        const RowAdapterData & d = kv.second;
        for (int l = 0; l < hp_.n_layer; ++l)
            for (int tg = 0; tg < kLoraTargets; ++tg) {
                rk::LoraEntry & e = table[((size_t)l * kLoraTargets + tg) * (size_t)lora_routes_ + (size_t)route];
                const size_t at = (size_t)l * kLoraTargets + tg;
                if (!d.a[at].ptr) continue;
                if (tg >= 4) lora_has_ffn_ = true;
                e.A = d.a[at].as<float>();
                e.B = d.b[at].as<float>();
                e.rank = d.rank;
                e.scale = (float)((double)d.scale * d.alpha / d.rank);
                e.a_type = ggml_activations_ ? d.a_type[at] : rk::WT_F32;
                e.b_type = ggml_activations_ ? d.b_type[at] : rk::WT_F32;
            }
        ++route;
    }
    hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
    lora_table_.alloc(table.size() * sizeof(rk::LoraEntry));
    hip_check(hipMemcpy(lora_table_.ptr, table.data(), table.size() * sizeof(rk::LoraEntry), hipMemcpyHostToDevice), "hipMemcpy");
    if (!lora_mid_.ptr) lora_mid_.alloc((size_t)3 * cfg_.n_batch * rk::LORA_MAX_RANK * 4);
}

// What the stacks cost as the reference builds them: every adapter padded to
// the widest rank, F32 (retro_gen_core.cpp:3008-3030).
void Engine::adapter_rows_info(retro_adapter_rows_info * out) const {
    *out = retro_adapter_rows_info{};
    out->struct_size = sizeof(retro_adapter_rows_info);
    uint32_t max_rank = 0;
    for (const auto & kv : row_adapters_)
        if (kv.first != kPolicyAdapter) max_rank = std::max<uint32_t>(max_rank, (uint32_t)kv.second.rank);
    out->n_adapters = (uint32_t)(row_adapters_.size() - row_adapters_.count(kPolicyAdapter));
    out->max_rank = max_rank;
    for (const auto & kv : row_adapters_) {
        if (kv.first == kPolicyAdapter) continue;
        out->stacked_bytes += kv.second.elements * max_rank * 4;
        out->unpadded_bytes += kv.second.elements * (uint64_t)kv.second.rank * 4;
    }
}

// ---- event timing -------------------------------------------------------------------------

size_t Engine::prof_begin(int cat) {
    if (prof_level_ == 0 || (prof_level_ == 1 && cat != PC_ATTN)) return (size_t)-1;
    if (prof_used_ + 2 > prof_events_.size()) {
        for (int i = 0; i < 2; ++i) {
            hipEvent_t e;
            hip_check(hipEventCreate(&e), "hipEventCreate");
            prof_events_.push_back(e);
        }
    }
    const size_t a = prof_used_;
    prof_used_ += 2;
    hip_check(hipEventRecord(prof_events_[a], stream_), "hipEventRecord");
    return a;
}

void Engine::prof_end(int cat, size_t token) {
    if (token == (size_t)-1) return;
    hip_check(hipEventRecord(prof_events_[token + 1], stream_), "hipEventRecord");
    prof_spans_.push_back({cat, token, token + 1});
}

void Engine::prof_resolve() {
    for (const ProfSpan & sp : prof_spans_) {
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, prof_events_[sp.a], prof_events_[sp.b]) == hipSuccess) {
            prof_ms_[sp.cat] += ms;
            prof_n_[sp.cat] += 1;
        }
    }
    prof_spans_.clear();
    prof_used_ = 0;
}

void Engine::profile_read(double * ms, uint64_t * launches, bool reset) {
    for (int c = 0; c < PC_COUNT; ++c) {
        ms[c] = prof_ms_[c];
        launches[c] = prof_n_[c];
        if (reset) { prof_ms_[c] = 0.0; prof_n_[c] = 0; }
    }
}

// ---- test hooks -------------------------------------------------------------------------

int Engine::debug_last_logits(float * out, size_t n_floats, size_t * out_rows) {
    if (out_rows) *out_rows = (size_t)last_n_out_;
    const size_t need = (size_t)last_n_out_ * hp_.n_vocab;
    if (!out) return 0;
    if (n_floats < need) {
        set_error("the logits buffer is too small");
        return -2;
    }
    if (need) hip_check(hipMemcpy(out, logits_.ptr, need * 4, hipMemcpyDeviceToHost), "hipMemcpy");
    return 0;
}

int Engine::debug_read_kv(int layer, int32_t slot, int32_t pos, int want_v, uint16_t * out) {
    if (layer < 0 || layer >= hp_.n_layer || slot < 0 || slot >= (int32_t)cfg_.n_seq_max) {
        set_error("layer or slot out of range");
        return -1;
    }
    const Slot & s = slots_[(size_t)slot];
    if (pos < s.begin || pos >= s.end) {
        set_error("position is not resident");
        return -1;
    }
    const int32_t cell = s.pages[(size_t)(pos / rk::PAGE)] * rk::PAGE + pos % rk::PAGE;
    // the row as kv_gather writes it: kv_dim f16 values, or (a Q8_0 cache) per kv head the code bytes and block scales
    const size_t kd = rk::kv_row_halves(hp_.n_head_kv, hp_.head_dim, kv_q8_);
    DevBuf dc, tmp;
    dc.alloc(4);
    tmp.alloc(kd * 2);
    hip_check(hipMemcpy(dc.ptr, &cell, 4, hipMemcpyHostToDevice), "hipMemcpy");
    const __half * pool = want_v ? v_pool_[(size_t)layer].as<__half>() : k_pool_[(size_t)layer].as<__half>();
    rk::kv_gather(stream_, pool, kv_strides_, hp_.n_head_kv, hp_.head_dim, want_v != 0, dc.as<int32_t>(), 1, tmp.as<__half>(), kv_q8_);
    hip_check(hipStreamSynchronize(stream_), "debug_read_kv");
    hip_check(hipMemcpy(out, tmp.ptr, kd * 2, hipMemcpyDeviceToHost), "hipMemcpy");
    return 0;
}

int Engine::debug_pack(int32_t * tok, int32_t * pos, int32_t * seq, int32_t * cell, int32_t * out_index,
                       int32_t * last_index, size_t cap_tokens, size_t cap_rows, int32_t * counts) {
    int32_t c[4];
    hip_check(hipMemcpy(c, pk_.counts, sizeof(c), hipMemcpyDeviceToHost), "hipMemcpy");
    std::memcpy(counts, c, sizeof(c));
    const size_t T = (size_t)c[0];
    if (T > cap_tokens) {
        set_error("the token buffers are too small");
        return -2;
    }
    auto get = [&](int32_t * dst, const int32_t * src, size_t n) {
        if (dst && n) hip_check(hipMemcpy(dst, src, n * 4, hipMemcpyDeviceToHost), "hipMemcpy");
    };
    get(tok, pk_.tok, T); get(pos, pk_.pos, T); get(seq, pk_.seq, T); get(cell, pk_.cell, T); get(out_index, pk_.out_index, T);
    get(last_index, pk_.last_index, std::min(cap_rows, (size_t)cfg_.n_batch));
    return 0;
}

void Engine::attention_timeline(bool on) {
    attn_timeline_ = on;
    if (!on) attn_stamped_wgs_ = 0;
}

int Engine::attention_timeline_read(unsigned long long * out, size_t cap_workgroups, size_t * n_workgroups) {
    hip_check(hipStreamSynchronize(stream_), "attention_timeline_read");
    if (n_workgroups) *n_workgroups = attn_stamped_wgs_;
    if (!out || attn_stamped_wgs_ == 0) return 0;
    if (cap_workgroups < attn_stamped_wgs_) { set_error("attention timeline: the buffer is too small"); return -2; }
    hip_check(hipMemcpy(out, attn_stamps_.ptr, attn_stamped_wgs_ * 6 * sizeof(unsigned long long), hipMemcpyDeviceToHost), "hipMemcpy");
    return 0;
}

int Engine::debug_page_table(int32_t slot, int32_t * out, size_t cap, size_t * out_n) {
    if (slot < 0 || slot >= (int32_t)cfg_.n_seq_max) {
        set_error("slot is outside the context's sequence range");
        return -1;
    }
    *out_n = (size_t)max_pages_;
    if (!out) return 0;
    if (cap < (size_t)max_pages_) {
        set_error("the page buffer is too small");
        return -2;
    }
    std::memcpy(out, slots_[(size_t)slot].pages.data(), (size_t)max_pages_ * 4);
    return 0;
}

}  // namespace retro
