// The engine behind the opaque retro_engine handle: a GGUF model resident in
// HBM, one paged KV pool, per-request sampler state, and the step that runs
// one forward pass over a caller-built ragged plan. Mirrors the state the
// reference keeps in engine_state (crates/retrograd-ffi/runtime/src/
// retro_engine.cpp:22-74) minus everything that belongs to llama.cpp.
#pragma once

#include "../../include/retro_step.h"
#include "gguf_file.hpp"
#include "kernels.hpp"
#include "tokenizer.hpp"
#include "grammar.hpp"
#include "sampler.hpp"

#include <map>
#include <memory>
#include <queue>
#include <string>
#include <unordered_map>
#include <vector>

// A grammar handle of the C ABI: an owned GBNF text (reference retro_grammar.cpp:20-33).
struct retro_grammar { std::string gbnf; };

namespace retro {

void set_error(std::string message);
void clear_error();
const std::string & last_error();

// A device allocation released with the object.
struct DevBuf {
    void * ptr = nullptr;
    size_t bytes = 0;
    DevBuf() = default;
    ~DevBuf();
    DevBuf(const DevBuf &) = delete;
    DevBuf & operator=(const DevBuf &) = delete;
    DevBuf(DevBuf && o) noexcept : ptr(o.ptr), bytes(o.bytes) { o.ptr = nullptr; o.bytes = 0; }
    DevBuf & operator=(DevBuf && o) noexcept;
    void alloc(size_t n);          // frees what it held; n = 0 leaves it empty
    void ensure(size_t n);         // grows (never shrinks); contents are not kept
    void release();
    template <typename T> T * as() const { return (T *)ptr; }
};

struct HostPinned {
    void * ptr = nullptr;
    size_t bytes = 0;
    ~HostPinned();
    void ensure(size_t n);
    template <typename T> T * as() const { return (T *)ptr; }
};

struct HParams {
    std::string arch;
    int n_layer = 0, n_embd = 0, n_head = 0, n_head_kv = 0, head_dim = 0, n_ff = 0, n_vocab = 0;
    int rope_dim = 0;
    bool rope_neox = false;
    float eps = 1e-5f;
    double rope_base = 10000.0;
    int n_expert = 0, n_expert_used = 0, n_ff_exp = 0;
};

struct DevWeight {
    rk::Weight w;
    DevBuf buf;
    DevBuf records;      // MXFP4 expert tensors: the rows again in the block-scaled kernels' records
};

struct LayerWeights {
    DevBuf attn_norm, ffn_norm, qkv_bias, q_norm, k_norm;
    std::vector<DevWeight> qkv;    // one fused matrix, or q, k, v separately
    DevWeight wo;
    std::vector<DevWeight> gate_up; // one fused matrix, or gate, up separately
    bool gate_up_interleaved = false;   // one matrix, 64 gate rows and 64 up rows in turn: SwiGLU runs in the matmul's epilogue
    DevWeight down;
    // mixture-of-experts layers: F32 router [n_expert][E] and the three expert tensors, tiled per expert
    DevWeight router, gate_exps, up_exps, down_exps;
};

struct Slot {
    int begin = 0, end = 0;         // resident positions [begin, end)
    std::vector<int32_t> pages;     // page id per page index (position / PAGE), -1 = none
};

struct Vocab {
    std::vector<std::string> pieces;
    std::vector<int32_t> types;
    int32_t eos = -1, eot = -1;
    Tokenizer tokenizer;            // text -> ids (sentencepiece-kind vocabularies)
    std::string tokenizer_error;    // why the vocabulary cannot tokenize, if it cannot
    GrammarVocab grammar_vocab;     // every token's text as a grammar reads it; built by the first grammar row
    bool grammar_vocab_ready = false;

    bool is_eog(int32_t t) const { return (eos >= 0 && t == eos) || (eot >= 0 && t == eot); }
    // The bytes token t stands for, appended to `text`: SentencePiece's U+2581 becomes a space, a byte token
    // "<0xXX>" its byte, a piece of a byte-pair vocabulary the bytes it spells; control and unknown tokens
    // contribute their text only with unparse_special.
    void append_text(int32_t t, bool unparse_special, std::string & text) const {
        if (t < 0 || (size_t)t >= pieces.size()) return;
        const int32_t type = (size_t)t < types.size() ? types[(size_t)t] : 1;
        const std::string & piece = pieces[(size_t)t];
        if (type == 3 || type == 2) {            // control / unknown
            if (unparse_special) text += piece;
            return;
        }
        if (type == 6) {
            const int v = byte_piece_value(piece);
            if (v >= 0) { text.push_back((char)v); return; }
        }
        if (tokenizer.model == "gpt2") {
            text += tokenizer.spelled_bytes(piece);
            return;
        }
        for (size_t j = 0; j < piece.size();) {
            if (j + 2 < piece.size() && (unsigned char)piece[j] == 0xE2 && (unsigned char)piece[j + 1] == 0x96
                    && (unsigned char)piece[j + 2] == 0x81) {
                text.push_back(' ');
                j += 3;
            } else {
                text.push_back(piece[j++]);
            }
        }
    }
    const GrammarVocab & for_grammars(int32_t n_vocab) {
        if (!grammar_vocab_ready) {
            grammar_vocab = GrammarVocab();
            for (int32_t t = 0; t < n_vocab; ++t) {
                std::string text;
                append_text(t, true, text);
                grammar_vocab.add(text, is_eog(t));
            }
            grammar_vocab_ready = true;
        }
        return grammar_vocab;
    }
};

// Kernel categories of one step, for the optional event-based timing.
enum ProfCat : int {
    PC_PACK = 0, PC_EMBED, PC_NORM, PC_QKV, PC_ROPE, PC_ATTN, PC_COMBINE, PC_OPROJ, PC_GATEUP, PC_SWIGLU,
    PC_DOWN, PC_HEAD, PC_SAMPLE, PC_COUNT
};

class Engine {
public:
    Engine(const std::string & path, const retro_engine_config & config);
    ~Engine();

    // The step; `v2` rows or `v1` rows (exactly one non-null).
    int step(const retro_step_row_v2 * rows2, const retro_step_row * rows1, size_t n_rows,
             retro_step_out_row_v2 * out2, retro_step_out_row * out1,
             int32_t * out_top_ids, float * out_top_logprobs, size_t n_top_stride);

    bool seq_rm(int32_t slot, int32_t p0, int32_t p1);
    bool seq_cp(int32_t src, int32_t dst, int32_t p0, int32_t p1);
    int seq_save(int32_t slot, uint32_t flags, uint8_t * buffer, size_t n_buffer, size_t * out_n_bytes);
    int seq_load(int32_t slot, uint32_t flags, const uint8_t * buffer, size_t n_bytes, size_t * out_n_read);
    int seq_pos(int32_t slot, int32_t * out_min, int32_t * out_max);
    int memory(retro_engine_memory_info * out);
    void request_free(int32_t request) { requests_.erase(request); }

    // Batched generators over the step (generate.cpp; reference retro_gen_core.cpp:317-707, 1696-2049).
    int generate_batch(const int32_t * prompt_tokens, size_t n_prompt, const retro_sampling_params * sampling,
                       size_t n_sequences, int32_t * out_tokens, float * out_logprobs, size_t n_out_max,
                       size_t * out_n_tokens, uint8_t * out_forced);
    int generate_continuous_batch(const retro_generation_sequence * sequences, size_t n_sequences,
                                  int32_t * out_tokens, float * out_logprobs, size_t n_out_max,
                                  size_t * out_n_tokens, uint8_t * out_forced);
    int generate_continuous_batch_v2(const retro_generation_sequence_v2 * sequences, size_t n_sequences,
                                     int32_t * out_tokens, float * out_logprobs, size_t n_out_max,
                                     size_t * out_n_tokens, uint8_t * out_forced);
    const retro_generation_stats & generation_stats() const { return gen_cache_.stats; }
    // A step or a raw sequence operation issued by a caller mutates the KV outside the
    // continuous generator's protocol: what its slots hold is forgotten (retro_gen_core.cpp:2569,
    // 2795, 2813, 2875), the KV itself stays.
    void forget_generation_bookkeeping() { gen_cache_.forget(); }
    void clear_generation_memory();
    // Per-row LoRA adapters (reference retro_engine.cpp:872-960): ids start at 1
    // and are never reused; loading leaves the resident KV alone.
    int adapter_load(const std::string & path, float scale, int32_t * out_id);
    // Rows of token_embd.weight of a model file, read from its header alone.
    static uint64_t vocab_size_of(const std::string & path) {
        GgufFile file(path);
        return (uint64_t)file.require("token_embd.weight").ne[1];
    }
    // context-wide adapters, registered by name, one active
    int load_lora(const std::string & path);
    int load_lora_named(const std::string & name, const std::string & path);
    int activate_lora(const std::string & name);
    int set_lora_enabled(bool enabled);
    const std::string & active_adapter() const { return active_adapter_; }
    // the generation side of a trainer handle
    int policy_adapter_load(const std::string & path);
    bool has_policy_adapter() const { return row_adapters_.count(kPolicyAdapter) != 0; }
    int adapter_snapshot(int32_t replace, float scale, int32_t * out_id);
    int set_default_adapter(int32_t adapter);
    int32_t default_adapter() const { return default_adapter_; }
    void forget_generation_kv();
    int adapter_unload(int32_t id);
    void adapter_rows_info(retro_adapter_rows_info * out) const;

    const retro_engine_config & config() const { return cfg_; }
    const HParams & hparams() const { return hp_; }
    const Vocab & vocab() const { return vocab_; }
    uint32_t context_size() const { return (uint32_t)n_ctx_seq_; }
    uint64_t weights_version() const { return weights_version_; }
    uint64_t fingerprint() const { return fingerprint_; }
    uint64_t steps_run() const { return steps_run_; }

    // Event timing of kernel categories: level 0 off, 1 attention only, 2 all.
    void profile_level(int level) { prof_level_ = level; }
    // The decode attention launch of the middle layer leaves six clock values per workgroup while this is on;
    // read returns those of the last such launch ([workgroup][6]) and the number of workgroups.
    void attention_timeline(bool on);
    void single_token_matvec(bool on) { gemv_exact_ = on; }
    int attention_timeline_read(unsigned long long * out, size_t cap_workgroups, size_t * n_workgroups);
    void profile_read(double * ms, uint64_t * launches, bool reset);

    // Test hooks: copies of device state.
    int debug_last_logits(float * out, size_t n_floats, size_t * out_rows);
    int debug_read_kv(int layer, int32_t slot, int32_t pos, int want_v, uint16_t * out);
    int debug_pack(int32_t * tok, int32_t * pos, int32_t * seq, int32_t * cell, int32_t * out_index,
                   int32_t * last_index, size_t cap_tokens, size_t cap_rows, int32_t * counts);
    int debug_page_table(int32_t slot, int32_t * out, size_t cap, size_t * out_n);

private:
    struct RowView {      // the fields both row versions share
        int32_t request, slot;
        const int32_t * tokens;
        uint32_t n;
        int32_t pos0;
        bool sample;
        const retro_sampling_params_v2 * v2;
        retro_sampling_params v1;
        uint32_t n_top;
        bool want_logprob;
        int32_t adapter;
    };

    void load_model(const std::string & path);
    void upload_weight(const TensorInfo & t, int64_t K, int64_t N, const uint8_t * data, size_t bytes,
                       bool keep_raw, DevWeight & out);
    void upload_fused(const std::vector<const TensorInfo *> & parts, std::vector<DevWeight> & out);
    bool upload_gate_up_interleaved(const TensorInfo & g, const TensorInfo & u, std::vector<DevWeight> & out);
    void upload_f32(const TensorInfo * t, DevBuf & out, size_t expect);
    void upload_experts(const TensorInfo & t, int64_t K, int64_t N, DevWeight & out);
    void build_buffers();

    int32_t alloc_page();
    void release_page(int32_t page);
    void copy_page(int32_t src, int32_t dst);
    void set_page(int32_t slot, int idx, int32_t page);
    void clear_slot(Slot & s, int32_t slot);
    void forward(int T, int n_out, int n_tiles, int n_items, bool one_token_rows, bool routed);

    retro_engine_config cfg_ {};
    HParams hp_;
    Vocab vocab_;
    uint64_t fingerprint_ = 0;
    uint64_t weights_version_ = 0;
    uint64_t steps_run_ = 0;
    int n_ctx_seq_ = 0;
    int max_pages_ = 0;       // page indices per slot
    int n_pages_ = 0;         // pages in the pool
    int qt_ = 1;              // query tokens per attention tile
    rk::KvStrides kv_strides_ {};   // layout of every KV pool

    hipStream_t stream_ = nullptr;

    // weights
    DevWeight tok_embd_;      // raw rows, gathered per token
    DevWeight lm_head_;
    DevBuf out_norm_, out_bias_;
    std::vector<LayerWeights> layers_;
    DevBuf inv_freq_;         // double[rope_dim/2]

    // KV
    // One allocation for every layer's K and V pool (one large mapping instead of 2 x n_layer medium ones);
    // the per-layer pools are views into it.
    struct PoolView {
        void * ptr = nullptr;
        size_t bytes = 0;
        template <typename T> T * as() const { return (T *)ptr; }
    };
    DevBuf kv_slab_;
    std::vector<PoolView> k_pool_, v_pool_;   // per layer
    DevBuf table_;                          // int32 [n_seq_max][max_pages]
    std::vector<Slot> slots_;
    std::vector<int32_t> page_ref_;
    std::priority_queue<int32_t, std::vector<int32_t>, std::greater<int32_t>> free_pages_;
    // Device block-table entries that changed since the last step, keyed by
    // slot * max_pages + index so that only the LAST value of an entry is
    // uploaded: the packing kernel applies the list with one thread per entry,
    // in no particular order.
    std::unordered_map<int64_t, int32_t> pending_updates_;

    // per-step device buffers
    DevBuf d_stage_;          // rows | tokens | table updates, as uploaded
    HostPinned h_stage_;
    rk::PackBuffers pk_ {};
    std::vector<DevBuf> pk_store_;
    DevBuf x_, qkv_, gu_, q_half_, partial_, logits_, sample_k_, sample_out_, sample_scratch_, out_rows_idx_;
    DevBuf act_e_x_, act_e_sums_;       // n_embd wide
    DevBuf act_q_x_, act_q_sums_;       // n_head * head_dim wide
    DevBuf act_f_x_, act_f_sums_;       // n_ff wide
    DevBuf act_o_x_, act_o_sums_;       // output rows, n_embd wide
    // the same rows after the conversion ggml's CPU matmul applies for a quantised weight
    DevBuf act_e_qx_, act_e_qsums_, act_q_qx_, act_q_qsums_, act_f_qx_, act_f_qsums_, act_o_qx_, act_o_qsums_;
    // ggml arithmetic only: the Q8_K / Q8_0 blocks themselves (codes, scales, block sums) of steps of at most
    // rk::GEMV_MAX_T tokens, for the integer matrix-vector kernel
    struct ActCodes { DevBuf codes, d, bsums; };
    ActCodes act_e_codes_, act_q_codes_, act_f_codes_, act_o_codes_;
    int gemv_max_t_ = rk::GEMV_MAX_T;
    bool fused_decode_attention_ = true;     // pure decode steps: rotation, KV store, attention and split merge in one launch (RETRO_FUSED_DECODE_ATTENTION=0: the three kernels)
    int32_t step_max_resident_ = 0;          // longest resident span (positions) among the rows of the step being run
    int merge_max_splits_ = 8;       // about a 1,000-token context: beyond it the merge kernel's own launch is cheaper
    bool gemv_fuse_ = true;      // small steps: the integer kernel makes its Q8_K blocks from the f32 rows itself where it can
    // Single-token steps of the exact arithmetic on the matrix-vector kernel with f32 rows (RETRO_GEMV_EXACT=1). Off by
    // default: its sums are added in another order than the tile kernels', so a sequence decoded alone would no longer
    // give bit for bit the logprobs it gives inside a batch - a relation the reference's tests hold
    // (tests/engine_runtime.rs:713-722).
    bool gemv_exact_ = false;
    DevBuf q_half_lo_;
    DevBuf item_meta_;        // the step's attention work items (PackBuffers::item_a, item_b), grown as needed
    DevBuf mm_ws_;            // matmul workspace: split-K partials, counters
    // mixture-of-experts scratch (allocated for MoE models only)
    DevBuf moe_logits_, moe_sel_, moe_wgt_, moe_n_, moe_off_, moe_tok_, moe_q_, moe_h_, moe_out_, moe_pair_;
    HostPinned h_sample_, h_logits_;
    int last_n_out_ = 0;

    // event timing
    struct ProfSpan { int cat; size_t a, b; };
    int prof_level_ = 0;
    DevBuf attn_stamps_;
    bool attn_timeline_ = false;
    size_t attn_stamped_wgs_ = 0;
    std::vector<hipEvent_t> prof_events_;
    size_t prof_used_ = 0;
    std::vector<ProfSpan> prof_spans_;
    double prof_ms_[PC_COUNT] = {};
    uint64_t prof_n_[PC_COUNT] = {};
    size_t prof_begin(int cat);
    int kv_q8_ = 0;            // rk::KV_F16, or KV_Q8 / KV_Q4: the KV pools hold Q8_0 / Q4_0 blocks (kv_dtype)
    uint32_t snap_magic() const;
    void prof_end(int cat, size_t token);
    void prof_resolve();

    // per-row adapters: targets attn_q, attn_k, attn_v, attn_output of every layer
    static constexpr int kLoraTargets = 7;      // attn_q, attn_k, attn_v, attn_output, ffn_gate, ffn_up, ffn_down
    bool lora_has_ffn_ = false;                 // some loaded adapter holds a pair for a feed-forward matrix
    struct RowAdapterData {
        float scale = 1.0f;
        double alpha = 0.0;
        int rank = 0;
        uint64_t elements = 0;                     // sum over pairs of (n_in + n_out)
        std::vector<DevBuf> a, b;                  // [layer * kLoraTargets + target], empty when the pair is absent
        std::vector<int32_t> a_type, b_type;       // storage types in the adapter file, same index
    };
    std::map<int32_t, RowAdapterData> row_adapters_;
    int32_t next_adapter_id_ = 1;
    DevBuf lora_table_;       // LoraEntry [layer][target][route - 1]
    DevBuf lora_mid_;         // [n_batch][LORA_MAX_RANK] f32
    int lora_routes_ = 0;
    bool ggml_activations_ = false;   // RETRO_ACTIVATIONS=ggml at construction
    bool moe_scaled_ = false;         // RETRO_MOE_SCALED=1: decode-sized steps multiply MXFP4 experts on the block-scaled matrix
                                      // instruction (measured slower than the f16 tile kernels end to end, so it is off by default)
    DevBuf moe_mx_ops_, moe_mx_scales_, moe_mx_h_;
    size_t moe_mx_slots_ = 0;
    void rebuild_lora_table();
    int read_adapter(const std::string & path, float scale, RowAdapterData & data);
    RowAdapterData clone_adapter(const RowAdapterData & src, float scale);
    void apply_active_adapter();
    std::map<std::string, RowAdapterData> named_adapters_;
    std::string active_adapter_;
    // id of the trained adapter among the per-row adapters: never handed out, never accepted from a caller
    static constexpr int32_t kPolicyAdapter = INT32_MAX;
    int32_t default_adapter_ = 0;
    const rk::LoraEntry * lora_entries(int layer, int target) const {
        return lora_table_.as<rk::LoraEntry>() + ((size_t)layer * kLoraTargets + target) * (size_t)lora_routes_;
    }

    std::map<int32_t, RequestState> requests_;

    // What the continuous generator's slots hold between calls (reference retro_runtime.hpp:244-263).
    struct GenCache {
        std::vector<std::vector<int32_t>> slots;   // resident tokens per slot
        std::vector<uint64_t> used_at;             // last call that extended the slot
        uint64_t clock = 0;
        retro_generation_stats stats {};
        void forget();
    };
    GenCache gen_cache_;
    bool gen_validate_sampling(const retro_sampling_params & s);
    bool gen_validate_tokens(const int32_t * tokens, size_t n);
    bool gen_prefill(int32_t slot, const int32_t * tokens, size_t p0, size_t p1);
    // how a generator's sequence samples: exactly one of the two is set
    struct GenSampling { const retro_sampling_params * v1 = nullptr; const retro_sampling_params_v2 * v2 = nullptr; };
    struct GenRow { size_t seq; int32_t slot; const int32_t * tokens; uint32_t n; int32_t pos0; bool sample; };
    int gen_sample_rows(const std::vector<GenRow> & specs, const std::vector<GenSampling> & sampling,
                        std::vector<retro_step_out_row> & outs);
    int generate_continuous_impl(const retro_generation_sequence * sequences, const std::vector<GenSampling> & sampling,
                                 const std::vector<uint32_t> & max_new, size_t n_sequences,
                                 int32_t * out_tokens, float * out_logprobs, size_t n_out_max,
                                 size_t * out_n_tokens, uint8_t * out_forced);
    int gen_decode_loop(const std::vector<size_t> & order, const std::vector<int32_t> & slot_of,
                        const std::vector<size_t> & n_prompt_of, const std::vector<GenSampling> & sampling,
                        const std::vector<size_t> & limits, std::vector<retro_step_out_row> produced,
                        int32_t * out_tokens, float * out_logprobs, size_t n_out_max, size_t * out_n_tokens,
                        uint8_t * out_forced);
    sampling::FullScratch scratch_;
};

}  // namespace retro

// The v2 sampling parameters' checks (engine.cpp), shared by the step and the v2 generator.
namespace retro { bool valid_sampling_v2(const retro_sampling_params_v2 & s, int32_t n_vocab); }

// The opaque handle of the C ABI.
struct retro_engine {
    retro::Engine impl;
    retro_engine(const std::string & path, const retro_engine_config & config) : impl(path, config) {}
};
