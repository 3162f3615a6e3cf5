// A deterministic in-memory DecodeBackend for tests of the policy that need no
// model (reference crates/retrograd-infer/src/fake.rs:22-575): slot spans in a
// fixed-size cell pool, a sampler that is a pure function of the request id and
// the number of tokens already generated, a piece table, and a log of every
// step, copy and removal.
#pragma once

#include <array>
#include <map>
#include <optional>
#include <string>
#include <unordered_map>
#include <vector>

#include "types.hpp"

namespace sched {

class FakeBackend : public DecodeBackend {
public:
    FakeBackend(uint32_t n_slots, uint32_t n_ctx_seq, uint64_t cells_total, uint32_t vocab, int32_t eos,
                std::vector<std::string> pieces);

    // script
    std::optional<size_t> eog_after;          // emit the EOG token after this many generated tokens of a request
    std::vector<int32_t> script;              // non-empty: sampling returns these tokens in order (per request)
    bool unified = true;
    bool recurrent = false;
    uint64_t version = 0;
    uint64_t fingerprint = 0xFACE;
    bool row_adapters_enabled = false;
    int fail_after_steps = -1;                // >= 0: that many more steps succeed, then one reports a backend failure
                                              // after committing (a partial decode failure)

    // log
    struct RowLog { int32_t slot; uint32_t n; int32_t request; };   // request = -1 on non-sampling rows
    std::vector<std::vector<RowLog>> steps;
    std::vector<std::vector<RowAdapter>> step_adapters;
    std::vector<std::array<int32_t, 4>> copies;
    std::vector<int32_t> removed;
    std::vector<int32_t> request_order;
    struct StateLog { int32_t slot; uint32_t flags; size_t len; };
    std::vector<StateLog> saves, loads;
    std::vector<std::pair<std::string, std::string>> adapter_ops;   // (op, name or "")

    void bump_weights_version() { version += 1; }
    void register_adapter(const std::string & name, const std::string & path);
    void apply_adapter(const std::optional<std::string> & name);

    void step(const std::vector<StepRow> & rows, StepOutput & out) override;
    void seq_rm(int32_t slot, int32_t p0, int32_t p1) override;
    void seq_cp(int32_t src, int32_t dst, int32_t p0, int32_t p1) override;
    std::pair<int32_t, int32_t> seq_pos(int32_t slot) override;
    size_t seq_save_len(int32_t slot, uint32_t flags) override;
    size_t seq_save_into(int32_t slot, uint32_t flags, uint8_t * buffer, size_t n) override;
    size_t seq_load(int32_t slot, uint32_t flags, const uint8_t * data, size_t n) override;
    bool kv_unified() override { return unified; }
    uint64_t weights_version() override { return version; }
    uint64_t model_fingerprint() override { return fingerprint; }
    bool is_hybrid() override { return recurrent; }
    KvCacheKey cache_key() override { return KvCacheKey{fingerprint, version, unified ? 1u : 0u}; }
    EngineMemory memory() override;
    void request_free(int32_t request) override { requests_.erase(request); }
    bool is_eog_token(int32_t token) override { return token == eos_; }
    std::string detokenize_bytes(const int32_t * tokens, size_t n, bool unparse_special) override;
    uint32_t context_size() override { return n_ctx_seq_; }
    uint32_t vocab_size() override { return vocab_; }
    void load_adapter(const std::string & name, const std::string & path) override;
    void activate_adapter(const std::optional<std::string> & name) override { apply_adapter(name); }
    std::optional<std::string> active_adapter() override { return active_adapter_; }
    bool supports_row_adapters() override { return row_adapters_enabled; }
    int32_t load_row_adapter(const std::string & path, float scale) override;
    void unload_row_adapter(int32_t id) override;

private:
    uint64_t cells_used() const;
    int32_t sample_token(int32_t request, size_t generated) const;
    std::optional<std::vector<uint8_t>> encode_snapshot(int32_t slot, uint32_t flags) const;

    uint32_t n_slots_, n_ctx_seq_;
    uint64_t cells_total_;
    uint32_t vocab_;
    int32_t eos_;
    std::vector<std::string> pieces_;
    std::vector<std::optional<std::pair<int32_t, int32_t>>> slots_;
    std::unordered_map<int32_t, size_t> requests_;
    std::map<std::string, std::string> adapters_;
    std::optional<std::string> active_adapter_;
    std::map<int32_t, std::string> row_adapters_;
    int32_t next_row_adapter_ = 1;
};

}  // namespace sched
