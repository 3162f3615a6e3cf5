#pragma once

#include <vector>

#include "../../../include/retro_step.h"
#include "types.hpp"

namespace sched {

// Borrows the engine handle: the caller keeps it alive and frees it.
class EngineBackend : public DecodeBackend {
public:
    explicit EngineBackend(retro_engine * engine) : engine_(engine) {}
    void step(const std::vector<StepRow> & rows, StepOutput & out) override;
    void seq_rm(int32_t slot, int32_t p0, int32_t p1) override;
    void seq_cp(int32_t src, int32_t dst, int32_t p0, int32_t p1) override;
    std::pair<int32_t, int32_t> seq_pos(int32_t slot) override;
    size_t seq_save_len(int32_t slot, uint32_t flags) override;
    size_t seq_save_into(int32_t slot, uint32_t flags, uint8_t * buffer, size_t n) override;
    size_t seq_load(int32_t slot, uint32_t flags, const uint8_t * data, size_t n) override;
    bool kv_unified() override;
    uint64_t weights_version() override;
    uint64_t model_fingerprint() override;
    bool is_hybrid() override;
    EngineMemory memory() override;
    void request_free(int32_t request) override;
    bool is_eog_token(int32_t token) override;
    std::string detokenize_bytes(const int32_t * tokens, size_t n, bool unparse_special) override;
    uint32_t context_size() override;
    uint32_t vocab_size() override;
    void load_adapter(const std::string & name, const std::string & path) override;
    void activate_adapter(const std::optional<std::string> & name) override;
    std::optional<std::string> active_adapter() override;
    bool supports_row_adapters() override { return true; }
    int32_t load_row_adapter(const std::string & path, float scale) override;
    void unload_row_adapter(int32_t id) override;
    AdapterRowsInfo adapter_rows_info() override;

private:
    retro_engine * engine_;
    std::vector<retro_step_row_v2> ffi_rows_;
    std::vector<retro_step_out_row_v2> ffi_out_;
    std::vector<int32_t> bias_ids_;
    std::vector<float> bias_values_;
};

}  // namespace sched
