"""ABI lane (no model, no GPU): struct sizes/alignments/offsets of the C header
against the values the reference pins in its own ABI test
(reference crates/retrograd-ffi/src/lib.rs:2899-2914, 2983-3058), the ctypes
mirrors against the same numbers, and every symbol the headers declare is
exported by the built library."""
import ctypes as C
import re
import subprocess
from pathlib import Path

import pytest

from retrograd_amd import engine as E
from retrograd_amd import trainer as T

ROOT = Path(__file__).resolve().parent.parent

# (struct, size, align, {field: offset})
EXPECT = [
    ("retro_sampling_params", 16, 4, {"max_new_tokens": 8}),
    ("retro_step_row", 64, 8, {"struct_size": 0, "request": 4, "slot": 8, "tokens": 16, "n": 24, "pos0": 28,
                               "sample": 32, "sampling": 36, "n_top_logprobs": 52, "adapter": 56}),
    ("retro_adapter_rows_info", 32, 8, {"max_rank": 8, "stacked_bytes": 16, "unpadded_bytes": 24}),
    ("retro_step_out_row", 20, 4, {"struct_size": 0, "token": 4, "logprob": 8, "n_top": 12, "forced": 16, "sampled": 17}),
    ("retro_sampling_params_v2", 72, 8, {"struct_size": 0, "temperature": 4, "top_p": 8, "max_new_tokens": 12,
                                         "seed": 16, "top_k": 20, "min_p": 24, "repeat_penalty": 28,
                                         "frequency_penalty": 32, "presence_penalty": 36, "penalty_window": 40,
                                         "n_logit_bias": 44, "logit_bias_ids": 48, "logit_bias_values": 56,
                                         "grammar": 64}),
    ("retro_step_row_v2", 128, 8, {"struct_size": 0, "request": 4, "slot": 8, "tokens": 16, "n": 24, "pos0": 28,
                                   "sample": 32, "sampling": 40, "n_top_logprobs": 112, "want_logprob": 116,
                                   "adapter": 120}),
    ("retro_step_out_row_v2", 24, 4, {"struct_size": 0, "token": 4, "logprob": 8, "n_top": 12, "forced": 16,
                                      "sampled": 17, "sampled_logprob": 20}),
    ("retro_engine_memory_info", 40, 8, {"struct_size": 0, "n_slots": 4, "cells_total": 8, "cells_used": 16,
                                         "kv_bytes": 24, "recurrent_bytes": 32}),
    # the reference's own layout assertions for RetroTrainConfig (crates/retrograd-ffi/src/lib.rs:2835-2880)
    ("retro_train_config", 176, 8, {"generation_concurrency": 16, "kv_dtype": 24, "learning_rate": 36, "warmup_steps": 56,
                                    "device": 68, "chunked_ce_seq_chunk": 80, "chunked_ce_offload_logsoftmax": 84,
                                    "checkpoint_every_n_layers": 88, "checkpoint_dtype": 92, "require_gpu_resident": 96,
                                    "generation_batch": 100, "shuffle_dataset": 104, "optimizer": 108,
                                    "shuffle_seed": 112, "trainable": 120, "muon_momentum": 124, "muon_ns_steps": 136,
                                    "muon_nesterov": 140, "gefen_variant": 144}),
    ("retro_engine_config", 64, 8, {"struct_size": 0, "n_ctx": 4, "n_seq_max": 8, "n_batch": 12, "n_ubatch": 16,
                                    "kv_dtype": 20, "flash_attn": 24, "device": 28, "threads": 32, "verbose": 36,
                                    "kv_unified": 40, "expert_placement": 44, "expert_host_layers": 48,
                                    "expert_device_cache_bytes": 56}),
]

CTYPES = {
    "retro_sampling_params": E.CSamplingParams, "retro_step_row": E.CStepRow,
    "retro_adapter_rows_info": E.CAdapterRowsInfo, "retro_step_out_row": E.CStepOutRow,
    "retro_sampling_params_v2": E.CSamplingParamsV2, "retro_step_row_v2": E.CStepRowV2,
    "retro_step_out_row_v2": E.CStepOutRowV2, "retro_engine_memory_info": E.CEngineMemoryInfo,
    "retro_engine_config": E.CEngineConfig, "retro_train_config": T.CTrainConfig,
}


def test_c_header_layout_matches_the_reference_abi(tmp_path):
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "retro_step.h"', '#include "retro_trainer.h"',
             "int main(void) {"]
    for name, size, align, fields in EXPECT:
        lines.append('printf("%s %%zu %%zu\\n", sizeof(%s), _Alignof(%s));' % (name, name, name))
        for f in fields:
            lines.append('printf("%s.%s %%zu\\n", offsetof(%s, %s));' % (name, f, name, f))
    lines += ['printf("consts %d %u %u %u\\n", RETRO_STEP_ADAPTER_BASE, RETRO_STATE_SEQ_FLAGS_NONE, '
              'RETRO_STATE_SEQ_FLAGS_PARTIAL_ONLY, RETRO_STATE_SEQ_FLAGS_ON_DEVICE);', "return 0; }"]
    src = tmp_path / "abi.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "abi"
    subprocess.run(["gcc", "-std=c11", "-I", str(ROOT / "include"), str(src), "-o", str(exe)], check=True)
    got = {}
    for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines():
        k, *v = line.split()
        got[k] = [int(x) for x in v]
    for name, size, align, fields in EXPECT:
        assert got[name] == [size, align], name
        for f, off in fields.items():
            assert got[name + "." + f] == [off], (name, f)
    assert got["consts"] == [-1, 0, 1, 2]


@pytest.mark.parametrize("name,size,align,fields", EXPECT)
def test_ctypes_mirrors_match(name, size, align, fields):
    ct = CTYPES[name]
    assert C.sizeof(ct) == size and C.alignment(ct) == align
    for f, off in fields.items():
        assert getattr(ct, f).offset == off, (name, f)


def _declared(header: Path):
    text = re.sub(r"/\*.*?\*/", "", header.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(retro_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = E.load_library()
    step = _declared(ROOT / "include" / "retro_step.h")
    kern = [s for s in _declared(ROOT / "include" / "retro_kernels.h") if s not in step]
    sched = [s for s in _declared(ROOT / "include" / "retro_scheduler.h") if s not in step]
    from retrograd_amd import scheduler as S
    trainer = [s for s in _declared(ROOT / "include" / "retro_trainer.h") if s not in step]
    assert sorted(trainer) == sorted(T.TRAINER_SYMBOLS)
    for sym in trainer:
        assert hasattr(lib, sym), sym
    assert sorted(step) == sorted(E.STEP_SYMBOLS)
    assert sorted(kern) == sorted(E.KERNEL_SYMBOLS)
    assert sorted(sched) == sorted(S.SCHED_SYMBOLS)
    for sym in step + kern + sched:
        assert hasattr(lib, sym), sym


def test_error_string_defaults_and_argument_checks_without_a_device():
    lib = E.load_library()
    # every entry point clears the thread's error first; a null handle is a
    # runtime failure with a message (reference retro_engine.cpp:76-82)
    assert lib.retro_engine_seq_rm(None, 0, -1, -1) == -1
    assert E.last_error() == "engine is required"
    assert lib.retro_engine_new(None, None) is None
    assert E.last_error() == "model_path is required"
    cfg = E.EngineConfig(n_ctx=0).to_ffi()
    assert lib.retro_engine_new(b"/nonexistent.gguf", C.byref(cfg)) is None
    assert E.last_error() == "engine n_ctx and n_seq_max must be greater than zero"
    cfg = E.EngineConfig(n_batch=8, n_ubatch=16).to_ffi()
    assert lib.retro_engine_new(b"/nonexistent.gguf", C.byref(cfg)) is None
    assert E.last_error() == "engine n_ubatch must be in (0, n_batch]"
    cfg = E.EngineConfig(n_seq_max=257, n_batch=512).to_ffi()
    assert lib.retro_engine_new(b"/nonexistent.gguf", C.byref(cfg)) is None
    assert "n_seq_max must not exceed" in E.last_error()
    cfg = E.EngineConfig(device=E.DEVICE_CPU).to_ffi()
    assert lib.retro_engine_new(b"/nonexistent.gguf", C.byref(cfg)) is None
    assert "only executes on an MI355X" in E.last_error()
    cfg = E.EngineConfig().to_ffi()
    cfg.struct_size = 16   # older than the oldest layout the reference accepts
    assert lib.retro_engine_new(b"/nonexistent.gguf", C.byref(cfg)) is None
    assert E.last_error() == "retro_engine_config.struct_size is too small for this build"
    g = lib.retro_grammar_from_gbnf(b'root ::= "a"')
    assert g and lib.retro_grammar_gbnf(g) == b'root ::= "a"'
    lib.retro_grammar_free(g)
    assert lib.retro_grammar_from_gbnf(b"") is None and E.last_error() == "gbnf is required"
    # the timing entry point hands its buffer to the tile kernels as Q4_K, Q6_K or Q8_0 tiles: any other type, or a
    # shape that is not whole tiles, would be read out of bounds and is refused before anything is allocated
    for args in ((39, 1024, 4096, 1), (1, 1024, 4096, 1), (12, 1000, 4096, 1), (14, 1024, 4000, 1), (8, 1024, 4096, 0)):
        with pytest.raises(E.EngineError):
            E.kernel_matmul_time(*args)
        assert "matmul_time" in E.last_error()


def test_engine_creation_fails_loudly_without_a_gpu(tmp_path):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from retrograd_amd import synth
    p = tmp_path / "m.gguf"
    synth.write_model(p, synth.TINY_LLAMA, seed=0, device="cpu")
    with pytest.raises(E.RuntimeFailure) as err:
        E.Engine(p)
    assert "no HIP device" in str(err.value) or "HIP" in str(err.value)


def test_trainer_creation_checks_its_configuration_and_fails_loudly_without_a_gpu(tmp_path):
    from retrograd_amd import synth
    lib = T._library()
    cfg = T.TrainConfig(n_ctx=64, n_batch=64, generation_concurrency=0).to_ffi()
    assert not lib.retro_trainer_new(b"/nonexistent.gguf", C.byref(cfg))
    assert E.last_error() == "generation_concurrency must be between 1 and 256"
    cfg = T.TrainConfig(n_ctx=64, n_batch=8, generation_concurrency=16).to_ffi()
    assert not lib.retro_trainer_new(b"/nonexistent.gguf", C.byref(cfg))
    assert E.last_error() == "generation_concurrency must not exceed n_batch"
    cfg = T.TrainConfig(n_ctx=64, n_batch=64, generation_kv_dtype=1, fast_generation_context=False).to_ffi()
    assert not lib.retro_trainer_new(b"/nonexistent.gguf", C.byref(cfg))
    assert E.last_error() == "a quantized generation_kv_dtype requires fast_generation_context"
    cfg = T.TrainConfig(n_ctx=64, n_batch=64, device=E.DEVICE_CPU).to_ffi()
    assert not lib.retro_trainer_new(b"/nonexistent.gguf", C.byref(cfg))
    assert "only executes on an MI355X GPU" in E.last_error()
    assert not lib.retro_trainer_new(None, C.byref(cfg)) and E.last_error() == "model_path is required"
    out = C.c_uint64()
    assert lib.retro_trainer_generation_weights_version(None, C.byref(out)) == -1
    assert E.last_error() == "trainer is required"
    import torch
    if not torch.cuda.is_available():
        path = tmp_path / "m.gguf"
        synth.write_model(path, synth.TINY_LLAMA, seed=1, device="cpu", std=0.02)
        with pytest.raises(E.RuntimeFailure, match="no HIP device"):
            T.Trainer(path, T.TrainConfig(n_ctx=64, n_batch=64, generation_concurrency=2))
