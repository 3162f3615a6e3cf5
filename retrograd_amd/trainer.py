"""Host-side mirror of the generation side of the reference's `Trainer`
(crates/retrograd-engine: Trainer::step, seq_*, memory, generate_batch,
generate_sampled_continuous, generation_adapter_snapshot ...; driven by
crates/retrograd-infer/src/backend.rs:376-461) over include/retro_trainer.h.

A Trainer is used exactly like an Engine: every method of Engine that has a
`retro_trainer_*` twin is inherited and reaches the library through that twin."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

from . import engine as E

_i32p = C.POINTER(C.c_int32)


class CTrainConfig(C.Structure):
    """retro_train_config (reference retro_lora_train.h:944-1059)."""
    _fields_ = [
        ("n_ctx", C.c_uint32), ("n_batch", C.c_uint32), ("n_ubatch", C.c_uint32), ("n_seq_max", C.c_uint32),
        ("generation_concurrency", C.c_uint32), ("fast_generation_context", C.c_bool), ("kv_dtype", C.c_int32),
        ("threads", C.c_uint32), ("epochs", C.c_uint32), ("learning_rate", C.c_float), ("weight_decay", C.c_float),
        ("max_grad_norm", C.c_float), ("lr_scheduler", C.c_int32), ("warmup_steps", C.c_uint64), ("verbose", C.c_bool),
        ("device", C.c_int32), ("chunked_cross_entropy", C.c_bool), ("chunked_ce_tiles", C.c_uint32),
        ("chunked_ce_seq_chunk", C.c_uint32), ("chunked_ce_offload_logsoftmax", C.c_bool),
        ("gradient_checkpointing", C.c_bool), ("checkpoint_every_n_layers", C.c_uint32), ("checkpoint_dtype", C.c_int32),
        ("require_gpu_resident", C.c_bool), ("generation_batch", C.c_uint32), ("shuffle_dataset", C.c_bool),
        ("optimizer", C.c_int32), ("shuffle_seed", C.c_uint64), ("trainable", C.c_int32), ("muon_momentum", C.c_float),
        ("muon_ns_epsilon", C.c_float), ("muon_fallback_learning_rate", C.c_float), ("muon_ns_steps", C.c_uint32),
        ("muon_nesterov", C.c_bool), ("gefen_variant", C.c_int32), ("gefen_block_size", C.c_uint32),
        ("gefen_beta1", C.c_float), ("gefen_beta2", C.c_float), ("gefen_eps", C.c_float), ("master_weights", C.c_int32),
        ("generation_kv_dtype", C.c_int32),
    ]


# engine entry point -> its twin on the trainer handle
TWINS = {
    "retro_engine_step": "retro_trainer_generation_step",
    "retro_engine_step_v2": "retro_trainer_generation_step_v2",
    "retro_engine_seq_rm": "retro_trainer_generation_seq_rm",
    "retro_engine_seq_cp": "retro_trainer_generation_seq_cp",
    "retro_engine_seq_save": "retro_trainer_generation_seq_save",
    "retro_engine_seq_load": "retro_trainer_generation_seq_load",
    "retro_engine_seq_pos": "retro_trainer_generation_seq_pos",
    "retro_engine_memory": "retro_trainer_generation_memory",
    "retro_engine_request_free": "retro_trainer_generation_request_free",
    "retro_engine_kv_unified": "retro_trainer_generation_kv_unified",
    "retro_engine_weights_version": "retro_trainer_generation_weights_version",
    "retro_engine_model_fingerprint": "retro_trainer_model_fingerprint",
    "retro_engine_is_hybrid": "retro_trainer_is_hybrid",
    "retro_engine_eos_token": "retro_trainer_eos_token",
    "retro_engine_vocab_size": "retro_trainer_vocab_size",
    "retro_engine_is_eog_token": "retro_trainer_is_eog_token",
    "retro_engine_context_size": "retro_trainer_context_size",
    "retro_engine_detokenize": "retro_trainer_detokenize",
    "retro_engine_tokenize_text": "retro_trainer_tokenize_text",
    "retro_engine_tokenize_fragment": "retro_trainer_tokenize_fragment",
    "retro_engine_tokenize": "retro_trainer_tokenize_with",
    "retro_engine_generate_batch": "retro_trainer_generate_batch",
    "retro_engine_generate_continuous_batch": "retro_trainer_generate_continuous_batch",
    "retro_engine_generation_stats": "retro_trainer_generation_stats",
    "retro_engine_adapter_unload": "retro_trainer_generation_adapter_unload",
    "retro_engine_adapter_rows_info": "retro_trainer_generation_adapter_rows_info",
}
TRAINER_SYMBOLS = sorted(set(TWINS.values()) | {
    "retro_trainer_new", "retro_trainer_free", "retro_trainer_load_lora", "retro_trainer_generation_adapter_snapshot",
    "retro_trainer_get_generation_adapter", "retro_trainer_set_generation_adapter",
    "retro_trainer_generate_continuous_batch_v2"})

_ready = False


def _library() -> C.CDLL:
    global _ready
    lib = E.load_library()
    if not _ready:
        lib.retro_trainer_new.restype = C.c_void_p
        lib.retro_trainer_new.argtypes = [C.c_char_p, C.POINTER(CTrainConfig)]
        lib.retro_trainer_free.restype = None
        lib.retro_trainer_free.argtypes = [C.c_void_p]
        lib.retro_trainer_load_lora.argtypes = [C.c_void_p, C.c_char_p]
        lib.retro_trainer_generation_adapter_snapshot.argtypes = [C.c_void_p, C.c_int32, C.c_float, _i32p]
        lib.retro_trainer_get_generation_adapter.argtypes = [C.c_void_p, _i32p]
        lib.retro_trainer_set_generation_adapter.argtypes = [C.c_void_p, C.c_int32]
        lib.retro_trainer_generate_continuous_batch_v2.argtypes = [
            C.c_void_p, C.POINTER(E.CGenerationSequenceV2), C.c_size_t, _i32p, C.POINTER(C.c_float), C.c_size_t,
            C.POINTER(C.c_size_t), C.POINTER(C.c_uint8)]
        for engine_name, twin in TWINS.items():
            getattr(lib, twin).argtypes = getattr(lib, engine_name).argtypes
        _ready = True
    return lib


class _Twins:
    """The library as an Engine sees it, with every engine entry point replaced by its trainer twin."""

    def __init__(self, lib: C.CDLL) -> None:
        self._lib = lib

    def __getattr__(self, name: str):
        if name.startswith("retro_engine_") and name not in TWINS:
            raise E.EngineError("%s has no twin on the trainer handle" % name)
        return getattr(self._lib, TWINS.get(name, name))


@dataclass
class TrainConfig:
    """The fields of retro_train_config the generation side reads; the rest keep the reference's
    defaults (retro_runtime.cpp:91-125)."""
    n_ctx: int = 128
    n_batch: int = 128
    generation_concurrency: int = 1
    fast_generation_context: bool = True
    generation_batch: int = 0
    device: int = E.DEVICE_AUTO
    generation_kv_dtype: int = 0

    def to_ffi(self) -> CTrainConfig:
        c = CTrainConfig()
        c.n_ctx, c.n_batch, c.n_ubatch, c.n_seq_max = self.n_ctx, self.n_batch, min(32, self.n_batch), 1
        c.generation_concurrency, c.fast_generation_context = self.generation_concurrency, self.fast_generation_context
        c.kv_dtype, c.threads, c.epochs, c.learning_rate, c.weight_decay, c.max_grad_norm = 0, 0, 1, 1e-4, 0.0, 1.0
        c.device, c.chunked_ce_tiles, c.checkpoint_every_n_layers = self.device, 8, 1
        c.generation_batch, c.shuffle_dataset, c.shuffle_seed = self.generation_batch, True, 42
        c.generation_kv_dtype = self.generation_kv_dtype
        return c


class Trainer(E.Engine):
    def __init__(self, model_path, config: TrainConfig | None = None) -> None:
        lib = _library()
        self._lib = _Twins(lib)
        cfg = (config or TrainConfig()).to_ffi()
        self._h = lib.retro_trainer_new(str(model_path).encode(), C.byref(cfg))
        if not self._h:
            raise E.RuntimeFailure(E.last_error())

    def close(self) -> None:
        if getattr(self, "_h", None):
            self._lib.retro_trainer_free(self._h)
            self._h = None

    def load_lora(self, path) -> None:
        """The trained adapter, from a LoRA adapter file: a weight change (the generation KV is dropped,
        the weights version moves on)."""
        s = self._lib.retro_trainer_load_lora(self._h, str(path).encode())
        if s != 0:
            E._raise(s)

    def generate_continuous_v2(self, sequences, n_out_max: int | None = None):
        """retro_trainer_generate_continuous_batch_v2 over (prompt, SamplingParamsV2) pairs (a grammar text among the
        parameters constrains the row). Returns [(tokens, logprobs, forced)] in input order."""
        import numpy as np
        n = len(sequences)
        n_out_max = n_out_max or max(p.max_new_tokens for _, p in sequences)
        keep = [np.ascontiguousarray(prompt, dtype=np.int32) for prompt, _ in sequences]
        ffi = (E.CGenerationSequenceV2 * n)()
        for i, (_, p) in enumerate(sequences):
            ffi[i].prompt_tokens = keep[i].ctypes.data_as(_i32p)
            ffi[i].n_prompt = keep[i].size
            self._fill_sampling_v2(ffi[i].sampling, p, keep)
        toks = np.zeros((n, n_out_max), np.int32)
        lps = np.zeros((n, n_out_max), np.float32)
        forced = np.zeros((n, n_out_max), np.uint8)
        counts = (C.c_size_t * n)()
        status = self._lib.retro_trainer_generate_continuous_batch_v2(
            self._h, ffi, n, toks.ctypes.data_as(_i32p), lps.ctypes.data_as(C.POINTER(C.c_float)), n_out_max, counts,
            forced.ctypes.data_as(C.POINTER(C.c_uint8)))
        if status != 0:
            E._raise(status)
        return self._collect(n, n_out_max, toks, lps, list(counts), forced)

    def generation_adapter_snapshot(self, replace: int = 0, scale: float = 1.0) -> int:
        out = C.c_int32()
        s = self._lib.retro_trainer_generation_adapter_snapshot(self._h, replace, scale, C.byref(out))
        if s != 0:
            E._raise(s)
        return out.value

    def generation_adapter_unload(self, adapter_id: int) -> None:
        self.adapter_unload(adapter_id)

    def generation_adapter(self) -> int:
        out = C.c_int32()
        s = self._lib.retro_trainer_get_generation_adapter(self._h, C.byref(out))
        if s != 0:
            E._raise(s)
        return out.value

    def set_generation_adapter(self, adapter: int) -> None:
        s = self._lib.retro_trainer_set_generation_adapter(self._h, adapter)
        if s != 0:
            E._raise(s)
