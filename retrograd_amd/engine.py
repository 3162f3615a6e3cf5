"""Host-side mirror of the reference's safe engine API over libretro_hip.so.

Same names and meaning as reference crates/retrograd-engine/src/step.rs
(`StepRow` :93-106, `StepOutRow` :208-221, `StepOutput` :256-263, `RowAdapter`
:61-80, `EngineMemory` :225-238) and crates/retrograd-engine/src/engine/step.rs
:19-189 (`Engine::step`, `seq_rm`, `seq_cp`, `seq_pos`, `seq_save*`,
`seq_load`, `memory`, `request_free`). Status -3 maps to `InvalidArgument`, any
other non-zero status to `RuntimeFailure(last_error)` (step.rs:497-502).

The library is loaded with ctypes; there is no fallback: a missing library or a
machine without a HIP device raises.
"""

from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass, field
from pathlib import Path
from typing import Iterable, Sequence

import numpy as np

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libretro_hip.so"

RETRO_STEP_ADAPTER_BASE = -1
STATE_SEQ_FLAGS_NONE = 0
STATE_SEQ_FLAGS_PARTIAL_ONLY = 1
STATE_SEQ_FLAGS_ON_DEVICE = 2
DEVICE_AUTO, DEVICE_CPU, DEVICE_GPU = 0, 1, 2
KV_F32, KV_F16, KV_Q8_0, KV_Q4_0 = 0, 1, 2, 3


class EngineError(RuntimeError):
    pass


class InvalidArgument(EngineError):
    """Status -3: a caller error reported before anything was decoded."""


class RuntimeFailure(EngineError):
    """Any other non-zero status."""


class BufferTooSmall(EngineError):
    """Status -2."""


# ---- C structs (layouts pinned by tests/test_abi.py) ------------------------------

class CSamplingParams(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_p", C.c_float),
                ("max_new_tokens", C.c_uint32), ("seed", C.c_uint32)]


class CGenerationSequence(C.Structure):
    _fields_ = [("prompt_tokens", C.POINTER(C.c_int32)), ("n_prompt", C.c_size_t), ("sampling", CSamplingParams)]


class CGenerationSequenceV2(C.Structure):
    pass      # fields set below, once CSamplingParamsV2 is known


class CGenerationStats(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("calls", "sequences", "prompt_tokens", "prefilled_tokens", "reused_tokens",
                                          "hits", "evictions")]


class CStepRow(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("request", C.c_int32), ("slot", C.c_int32),
                ("tokens", C.POINTER(C.c_int32)), ("n", C.c_uint32), ("pos0", C.c_int32),
                ("sample", C.c_bool), ("sampling", CSamplingParams), ("n_top_logprobs", C.c_uint32),
                ("adapter", C.c_int32)]


class CStepOutRow(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("token", C.c_int32), ("logprob", C.c_float),
                ("n_top", C.c_uint32), ("forced", C.c_uint8), ("sampled", C.c_uint8)]


class CSamplingParamsV2(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("temperature", C.c_float), ("top_p", C.c_float),
                ("max_new_tokens", C.c_uint32), ("seed", C.c_uint32), ("top_k", C.c_int32),
                ("min_p", C.c_float), ("repeat_penalty", C.c_float), ("frequency_penalty", C.c_float),
                ("presence_penalty", C.c_float), ("penalty_window", C.c_uint32), ("n_logit_bias", C.c_uint32),
                ("logit_bias_ids", C.POINTER(C.c_int32)), ("logit_bias_values", C.POINTER(C.c_float)),
                ("grammar", C.c_void_p)]


CGenerationSequenceV2._fields_ = [("prompt_tokens", C.POINTER(C.c_int32)), ("n_prompt", C.c_size_t), ("sampling", CSamplingParamsV2)]


class CStepRowV2(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("request", C.c_int32), ("slot", C.c_int32),
                ("tokens", C.POINTER(C.c_int32)), ("n", C.c_uint32), ("pos0", C.c_int32),
                ("sample", C.c_bool), ("sampling", CSamplingParamsV2), ("n_top_logprobs", C.c_uint32),
                ("want_logprob", C.c_uint8), ("adapter", C.c_int32)]


def _ffi_row_dtype() -> np.dtype:
    """CStepRowV2 as a numpy record (pointers as addresses, the sampling block's fields under "s.")."""
    kinds = {C.c_uint32: "<u4", C.c_int32: "<i4", C.c_float: "<f4", C.c_bool: "?", C.c_uint8: "u1"}
    names, formats, offsets = [], [], []

    def walk(struct, base, prefix):
        for name, ctype in struct._fields_:
            at = base + getattr(struct, name).offset
            if isinstance(ctype, type) and issubclass(ctype, C.Structure):
                walk(ctype, at, "s.")
                continue
            names.append(prefix + name)
            formats.append(kinds.get(ctype, "<u8"))        # the rest are pointers
            offsets.append(at)

    walk(CStepRowV2, 0, "")
    return np.dtype({"names": names, "formats": formats, "offsets": offsets, "itemsize": C.sizeof(CStepRowV2)})


_FFI_ROW_DTYPE = _ffi_row_dtype()


class CStepOutRowV2(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("token", C.c_int32), ("logprob", C.c_float),
                ("n_top", C.c_uint32), ("forced", C.c_uint8), ("sampled", C.c_uint8),
                ("sampled_logprob", C.c_float)]


class CAdapterRowsInfo(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("n_adapters", C.c_uint32), ("max_rank", C.c_uint32),
                ("stacked_bytes", C.c_uint64), ("unpadded_bytes", C.c_uint64)]


class CEngineMemoryInfo(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("n_slots", C.c_uint32), ("cells_total", C.c_uint64),
                ("cells_used", C.c_uint64), ("kv_bytes", C.c_uint64), ("recurrent_bytes", C.c_uint64)]


class CEngineConfig(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("n_ctx", C.c_uint32), ("n_seq_max", C.c_uint32),
                ("n_batch", C.c_uint32), ("n_ubatch", C.c_uint32), ("kv_dtype", C.c_int32),
                ("flash_attn", C.c_bool), ("device", C.c_int32), ("threads", C.c_uint32),
                ("verbose", C.c_bool), ("kv_unified", C.c_uint32), ("expert_placement", C.c_int32),
                ("expert_host_layers", C.c_uint32), ("expert_device_cache_bytes", C.c_uint64)]


# Every symbol include/retro_step.h and include/retro_kernels.h declare.
STEP_SYMBOLS = [
    "retro_engine_new", "retro_engine_new_checked", "retro_engine_free", "retro_engine_step",
    "retro_engine_step_v2", "retro_engine_seq_rm", "retro_engine_seq_cp", "retro_engine_seq_save",
    "retro_engine_seq_load", "retro_engine_seq_pos", "retro_engine_memory", "retro_engine_request_free",
    "retro_engine_generate_batch", "retro_engine_generate_continuous_batch", "retro_engine_generation_stats",
    "retro_engine_kv_unified", "retro_engine_weights_version", "retro_engine_model_fingerprint",
    "retro_engine_is_hybrid", "retro_engine_eos_token", "retro_engine_vocab_size", "retro_engine_is_eog_token",
    "retro_engine_context_size", "retro_engine_detokenize", "retro_engine_graphs_reused",
    "retro_engine_tokenize_text", "retro_engine_tokenize_fragment", "retro_engine_tokenize", "retro_engine_token_piece",
    "retro_engine_load_lora", "retro_engine_set_lora_enabled",
    "retro_engine_load_lora_named", "retro_engine_activate_lora", "retro_engine_active_adapter",
    "retro_engine_adapter_load", "retro_engine_adapter_unload", "retro_engine_adapter_rows_info",
    "retro_grammar_from_json_schema", "retro_grammar_from_gbnf", "retro_grammar_json_object",
    "retro_grammar_gbnf", "retro_grammar_free", "retro_last_error",
]
KERNEL_SYMBOLS = [
    "retro_kernel_matmul", "retro_kernel_gemv_fused", "retro_kernel_matmul_time", "retro_kernel_mxfp4_scaled", "retro_kernel_mxfp4_scaled_time", "retro_kernel_stream_time", "retro_kernel_sample_prepare", "retro_kernel_sample_greedy_noalloc", "retro_kernel_sample_greedy_noalloc_max_rows", "retro_kernel_page_size", "retro_kernel_max_topk",
    "retro_engine_debug_logits", "retro_engine_debug_kv", "retro_engine_debug_pack", "retro_engine_debug_pages",
    "retro_engine_debug_profile", "retro_engine_debug_profile_categories", "retro_engine_debug_profile_read",
    "retro_engine_debug_attention_timeline", "retro_engine_debug_attention_timeline_read", "retro_engine_debug_single_token_matvec",
]
PROFILE_CATEGORIES = ["pack", "embed", "norm", "qkv", "rope", "attention", "combine", "o_proj", "gate_up", "swiglu",
                      "down", "head", "sample"]

_lib = None
_i32p, _f32p, _u8p = C.POINTER(C.c_int32), C.POINTER(C.c_float), C.POINTER(C.c_uint8)


def load_library() -> C.CDLL:
    """Loads the built library; raises when it is missing (build it with
    `python -m retrograd_amd.build` or `__graft_entry__.build()`)."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise EngineError("libretro_hip.so is not built: %s is missing" % LIB_PATH)
    lib = C.CDLL(str(LIB_PATH))
    lib.retro_last_error.restype = C.c_char_p
    lib.retro_engine_new.restype = C.c_void_p
    lib.retro_engine_new.argtypes = [C.c_char_p, C.POINTER(CEngineConfig)]
    lib.retro_engine_new_checked.restype = C.c_void_p
    lib.retro_engine_new_checked.argtypes = [C.c_char_p, C.POINTER(CEngineConfig), C.POINTER(C.c_bool)]
    lib.retro_engine_free.restype = None
    lib.retro_engine_free.argtypes = [C.c_void_p]
    lib.retro_engine_step.argtypes = [C.c_void_p, C.POINTER(CStepRow), C.c_size_t, C.POINTER(CStepOutRow),
                                      _i32p, _f32p, C.c_size_t]
    lib.retro_engine_step_v2.argtypes = [C.c_void_p, C.POINTER(CStepRowV2), C.c_size_t, C.POINTER(CStepOutRowV2),
                                         _i32p, _f32p, C.c_size_t]
    lib.retro_engine_generate_batch.argtypes = [C.c_void_p, _i32p, C.c_size_t, C.POINTER(CSamplingParams), C.c_size_t,
                                                _i32p, _f32p, C.c_size_t, C.POINTER(C.c_size_t), _u8p]
    lib.retro_engine_generate_continuous_batch.argtypes = [C.c_void_p, C.POINTER(CGenerationSequence), C.c_size_t,
                                                           _i32p, _f32p, C.c_size_t, C.POINTER(C.c_size_t), _u8p]
    lib.retro_engine_generation_stats.argtypes = [C.c_void_p, C.POINTER(CGenerationStats)]
    lib.retro_engine_seq_rm.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_int32]
    lib.retro_engine_seq_cp.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32]
    lib.retro_engine_seq_save.argtypes = [C.c_void_p, C.c_int32, C.c_uint32, _u8p, C.c_size_t, C.POINTER(C.c_size_t)]
    lib.retro_engine_seq_load.argtypes = [C.c_void_p, C.c_int32, C.c_uint32, _u8p, C.c_size_t, C.POINTER(C.c_size_t)]
    lib.retro_engine_seq_pos.argtypes = [C.c_void_p, C.c_int32, _i32p, _i32p]
    lib.retro_engine_memory.argtypes = [C.c_void_p, C.POINTER(CEngineMemoryInfo)]
    lib.retro_engine_request_free.argtypes = [C.c_void_p, C.c_int32]
    lib.retro_engine_kv_unified.argtypes = [C.c_void_p, C.POINTER(C.c_bool)]
    lib.retro_engine_weights_version.argtypes = [C.c_void_p, C.POINTER(C.c_uint64)]
    lib.retro_engine_model_fingerprint.argtypes = [C.c_void_p, C.POINTER(C.c_uint64)]
    lib.retro_engine_is_hybrid.argtypes = [C.c_void_p, C.POINTER(C.c_bool)]
    lib.retro_engine_eos_token.argtypes = [C.c_void_p, _i32p]
    lib.retro_engine_vocab_size.argtypes = [C.c_void_p, C.POINTER(C.c_uint32)]
    lib.retro_engine_is_eog_token.argtypes = [C.c_void_p, C.c_int32, C.POINTER(C.c_bool)]
    lib.retro_engine_context_size.argtypes = [C.c_void_p, C.POINTER(C.c_uint32)]
    lib.retro_engine_tokenize.argtypes = [C.c_void_p, C.c_char_p, C.c_bool, C.c_bool, _i32p, C.c_size_t, C.POINTER(C.c_size_t)]
    lib.retro_engine_tokenize_text.argtypes = [C.c_void_p, C.c_char_p, _i32p, C.c_size_t, C.POINTER(C.c_size_t)]
    lib.retro_engine_tokenize_fragment.argtypes = [C.c_void_p, C.c_char_p, _i32p, C.c_size_t, C.POINTER(C.c_size_t)]
    lib.retro_engine_token_piece.argtypes = [C.c_void_p, C.c_int32, C.c_bool, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)]
    lib.retro_engine_detokenize.argtypes = [C.c_void_p, _i32p, C.c_size_t, C.c_bool, C.c_char_p, C.c_size_t,
                                            C.POINTER(C.c_size_t)]
    lib.retro_engine_graphs_reused.argtypes = [C.c_void_p, C.POINTER(C.c_uint64)]
    lib.retro_engine_load_lora.argtypes = [C.c_void_p, C.c_char_p]
    lib.retro_engine_set_lora_enabled.argtypes = [C.c_void_p, C.c_bool]
    lib.retro_engine_load_lora_named.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p]
    lib.retro_engine_activate_lora.argtypes = [C.c_void_p, C.c_char_p]
    lib.retro_engine_active_adapter.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)]
    lib.retro_engine_adapter_load.argtypes = [C.c_void_p, C.c_char_p, C.c_float, _i32p]
    lib.retro_engine_adapter_unload.argtypes = [C.c_void_p, C.c_int32]
    lib.retro_engine_adapter_rows_info.argtypes = [C.c_void_p, C.POINTER(CAdapterRowsInfo)]
    lib.retro_grammar_from_gbnf.restype = C.c_void_p
    lib.retro_grammar_from_gbnf.argtypes = [C.c_char_p]
    lib.retro_grammar_from_json_schema.restype = C.c_void_p
    lib.retro_grammar_from_json_schema.argtypes = [C.c_char_p]
    lib.retro_grammar_json_object.restype = C.c_void_p
    lib.retro_grammar_gbnf.restype = C.c_char_p
    lib.retro_grammar_gbnf.argtypes = [C.c_void_p]
    lib.retro_grammar_free.restype = None
    lib.retro_grammar_free.argtypes = [C.c_void_p]
    # kernel-level entry points
    lib.retro_kernel_matmul.argtypes = [C.c_int32, _u8p, C.c_int64, C.c_int64, _f32p, C.c_int32, C.c_int32,
                                        _f32p, C.c_int32, _f32p]
    lib.retro_kernel_sample_prepare.argtypes = [_f32p, C.c_int32, C.c_int32, _i32p, _i32p, _f32p,
                                                C.POINTER(C.c_double), _i32p, _f32p]
    lib.retro_kernel_sample_greedy_noalloc.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
                                                       C.c_void_p, C.c_void_p]
    lib.retro_kernel_sample_greedy_noalloc_max_rows.restype = C.c_int32
    lib.retro_kernel_gemv_fused.argtypes = [C.c_int32, C.c_int32, _u8p, C.c_int64, C.c_int64, _f32p, _f32p, C.c_float, C.c_int32, C.c_int32,
                                            _f32p, _f32p]
    lib.retro_kernel_gemv_fused.restype = C.c_int
    lib.retro_kernel_matmul_time.argtypes = [C.c_int32, C.c_int64, C.c_int64, C.c_int32, C.c_int32, C.c_int32,
                                             C.c_int32, C.c_int32, C.POINTER(C.c_double)]
    lib.retro_kernel_mxfp4_scaled.argtypes = [_u8p, C.c_int64, C.c_int64, _f32p, C.c_int32, C.c_int32, _f32p]
    lib.retro_kernel_mxfp4_scaled_time.argtypes = [C.c_int64, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_double)]
    lib.retro_kernel_stream_time.argtypes = [C.c_int64, C.c_int32, C.c_int32, C.POINTER(C.c_double)]
    lib.retro_kernel_page_size.restype = C.c_int32
    lib.retro_kernel_max_topk.restype = C.c_int32
    lib.retro_engine_debug_logits.argtypes = [C.c_void_p, _f32p, C.c_size_t, C.POINTER(C.c_size_t)]
    lib.retro_engine_debug_kv.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                          C.POINTER(C.c_uint16)]
    lib.retro_engine_debug_pack.argtypes = [C.c_void_p, _i32p, _i32p, _i32p, _i32p, _i32p, _i32p, C.c_size_t,
                                            C.c_size_t, _i32p]
    lib.retro_engine_debug_pages.argtypes = [C.c_void_p, C.c_int32, _i32p, C.c_size_t, C.POINTER(C.c_size_t)]
    lib.retro_engine_debug_profile.argtypes = [C.c_void_p, C.c_int32]
    lib.retro_engine_debug_attention_timeline.argtypes = [C.c_void_p, C.c_int32]
    lib.retro_engine_debug_single_token_matvec.argtypes = [C.c_void_p, C.c_int32]
    lib.retro_engine_debug_attention_timeline_read.argtypes = [C.c_void_p, C.POINTER(C.c_uint64), C.c_size_t, C.POINTER(C.c_size_t)]
    lib.retro_engine_debug_profile_categories.restype = C.c_int32
    lib.retro_engine_debug_profile_read.argtypes = [C.c_void_p, C.POINTER(C.c_double), C.POINTER(C.c_uint64), C.c_int32]
    _lib = lib
    return lib


def last_error() -> str:
    return load_library().retro_last_error().decode("utf-8", "replace")


def _raise(status: int) -> None:
    msg = last_error()
    if status == -3:
        raise InvalidArgument(msg)
    if status == -2:
        raise BufferTooSmall(msg)
    raise RuntimeFailure(msg)


# ---- safe types ---------------------------------------------------------------------

@dataclass
class SamplingParamsV2:
    """reference crates/retrograd-core/src/types.rs:1353-1374."""
    temperature: float = 1.0
    top_p: float = 1.0
    max_new_tokens: int = 1
    seed: int = 0
    top_k: int = 0
    min_p: float = 0.0
    repeat_penalty: float = 1.0
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0
    penalty_window: int = 0
    logit_bias: Sequence[tuple] = ()
    grammar: str | None = None

    @staticmethod
    def greedy(seed: int = 0, max_new_tokens: int = 1) -> "SamplingParamsV2":
        # "greedy" in the reference is temperature 1, top_p 1, top_k 1
        # (tests/expert_placement.rs:355-356); temperature 0 is refused.
        return SamplingParamsV2(temperature=1.0, top_p=1.0, top_k=1, seed=seed, max_new_tokens=max_new_tokens)


@dataclass
class RowAdapter:
    value: int = 0

    @staticmethod
    def context() -> "RowAdapter":
        return RowAdapter(0)

    @staticmethod
    def base() -> "RowAdapter":
        return RowAdapter(RETRO_STEP_ADAPTER_BASE)

    @staticmethod
    def loaded(adapter_id: int) -> "RowAdapter":
        return RowAdapter(adapter_id)


@dataclass
class StepRow:
    request: int
    slot: int
    tokens: Sequence[int]
    pos0: int
    sample: bool = False
    sampling: SamplingParamsV2 = field(default_factory=SamplingParamsV2)
    n_top_logprobs: int = 0
    want_logprob: bool = False
    adapter: RowAdapter = field(default_factory=RowAdapter)

    @staticmethod
    def prefill(request: int, slot: int, tokens: Sequence[int], pos0: int) -> "StepRow":
        return StepRow(request, slot, tokens, pos0)

    @staticmethod
    def decode(request: int, slot: int, token: int, pos0: int, sampling: SamplingParamsV2) -> "StepRow":
        return StepRow(request, slot, [token], pos0, sample=True, sampling=sampling)


@dataclass
class StepOutRow:
    token: int = 0
    logprob: float = 0.0
    forced: bool = False
    sampled: bool = False
    n_top: int = 0
    sampled_logprob: float = 0.0


@dataclass
class EngineMemory:
    n_slots: int
    cells_total: int
    cells_used: int
    kv_bytes: int
    recurrent_bytes: int


@dataclass
class EngineConfig:
    """reference crates/retrograd-core/src/types.rs:158-175 / retro_engine_config."""
    n_ctx: int = 4096
    n_seq_max: int = 8
    n_batch: int = 512
    n_ubatch: int = 512
    kv_dtype: int = KV_F16
    flash_attn: bool = True
    device: int = DEVICE_AUTO
    threads: int = 0
    verbose: bool = False
    kv_unified: bool = True

    def to_ffi(self) -> CEngineConfig:
        c = CEngineConfig()
        c.struct_size = C.sizeof(CEngineConfig)
        c.n_ctx, c.n_seq_max, c.n_batch, c.n_ubatch = self.n_ctx, self.n_seq_max, self.n_batch, self.n_ubatch
        c.kv_dtype, c.flash_attn, c.device, c.threads = self.kv_dtype, self.flash_attn, self.device, self.threads
        c.verbose, c.kv_unified = self.verbose, 1 if self.kv_unified else 0
        c.expert_placement, c.expert_host_layers, c.expert_device_cache_bytes = 0, 0, 0
        return c


class StepOutput:
    """Reused buffers of Engine.step: FFI row staging, one output row per step
    row, and the row-major top-logprob arrays of stride n_top_stride."""

    def __init__(self, capacity: int = 0, n_top_stride: int = 0) -> None:
        self._cap = 0
        self.n_top_stride = 0
        self.n_rows = 0
        self._ffi_rows = None
        self._view = None
        self._rows = None
        self.top_ids = np.zeros(0, np.int32)
        self.top_logprobs = np.zeros(0, np.float32)
        self._keep: list = []
        self._reserve(capacity, n_top_stride)

    def _reserve(self, n_rows: int, stride: int) -> None:
        if n_rows > self._cap:
            self._cap = max(n_rows, 2 * self._cap)
            self._ffi_rows = (CStepRowV2 * self._cap)()
            self._view = np.frombuffer(self._ffi_rows, dtype=_FFI_ROW_DTYPE)
            self._rows = (CStepOutRowV2 * self._cap)()
        if stride != self.n_top_stride or self.top_ids.size < self._cap * stride:
            self.n_top_stride = stride
            self.top_ids = np.zeros(self._cap * stride, np.int32)
            self.top_logprobs = np.zeros(self._cap * stride, np.float32)

    def rows(self) -> list:
        return [StepOutRow(r.token, r.logprob, bool(r.forced), bool(r.sampled), r.n_top, r.sampled_logprob)
                for r in self._rows[:self.n_rows]]

    def row(self, i: int) -> StepOutRow:
        r = self._rows[i]
        return StepOutRow(r.token, r.logprob, bool(r.forced), bool(r.sampled), r.n_top, r.sampled_logprob)

    def top(self, i: int):
        n = self._rows[i].n_top
        s = self.n_top_stride
        return self.top_ids[i * s:i * s + n].copy(), self.top_logprobs[i * s:i * s + n].copy()


class Engine:
    """One model, one KV pool, single-threaded use."""

    def __init__(self, model_path, config: EngineConfig | None = None) -> None:
        self._lib = load_library()
        cfg = (config or EngineConfig()).to_ffi()
        self._h = self._lib.retro_engine_new(os.fsencode(str(model_path)), C.byref(cfg))
        if not self._h:
            raise RuntimeFailure(last_error())
        self.config = config or EngineConfig()

    def close(self) -> None:
        if getattr(self, "_h", None):
            self._lib.retro_engine_free(self._h)
            self._h = None

    def __del__(self) -> None:
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- the step ------------------------------------------------------------------
    def step(self, rows: Sequence[StepRow], out: StepOutput) -> None:
        n = len(rows)
        stride = max((r.n_top_logprobs for r in rows), default=0)
        out._reserve(n, stride)
        out._keep = keep = []
        lens = [len(r.tokens) for r in rows]
        requests = [r.request for r in rows]
        pos0 = [r.pos0 for r in rows]
        sample = [bool(r.sample) for r in rows]
        sp = [r.sampling for r in rows]
        self._check_rows(rows, lens, requests, pos0, sample, sp)
        if n:
            # The FFI rows are filled column by column through a numpy view of the ctypes array (a Python
            # assignment per field and row costs several times the C call's own host work at 64 rows).
            v = out._view[:n]
            if max(lens) == 1:
                flat = np.array([r.tokens[0] for r in rows], dtype=np.int32)
            else:
                flat = np.concatenate([np.asarray(r.tokens, dtype=np.int32).ravel() for r in rows])
            keep.append(flat)
            lens_a = np.array(lens, dtype=np.uint64)
            v["struct_size"] = C.sizeof(CStepRowV2)
            v["tokens"] = flat.ctypes.data + 4 * (np.cumsum(lens_a) - lens_a)
            v["n"] = lens_a
            # integer fields wrap to their C width as a ctypes field assignment does
            i32 = lambda values: np.array(values, dtype=np.int64).astype(np.int32)
            u32 = lambda values: np.array(values, dtype=np.int64).astype(np.uint32)
            v["request"] = i32(requests)
            v["slot"] = i32([r.slot for r in rows])
            v["pos0"] = pos0
            v["sample"] = sample
            v["n_top_logprobs"] = u32([r.n_top_logprobs for r in rows])
            v["want_logprob"] = [1 if r.want_logprob else 0 for r in rows]
            v["adapter"] = i32([r.adapter.value for r in rows])
            v["s.struct_size"] = C.sizeof(CSamplingParamsV2)
            one = sp[0] if all(s is sp[0] for s in sp) else None        # rows that share one parameter object
            for name in ("temperature", "top_p", "min_p", "repeat_penalty", "frequency_penalty", "presence_penalty"):
                v["s." + name] = getattr(one, name) if one is not None else [getattr(s, name) for s in sp]
            for name, conv in (("max_new_tokens", u32), ("top_k", i32), ("penalty_window", u32)):
                v["s." + name] = conv([getattr(one, name)])[0] if one is not None else conv([getattr(s, name) for s in sp])
            v["s.seed"] = one.seed & 0xFFFFFFFF if one is not None else [s.seed & 0xFFFFFFFF for s in sp]
            v["s.n_logit_bias"] = 0
            v["s.logit_bias_ids"] = 0
            v["s.logit_bias_values"] = 0
            v["s.grammar"] = 0
            for i, s in enumerate(sp):           # the rows that point at more: bias lists, a grammar text
                if s.logit_bias or s.grammar is not None:
                    self._fill_sampling_v2(out._ffi_rows[i].sampling, s, keep)
        top_ids = out.top_ids.ctypes.data_as(_i32p) if stride else None
        top_lps = out.top_logprobs.ctypes.data_as(_f32p) if stride else None
        status = self._lib.retro_engine_step_v2(self._h, out._ffi_rows, n, out._rows, top_ids, top_lps, stride)
        out._keep = []
        if status != 0:
            _raise(status)
        out.n_rows = n

    @staticmethod
    def _check_rows(rows, lens, requests, pos0, sample, sp) -> None:
        """The caller-side checks of StepRow::to_ffi_v2 / step_with (reference step.rs:150-203, 412-505): one
        pass over the columns decides whether anything is wrong; the error is then the first in row order."""
        if not rows:
            return
        live = [q for q in requests if q >= 0]
        if (min(lens) > 0 and min(pos0) >= 0 and max(p + n for p, n in zip(pos0, lens)) <= 2 ** 31 - 1
                and len(set(live)) == len(live) and not any(s and q < 0 for s, q in zip(sample, requests))
                and not any(len(s.logit_bias) > 4096 for s in sp if s.logit_bias)):
            return
        seen = set()
        for r, n_tok in zip(rows, lens):
            if n_tok == 0:
                raise InvalidArgument("a step row requires at least one token")
            if r.pos0 < 0:
                raise InvalidArgument("a step row's pos0 must be >= 0")
            if r.pos0 + n_tok > 2 ** 31 - 1:
                raise EngineError("a step row's position range overflows i32")
            if r.sample and r.request < 0:
                raise InvalidArgument("a sampling step row requires a request id >= 0")
            if len(r.sampling.logit_bias) > 4096:
                raise InvalidArgument("logit_bias takes at most 4096 entries")
            if r.request >= 0:
                if r.request in seen:
                    raise InvalidArgument("a request id appears twice in one step")
                seen.add(r.request)

    def step_v1(self, rows: Sequence[tuple], n_top_stride: int = 0):
        """retro_engine_step with v1 rows: (request, slot, tokens, pos0, sample,
        temperature, top_p, seed, n_top_logprobs). Returns (out rows, ids, logprobs)."""
        n = len(rows)
        ffi = (CStepRow * n)()
        outs = (CStepOutRow * n)()
        keep = []
        for i, (request, slot, tokens, pos0, sample, temperature, top_p, seed, n_top) in enumerate(rows):
            toks = np.ascontiguousarray(tokens, dtype=np.int32)
            keep.append(toks)
            f = ffi[i]
            f.struct_size = C.sizeof(CStepRow)
            f.request, f.slot, f.tokens, f.n, f.pos0, f.sample = request, slot, toks.ctypes.data_as(_i32p), toks.size, pos0, sample
            f.sampling.temperature, f.sampling.top_p, f.sampling.max_new_tokens, f.sampling.seed = temperature, top_p, 1, seed
            f.n_top_logprobs, f.adapter = n_top, 0
        ids = np.zeros(n * max(n_top_stride, 1), np.int32)
        lps = np.zeros(n * max(n_top_stride, 1), np.float32)
        status = self._lib.retro_engine_step(self._h, ffi, n, outs, ids.ctypes.data_as(_i32p) if n_top_stride else None,
                                             lps.ctypes.data_as(_f32p) if n_top_stride else None, n_top_stride)
        if status != 0:
            _raise(status)
        return ([StepOutRow(o.token, o.logprob, bool(o.forced), bool(o.sampled), o.n_top) for o in outs],
                ids.reshape(n, -1), lps.reshape(n, -1))

    # -- batched generators -----------------------------------------------------------
    @staticmethod
    def _sampling_v1(p) -> CSamplingParams:
        """p: (temperature, top_p, max_new_tokens, seed)."""
        c = CSamplingParams()
        c.temperature, c.top_p, c.max_new_tokens, c.seed = p
        return c

    def _collect(self, n, n_out_max, toks, lps, counts, forced):
        return [(toks[i, :counts[i]].tolist(), lps[i, :counts[i]].copy(), forced[i, :counts[i]].astype(bool).tolist())
                for i in range(n)]

    def generate_batch(self, prompt: Sequence[int], sampling: Sequence[tuple], n_out_max: int | None = None):
        """retro_engine_generate_batch: one completion per entry of `sampling`
        ((temperature, top_p, max_new_tokens, seed) each) of the one prompt.
        Returns [(tokens, logprobs, forced)] per member."""
        n = len(sampling)
        n_out_max = n_out_max or max(p[2] for p in sampling)
        prompt_arr = np.ascontiguousarray(prompt, dtype=np.int32)
        params = (CSamplingParams * n)(*[self._sampling_v1(p) for p in sampling])
        toks = np.zeros((n, n_out_max), np.int32)
        lps = np.zeros((n, n_out_max), np.float32)
        forced = np.zeros((n, n_out_max), np.uint8)
        counts = (C.c_size_t * n)()
        status = self._lib.retro_engine_generate_batch(self._h, prompt_arr.ctypes.data_as(_i32p), prompt_arr.size, params, n,
                                                       toks.ctypes.data_as(_i32p), lps.ctypes.data_as(_f32p), n_out_max,
                                                       counts, forced.ctypes.data_as(_u8p))
        if status != 0:
            _raise(status)
        return self._collect(n, n_out_max, toks, lps, list(counts), forced)

    def _fill_sampling_v2(self, p, s, keep: list) -> None:
        """Stages SamplingParamsV2 `s` into the FFI struct `p`; what `p` points at is appended to `keep`."""
        p.struct_size = C.sizeof(CSamplingParamsV2)
        p.temperature, p.top_p, p.max_new_tokens, p.seed = s.temperature, s.top_p, s.max_new_tokens, s.seed & 0xFFFFFFFF
        p.top_k, p.min_p, p.repeat_penalty = s.top_k, s.min_p, s.repeat_penalty
        p.frequency_penalty, p.presence_penalty, p.penalty_window = s.frequency_penalty, s.presence_penalty, s.penalty_window
        if s.logit_bias:
            ids = np.array([b[0] for b in s.logit_bias], np.int32)
            vals = np.array([b[1] for b in s.logit_bias], np.float32)
            keep.extend((ids, vals))
            p.n_logit_bias = ids.size
            p.logit_bias_ids = ids.ctypes.data_as(_i32p)
            p.logit_bias_values = vals.ctypes.data_as(_f32p)
        else:
            p.n_logit_bias = 0
            p.logit_bias_ids = None
            p.logit_bias_values = None
        if s.grammar is not None:
            g = self._lib.retro_grammar_from_gbnf(s.grammar.encode())
            if not g:
                raise InvalidArgument(last_error())
            keep.append(_GrammarHandle(self._lib, g))
            p.grammar = g
        else:
            p.grammar = None

    def generate_continuous(self, sequences: Sequence[tuple], n_out_max: int | None = None):
        """retro_engine_generate_continuous_batch over (prompt, (temperature, top_p,
        max_new_tokens, seed)) pairs. Returns [(tokens, logprobs, forced)] in input order."""
        n = len(sequences)
        n_out_max = n_out_max or max(p[2] for _, p in sequences)
        keep = [np.ascontiguousarray(prompt, dtype=np.int32) for prompt, _ in sequences]
        ffi = (CGenerationSequence * n)()
        for i, (_, p) in enumerate(sequences):
            ffi[i].prompt_tokens = keep[i].ctypes.data_as(_i32p)
            ffi[i].n_prompt = keep[i].size
            ffi[i].sampling = self._sampling_v1(p)
        toks = np.zeros((n, n_out_max), np.int32)
        lps = np.zeros((n, n_out_max), np.float32)
        forced = np.zeros((n, n_out_max), np.uint8)
        counts = (C.c_size_t * n)()
        status = self._lib.retro_engine_generate_continuous_batch(self._h, ffi, n, toks.ctypes.data_as(_i32p),
                                                                  lps.ctypes.data_as(_f32p), n_out_max, counts,
                                                                  forced.ctypes.data_as(_u8p))
        if status != 0:
            _raise(status)
        return self._collect(n, n_out_max, toks, lps, list(counts), forced)

    def generation_stats(self) -> dict:
        st = CGenerationStats()
        if self._lib.retro_engine_generation_stats(self._h, C.byref(st)) != 0:
            _raise(-1)
        return {name: int(getattr(st, name)) for name, _ in CGenerationStats._fields_}

    # -- sequence operations -----------------------------------------------------------
    def seq_rm(self, slot: int, p0: int = -1, p1: int = -1) -> None:
        s = self._lib.retro_engine_seq_rm(self._h, slot, p0, p1)
        if s != 0:
            _raise(s)

    def seq_cp(self, src: int, dst: int, p0: int = -1, p1: int = -1) -> None:
        s = self._lib.retro_engine_seq_cp(self._h, src, dst, p0, p1)
        if s != 0:
            _raise(s)

    def seq_pos(self, slot: int):
        a, b = C.c_int32(), C.c_int32()
        s = self._lib.retro_engine_seq_pos(self._h, slot, C.byref(a), C.byref(b))
        if s != 0:
            _raise(s)
        return a.value, b.value

    def seq_save_len(self, slot: int, flags: int = 0) -> int:
        n = C.c_size_t()
        s = self._lib.retro_engine_seq_save(self._h, slot, flags, None, 0, C.byref(n))
        if s != 0:
            _raise(s)
        return n.value

    def seq_save(self, slot: int, flags: int = 0) -> bytes:
        need = self.seq_save_len(slot, flags)
        buf = (C.c_uint8 * need)()
        n = C.c_size_t()
        s = self._lib.retro_engine_seq_save(self._h, slot, flags, buf, need, C.byref(n))
        if s != 0:
            _raise(s)
        return bytes(buf[:n.value])

    def seq_save_into(self, slot: int, flags: int, buffer: bytearray) -> int:
        arr = (C.c_uint8 * len(buffer)).from_buffer(buffer)
        n = C.c_size_t()
        s = self._lib.retro_engine_seq_save(self._h, slot, flags, arr, len(buffer), C.byref(n))
        if s != 0:
            _raise(s)
        return n.value

    def seq_load(self, slot: int, data: bytes, flags: int = 0) -> int:
        buf = (C.c_uint8 * len(data)).from_buffer_copy(data)
        n = C.c_size_t()
        s = self._lib.retro_engine_seq_load(self._h, slot, flags, buf, len(data), C.byref(n))
        if s != 0:
            _raise(s)
        return n.value

    def memory(self) -> EngineMemory:
        info = CEngineMemoryInfo()
        s = self._lib.retro_engine_memory(self._h, C.byref(info))
        if s != 0:
            _raise(s)
        return EngineMemory(info.n_slots, info.cells_total, info.cells_used, info.kv_bytes, info.recurrent_bytes)

    def request_free(self, request: int) -> None:
        s = self._lib.retro_engine_request_free(self._h, request)
        if s != 0:
            _raise(s)

    # -- introspection -----------------------------------------------------------------
    def _get(self, fn, ctype):
        v = ctype()
        s = fn(self._h, C.byref(v))
        if s != 0:
            _raise(s)
        return v.value

    def kv_unified(self) -> bool:
        return bool(self._get(self._lib.retro_engine_kv_unified, C.c_bool))

    def weights_version(self) -> int:
        return self._get(self._lib.retro_engine_weights_version, C.c_uint64)

    def model_fingerprint(self) -> int:
        return self._get(self._lib.retro_engine_model_fingerprint, C.c_uint64)

    def is_hybrid(self) -> bool:
        return bool(self._get(self._lib.retro_engine_is_hybrid, C.c_bool))

    def vocab_size(self) -> int:
        return self._get(self._lib.retro_engine_vocab_size, C.c_uint32)

    def context_size(self) -> int:
        return self._get(self._lib.retro_engine_context_size, C.c_uint32)

    def eos_token(self) -> int:
        return self._get(self._lib.retro_engine_eos_token, C.c_int32)

    def graphs_reused(self) -> int:
        return self._get(self._lib.retro_engine_graphs_reused, C.c_uint64)

    def is_eog_token(self, token: int) -> bool:
        v = C.c_bool()
        s = self._lib.retro_engine_is_eog_token(self._h, token, C.byref(v))
        if s != 0:
            _raise(s)
        return bool(v.value)

    def tokenize(self, text: str, add_special: bool = True, parse_special: bool = True) -> list:
        """Text -> token ids (sentencepiece-kind vocabularies); the reference's two-call contract."""
        raw = text.encode()
        n = C.c_size_t()
        s = self._lib.retro_engine_tokenize(self._h, raw, add_special, parse_special, None, 0, C.byref(n))
        if s != 0:
            _raise(s)
        out = np.zeros(max(n.value, 1), np.int32)
        s = self._lib.retro_engine_tokenize(self._h, raw, add_special, parse_special, out.ctypes.data_as(_i32p), n.value, C.byref(n))
        if s != 0:
            _raise(s)
        return [int(t) for t in out[:n.value]]

    def token_piece(self, token: int, special: bool = False) -> bytes:
        n = C.c_size_t()
        s = self._lib.retro_engine_token_piece(self._h, token, special, None, 0, C.byref(n))
        if s != 0:
            _raise(s)
        buf = C.create_string_buffer(n.value + 1)
        s = self._lib.retro_engine_token_piece(self._h, token, special, buf, n.value + 1, C.byref(n))
        if s != 0:
            _raise(s)
        return buf.raw[:n.value]

    def detokenize_bytes(self, tokens: Sequence[int], unparse_special: bool = False) -> bytes:
        toks = np.ascontiguousarray(tokens, dtype=np.int32)
        n = C.c_size_t()
        ptr = toks.ctypes.data_as(_i32p) if toks.size else None
        s = self._lib.retro_engine_detokenize(self._h, ptr, toks.size, unparse_special, None, 0, C.byref(n))
        if s != 0:
            _raise(s)
        buf = C.create_string_buffer(n.value + 1)
        s = self._lib.retro_engine_detokenize(self._h, ptr, toks.size, unparse_special, buf, n.value + 1, C.byref(n))
        if s != 0:
            _raise(s)
        return buf.raw[:n.value]

    # -- context-wide adapters: what rows with adapter 0 decode under ---------------------------
    def load_lora(self, path) -> None:
        """The one context-wide adapter: every other registered adapter goes, this one is active."""
        s = self._lib.retro_engine_load_lora(self._h, os.fsencode(str(path)))
        if s != 0:
            _raise(s)

    def set_lora_enabled(self, enabled: bool) -> None:
        s = self._lib.retro_engine_set_lora_enabled(self._h, enabled)
        if s != 0:
            _raise(s)

    def load_lora_named(self, name: str, path) -> None:
        s = self._lib.retro_engine_load_lora_named(self._h, name.encode(), os.fsencode(str(path)))
        if s != 0:
            _raise(s)

    def activate_lora(self, name: str | None) -> None:
        """None or "": the base model."""
        s = self._lib.retro_engine_activate_lora(self._h, (name or "").encode())
        if s != 0:
            _raise(s)

    def active_adapter(self) -> str:
        n = C.c_size_t()
        s = self._lib.retro_engine_active_adapter(self._h, None, 0, C.byref(n))
        if s != 0:
            _raise(s)
        buf = C.create_string_buffer(n.value + 1)
        s = self._lib.retro_engine_active_adapter(self._h, buf, n.value + 1, C.byref(n))
        if s != 0:
            _raise(s)
        return buf.raw[:n.value].decode()

    # -- per-row adapters --------------------------------------------------------------------
    def adapter_load(self, path, scale: float = 1.0) -> int:
        out = C.c_int32()
        s = self._lib.retro_engine_adapter_load(self._h, os.fsencode(str(path)), scale, C.byref(out))
        if s != 0:
            _raise(s)
        return out.value

    def adapter_unload(self, adapter_id: int) -> None:
        s = self._lib.retro_engine_adapter_unload(self._h, adapter_id)
        if s != 0:
            _raise(s)

    def adapter_rows_info(self) -> "CAdapterRowsInfo":
        """n_adapters, max_rank, stacked_bytes, unpadded_bytes (retrograd-engine AdapterRowsInfo)."""
        info = CAdapterRowsInfo()
        s = self._lib.retro_engine_adapter_rows_info(self._h, C.byref(info))
        if s != 0:
            _raise(s)
        return info

    # -- state inspection (tests) --------------------------------------------------------
    def debug_logits(self) -> np.ndarray:
        rows = C.c_size_t()
        s = self._lib.retro_engine_debug_logits(self._h, None, 0, C.byref(rows))
        if s != 0:
            _raise(s)
        v = self.vocab_size()
        out = np.empty((rows.value, v), np.float32)
        s = self._lib.retro_engine_debug_logits(self._h, out.ctypes.data_as(_f32p), out.size, C.byref(rows))
        if s != 0:
            _raise(s)
        return out

    def debug_kv(self, layer: int, slot: int, pos: int, want_v: bool, kv_dim: int) -> np.ndarray:
        out = np.empty(kv_dim, np.uint16)
        s = self._lib.retro_engine_debug_kv(self._h, layer, slot, pos, 1 if want_v else 0,
                                            out.ctypes.data_as(C.POINTER(C.c_uint16)))
        if s != 0:
            _raise(s)
        return out.view(np.float16)

    def debug_kv_q8(self, layer: int, slot: int, pos: int, want_v: bool, n_kv: int, head_dim: int, bits: int = 8) -> np.ndarray:
        """The K or V row of a Q8_0 (bits 8) or Q4_0 (bits 4) cache as the values it stands for (scale times code),
        f32, kv_dim of them."""
        code_units = head_dim // 2 if bits == 8 else head_dim // 4
        per_head = code_units + head_dim // 32
        raw = np.empty(n_kv * per_head, np.uint16)
        s = self._lib.retro_engine_debug_kv(self._h, layer, slot, pos, 1 if want_v else 0,
                                            raw.ctypes.data_as(C.POINTER(C.c_uint16)))
        if s != 0:
            _raise(s)
        out = np.empty((n_kv, head_dim), np.float32)
        for h in range(n_kv):
            row = raw[h * per_head:(h + 1) * per_head]
            packed = row[:code_units].view(np.uint8).astype(np.int32)
            if bits == 8:
                codes = packed - 128
            else:               # element 2 k in the low nibble of byte k, a value is scale times (code - 8)
                codes = np.stack([packed & 15, packed >> 4], axis=-1).reshape(-1) - 8
            scales = row[code_units:].view(np.float16).astype(np.float32)
            out[h] = (codes.reshape(-1, 32) * scales[:, None]).reshape(-1)
        return out.reshape(-1)

    def debug_pack(self, cap_tokens: int, cap_rows: int) -> dict:
        arrs = {k: np.full(cap_tokens, -7, np.int32) for k in ("token", "pos", "seq", "cell", "out_index")}
        last = np.full(cap_rows, -7, np.int32)
        counts = np.zeros(4, np.int32)
        s = self._lib.retro_engine_debug_pack(self._h, *(arrs[k].ctypes.data_as(_i32p) for k in ("token", "pos", "seq", "cell", "out_index")),
                                              last.ctypes.data_as(_i32p), cap_tokens, cap_rows, counts.ctypes.data_as(_i32p))
        if s != 0:
            _raise(s)
        T = int(counts[0])
        out = {k: v[:T] for k, v in arrs.items()}
        out["last_index"] = last
        out["counts"] = counts
        return out

    def profile(self, level: int) -> None:
        """HIP-event timing of kernel categories: 0 off, 1 attention only, 2 all."""
        s = self._lib.retro_engine_debug_profile(self._h, level)
        if s != 0:
            _raise(s)

    def single_token_matvec(self, on: bool) -> None:
        """Single-token steps of the exact arithmetic on the matrix-vector kernel with f32 rows instead of the tile
        kernels (what RETRO_GEMV_EXACT=1 selects at creation; off by default, see include/retro_kernels.h)."""
        s = self._lib.retro_engine_debug_single_token_matvec(self._h, 1 if on else 0)
        if s != 0:
            _raise(s)

    def attention_timeline(self, on: bool) -> None:
        """While on, the decode attention launch of the middle layer records six clock values per workgroup."""
        s = self._lib.retro_engine_debug_attention_timeline(self._h, 1 if on else 0)
        if s != 0:
            _raise(s)

    def attention_timeline_read(self) -> np.ndarray:
        """[workgroups][6] of the last recorded launch: start, after the prologue, first wave done, all waves done,
        end (ticks of the 100 MHz clock) and the row's KV pages; empty when no step took that launch."""
        n = C.c_size_t()
        s = self._lib.retro_engine_debug_attention_timeline_read(self._h, None, 0, C.byref(n))
        if s != 0:
            _raise(s)
        out = np.zeros((n.value, 6), np.uint64)
        if n.value:
            s = self._lib.retro_engine_debug_attention_timeline_read(self._h, out.ctypes.data_as(C.POINTER(C.c_uint64)), n.value, C.byref(n))
            if s != 0:
                _raise(s)
        return out

    def profile_read(self, reset: bool = True) -> dict:
        n = self._lib.retro_engine_debug_profile_categories()
        assert n == len(PROFILE_CATEGORIES)
        ms = (C.c_double * n)()
        cnt = (C.c_uint64 * n)()
        s = self._lib.retro_engine_debug_profile_read(self._h, ms, cnt, 1 if reset else 0)
        if s != 0:
            _raise(s)
        return {name: (ms[i], int(cnt[i])) for i, name in enumerate(PROFILE_CATEGORIES)}

    def debug_pages(self, slot: int) -> np.ndarray:
        n = C.c_size_t()
        s = self._lib.retro_engine_debug_pages(self._h, slot, None, 0, C.byref(n))
        if s != 0:
            _raise(s)
        out = np.empty(n.value, np.int32)
        s = self._lib.retro_engine_debug_pages(self._h, slot, out.ctypes.data_as(_i32p), out.size, C.byref(n))
        if s != 0:
            _raise(s)
        return out


class _GrammarHandle:
    def __init__(self, lib, handle) -> None:
        self._lib, self._h = lib, handle

    def __del__(self) -> None:
        try:
            self._lib.retro_grammar_free(self._h)
        except Exception:
            pass


# ---- kernel-level calls (tests, micro-benchmarks) -----------------------------------------

def kernel_matmul(ggml_type: int, raw: np.ndarray, n_rows: int, k: int, x: np.ndarray, use_tiles,
                  bias: np.ndarray | None = None, accumulate_into: np.ndarray | None = None,
                  ggml_activations: bool = False, integer: bool = False) -> np.ndarray:
    """One matmul kernel on host data; ggml_activations: the rows are converted as ggml's CPU matmul does;
    integer (with it, Q4_K or Q8_0 tiles, at most two rows): the converted blocks go through the integer matrix-vector kernel."""
    lib = load_library()
    use_tiles = int(use_tiles) | (0x100 if ggml_activations else 0) | (0x200 if integer else 0)
    raw = np.ascontiguousarray(raw, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    T = x.shape[0]
    y = np.zeros((T, n_rows), np.float32) if accumulate_into is None else np.ascontiguousarray(accumulate_into, np.float32).copy()
    b = None
    if bias is not None:
        bias = np.ascontiguousarray(bias, np.float32)
        b = bias.ctypes.data_as(_f32p)
    s = lib.retro_kernel_matmul(ggml_type, raw.ctypes.data_as(_u8p), n_rows, k, x.ctypes.data_as(_f32p), T,
                                int(use_tiles), b, 0 if accumulate_into is None else 1, y.ctypes.data_as(_f32p))
    if s != 0:
        _raise(s)
    return y


def kernel_gemv_fused(kind: int, ggml_type: int, raw: np.ndarray, n_rows: int, k: int, x: np.ndarray, norm_w: np.ndarray | None = None,
                      eps: float = 1e-5, group: int = 0):
    """The integer matrix-vector kernel with RMSNorm (kind 1) or SwiGLU (kind 2) fused into its staging, and the same
    product as producer launch plus kernel: returns (fused, unfused), each [tokens][n_rows]."""
    lib = load_library()
    raw = np.ascontiguousarray(raw, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    T = x.shape[0]
    w = None
    if norm_w is not None:
        norm_w = np.ascontiguousarray(norm_w, np.float32)
        w = norm_w.ctypes.data_as(_f32p)
    fused, unfused = np.zeros((T, n_rows), np.float32), np.zeros((T, n_rows), np.float32)
    s = lib.retro_kernel_gemv_fused(kind, ggml_type, raw.ctypes.data_as(_u8p), n_rows, k, x.ctypes.data_as(_f32p), w, eps, T, group,
                                    fused.ctypes.data_as(_f32p), unfused.ctypes.data_as(_f32p))
    if s != 0:
        _raise(s)
    return fused, unfused


def kernel_matmul_time(ggml_type: int, n_rows: int, k: int, n_tokens: int, mode: int = 2, iters: int = 50,
                       debug: int = 0, force_ksplit: int = 0) -> float:
    """Microseconds per launch of one tile matmul on device-only data."""
    out = C.c_double()
    s = load_library().retro_kernel_matmul_time(ggml_type, n_rows, k, n_tokens, mode, iters, debug, force_ksplit,
                                                C.byref(out))
    if s != 0:
        _raise(s)
    return out.value


def kernel_mxfp4_scaled(raw, n_rows: int, k: int, x: np.ndarray, exact: bool = False) -> np.ndarray:
    """MXFP4 rows times at most 16 tokens on the block-scaled matrix instruction: ggml's arithmetic (Q8_0 activation
    blocks), or with `exact` the f32 activations themselves."""
    src = np.ascontiguousarray(raw, np.uint8)
    x = np.ascontiguousarray(x, np.float32).reshape(-1, k)
    y = np.empty((x.shape[0], n_rows), np.float32)
    s = load_library().retro_kernel_mxfp4_scaled(src.ctypes.data_as(C.POINTER(C.c_uint8)), n_rows, k,
                                                 x.ctypes.data_as(C.POINTER(C.c_float)), x.shape[0], 1 if exact else 0,
                                                 y.ctypes.data_as(C.POINTER(C.c_float)))
    if s != 0:
        _raise(s)
    return y


def kernel_mxfp4_scaled_time(n_rows: int, k: int, n_tokens: int, cold: bool = True, iters: int = 50, exact: bool = False) -> float:
    """Microseconds per launch of kernel_mxfp4_scaled's product on device-only data."""
    out = C.c_double()
    s = load_library().retro_kernel_mxfp4_scaled_time(n_rows, k, n_tokens, 1 if exact else 0, 1 if cold else 0, iters, C.byref(out))
    if s != 0:
        _raise(s)
    return out.value


def kernel_stream_time(n_bytes: int, read_only: bool = False, iters: int = 20) -> float:
    """Microseconds per launch of a plain copy (or pure read) of n_bytes."""
    out = C.c_double()
    s = load_library().retro_kernel_stream_time(n_bytes, 1 if read_only else 0, iters, C.byref(out))
    if s != 0:
        _raise(s)
    return out.value


def kernel_sample_prepare(logits: np.ndarray, k: Sequence[int]):
    lib = load_library()
    logits = np.ascontiguousarray(logits, np.float32)
    n, v = logits.shape
    kk = np.ascontiguousarray(k, np.int32)
    m = lib.retro_kernel_max_topk()
    argmax = np.zeros(n, np.int32)
    mx = np.zeros(n, np.float32)
    se = np.zeros(n, np.float64)
    ids = np.zeros((n, m), np.int32)
    vals = np.zeros((n, m), np.float32)
    s = lib.retro_kernel_sample_prepare(logits.ctypes.data_as(_f32p), n, v, kk.ctypes.data_as(_i32p),
                                        argmax.ctypes.data_as(_i32p), mx.ctypes.data_as(_f32p),
                                        se.ctypes.data_as(C.POINTER(C.c_double)), ids.ctypes.data_as(_i32p),
                                        vals.ctypes.data_as(_f32p))
    if s != 0:
        _raise(s)
    return argmax, mx, se, ids, vals


def kernel_sample_greedy_noalloc(d_logits: int, n_rows: int, n_vocab: int, d_argmax: int, d_max: int, d_sum_exp: int,
                                 stream: int = 0) -> None:
    """retro_kernel_sample_greedy_noalloc over raw device addresses (e.g. torch tensors' data_ptr()) on a HIP
    stream handle (0 = the default stream). Launches only: the caller synchronises its stream."""
    s = load_library().retro_kernel_sample_greedy_noalloc(d_logits, n_rows, n_vocab, d_argmax, d_max, d_sum_exp,
                                                          stream or None)
    if s != 0:
        _raise(s)
