"""CPU oracle of the decode step - TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; the product (retrograd_amd) never does. It loads
oracle/_build/liboracle.so, built by oracle/Makefile from the C++ restatement
in this directory.
"""

from __future__ import annotations

import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
_LIB_PATH = _DIR / "_build" / "liboracle.so"
_lib = None


def build(force: bool = False) -> Path:
    """Compiles the oracle with g++ (seconds)."""
    args = ["make", "-C", str(_DIR)] + (["-B"] if force else [])
    subprocess.run(args, check=True, capture_output=True)
    return _LIB_PATH


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        _lib = C.CDLL(str(_LIB_PATH))
        _declare(_lib)
    return _lib


_i32p = C.POINTER(C.c_int32)
_u32p = C.POINTER(C.c_uint32)
_u8p = C.POINTER(C.c_uint8)
_u16p = C.POINTER(C.c_uint16)
_f32p = C.POINTER(C.c_float)
_f64p = C.POINTER(C.c_double)
_i64p = C.POINTER(C.c_int64)


def _declare(l: C.CDLL) -> None:
    l.orc_last_error.restype = C.c_char_p
    l.orc_decode_row.argtypes = [C.c_uint32, _u8p, C.c_size_t, _f32p]
    l.orc_row_bytes.argtypes = [C.c_uint32, C.c_size_t, C.POINTER(C.c_size_t)]
    l.orc_quantize_q8_0.argtypes = [_f32p, C.c_size_t, _u8p]
    l.orc_half_to_float.argtypes = [_u16p, C.c_size_t, _f32p]
    l.orc_half_to_float.restype = None
    l.orc_float_to_half.argtypes = [_f32p, C.c_size_t, _u16p]
    l.orc_float_to_half.restype = None
    l.orc_double_to_half.argtypes = [_f64p, C.c_size_t, _u16p]
    l.orc_double_to_half.restype = None
    l.orc_activation_row.argtypes = [C.c_uint32, _f32p, C.c_size_t, _f32p]
    l.orc_matmul.argtypes = [C.c_uint32, _u8p, C.c_size_t, C.c_size_t, _f32p, C.c_int, _f32p]
    l.orc_set_exact_activations.argtypes = [C.c_int]
    l.orc_set_exact_activations.restype = None
    l.orc_e8m0_half.argtypes = [C.c_uint8]
    l.orc_e8m0_half.restype = C.c_float
    l.orc_pack_rows.argtypes = [C.c_size_t, _i32p, _i32p, _u32p, _u8p, _i32p,
                                _i32p, _i32p, _i32p, _u8p, _i32p, _i32p, _i32p, C.POINTER(C.c_size_t)]
    l.orc_pack_cells.argtypes = [C.c_size_t, _i32p, _i32p, _i32p, C.c_size_t, C.c_int32, _i64p]
    l.orc_model_load.argtypes = [C.c_char_p]
    l.orc_model_load.restype = C.c_void_p
    l.orc_model_free.argtypes = [C.c_void_p]
    l.orc_model_free.restype = None
    l.orc_model_info.argtypes = [C.c_void_p, _i32p]
    l.orc_adapter_load.argtypes = [C.c_void_p, C.c_char_p, C.c_float, _i32p]
    l.orc_ctx_new.argtypes = [C.c_void_p, C.c_int]
    l.orc_ctx_new.restype = C.c_void_p
    l.orc_ctx_set_exact.argtypes = [C.c_void_p, C.c_int]
    l.orc_ctx_set_exact.restype = None
    l.orc_ctx_set_kv_q8.argtypes = [C.c_void_p, C.c_int]
    l.orc_ctx_set_kv_q8.restype = None
    l.orc_ctx_read_kv_f32.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, _f32p]
    l.orc_ctx_import_kv_f32.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, _f32p, _f32p]
    l.orc_ctx_free.argtypes = [C.c_void_p]
    l.orc_ctx_free.restype = None
    l.orc_ctx_step.argtypes = [C.c_void_p, C.c_int, _i32p, _i32p, _i32p, _i32p, _u8p, _f32p]
    l.orc_ctx_seq_rm.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int]
    l.orc_ctx_seq_cp.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int]
    l.orc_ctx_seq_pos.argtypes = [C.c_void_p, C.c_int, _i32p, _i32p]
    l.orc_ctx_read_kv.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, _u16p]
    l.orc_ctx_import_kv.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, _u16p, _u16p]
    l.orc_rng_new.argtypes = [C.c_uint32]
    l.orc_rng_new.restype = C.c_void_p
    l.orc_rng_free.argtypes = [C.c_void_p]
    l.orc_rng_free.restype = None
    l.orc_rng_uniform.argtypes = [C.c_void_p, C.c_double]
    l.orc_rng_uniform.restype = C.c_double
    l.orc_rng_u32.argtypes = [C.c_void_p]
    l.orc_rng_u32.restype = C.c_uint32
    l.orc_sample_v1.argtypes = [_f32p, C.c_size_t, C.c_float, C.c_float, C.c_void_p,
                                _i32p, _f32p, C.c_size_t, _i32p, _f32p]
    l.orc_sample_v2.argtypes = [_f32p, C.c_size_t, C.c_float, C.c_float, C.c_int32, C.c_float,
                                C.c_float, C.c_float, C.c_float, C.c_uint32, C.c_uint32, _i32p, _f32p,
                                C.c_void_p, _i32p, C.c_size_t, _i32p, _f32p, _f32p,
                                C.c_size_t, _i32p, _f32p, _u8p]
    l.orc_token_logprob.argtypes = [_f32p, C.c_size_t, C.c_int32]
    l.orc_token_logprob.restype = C.c_float
    l.orc_top_logprobs.argtypes = [_f32p, C.c_size_t, C.c_size_t, _i32p, _f32p]


class OracleError(RuntimeError):
    pass


def _check(status: int) -> None:
    if status != 0:
        raise OracleError(lib().orc_last_error().decode())


def _ptr(a: np.ndarray, t):
    return a.ctypes.data_as(t)


# ---- block formats -----------------------------------------------------------

def decode_row(ggml_type: int, raw, n: int) -> np.ndarray:
    src = np.frombuffer(bytes(raw), dtype=np.uint8) if not isinstance(raw, np.ndarray) else np.ascontiguousarray(raw, dtype=np.uint8)
    out = np.empty(n, dtype=np.float32)
    _check(lib().orc_decode_row(ggml_type, _ptr(src, _u8p), n, _ptr(out, _f32p)))
    return out


def activation_row(weight_type: int, x: np.ndarray) -> np.ndarray:
    """The activations a weight of `weight_type` is multiplied with on ggml's CPU path."""
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    out = np.empty_like(x)
    _check(lib().orc_activation_row(weight_type, _ptr(x, _f32p), x.size, _ptr(out, _f32p)))
    return out


def matmul(ggml_type: int, raw, n_rows: int, k: int, x: np.ndarray) -> np.ndarray:
    """x [T, k] times the n_rows raw rows, activations converted as ggml's CPU path does."""
    src = np.ascontiguousarray(raw, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k)
    y = np.empty((x.shape[0], n_rows), np.float32)
    _check(lib().orc_matmul(ggml_type, _ptr(src, _u8p), k, n_rows, _ptr(x, _f32p), x.shape[0], _ptr(y, _f32p)))
    return y


def set_exact_activations(on: bool) -> None:
    """Matmuls of the forward pass take f32 activations as they are (measurements only)."""
    lib().orc_set_exact_activations(1 if on else 0)


def row_bytes(ggml_type: int, n: int) -> int:
    out = C.c_size_t()
    _check(lib().orc_row_bytes(ggml_type, n, C.byref(out)))
    return out.value


def quantize_q8_0(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    out = np.empty(x.size // 32 * 34, dtype=np.uint8)
    _check(lib().orc_quantize_q8_0(_ptr(x, _f32p), x.size, _ptr(out, _u8p)))
    return out


def half_to_float(h: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().orc_half_to_float(_ptr(h, _u16p), h.size, _ptr(out, _f32p))
    return out


def float_to_half(f: np.ndarray) -> np.ndarray:
    f = np.ascontiguousarray(f, dtype=np.float32)
    out = np.empty(f.shape, dtype=np.uint16)
    lib().orc_float_to_half(_ptr(f, _f32p), f.size, _ptr(out, _u16p))
    return out


def double_to_half(f: np.ndarray) -> np.ndarray:
    f = np.ascontiguousarray(f, dtype=np.float64)
    out = np.empty(f.shape, dtype=np.uint16)
    lib().orc_double_to_half(_ptr(f, _f64p), f.size, _ptr(out, _u16p))
    return out


def e8m0_half(x: int) -> float:
    return float(lib().orc_e8m0_half(x))


# ---- packing -----------------------------------------------------------------

def pack_rows(rows):
    """rows: iterable of (slot, pos0, tokens, sample). Returns a dict of the flat
    arrays of one step's batch."""
    rows = list(rows)
    slot = np.array([r[0] for r in rows], dtype=np.int32)
    pos0 = np.array([r[1] for r in rows], dtype=np.int32)
    n = np.array([len(r[2]) for r in rows], dtype=np.uint32)
    sample = np.array([1 if r[3] else 0 for r in rows], dtype=np.uint8)
    toks = np.concatenate([np.asarray(r[2], dtype=np.int32) for r in rows]) if rows else np.zeros(0, np.int32)
    total = int(n.sum())
    out = {
        "token": np.empty(total, np.int32), "pos": np.empty(total, np.int32),
        "seq": np.empty(total, np.int32), "output": np.empty(total, np.uint8),
        "row": np.empty(total, np.int32), "last_index": np.full(len(rows), -1, np.int32),
        "row_offset": np.empty(len(rows) + 1, np.int32),
    }
    got = C.c_size_t()
    _check(lib().orc_pack_rows(len(rows), _ptr(slot, _i32p), _ptr(pos0, _i32p), _ptr(n, _u32p),
                               _ptr(sample, _u8p), _ptr(toks, _i32p),
                               _ptr(out["token"], _i32p), _ptr(out["pos"], _i32p), _ptr(out["seq"], _i32p),
                               _ptr(out["output"], _u8p), _ptr(out["row"], _i32p),
                               _ptr(out["last_index"], _i32p), _ptr(out["row_offset"], _i32p), C.byref(got)))
    assert got.value == total
    return out


def pack_cells(pos: np.ndarray, seq: np.ndarray, table: np.ndarray, page: int) -> np.ndarray:
    pos = np.ascontiguousarray(pos, np.int32)
    seq = np.ascontiguousarray(seq, np.int32)
    table = np.ascontiguousarray(table, np.int32)
    out = np.empty(pos.size, np.int64)
    _check(lib().orc_pack_cells(pos.size, _ptr(pos, _i32p), _ptr(seq, _i32p), _ptr(table, _i32p),
                                table.shape[1], page, _ptr(out, _i64p)))
    return out


# ---- model -------------------------------------------------------------------

class Model:
    def __init__(self, path) -> None:
        self._h = lib().orc_model_load(os.fsencode(str(path)))
        if not self._h:
            raise OracleError(lib().orc_last_error().decode())
        info = np.zeros(12, np.int32)
        _check(lib().orc_model_info(self._h, _ptr(info, _i32p)))
        (self.n_layer, self.n_embd, self.n_head, self.n_head_kv, self.head_dim, self.n_ff,
         self.n_vocab, self.n_expert, self.n_expert_used, self.n_ff_exp, neox, self.rope_dim) = (int(v) for v in info)
        self.rope_neox = bool(neox)

    def load_adapter(self, path, scale: float = 1.0) -> int:
        out = C.c_int32()
        _check(lib().orc_adapter_load(self._h, os.fsencode(str(path)), scale, C.byref(out)))
        return out.value

    def close(self) -> None:
        if self._h:
            lib().orc_model_free(self._h)
            self._h = None

    def __del__(self) -> None:
        try:
            self.close()
        except Exception:
            pass


class Context:
    """Per-slot dense KV (f16, or Q8_0 / Q4_0 blocks with kv="q8_0" / "q4_0") and one decode per step() over a packed batch.

    activations: "exact" multiplies every weight with the f32 activations as they
    are (the product's default arithmetic, on which the logit tolerances are
    demonstrated); "ggml" converts them first as ggml's CPU matmul does (Q8_K /
    Q8_0 codes, f16 / bf16 rounding: the reference's CPU arithmetic, which the
    product runs under RETRO_ACTIVATIONS=ggml)."""

    def __init__(self, model: Model, n_seq_max: int, activations: str = "exact", kv: str = "f16") -> None:
        if activations not in ("exact", "ggml"):
            raise ValueError("activations must be 'exact' or 'ggml'")
        if kv not in ("f16", "q8_0", "q4_0"):
            raise ValueError("kv must be 'f16', 'q8_0' or 'q4_0'")
        self.model = model
        self._h = lib().orc_ctx_new(model._h, n_seq_max)
        if not self._h:
            raise OracleError(lib().orc_last_error().decode())
        lib().orc_ctx_set_exact(self._h, 1 if activations == "exact" else 0)
        lib().orc_ctx_set_kv_q8(self._h, {"f16": 0, "q8_0": 8, "q4_0": 4}[kv])

    def step(self, token, pos, slot, want, adapter_of=None) -> np.ndarray:
        token = np.ascontiguousarray(token, np.int32)
        pos = np.ascontiguousarray(pos, np.int32)
        slot = np.ascontiguousarray(slot, np.int32)
        want = np.ascontiguousarray(want, np.uint8)
        n_out = int(want.astype(bool).sum())
        logits = np.empty((n_out, self.model.n_vocab), np.float32)
        ad = None
        if adapter_of is not None:
            ad_arr = np.ascontiguousarray(adapter_of, np.int32)
            ad = _ptr(ad_arr, _i32p)
        _check(lib().orc_ctx_step(self._h, token.size, _ptr(token, _i32p), _ptr(pos, _i32p), _ptr(slot, _i32p),
                                  ad, _ptr(want, _u8p), _ptr(logits, _f32p)))
        return logits

    def step_rows(self, rows, adapters=None) -> np.ndarray:
        """rows: (slot, pos0, tokens, sample); returns the logits of sampling rows."""
        p = pack_rows(rows)
        adapter_of = None
        if adapters is not None:
            adapter_of = np.array([adapters[r] for r in p["row"]], np.int32)
        return self.step(p["token"], p["pos"], p["seq"], p["output"], adapter_of)

    def seq_rm(self, slot, p0=-1, p1=-1) -> None:
        _check(lib().orc_ctx_seq_rm(self._h, slot, p0, p1))

    def seq_cp(self, src, dst, p0=-1, p1=-1) -> None:
        _check(lib().orc_ctx_seq_cp(self._h, src, dst, p0, p1))

    def seq_pos(self, slot):
        a, b = C.c_int32(), C.c_int32()
        _check(lib().orc_ctx_seq_pos(self._h, slot, C.byref(a), C.byref(b)))
        return a.value, b.value

    def read_kv_values(self, layer, slot, pos, want_v=False) -> np.ndarray:
        """The stored K or V row as the values the cache holds (f16-rounded, or scale times code of a Q8_0 cache)."""
        out = np.empty(self.model.n_head_kv * self.model.head_dim, np.float32)
        _check(lib().orc_ctx_read_kv_f32(self._h, layer, slot, pos, 1 if want_v else 0, _ptr(out, _f32p)))
        return out

    def read_kv(self, layer, slot, pos, want_v=False) -> np.ndarray:
        out = np.empty(self.model.n_head_kv * self.model.head_dim, np.uint16)
        _check(lib().orc_ctx_read_kv(self._h, layer, slot, pos, 1 if want_v else 0, _ptr(out, _u16p)))
        return out.view(np.float16)

    def import_kv(self, layer, slot, begin, end, k_rows: np.ndarray, v_rows: np.ndarray) -> None:
        k = np.ascontiguousarray(k_rows).view(np.uint16)
        v = np.ascontiguousarray(v_rows).view(np.uint16)
        _check(lib().orc_ctx_import_kv(self._h, layer, slot, begin, end, _ptr(k, _u16p), _ptr(v, _u16p)))

    def import_snapshot(self, slot: int, snapshot: bytes) -> None:
        """Loads a sequence snapshot written by the engine's seq_save (header of
        six 32-bit words: magic, flags, n_layer, kv_dim, begin, end; then per
        layer the K rows and the V rows as f16)."""
        head = np.frombuffer(snapshot, np.int32, 6)
        n_layer, kd, begin, end = (int(v) for v in head[2:6])
        n = end - begin
        body = np.frombuffer(snapshot, np.uint16, offset=24)
        per = n * kd
        if int(head[0]) == 0x38564b52:
            # a Q8_0 cache ("RKV8"): per row and kv head head_dim code bytes (code + 128), then head_dim / 32 f16 scales
            hd, n_kv = self.model.head_dim, self.model.n_head_kv
            per_head = hd // 2 + hd // 32
            assert kd == n_kv * per_head

            def values(units):
                rows = units.reshape(n, n_kv, per_head)
                codes = np.ascontiguousarray(rows[:, :, :hd // 2]).view(np.uint8).astype(np.float32) - 128.0
                scales = np.ascontiguousarray(rows[:, :, hd // 2:]).view(np.float16).astype(np.float32)
                return np.ascontiguousarray((codes.reshape(n, n_kv, hd // 32, 32) * scales[..., None]).reshape(n, n_kv * hd))
            for l in range(n_layer):
                k = values(body[(2 * l) * per:(2 * l + 1) * per])
                v = values(body[(2 * l + 1) * per:(2 * l + 2) * per])
                _check(lib().orc_ctx_import_kv_f32(self._h, l, slot, begin, end, _ptr(k, _f32p), _ptr(v, _f32p)))
            return
        if int(head[0]) == 0x34564b52:
            # a Q4_0 cache ("RKV4"): per row and kv head head_dim / 2 code bytes (element 2 k in the low nibble of
            # byte k), then head_dim / 32 f16 scales; a value is scale times (code - 8)
            hd, n_kv = self.model.head_dim, self.model.n_head_kv
            per_head = hd // 4 + hd // 32
            assert kd == n_kv * per_head

            def values4(units):
                rows = units.reshape(n, n_kv, per_head)
                packed = np.ascontiguousarray(rows[:, :, :hd // 4]).view(np.uint8)
                codes = np.stack([packed & 15, packed >> 4], axis=-1).reshape(n, n_kv, hd).astype(np.float32) - 8.0
                scales = np.ascontiguousarray(rows[:, :, hd // 4:]).view(np.float16).astype(np.float32)
                return np.ascontiguousarray((codes.reshape(n, n_kv, hd // 32, 32) * scales[..., None]).reshape(n, n_kv * hd))
            for l in range(n_layer):
                k = values4(body[(2 * l) * per:(2 * l + 1) * per])
                v = values4(body[(2 * l + 1) * per:(2 * l + 2) * per])
                _check(lib().orc_ctx_import_kv_f32(self._h, l, slot, begin, end, _ptr(k, _f32p), _ptr(v, _f32p)))
            return
        for l in range(n_layer):
            k = body[(2 * l) * per:(2 * l + 1) * per]
            v = body[(2 * l + 1) * per:(2 * l + 2) * per]
            self.import_kv(l, slot, begin, end, k, v)

    def close(self) -> None:
        if self._h:
            lib().orc_ctx_free(self._h)
            self._h = None

    def __del__(self) -> None:
        try:
            self.close()
        except Exception:
            pass


# ---- sampling ----------------------------------------------------------------

class Rng:
    """std::mt19937 seeded once, as the reference seeds a request's generator."""

    def __init__(self, seed: int) -> None:
        self._h = lib().orc_rng_new(seed & 0xFFFFFFFF)

    def uniform(self, hi: float = 1.0) -> float:
        return float(lib().orc_rng_uniform(self._h, hi))

    def u32(self) -> int:
        return int(lib().orc_rng_u32(self._h))

    def __del__(self) -> None:
        try:
            lib().orc_rng_free(self._h)
        except Exception:
            pass


def sample_v1(logits: np.ndarray, temperature: float, top_p: float, rng: Rng, k: int = 0):
    logits = np.ascontiguousarray(logits, np.float32)
    tok, lp = C.c_int32(), C.c_float()
    ids = np.empty(max(k, 1), np.int32)
    lps = np.empty(max(k, 1), np.float32)
    _check(lib().orc_sample_v1(_ptr(logits, _f32p), logits.size, temperature, top_p, rng._h,
                               C.byref(tok), C.byref(lp), k, _ptr(ids, _i32p), _ptr(lps, _f32p)))
    return tok.value, lp.value, ids[:k], lps[:k]


def sample_v2(logits: np.ndarray, rng: Rng, *, temperature=1.0, top_p=1.0, top_k=0, min_p=0.0,
              repeat_penalty=1.0, frequency_penalty=0.0, presence_penalty=0.0, penalty_window=0,
              bias_ids=(), bias_values=(), history=(), k: int = 0, allowed=None):
    """`allowed`: one flag per token, the set a grammar leaves at this position (None: no grammar)."""
    logits = np.ascontiguousarray(logits, np.float32)
    mask = None if allowed is None else np.ascontiguousarray(allowed, np.uint8)
    assert mask is None or mask.size == logits.size
    bi = np.asarray(bias_ids, np.int32)
    bv = np.asarray(bias_values, np.float32)
    hist = np.asarray(history, np.int32)
    tok, lp, slp = C.c_int32(), C.c_float(), C.c_float()
    ids = np.empty(max(k, 1), np.int32)
    lps = np.empty(max(k, 1), np.float32)
    _check(lib().orc_sample_v2(_ptr(logits, _f32p), logits.size, temperature, top_p, top_k, min_p,
                               repeat_penalty, frequency_penalty, presence_penalty, penalty_window,
                               bi.size, _ptr(bi, _i32p), _ptr(bv, _f32p), rng._h,
                               _ptr(hist, _i32p), hist.size, C.byref(tok), C.byref(lp), C.byref(slp),
                               k, _ptr(ids, _i32p), _ptr(lps, _f32p), None if mask is None else _ptr(mask, _u8p)))
    return tok.value, lp.value, slp.value, ids[:k], lps[:k]


def token_logprob(logits: np.ndarray, token: int) -> float:
    logits = np.ascontiguousarray(logits, np.float32)
    return float(lib().orc_token_logprob(_ptr(logits, _f32p), logits.size, token))


def top_logprobs(logits: np.ndarray, k: int):
    logits = np.ascontiguousarray(logits, np.float32)
    ids = np.empty(k, np.int32)
    lps = np.empty(k, np.float32)
    _check(lib().orc_top_logprobs(_ptr(logits, _f32p), logits.size, k, _ptr(ids, _i32p), _ptr(lps, _f32p)))
    return ids, lps
