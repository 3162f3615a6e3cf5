"""Rebuilds the reference's tiny GGUF fixtures byte for byte.

The reference pins the bytes of its generated fixtures by sha256
(reference tests/fixtures/TINY_FIXTURE.toml, TINY_F16_FIXTURE.toml,
TINY_Q8_FIXTURE.toml, TINY_MOE_FIXTURE.toml). Reproducing those digests with
this repository's own GGUF writer, f16 rounding and Q8_0 quantiser is a
known-answer test of all three: a wrong alignment, key order, rounding mode or
quantiser step changes the digest.

Recipe restated from reference scripts/gen-tiny-fixture.py:116-133 (xorshift64*
weights in [-1,1) from the 24 high bits), :167-170 (value = offset + scale*unit
snapped to the f16 grid), :226-262 (tensor order, per-tensor seed chain),
:294-335 (metadata order) and scripts/gen-tiny-moe-fixture.py:195-244, 272-323.
"""

from __future__ import annotations

import hashlib

import numpy as np

from retrograd_amd import gguf_writer as gw

MASK = (1 << 64) - 1

DIGESTS = {
    # name: (size_bytes, sha256)
    "qwen2-f32": (737952, "218570a8f7793864c8c1b4a6eb6d132c5ecff9e2432b8c0b41270a6901971f07"),
    "qwen2-f16": (376480, "f2abf21a1f4ffd7fe6cf433d2186027f3be9b7469c8cd0e3f8fa50dced4cf052"),
    "qwen2-q8_0": (207072, "f48a0e831ab1c16b07aa98b645205fb08e5c390ada539fa36052fc9e93463890"),
    "olmoe-f32": (1065440, "951939411c8fcfb8ededc826c4dd558674f04abfb9d751b53c62033436957a03"),
}


def xorshift_units(seed: int, count: int) -> np.ndarray:
    """`count` values in [-1, 1) of the xorshift64* stream seeded with seed|1."""
    state = (seed | 1) & MASK
    bits = np.empty(count, dtype=np.float64)
    for i in range(count):
        state ^= state >> 12
        state = (state ^ (state << 25)) & MASK
        state ^= state >> 27
        bits[i] = ((state * 0x2545F4914F6CDD1D) & MASK) >> 40
    return bits / float(1 << 24) * 2.0 - 1.0


def grid_values(seed: int, count: int, scale: float, offset: float) -> np.ndarray:
    """float64 values offset + scale*unit, rounded once to f16 (as float16)."""
    return (offset + scale * xorshift_units(seed, count)).astype(np.float16)


def next_seed(seed: int) -> int:
    return (seed * 6364136223846793005 + 1442695040888963407) & MASK


def vocabulary():
    tokens = ["<unk>", "<s>", "</s>"] + ["<0x%02X>" % b for b in range(256)] + ["▁the"]
    types = [2, 3, 3] + [6] * 256 + [1]
    return tokens, types


def encode_matrix(values_f16: np.ndarray, ggml_type: int, quantize_q8_0=None) -> np.ndarray:
    if ggml_type == gw.GGML_F32:
        return values_f16.astype(np.float32)
    if ggml_type == gw.GGML_F16:
        return values_f16
    if ggml_type == gw.GGML_Q8_0:
        return quantize_q8_0(values_f16.astype(np.float32))
    raise ValueError(ggml_type)


def _metadata(w: gw.GGUFWriter, arch: str, name: str, file_type: int, shape: dict, extra=()) -> None:
    tokens, types = vocabulary()
    w.add("general.architecture", gw.T_STRING, arch)
    w.add("general.name", gw.T_STRING, name)
    w.add("general.file_type", gw.T_UINT32, file_type)
    w.add(arch + ".block_count", gw.T_UINT32, shape["layers"])
    w.add(arch + ".context_length", gw.T_UINT32, 256)
    w.add(arch + ".embedding_length", gw.T_UINT32, shape["embd"])
    w.add(arch + ".feed_forward_length", gw.T_UINT32, shape["ff"])
    w.add(arch + ".attention.head_count", gw.T_UINT32, shape["heads"])
    w.add(arch + ".attention.head_count_kv", gw.T_UINT32, shape["heads_kv"])
    w.add(arch + ".attention.layer_norm_rms_epsilon", gw.T_FLOAT32, 1.0e-5)
    for key, value in extra:
        w.add(arch + "." + key, gw.T_UINT32, value)
    w.add(arch + ".rope.dimension_count", gw.T_UINT32, shape["embd"] // shape["heads"])
    w.add(arch + ".rope.freq_base", gw.T_FLOAT32, 10000.0)
    w.add("tokenizer.ggml.model", gw.T_STRING, "llama")
    w.add("tokenizer.ggml.tokens", gw.T_ARRAY, tokens, gw.T_STRING)
    w.add("tokenizer.ggml.scores", gw.T_ARRAY, [0.0] * len(tokens), gw.T_FLOAT32)
    w.add("tokenizer.ggml.token_type", gw.T_ARRAY, types, gw.T_INT32)
    w.add("tokenizer.ggml.bos_token_id", gw.T_UINT32, 1)
    w.add("tokenizer.ggml.eos_token_id", gw.T_UINT32, 2)
    w.add("tokenizer.ggml.unknown_token_id", gw.T_UINT32, 0)
    w.add("tokenizer.ggml.add_bos_token", gw.T_BOOL, True)
    w.add("tokenizer.ggml.add_eos_token", gw.T_BOOL, False)
    w.add("general.alignment", gw.T_UINT32, 32)


class _Chain:
    """Adds tensors in order, advancing the per-tensor seed chain."""

    def __init__(self, writer: gw.GGUFWriter, matrix_type: int, quantize_q8_0=None) -> None:
        self.w = writer
        self.matrix_type = matrix_type
        self.q8 = quantize_q8_0
        self.seed = 0x9E3779B97F4A7C15

    def add(self, name, ne, scale, offset=0.0, patch=None) -> None:
        count = int(np.prod(ne))
        values = grid_values(self.seed, count, scale, offset)
        if patch is not None:
            patch(values)
        self.put(name, ne, values)

    def put(self, name, ne, values_f16: np.ndarray) -> None:
        ggml_type = self.matrix_type if len(ne) > 1 else gw.GGML_F32
        self.w.add_tensor(name, ne, ggml_type, encode_matrix(values_f16, ggml_type, self.q8))
        self.seed = next_seed(self.seed)


def build_qwen2(dtype: str, quantize_q8_0=None) -> bytes:
    """The reference's tiny qwen2 fixture: 4 layers, embd 64, 4 heads / 2 kv, ff 128."""
    matrix_type, file_type = {"f32": (gw.GGML_F32, 0), "f16": (gw.GGML_F16, 1), "q8_0": (gw.GGML_Q8_0, 7)}[dtype]
    shape = dict(layers=4, embd=64, heads=4, heads_kv=2, ff=128)
    E, F = shape["embd"], shape["ff"]
    GQA = E // shape["heads"] * shape["heads_kv"]
    V = len(vocabulary()[0])
    w = gw.GGUFWriter()
    _metadata(w, "qwen2", "retrograd-tiny-qwen2", file_type, shape)
    c = _Chain(w, matrix_type, quantize_q8_0)
    c.add("token_embd.weight", [E, V], 0.08)
    for l in range(shape["layers"]):
        b = "blk.%d." % l
        c.add(b + "attn_norm.weight", [E], 0.02, 1.0)
        c.add(b + "attn_q.weight", [E, E], 0.08)
        c.add(b + "attn_q.bias", [E], 0.01)
        c.add(b + "attn_k.weight", [E, GQA], 0.08)
        c.add(b + "attn_k.bias", [GQA], 0.01)
        c.add(b + "attn_v.weight", [E, GQA], 0.08)
        c.add(b + "attn_v.bias", [GQA], 0.01)
        c.add(b + "attn_output.weight", [E, E], 0.08)
        c.add(b + "ffn_norm.weight", [E], 0.02, 1.0)
        c.add(b + "ffn_gate.weight", [E, F], 0.08)
        c.add(b + "ffn_up.weight", [E, F], 0.08)
        c.add(b + "ffn_down.weight", [F, E], 0.08)
    c.add("output_norm.weight", [E], 0.02, 1.0)
    c.add("output.weight", [E, V], 0.08)
    c.add("output.bias", [V], 0.01)
    return w.to_bytes()


def build_olmoe_f32() -> bytes:
    """The reference's tiny OLMoE fixture (concentrated router): 2 layers, embd 64,
    4 heads, ff 64, 8 experts of which 2 are used."""
    shape = dict(layers=2, embd=64, heads=4, heads_kv=4, ff=64)
    E, F, NE, NU = 64, 64, 8, 2
    V = len(vocabulary()[0])
    w = gw.GGUFWriter()
    _metadata(w, "olmoe", "retrograd-tiny-olmoe", 0, shape,
              extra=(("expert_count", NE), ("expert_used_count", NU)))
    c = _Chain(w, gw.GGML_F32)

    def embd_patch(v):
        v[::E] = np.float16(0.125)

    def attn_out_patch(v):
        v[:E] = 0

    def down_patch(v):
        stride = F * E
        for start in range(0, v.size, stride):
            v[start:start + F] = 0

    c.add("token_embd.weight", [E, V], 0.08, patch=embd_patch)
    for l in range(shape["layers"]):
        b = "blk.%d." % l
        c.add(b + "attn_norm.weight", [E], 0.02, 1.0)
        c.add(b + "attn_q.weight", [E, E], 0.08)
        c.add(b + "attn_k.weight", [E, E], 0.08)
        c.add(b + "attn_v.weight", [E, E], 0.08)
        c.add(b + "attn_q_norm.weight", [E], 0.02, 1.0)
        c.add(b + "attn_k_norm.weight", [E], 0.02, 1.0)
        c.add(b + "attn_output.weight", [E, E], 0.08, patch=attn_out_patch)
        c.add(b + "ffn_norm.weight", [E], 0.02, 1.0)
        router = np.zeros(E * NE, np.float16)
        router[::E] = [0.0625 if e < NU else -0.0625 for e in range(NE)]
        c.put(b + "ffn_gate_inp.weight", [E, NE], router)
        c.add(b + "ffn_gate_exps.weight", [E, F, NE], 0.08)
        c.add(b + "ffn_up_exps.weight", [E, F, NE], 0.08)
        c.add(b + "ffn_down_exps.weight", [F, E, NE], 0.08, patch=down_patch)
    c.add("output_norm.weight", [E], 0.02, 1.0)
    c.add("output.weight", [E, V], 0.08)
    return w.to_bytes()


def digest(data: bytes):
    return len(data), hashlib.sha256(data).hexdigest()


if __name__ == "__main__":
    import oracle

    for name, blob in (("qwen2-f32", build_qwen2("f32")), ("qwen2-f16", build_qwen2("f16")),
                       ("qwen2-q8_0", build_qwen2("q8_0", oracle.quantize_q8_0)), ("olmoe-f32", build_olmoe_f32())):
        print(name, digest(blob), digest(blob) == DIGESTS[name])
