"""Synthetic random-weight GGUF models of the benchmark shapes.

Weights are N(0, 0.02) from a seeded torch generator, norm vectors are 1, and
matrices are quantised block by block into the GGUF storage formats the decode
step reads (Q8_0, Q4_K, MXFP4, F16). The quantisers here only have to produce
*valid blocks*: parity is always "the same stored bytes decoded two ways"
(reference crates/rir-core/src/quant.rs:1-6), never two quantisations compared.
Block layouts follow reference crates/rir-core/src/quant.rs:119-128 (Q4_K 6-bit
scale/min packing), :286-295 (MXFP4: E8M0 byte then low/high nibble halves) and
scripts/gen-tiny-fixture.py:173-197 (Q8_0).
"""

from __future__ import annotations

from dataclasses import dataclass, field, replace
from pathlib import Path

import numpy as np
import torch

from . import gguf_writer as gw


@dataclass(frozen=True)
class ModelShape:
    arch: str
    n_layer: int
    n_embd: int
    n_head: int
    n_head_kv: int
    head_dim: int
    n_ff: int
    n_vocab: int
    rope_base: float
    matrix_type: int                 # ggml type of the 2-D matrices
    n_expert: int = 0
    n_expert_used: int = 0
    n_ff_exp: int = 0
    expert_type: int = gw.GGML_MXFP4
    expert_down_type: int = -1       # ffn_down_exps on the finer layers (-1: expert_type)
    qkv_bias: bool = False
    eps: float = 1e-5
    name: str = "synthetic"
    # the mix of a Q4_K_M file: some matrices kept at a finer type (-1: matrix_type)
    output_type: int = -1            # output.weight
    down_type: int = -1              # ffn_down.weight
    v_type: int = -1                 # attn_v.weight
    rope_freqs: bool = False         # write rope_freqs.weight: per-frequency divisors of the rotation angle as
                                     # Llama 3.1's rule gives them (1 for short wavelengths, 8 for long, a ramp between)
    rope_scaling_linear: float = 0.0 # > 0: rope.scaling.type = linear with this factor
    rope_scaling_yarn: float = 0.0   # > 0: rope.scaling.type = yarn with this factor ...
    rope_original_context: int = 0   # ... over this original context length
    norm_std: float = 0.0            # > 0: norm vectors are 1 + norm_std * N(0, 1) instead of all ones, so that a test
                                     # can tell whether (and where) a norm weight is applied
    finer_layers: str = "all"        # layers whose ffn_down / attn_v take the finer type: "all", or "more_bits" =
                                     # the first and last eighth and every third layer between (llama.cpp's rule for Q4_K_M)


# The five benchmark configurations.
TINY_LLAMA = ModelShape("llama", 2, 128, 4, 2, 32, 344, 512, 10000.0, gw.GGML_Q8_0, name="tiny-llama-q8_0")
LLAMA3_8B_Q4K = ModelShape("llama", 32, 4096, 32, 8, 128, 14336, 128256, 500000.0, gw.GGML_Q4_K,
                           name="llama3-8b-shape-q4_k")
# the same shape with the type mix of a Q4_K_M file: output.weight in Q6_K, ffn_down and attn_v in Q6_K on llama.cpp's layers
LLAMA3_8B_Q4K_M = ModelShape("llama", 32, 4096, 32, 8, 128, 14336, 128256, 500000.0, gw.GGML_Q4_K,
                             output_type=gw.GGML_Q6_K, down_type=gw.GGML_Q6_K, v_type=gw.GGML_Q6_K, finer_layers="more_bits",
                             name="llama3-8b-shape-q4_k_m")
QWEN25_7B_Q8 = ModelShape("qwen2", 28, 3584, 28, 4, 128, 18944, 152064, 1000000.0, gw.GGML_Q8_0,
                          qkv_bias=True, name="qwen2.5-7b-shape-q8_0")
QWEN3_30B_A3B = ModelShape("qwen3moe", 48, 2048, 32, 4, 128, 6144, 151936, 1000000.0, gw.GGML_Q8_0,
                           n_expert=128, n_expert_used=8, n_ff_exp=768, eps=1e-6,
                           name="qwen3-30b-a3b-shape-mxfp4")


def finer_layer(shape: ModelShape, layer: int) -> bool:
    """Whether `layer` stores ffn_down and attn_v at the finer type (down_type / v_type)."""
    if shape.finer_layers == "all":
        return True
    n = shape.n_layer
    return layer < n // 8 or layer >= 7 * n // 8 or (layer - n // 8) % 3 == 2


def matrix_types(shape: ModelShape):
    """(name, n_in, n_out, ggml type) of every dense 2-D matrix of a non-expert model, in file order without the
    token embedding: what a decode step streams once."""
    s = shape
    E, QD, KD = s.n_embd, s.n_head * s.head_dim, s.n_head_kv * s.head_dim
    out = []
    for l in range(s.n_layer):
        fine = finer_layer(s, l)
        b = "blk.%d." % l
        out.append((b + "attn_q.weight", E, QD, s.matrix_type))
        out.append((b + "attn_k.weight", E, KD, s.matrix_type))
        out.append((b + "attn_v.weight", E, KD, s.v_type if (s.v_type >= 0 and fine) else s.matrix_type))
        out.append((b + "attn_output.weight", QD, E, s.matrix_type))
        out.append((b + "ffn_gate.weight", E, s.n_ff, s.matrix_type))
        out.append((b + "ffn_up.weight", E, s.n_ff, s.matrix_type))
        out.append((b + "ffn_down.weight", s.n_ff, E, s.down_type if (s.down_type >= 0 and fine) else s.matrix_type))
    out.append(("output.weight", E, s.n_vocab, s.output_type if s.output_type >= 0 else s.matrix_type))
    return out


def streamed_weight_bytes(shape: ModelShape) -> int:
    """Bytes of the matrices a decode step of a non-expert model reads once (stored types as written)."""
    total = 0
    for _, n_in, n_out, t in matrix_types(shape):
        el, by = gw.BLOCK_GEOMETRY[storage_type(t, n_in)]
        total += n_in // el * by * n_out
    return total


def scaled(shape: ModelShape, **kw) -> ModelShape:
    """The same architecture at reduced depth/width, for parity runs the CPU oracle finishes in seconds."""
    return replace(shape, **kw)


# ---- quantisers (torch, any device) -------------------------------------------

def _round_half_away(x: torch.Tensor) -> torch.Tensor:
    return torch.sign(x) * torch.floor(torch.abs(x) + 0.5)


def quantize_q8_0(x: torch.Tensor) -> torch.Tensor:
    """[rows, K] float -> uint8 [rows, K/32*34]."""
    rows, K = x.shape
    b = x.reshape(rows, K // 32, 32).float()
    amax = b.abs().amax(dim=-1, keepdim=True)
    d = amax / 127.0
    inv = torch.where(d != 0, 1.0 / d, torch.zeros_like(d))
    q = _round_half_away(b * inv).clamp_(-127, 127).to(torch.int8)
    out = torch.empty(rows, K // 32, 34, dtype=torch.uint8, device=x.device)
    out[..., 0:2] = d.to(torch.float16).view(torch.uint8).reshape(rows, K // 32, 2)
    out[..., 2:] = q.view(torch.uint8)
    return out.reshape(rows, -1)


def quantize_q4_k(x: torch.Tensor) -> torch.Tensor:
    """[rows, K] float -> uint8 [rows, K/256*144]. Min/max affine per 32-element
    sub-block, 6-bit sub-block scales and mins against f16 super-block d/dmin."""
    rows, K = x.shape
    nb = K // 256
    b = x.reshape(rows, nb, 8, 32).float()
    mn = b.amin(dim=-1).clamp(max=0.0)
    mx = b.amax(dim=-1).clamp(min=0.0)
    scale = (mx - mn) / 15.0
    nmin = -mn
    d = (scale.amax(dim=-1, keepdim=True) / 63.0).to(torch.float16)
    dmin = (nmin.amax(dim=-1, keepdim=True) / 63.0).to(torch.float16)
    df, dminf = d.float(), dmin.float()
    sc = torch.where(df > 0, torch.round(scale / df.clamp(min=1e-30)), torch.zeros_like(scale)).clamp_(0, 63)
    m = torch.where(dminf > 0, torch.round(nmin / dminf.clamp(min=1e-30)), torch.zeros_like(nmin)).clamp_(0, 63)
    dl = (df * sc).unsqueeze(-1)
    ml = (dminf * m).unsqueeze(-1)
    q = torch.where(dl > 0, torch.round((b + ml) / dl.clamp(min=1e-30)), torch.zeros_like(b)).clamp_(0, 15).to(torch.uint8)
    sc = sc.to(torch.uint8)
    m = m.to(torch.uint8)
    out = torch.empty(rows, nb, 144, dtype=torch.uint8, device=x.device)
    out[..., 0:2] = d.view(torch.uint8).reshape(rows, nb, 2)
    out[..., 2:4] = dmin.view(torch.uint8).reshape(rows, nb, 2)
    out[..., 4:8] = (sc[..., 0:4] & 63) | ((sc[..., 4:8] >> 4) << 6)
    out[..., 8:12] = (m[..., 0:4] & 63) | ((m[..., 4:8] >> 4) << 6)
    out[..., 12:16] = (sc[..., 4:8] & 0x0F) | ((m[..., 4:8] & 0x0F) << 4)
    qp = q.reshape(rows, nb, 4, 2, 32)
    out[..., 16:] = (qp[..., 0, :] | (qp[..., 1, :] << 4)).reshape(rows, nb, 128)
    return out.reshape(rows, -1)


def quantize_q5_k(x: torch.Tensor) -> torch.Tensor:
    """[rows, K] float -> uint8 [rows, K/256*176]: as Q4_K with five-bit codes, the fifth bit of element l of
    sub-block s in bit s of qh[l]; stored as d, dmin | scales[12] | qh[32] | qs[128]."""
    rows, K = x.shape
    nb = K // 256
    b = x.reshape(rows, nb, 8, 32).float()
    mn = b.amin(dim=-1).clamp(max=0.0)
    mx = b.amax(dim=-1).clamp(min=0.0)
    scale = (mx - mn) / 31.0
    nmin = -mn
    d = (scale.amax(dim=-1, keepdim=True) / 63.0).to(torch.float16)
    dmin = (nmin.amax(dim=-1, keepdim=True) / 63.0).to(torch.float16)
    df, dminf = d.float(), dmin.float()
    sc = torch.where(df > 0, torch.round(scale / df.clamp(min=1e-30)), torch.zeros_like(scale)).clamp_(0, 63)
    m = torch.where(dminf > 0, torch.round(nmin / dminf.clamp(min=1e-30)), torch.zeros_like(nmin)).clamp_(0, 63)
    dl = (df * sc).unsqueeze(-1)
    ml = (dminf * m).unsqueeze(-1)
    q = torch.where(dl > 0, torch.round((b + ml) / dl.clamp(min=1e-30)), torch.zeros_like(b)).clamp_(0, 31).to(torch.uint8)
    sc = sc.to(torch.uint8)
    m = m.to(torch.uint8)
    out = torch.empty(rows, nb, 176, dtype=torch.uint8, device=x.device)
    out[..., 0:2] = d.view(torch.uint8).reshape(rows, nb, 2)
    out[..., 2:4] = dmin.view(torch.uint8).reshape(rows, nb, 2)
    out[..., 4:8] = (sc[..., 0:4] & 63) | ((sc[..., 4:8] >> 4) << 6)
    out[..., 8:12] = (m[..., 0:4] & 63) | ((m[..., 4:8] >> 4) << 6)
    out[..., 12:16] = (sc[..., 4:8] & 0x0F) | ((m[..., 4:8] & 0x0F) << 4)
    top = q >> 4                                                   # [rows, nb, 8, 32]
    shifts = torch.arange(8, device=x.device, dtype=torch.uint8).reshape(1, 1, 8, 1)
    out[..., 16:48] = (top << shifts).sum(dim=2).to(torch.uint8)
    qp = (q & 0x0F).reshape(rows, nb, 4, 2, 32)
    out[..., 48:] = (qp[..., 0, :] | (qp[..., 1, :] << 4)).reshape(rows, nb, 128)
    return out.reshape(rows, -1)


def quantize_q6_k(x: torch.Tensor) -> torch.Tensor:
    """[rows, K] float -> uint8 [rows, K/256*210]: six-bit codes (offset 32) with an int8 scale per 16
    elements against an f16 super-block d, stored as ql[128] | qh[64] | scales[16] | d."""
    rows, K = x.shape
    nb = K // 256
    b = x.reshape(rows, nb, 16, 16).float()
    sub = b.abs().amax(dim=-1) / 31.0
    d = (sub.amax(dim=-1, keepdim=True) / 127.0).to(torch.float16)
    df = d.float()
    sc = torch.where(df > 0, torch.round(sub / df.clamp(min=1e-30)), torch.zeros_like(sub)).clamp_(0, 127)
    step = (df * sc).unsqueeze(-1)
    code = torch.where(step > 0, torch.round(b / step.clamp(min=1e-30)), torch.zeros_like(b)).clamp_(-32, 31) + 32
    code = code.to(torch.uint8).reshape(rows, nb, 2, 4, 32)          # [half][group of 32][l]
    low, top = code & 0x0F, code >> 4
    out = torch.empty(rows, nb, 210, dtype=torch.uint8, device=x.device)
    ql = torch.empty(rows, nb, 2, 64, dtype=torch.uint8, device=x.device)
    ql[..., 0:32] = low[..., 0, :] | (low[..., 2, :] << 4)
    ql[..., 32:64] = low[..., 1, :] | (low[..., 3, :] << 4)
    out[..., 0:128] = ql.reshape(rows, nb, 128)
    qh = top[..., 0, :] | (top[..., 1, :] << 2) | (top[..., 2, :] << 4) | (top[..., 3, :] << 6)
    out[..., 128:192] = qh.reshape(rows, nb, 64)
    out[..., 192:208] = sc.to(torch.int8).view(torch.uint8)
    out[..., 208:210] = d.view(torch.uint8).reshape(rows, nb, 2)
    return out.reshape(rows, -1)


_FP4_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


def quantize_mxfp4(x: torch.Tensor) -> torch.Tensor:
    """[rows, K] float -> uint8 [rows, K/32*17]: E8M0 block exponent, E2M1 codes."""
    rows, K = x.shape
    nb = K // 32
    b = x.reshape(rows, nb, 32).float()
    amax = b.abs().amax(dim=-1, keepdim=True)
    # floor(log2(amax)) from the float's own exponent (frexp is exact; log2 differs between machines near powers of two)
    _, ex = torch.frexp(amax.clamp(min=1e-38))
    e = torch.where(amax > 0, ex.to(amax.dtype) - 3.0, torch.full_like(amax, -127.0))
    e = e.clamp_(-127, 127)
    s = torch.exp2(e)
    grid = torch.tensor(_FP4_VALUES, device=x.device)
    mag = (b.abs() / s).clamp_(max=6.0)
    code = (mag.unsqueeze(-1) - grid).abs().argmin(dim=-1).to(torch.uint8)
    code = code | ((b < 0).to(torch.uint8) << 3)
    out = torch.empty(rows, nb, 17, dtype=torch.uint8, device=x.device)
    out[..., 0] = (e.squeeze(-1) + 127).to(torch.uint8)
    out[..., 1:] = code[..., :16] | (code[..., 16:] << 4)
    return out.reshape(rows, -1)


# type -> (offsets of the block's f16 scale fields with their factors, the standard deviation of a block of
# uniformly random codes at scale 1): Q4_1 and Q5_1 get the min -7.5 d / -15.5 d and Q2_K dmin = 1.5 d, which
# centre their values on zero
_RANDOM_BLOCKS = {
    gw.GGML_Q4_0: ([(0, 1.0)], 4.61), gw.GGML_Q5_0: ([(0, 1.0)], 9.23), gw.GGML_IQ4_NL: ([(0, 1.0)], 67.1),
    gw.GGML_Q4_1: ([(0, 1.0), (2, -7.5)], 4.61), gw.GGML_Q5_1: ([(0, 1.0), (2, -15.5)], 9.23),
    gw.GGML_Q2_K: ([(80, 1.0), (82, 1.5)], 13.9), gw.GGML_Q3_K: ([(108, 1.0)], 43.3), gw.GGML_IQ4_XS: ([(0, 1.0)], 1247.5),
}


def random_blocks(x: torch.Tensor, ggml_type: int) -> np.ndarray:
    """Rows of the legacy and i-quant types for a test model: every payload byte uniformly random (so every code,
    sub-block scale and high bit occurs), the f16 scale fields set so that the decoded values have about the
    standard deviation of `x`, with a random sign and a spread of two octaves per block. `x` gives the shape, the
    spread and the seed; its values are not fitted (no quantiser of these types is needed where the same bytes are
    decoded on both sides of a comparison)."""
    rows, K = x.shape
    el, nb = gw.BLOCK_GEOMETRY[ggml_type]
    fields, unit = _RANDOM_BLOCKS[ggml_type]
    sd = float(x.float().std())
    rng = np.random.default_rng(int(abs(float(x.float().sum())) * 1e6) % (2 ** 32))
    n = rows * (K // el)
    raw = rng.integers(0, 256, (n, nb), dtype=np.uint8)
    d = (sd / unit) * np.exp2(rng.uniform(-1.0, 1.0, n)) * rng.choice([-1.0, 1.0], n)
    for off, factor in fields:
        raw[:, off:off + 2] = (d * factor).astype(np.float16).view(np.uint8).reshape(n, 2)
    return raw.reshape(rows, -1)


def encode(x: torch.Tensor, ggml_type: int) -> np.ndarray:
    """[rows, K] float tensor -> numpy bytes of the stored representation."""
    if ggml_type in _RANDOM_BLOCKS:
        return random_blocks(x, ggml_type)
    if ggml_type == gw.GGML_F32:
        return x.float().cpu().numpy()
    if ggml_type == gw.GGML_F16:
        return x.to(torch.float16).cpu().numpy()
    if ggml_type == gw.GGML_Q8_0:
        return quantize_q8_0(x).cpu().numpy()
    if ggml_type == gw.GGML_Q4_K:
        return quantize_q4_k(x).cpu().numpy()
    if ggml_type == gw.GGML_MXFP4:
        return quantize_mxfp4(x).cpu().numpy()
    if ggml_type == gw.GGML_Q5_K:
        return quantize_q5_k(x).cpu().numpy()
    if ggml_type == gw.GGML_Q6_K:
        return quantize_q6_k(x).cpu().numpy()
    raise ValueError("unsupported ggml type %d" % ggml_type)


def storage_type(ggml_type: int, row_len: int) -> int:
    """A matrix whose row length is not a whole number of blocks is kept F16
    (the tiny config's ffn_down, row length 344)."""
    return ggml_type if row_len % gw.BLOCK_GEOMETRY[ggml_type][0] == 0 else gw.GGML_F16


# ---- model files ----------------------------------------------------------------

def _common_metadata(w: gw.GGUFWriter, s: ModelShape, with_eos: bool, vocab: dict | None = None) -> None:
    a = s.arch
    w.add("general.architecture", gw.T_STRING, a)
    w.add("general.name", gw.T_STRING, s.name)
    w.add(a + ".block_count", gw.T_UINT32, s.n_layer)
    w.add(a + ".context_length", gw.T_UINT32, 131072)
    w.add(a + ".embedding_length", gw.T_UINT32, s.n_embd)
    w.add(a + ".feed_forward_length", gw.T_UINT32, s.n_ff)
    w.add(a + ".attention.head_count", gw.T_UINT32, s.n_head)
    w.add(a + ".attention.head_count_kv", gw.T_UINT32, s.n_head_kv)
    w.add(a + ".attention.key_length", gw.T_UINT32, s.head_dim)
    w.add(a + ".attention.value_length", gw.T_UINT32, s.head_dim)
    w.add(a + ".attention.layer_norm_rms_epsilon", gw.T_FLOAT32, s.eps)
    w.add(a + ".rope.dimension_count", gw.T_UINT32, s.head_dim)
    w.add(a + ".rope.freq_base", gw.T_FLOAT32, s.rope_base)
    if s.rope_scaling_linear > 0:
        w.add(a + ".rope.scaling.type", gw.T_STRING, "linear")
        w.add(a + ".rope.scaling.factor", gw.T_FLOAT32, s.rope_scaling_linear)
    if s.rope_scaling_yarn > 0:
        w.add(a + ".rope.scaling.type", gw.T_STRING, "yarn")
        w.add(a + ".rope.scaling.factor", gw.T_FLOAT32, s.rope_scaling_yarn)
        w.add(a + ".rope.scaling.original_context_length", gw.T_UINT32, s.rope_original_context)
    if s.n_expert:
        w.add(a + ".expert_count", gw.T_UINT32, s.n_expert)
        w.add(a + ".expert_used_count", gw.T_UINT32, s.n_expert_used)
        w.add(a + ".expert_feed_forward_length", gw.T_UINT32, s.n_ff_exp)
    w.add("tokenizer.ggml.model", gw.T_STRING, (vocab or {}).get("model", "llama"))
    if vocab is not None:
        # a real vocabulary (n_vocab pieces): sentencepiece-kind with scores and the unknown id, or byte-pair
        # (model "gpt2") with the pre-tokeniser's name and the merges
        assert len(vocab["tokens"]) == s.n_vocab
        w.add("tokenizer.ggml.tokens", gw.T_ARRAY, list(vocab["tokens"]), gw.T_STRING)
        if "scores" in vocab:
            w.add("tokenizer.ggml.scores", gw.T_ARRAY, [float(x) for x in vocab["scores"]], gw.T_FLOAT32)
        w.add("tokenizer.ggml.token_type", gw.T_ARRAY, [int(x) for x in vocab["types"]], gw.T_INT32)
        if "pre" in vocab:
            w.add("tokenizer.ggml.pre", gw.T_STRING, vocab["pre"])
            w.add("tokenizer.ggml.merges", gw.T_ARRAY, list(vocab["merges"]), gw.T_STRING)
        w.add("tokenizer.ggml.bos_token_id", gw.T_UINT32, int(vocab["bos"]))
        w.add("tokenizer.ggml.eos_token_id", gw.T_UINT32, int(vocab["eos"]))
        if "unk" in vocab:
            w.add("tokenizer.ggml.unknown_token_id", gw.T_UINT32, int(vocab["unk"]))
        w.add("general.alignment", gw.T_UINT32, 32)
        return
    w.add("tokenizer.ggml.tokens", gw.T_ARRAY, ["<t%d>" % i for i in range(s.n_vocab)], gw.T_STRING)
    w.add("tokenizer.ggml.token_type", gw.T_ARRAY, [1] * s.n_vocab, gw.T_INT32)
    if with_eos:
        w.add("tokenizer.ggml.eos_token_id", gw.T_UINT32, 2)
    w.add("general.alignment", gw.T_UINT32, 32)


def write_model(path, shape: ModelShape, seed: int = 0, device: str | None = None,
                with_eos: bool = False, std: float = 0.02, vocab: dict | None = None) -> int:
    """Writes a random-weight GGUF of `shape`; returns the file size. One tensor
    is materialised at a time, on `device` (cuda if available)."""
    if device is None:
        device = "cuda" if torch.cuda.is_available() else "cpu"
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    s = shape
    w = gw.GGUFWriter()
    _common_metadata(w, s, with_eos, vocab)

    def matrix(name, n_in, n_out, ggml_type=None, n_mats=1, sd=std):
        t = storage_type(s.matrix_type if ggml_type is None else ggml_type, n_in)
        ne = [n_in, n_out] if n_mats == 1 else [n_in, n_out, n_mats]

        def make():
            x = torch.randn(n_out * n_mats, n_in, generator=gen, device=device) * sd
            return encode(x, t)
        w.add_tensor(name, ne, t, make)

    def vector(name, n, value=None, sd=std):
        def make():
            if value is not None and s.norm_std > 0 and value == 1.0:
                return (1.0 + torch.randn(n, generator=gen, device=device) * s.norm_std).float().cpu().numpy()
            if value is not None:
                return np.full(n, value, np.float32)
            return (torch.randn(n, generator=gen, device=device) * sd).float().cpu().numpy()
        w.add_tensor(name, [n], gw.GGML_F32, make)

    E, QD, KD = s.n_embd, s.n_head * s.head_dim, s.n_head_kv * s.head_dim
    matrix("token_embd.weight", E, s.n_vocab)
    for l in range(s.n_layer):
        b = "blk.%d." % l
        vector(b + "attn_norm.weight", E, 1.0)
        matrix(b + "attn_q.weight", E, QD)
        matrix(b + "attn_k.weight", E, KD)
        fine = finer_layer(s, l)
        matrix(b + "attn_v.weight", E, KD, None if (s.v_type < 0 or not fine) else s.v_type)
        if s.qkv_bias:
            vector(b + "attn_q.bias", QD)
            vector(b + "attn_k.bias", KD)
            vector(b + "attn_v.bias", KD)
        if s.arch == "qwen3moe":
            vector(b + "attn_q_norm.weight", s.head_dim, 1.0)
            vector(b + "attn_k_norm.weight", s.head_dim, 1.0)
        matrix(b + "attn_output.weight", QD, E)
        vector(b + "ffn_norm.weight", E, 1.0)
        if s.n_expert:
            # Router logits ~ N(0, 1) on unit-RMS inputs: weights N(0, 1/E).
            matrix(b + "ffn_gate_inp.weight", E, s.n_expert, gw.GGML_F32, sd=E ** -0.5)
            matrix(b + "ffn_gate_exps.weight", E, s.n_ff_exp, s.expert_type, s.n_expert)
            matrix(b + "ffn_up_exps.weight", E, s.n_ff_exp, s.expert_type, s.n_expert)
            matrix(b + "ffn_down_exps.weight", s.n_ff_exp, E,
                   s.expert_down_type if (s.expert_down_type >= 0 and fine) else s.expert_type, s.n_expert)
        else:
            matrix(b + "ffn_gate.weight", E, s.n_ff)
            matrix(b + "ffn_up.weight", E, s.n_ff)
            matrix(b + "ffn_down.weight", s.n_ff, E, None if (s.down_type < 0 or not fine) else s.down_type)
    if s.rope_freqs:
        def llama3_factors():
            # llama.cpp's convert script for Llama 3.1: factor 8, low / high frequency factors 1 / 4, over an
            # original context of 8192 (scaled here to the rotary base in use)
            half = s.head_dim // 2
            freqs = 1.0 / (s.rope_base ** (np.arange(half, dtype=np.float64) * 2.0 / s.head_dim))
            wavelen = 2.0 * np.pi / freqs
            old_ctx, factor, lo, hi = 8192.0, 8.0, 1.0, 4.0
            smooth = np.clip((old_ctx / wavelen - lo) / (hi - lo), 0.0, 1.0)
            out = np.where(wavelen < old_ctx / hi, 1.0, np.where(wavelen > old_ctx / lo, factor, 1.0 / ((1.0 - smooth) / factor + smooth)))
            return out.astype(np.float32)
        w.add_tensor("rope_freqs.weight", [s.head_dim // 2], gw.GGML_F32, llama3_factors)
    vector("output_norm.weight", E, 1.0)
    matrix("output.weight", E, s.n_vocab, None if s.output_type < 0 else s.output_type)
    return w.write(Path(path))


def write_lora_adapter(path, shape: ModelShape, rank: int = 16, alpha: float = 16.0, seed: int = 0,
                       targets=("attn_q", "attn_k", "attn_v", "attn_output"), dtype: int = gw.GGML_F16,
                       std_a: float = 0.02, std_b: float = 0.01) -> int:
    """A LoRA adapter file as the reference writes it (reference
    crates/retrograd-ffi/runtime/src/retro_lora.cpp:1004-1043, 1143-1153):
    general.type = "adapter", adapter.type = "lora", adapter.lora.alpha, and per
    target "<weight>.lora_a" ne=[n_in, r] / "<weight>.lora_b" ne=[r, n_out]."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    s = shape
    w = gw.GGUFWriter()
    w.add("general.type", gw.T_STRING, "adapter")
    w.add("general.architecture", gw.T_STRING, s.arch)
    w.add("adapter.type", gw.T_STRING, "lora")
    w.add("adapter.lora.alpha", gw.T_FLOAT32, float(alpha))
    E, QD, KD = s.n_embd, s.n_head * s.head_dim, s.n_head_kv * s.head_dim
    dims = {"attn_q": (E, QD), "attn_k": (E, KD), "attn_v": (E, KD), "attn_output": (QD, E),
            "ffn_gate": (E, s.n_ff), "ffn_up": (E, s.n_ff), "ffn_down": (s.n_ff, E)}
    for l in range(s.n_layer):
        for t in targets:
            n_in, n_out = dims[t]
            name = "blk.%d.%s.weight" % (l, t)
            a = torch.randn(rank, n_in, generator=gen) * std_a
            b = torch.randn(n_out, rank, generator=gen) * std_b
            w.add_tensor(name + ".lora_a", [n_in, rank], dtype, encode(a, dtype))
            w.add_tensor(name + ".lora_b", [rank, n_out], dtype, encode(b, dtype))
    return w.write(Path(path))
