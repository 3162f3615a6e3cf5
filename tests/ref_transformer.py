"""float64 numpy transformer written from the textbook formulas, independent of
oracle/model.hpp: used to pin the oracle's forward (tests only)."""
import numpy as np

import oracle
from gguf_reader import Reader


F32, F16, Q8_0, Q4_K, Q5_K, Q6_K, BF16, MXFP4 = 0, 1, 8, 12, 13, 14, 30, 39


def q4_0_cache_rows(v):
    """Rows as a Q4_0 KV cache holds them (ggml's quantize_row_q4_0_ref, in numpy's float32 arithmetic): per 32
    values the first value m of largest magnitude, d = m / -8, codes min(15, trunc(x / d + 8.5)) with the unrounded
    d, values (code - 8) times d rounded to f16."""
    x = np.asarray(v, np.float32)
    f32 = np.float32
    b = x.reshape(-1, 32)
    first = np.abs(b).argmax(-1)
    d = (b[np.arange(len(b)), first] / f32(-8.0)).astype(f32)
    inv = np.where(d != 0, f32(1.0) / np.where(d != 0, d, f32(1.0)), f32(0.0)).astype(f32)
    codes = np.minimum(np.trunc((b * inv[:, None]).astype(f32) + f32(8.5)), 15)
    out = d.astype(np.float16).astype(f32)[:, None] * (codes - 8).astype(f32)
    return out.reshape(x.shape).astype(np.float64)


def ggml_activations(v, weight_type):
    """The rows of v as ggml's CPU matmul multiplies them with a weight of this
    type: re-quantised to Q8_K (Q4_K and Q6_K weights; blocks of 256, the first value of
    largest magnitude maps to -127, codes rounded half to even and capped at
    127), to Q8_0 (Q8_0 and MXFP4 weights; blocks of 32, scale amax / 127 kept
    as f16, codes rounded half away from zero with the unrounded scale), or
    rounded to f16 (F16 weights). Written with numpy's float32 arithmetic,
    independently of oracle/model.hpp."""
    x = np.asarray(v, np.float32)
    f32 = np.float32
    if weight_type in (Q4_K, Q5_K, Q6_K):
        b = x.reshape(-1, 256)
        first = np.abs(b).argmax(-1)                      # argmax returns the first maximum
        mx = b[np.arange(len(b)), first]
        out = np.zeros_like(b)
        nz = mx != 0
        iscale = (f32(-127.0) / mx[nz]).astype(f32)
        codes = np.minimum(np.rint((b[nz] * iscale[:, None]).astype(f32)), 127)
        out[nz] = ((f32(1.0) / iscale).astype(f32)[:, None] * codes.astype(f32)).astype(f32)
        return out.reshape(x.shape).astype(np.float64)
    if weight_type in (Q8_0, MXFP4):
        b = x.reshape(-1, 32)
        d = (np.abs(b).max(-1) / f32(127.0)).astype(f32)
        inv = np.where(d != 0, f32(1.0) / np.where(d != 0, d, f32(1.0)), f32(0.0)).astype(f32)
        scaled = (b * inv[:, None]).astype(f32)
        codes = np.sign(scaled) * np.floor(np.abs(scaled) + f32(0.5))
        out = d.astype(np.float16).astype(f32)[:, None] * codes.astype(f32)
        return out.reshape(x.shape).astype(np.float64)
    if weight_type == F16:
        return x.astype(np.float16).astype(np.float64)
    if weight_type == BF16:
        u = x.view(np.uint32).astype(np.uint64)
        u = (u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000
        return u.astype(np.uint32).view(np.float32).reshape(x.shape).astype(np.float64)
    return np.asarray(v, np.float64)


class NumpyModel:
    def __init__(self, path, activations="exact", kv="f16"):
        self.kv = kv          # "f16", or "q8_0": K and V rows stored as Q8_0 blocks of 32 along a head's row
        """activations: "exact" (the f32 values are multiplied) or "ggml" (converted first)."""
        self.ggml = activations == "ggml"
        r = Reader(path)
        self.r = r
        a = r.kv["general.architecture"]
        self.arch = a
        g = lambda k, d=None: r.kv.get(a + "." + k, d)
        self.L = g("block_count")
        self.E = g("embedding_length")
        self.H = g("attention.head_count")
        self.KV = g("attention.head_count_kv", self.H)
        self.D = g("attention.key_length", self.E // self.H)
        self.eps = g("attention.layer_norm_rms_epsilon", 1e-5)
        self.base = g("rope.freq_base", 10000.0)
        self.n_expert = g("expert_count", 0)
        self.n_used = g("expert_used_count", 0)
        self.neox = a != "llama"
        self.w = {}
        # divisors of the rotation angle per frequency: linear scaling and the model's rope_freqs.weight
        scaling = g("rope.scaling.type", "none")
        assert scaling in ("none", "linear", "yarn"), scaling
        self.rope_div = np.full(self.D // 2, float(g("rope.scaling.factor", 1.0)) if scaling == "linear" else 1.0)
        self.rope_magnitude = 1.0
        if "rope_freqs.weight" in r.tensors:
            self.rope_div = self.rope_div * np.asarray(self.t("rope_freqs.weight"), np.float64).reshape(-1)
        if scaling == "yarn":
            # the YaRN rule as its paper states it: below the correction range interpolate (1 / factor), above it keep,
            # a linear ramp over the pair index between; amplitudes times 0.1 ln(factor) + 1
            factor, n_orig = float(g("rope.scaling.factor")), float(g("rope.scaling.original_context_length"))
            corr = lambda rot: self.D * np.log(n_orig / (rot * 2 * np.pi)) / (2 * np.log(self.base))
            low, high = max(np.floor(corr(32.0)), 0), min(np.ceil(corr(1.0)), self.D - 1)
            keep = 1 - np.clip((np.arange(self.D // 2) - low) / max(high - low, 0.001), 0, 1)
            self.rope_div = self.rope_div / ((1 - keep) / factor + keep)
            self.rope_magnitude = 0.1 * np.log(factor) + 1.0

    def t(self, name):
        if name not in self.w:
            self.w[name] = self.r.dense(name, oracle.decode_row) if name in self.r.tensors else None
        return self.w[name]

    def act(self, name, v):
        return ggml_activations(v, self.r.tensors[name][1]) if self.ggml else v

    def norm(self, x, w):
        return x / np.sqrt((x * x).mean(-1, keepdims=True) + self.eps) * w

    def rope(self, v, pos):
        # v: [heads, D]
        D = self.D
        i = np.arange(D // 2)
        ang = pos * self.base ** (-2.0 * i / D) / self.rope_div
        c, s = np.cos(ang) * self.rope_magnitude, np.sin(ang) * self.rope_magnitude
        out = v.copy()
        if self.neox:
            a, b = v[:, :D // 2], v[:, D // 2:]
            out[:, :D // 2] = a * c - b * s
            out[:, D // 2:] = a * s + b * c
        else:
            a, b = v[:, 0::2], v[:, 1::2]
            out[:, 0::2] = a * c - b * s
            out[:, 1::2] = a * s + b * c
        return out

    def forward(self, tokens, pos0=0, lora=None):
        """Full causal forward of one sequence; returns logits [T, V].
        lora: dict name -> (A [r, in], B [out, r], scale*alpha/r, storage type of A and B)."""
        T = len(tokens)
        x = self.t("token_embd.weight")[np.asarray(tokens)]
        G = self.H // self.KV

        def mm(name, v):
            y = self.act(name, v) @ self.t(name).T
            if lora and name in lora:
                A, B, s, adapter_type = lora[name]
                if self.ggml:
                    y = y + s * (ggml_activations(ggml_activations(v, adapter_type) @ A.T, adapter_type) @ B.T)
                else:
                    y = y + s * ((v @ A.T) @ B.T)
            return y

        for l in range(self.L):
            b = "blk.%d." % l
            h = self.norm(x, self.t(b + "attn_norm.weight"))
            q, k, v = mm(b + "attn_q.weight", h), mm(b + "attn_k.weight", h), mm(b + "attn_v.weight", h)
            if self.t(b + "attn_q.bias") is not None:
                q = q + self.t(b + "attn_q.bias"); k = k + self.t(b + "attn_k.bias"); v = v + self.t(b + "attn_v.bias")
            q = q.reshape(T, self.H, self.D); k = k.reshape(T, self.KV, self.D); v = v.reshape(T, self.KV, self.D)
            if self.t(b + "attn_q_norm.weight") is not None:
                q = self.norm(q, self.t(b + "attn_q_norm.weight"))
                k = self.norm(k, self.t(b + "attn_k_norm.weight"))
            q = np.stack([self.rope(q[t], pos0 + t) for t in range(T)])
            k = np.stack([self.rope(k[t], pos0 + t) for t in range(T)])
            if self.kv in ("q8_0", "q4_0"):
                # blocks of 32 never straddle heads (head_dim is a multiple of 32); under the ggml arithmetic the
                # query row meets a Q8_0 or Q4_0 K row converted to Q8_0 itself
                if self.kv == "q4_0":
                    k, v = q4_0_cache_rows(k), q4_0_cache_rows(v)
                else:
                    k = ggml_activations(k.astype(np.float32), Q8_0)
                    v = ggml_activations(v.astype(np.float32), Q8_0)
                if self.ggml:
                    q = ggml_activations(q.astype(np.float32), Q8_0)
            else:
                k = k.astype(np.float16).astype(np.float64)   # f16 KV cache
                v = v.astype(np.float16).astype(np.float64)
            att = np.zeros((T, self.H, self.D))
            for hh in range(self.H):
                s = q[:, hh] @ k[:, hh // G].T / np.sqrt(self.D)
                s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
                p = np.exp(s - s.max(-1, keepdims=True))
                p /= p.sum(-1, keepdims=True)
                att[:, hh] = p @ v[:, hh // G]
            x = x + mm(b + "attn_output.weight", att.reshape(T, -1))
            h = self.norm(x, self.t(b + "ffn_norm.weight"))
            if self.n_expert:
                x = x + self.moe(b, h)
            else:
                gate, up = mm(b + "ffn_gate.weight", h), mm(b + "ffn_up.weight", h)
                x = x + mm(b + "ffn_down.weight", gate / (1 + np.exp(-gate)) * up)
        h = self.norm(x, self.t("output_norm.weight"))
        head = self.t("output.weight")
        if head is None:
            head = self.t("token_embd.weight")
        logits = self.act("output.weight" if self.t("output.weight") is not None else "token_embd.weight", h) @ head.T
        if self.t("output.bias") is not None:
            logits = logits + self.t("output.bias")
        return logits

    def moe(self, b, h):
        router = self.act(b + "ffn_gate_inp.weight", h) @ self.t(b + "ffn_gate_inp.weight").T
        p = np.exp(router - router.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        Wg, Wu, Wd = self.t(b + "ffn_gate_exps.weight"), self.t(b + "ffn_up_exps.weight"), self.t(b + "ffn_down_exps.weight")
        out = np.zeros_like(h)
        for t in range(h.shape[0]):
            top = np.argsort(-p[t], kind="stable")[:self.n_used]
            wsum = p[t, top].sum()
            for e in top:
                g, u = Wg[e] @ self.act(b + "ffn_gate_exps.weight", h[t]), Wu[e] @ self.act(b + "ffn_up_exps.weight", h[t])
                out[t] += p[t, e] / wsum * (Wd[e] @ self.act(b + "ffn_down_exps.weight", g / (1 + np.exp(-g)) * u))
        return out
