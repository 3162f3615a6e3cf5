"""Writes tests/golden/hf_reference_logits.npz: logits of Hugging Face `transformers` models
(LlamaForCausalLM, Qwen2ForCausalLM, Qwen3MoeForCausalLM, float64, eager attention) built from
the dequantised weights of small synthetic GGUF files. tests/test_oracle_model.py regenerates
the same files (seeded, CPU) and requires oracle.Context(..., "exact") to reproduce these logits,
which pins the oracle's forward pass against a library that is not this repository's code:

  * RoPE pairing: a `llama` GGUF stores attn_q / attn_k with llama.cpp's row permutation and rotates
    adjacent pairs (2i, 2i+1); Hugging Face rotates (i, i + D/2). Row 2i+h of a head in the file is row
    h*D/2 + i of the Hugging Face matrix (convert_hf_to_gguf.py's `permute`, inverted here). qwen2 and
    qwen3moe files keep the Hugging Face order and rotate (i, i + D/2).
  * grouped-query head mapping (query head h reads KV head h // (H / KV)), 1/sqrt(D) scaling, causal mask;
  * q/k/v biases (qwen2); per-head q/k RMSNorm before the rotation (qwen3moe); RMSNorm with its weight
    (norm vectors are random here, not all ones);
  * rope_freqs.weight (Llama 3.1's frequency divisors = Hugging Face rope_type "llama3"), linear and yarn scaling;
  * the expert router: softmax over all experts, top-k, renormalise (norm_topk_prob), SwiGLU experts;
  * the LoRA delta scale * alpha / r * B (A x): merged into the dense Hugging Face matrices.

The K and V an attention layer reads are rounded to f16, as the f16 KV cache stores them (K after the
rotation): done here by wrapping the library's apply_rotary_pos_emb and hooking v_proj, so that the
comparison can be tight (1e-4) rather than at the 1e-3 the cache rounding alone would leave.

The block decoders below (F32, F16, Q8_0, MXFP4) are written from the format definitions
(reference crates/rir-core/src/quant.rs:82-128, 286-295), independently of oracle/quant.hpp.

Runs only where `transformers` is importable (the build container); the tests read the .npz.
Usage: python tests/golden/hf_reference_logits.py
"""
import hashlib
import sys
import tempfile
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

from retrograd_amd import synth  # noqa: E402
from gguf_reader import Reader  # noqa: E402

OUT = Path(__file__).resolve().parent / "hf_reference_logits.npz"

# name -> (shape, seed, std). Every matrix type here decodes with the few lines below.
CASES = {
    "llama": (synth.scaled(synth.TINY_LLAMA, norm_std=0.2, name="hf-llama"), 41, 0.08),
    "llama-rope-freqs": (synth.scaled(synth.TINY_LLAMA, norm_std=0.2, rope_freqs=True, rope_base=500000.0,
                                      name="hf-llama-rope-freqs"), 42, 0.08),
    "llama-linear": (synth.scaled(synth.TINY_LLAMA, norm_std=0.2, rope_scaling_linear=4.0, name="hf-llama-linear"), 43, 0.08),
    # yarn: with 32 rotary dims, base 1e4 and an original context of 32 the correction range is pairs 0..3
    "llama-yarn": (synth.scaled(synth.TINY_LLAMA, norm_std=0.2, rope_scaling_yarn=4.0, rope_original_context=32,
                                name="hf-llama-yarn"), 46, 0.08),
    "qwen2": (synth.scaled(synth.QWEN25_7B_Q8, n_layer=2, n_embd=128, n_head=4, n_head_kv=2, head_dim=32, n_ff=256,
                           n_vocab=300, norm_std=0.2, name="hf-qwen2"), 44, 0.08),
    "qwen3moe": (synth.scaled(synth.QWEN3_30B_A3B, n_layer=2, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_vocab=288,
                              n_expert=8, n_expert_used=2, n_ff_exp=256, norm_std=0.2, name="hf-qwen3moe"), 45, 0.08),
}
LORA = {"case": "qwen2", "rank": 4, "alpha": 8.0, "seed": 3, "scale": 0.5, "std_a": 0.1, "std_b": 0.1,
        # every true matrix of a layer is a target (reference retro_lora.cpp:165-169)
        "targets": ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")}
PROMPT_SEED = 77
N_TOKENS = 14
POS0 = {"llama-linear": 0}


def sha256(path):
    return hashlib.sha256(open(path, "rb").read()).hexdigest()


def decode_row(t, raw, n):
    """One row of n elements of a GGUF tensor of type t as float64."""
    raw = np.asarray(raw, np.uint8)
    if t == 0:
        return raw.view(np.float32).astype(np.float64)
    if t == 1:
        return raw.view(np.float16).astype(np.float64)
    if t == 8:       # Q8_0: f16 d, 32 int8
        b = raw.reshape(n // 32, 34)
        d = b[:, :2].copy().view(np.float16).astype(np.float64)
        return (d * b[:, 2:].view(np.int8).astype(np.float64)).reshape(-1)
    if t == 39:      # MXFP4: E8M0 byte, 16 bytes of E2M1 codes (low nibbles = elements 0..15, high = 16..31)
        b = raw.reshape(n // 32, 17)
        e = b[:, 0].astype(np.int32)
        # the code table holds twice the E2M1 values and the block scale is 2^(e - 127) / 2 = 2^(e - 128), down to
        # the subnormal 2^-128 at e = 0 (reference quant.rs:105-117, 543-552)
        half = np.ldexp(1.0, e - 128)
        table = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.float64)
        lo, hi = b[:, 1:] & 15, b[:, 1:] >> 4
        vals = np.concatenate([table[lo], table[hi]], axis=1) * half[:, None]
        return vals.reshape(-1)
    raise ValueError("type %d is not decoded here" % t)


def unpermute(w, n_head):
    """File order (adjacent pairs) -> Hugging Face order (halves) of the rows of attn_q / attn_k."""
    rows, cols = w.shape
    d = rows // n_head
    return w.reshape(n_head, d // 2, 2, cols).swapaxes(1, 2).reshape(rows, cols)


def build_hf(path, shape, lora=None):
    import torch
    import transformers
    from transformers import (LlamaConfig, LlamaForCausalLM, Qwen2Config, Qwen2ForCausalLM, Qwen3MoeConfig,
                              Qwen3MoeForCausalLM)

    s = shape
    r = Reader(path)
    W = lambda name: r.dense(name, decode_row)
    rope = {"rope_theta": float(s.rope_base), "rope_type": "default"}
    if s.rope_freqs:
        rope = {"rope_theta": float(s.rope_base), "rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}
    if s.rope_scaling_linear > 0:
        rope = {"rope_theta": float(s.rope_base), "rope_type": "linear", "factor": float(s.rope_scaling_linear)}
    if s.rope_scaling_yarn > 0:
        rope = {"rope_theta": float(s.rope_base), "rope_type": "yarn", "factor": float(s.rope_scaling_yarn),
                "original_max_position_embeddings": int(s.rope_original_context), "beta_fast": 32.0, "beta_slow": 1.0}
    common = dict(vocab_size=s.n_vocab, hidden_size=s.n_embd, num_hidden_layers=s.n_layer, num_attention_heads=s.n_head,
                  num_key_value_heads=s.n_head_kv, rms_norm_eps=s.eps, max_position_embeddings=131072,
                  tie_word_embeddings=False, rope_parameters=rope, attn_implementation="eager", experts_implementation="eager")
    if s.arch == "llama":
        cfg = LlamaConfig(intermediate_size=s.n_ff, head_dim=s.head_dim, attention_bias=False, mlp_bias=False, **common)
        model = LlamaForCausalLM(cfg)
    elif s.arch == "qwen2":
        cfg = Qwen2Config(intermediate_size=s.n_ff, **common)
        model = Qwen2ForCausalLM(cfg)
    else:
        cfg = Qwen3MoeConfig(intermediate_size=s.n_ff, head_dim=s.head_dim, num_experts=s.n_expert,
                             num_experts_per_tok=s.n_expert_used, moe_intermediate_size=s.n_ff_exp, norm_topk_prob=True,
                             decoder_sparse_step=1, mlp_only_layers=[], attention_bias=False, **common)
        model = Qwen3MoeForCausalLM(cfg)
    model.config._experts_implementation = "eager"
    model = model.to(torch.float64).eval()
    sd = {}
    T = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float64))

    def merged(name):
        w = W(name)
        if lora and name in lora:
            A, B, scale = lora[name]
            w = w + scale * (B @ A)
        return w

    sd["model.embed_tokens.weight"] = T(W("token_embd.weight"))
    sd["model.norm.weight"] = T(W("output_norm.weight").reshape(-1))
    sd["lm_head.weight"] = T(W("output.weight"))
    for l in range(s.n_layer):
        b, h = "blk.%d." % l, "model.layers.%d." % l
        q, k = merged(b + "attn_q.weight"), merged(b + "attn_k.weight")
        if s.arch == "llama":
            q, k = unpermute(q, s.n_head), unpermute(k, s.n_head_kv)
        sd[h + "self_attn.q_proj.weight"], sd[h + "self_attn.k_proj.weight"] = T(q), T(k)
        sd[h + "self_attn.v_proj.weight"] = T(merged(b + "attn_v.weight"))
        sd[h + "self_attn.o_proj.weight"] = T(merged(b + "attn_output.weight"))
        if s.qkv_bias:
            for x in "qkv":
                sd[h + "self_attn.%s_proj.bias" % x] = T(W(b + "attn_%s.bias" % x).reshape(-1))
        if s.arch == "qwen3moe":
            sd[h + "self_attn.q_norm.weight"] = T(W(b + "attn_q_norm.weight").reshape(-1))
            sd[h + "self_attn.k_norm.weight"] = T(W(b + "attn_k_norm.weight").reshape(-1))
        sd[h + "input_layernorm.weight"] = T(W(b + "attn_norm.weight").reshape(-1))
        sd[h + "post_attention_layernorm.weight"] = T(W(b + "ffn_norm.weight").reshape(-1))
        if s.n_expert:
            sd[h + "mlp.gate.weight"] = T(W(b + "ffn_gate_inp.weight"))
            gate, up = W(b + "ffn_gate_exps.weight"), W(b + "ffn_up_exps.weight")       # [expert][F][E]
            sd[h + "mlp.experts.gate_up_proj"] = T(np.concatenate([gate, up], axis=1))
            sd[h + "mlp.experts.down_proj"] = T(W(b + "ffn_down_exps.weight"))          # [expert][E][F]
        else:
            sd[h + "mlp.gate_proj.weight"] = T(merged(b + "ffn_gate.weight"))
            sd[h + "mlp.up_proj.weight"] = T(merged(b + "ffn_up.weight"))
            sd[h + "mlp.down_proj.weight"] = T(merged(b + "ffn_down.weight"))
    missing, unexpected = model.load_state_dict(sd, strict=False)
    assert not unexpected, unexpected
    assert all("rotary" in m or "inv_freq" in m for m in missing), missing

    # the f16 KV cache: K after the rotation and V as projected are rounded to f16 before attention reads them
    mod = sys.modules[type(model).__module__]
    plain = mod.apply_rotary_pos_emb
    if not getattr(plain, "_rounds_k", False):
        def rounding(q, k, cos, sin, *a, **kw):
            q2, k2 = plain(q, k, cos, sin, *a, **kw)
            return q2, k2.to(torch.float16).to(k2.dtype)
        rounding._rounds_k = True
        mod.apply_rotary_pos_emb = rounding
    for layer in model.model.layers:
        layer.self_attn.v_proj.register_forward_hook(lambda m, i, o: o.to(torch.float16).to(o.dtype))
    return model, transformers.__version__


def main():
    import torch
    out = {}
    with tempfile.TemporaryDirectory() as d:
        for key, (shape, seed, std) in CASES.items():
            path = Path(d) / (key + ".gguf")
            synth.write_model(path, shape, seed=seed, device="cpu", std=std)
            toks = np.random.default_rng(PROMPT_SEED + seed).integers(0, shape.n_vocab, N_TOKENS)
            model, version = build_hf(path, shape)
            with torch.no_grad():
                logits = model(torch.from_numpy(toks)[None]).logits[0].numpy()
            out[key + ".tokens"] = toks.astype(np.int32)
            out[key + ".logits"] = logits.astype(np.float32)
            out[key + ".sha256"] = np.frombuffer(bytes.fromhex(sha256(path)), np.uint8)
            print(key, "logits", logits.shape, "abs mean %.3f" % np.abs(logits).mean(), "transformers", version)
            if key == LORA["case"]:
                ad = Path(d) / "adapter.gguf"
                synth.write_lora_adapter(ad, shape, rank=LORA["rank"], alpha=LORA["alpha"], seed=LORA["seed"],
                                         std_a=LORA["std_a"], std_b=LORA["std_b"], targets=LORA["targets"])
                ar = Reader(ad)
                pairs = {}
                for name in ar.tensors:
                    if name.endswith(".lora_a"):
                        base = name[:-7]
                        pairs[base] = (ar.dense(name, decode_row), ar.dense(base + ".lora_b", decode_row),
                                       LORA["scale"] * LORA["alpha"] / LORA["rank"])
                model, _ = build_hf(path, shape, lora=pairs)
                with torch.no_grad():
                    with_adapter = model(torch.from_numpy(toks)[None]).logits[0].numpy()
                out[key + ".lora.logits"] = with_adapter.astype(np.float32)
                out[key + ".lora.sha256"] = np.frombuffer(bytes.fromhex(sha256(ad)), np.uint8)
                print(key, "with adapter: moves the logits by %.3f" % np.abs(with_adapter - logits).mean())
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
