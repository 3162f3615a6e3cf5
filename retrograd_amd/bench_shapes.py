"""Decode-step measurements of the other full-shape configurations of the
benchmark set on one MI355X (secondary figures; bench.py at the repository root
measures the headline):

    python -m retrograd_amd.bench_shapes c4        # multi-LoRA decode, Qwen2.5-7B shape, Q8_0 base
    python -m retrograd_amd.bench_shapes c5        # mixture of experts, Qwen3-30B-A3B shape, MXFP4 experts
    python -m retrograd_amd.bench_shapes c5-q4km   # the same shape with the type mix of a Q4_K_M file
    python -m retrograd_amd.bench_shapes mxfp4-scaled   # the block-scaled FP4 x FP8 product at c5's expert sizes

c4: 28 layers, hidden 3584, 28 / 4 heads, FFN 18944, vocabulary 152064, eight
rank-16 F16 adapters on q/k/v/o (A ~ N(0, 0.02), B ~ N(0, 0.01)), 64 sequences
each routed at random to one adapter or to the base, prompts uniform in
[256, 2048], 128 greedy tokens.
c5: 48 layers, hidden 2048, 32 / 4 heads, 128 experts of width 768 with top-8
routing, attention in Q8_0, experts in MXFP4, 128 sequences with prompts
log-uniform in [64, 2048], 128 greedy tokens.

Weights are synthetic (seeded), prompts random token ids. Prefill runs first,
untimed for the decode figure; then `--new` decode steps over all sequences: the
first part is timed as it is, the last `--profiled` steps run with an event pair
around every kernel category (which slows them a little) for the breakdown.
Prints one JSON line.

mxfp4-scaled times two kernels, not a step: MXFP4 rows times 1 to 16 tokens on the block-scaled matrix instruction,
under ggml's arithmetic and under the exact one, as one dense matrix of the size of a layer's expert weights (gate and up of 128
experts: 196608 rows of 2048; down: 262144 rows of 768), every launch on another copy of the weights so that they
come from HBM."""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np


def step_algorithmic_bytes(shape, synth, gw, n_seq: int, mean_context: float) -> dict:
    """HBM bytes one decode step has to move: every dense matrix once at its stored type, the experts the step's rows
    touch (their expected number under uniform routing), and K and V of every attended cell (f16)."""
    kv = shape.n_layer * 2 * shape.n_head_kv * shape.head_dim * 2 * mean_context * n_seq
    if shape.n_expert == 0:
        return {"weights": synth.streamed_weight_bytes(shape), "experts": 0, "kv": round(kv)}
    dense = 0
    for name, n_in, n_out, t in synth.matrix_types(shape):
        if ".ffn_" in name:
            continue
        el, by = gw.BLOCK_GEOMETRY[synth.storage_type(t, n_in)]
        dense += n_in // el * by * n_out
    dense += shape.n_layer * shape.n_embd * shape.n_expert * 4          # the F32 routers
    touched = shape.n_expert * (1.0 - (1.0 - shape.n_expert_used / shape.n_expert) ** n_seq)
    el, by = gw.BLOCK_GEOMETRY[shape.expert_type]
    gate_up = 2 * shape.n_embd // el * by * shape.n_ff_exp
    el, by = gw.BLOCK_GEOMETRY[shape.expert_down_type if shape.expert_down_type >= 0 else shape.expert_type]
    down = shape.n_ff_exp // el * by * shape.n_embd
    return {"weights": dense, "experts": round(shape.n_layer * touched * (gate_up + down)), "kv": round(kv),
            "experts_touched_per_layer": round(touched, 2)}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("config", choices=["c4", "c5", "c5-q4km", "mxfp4-scaled"])
    ap.add_argument("--new", type=int, default=128)
    ap.add_argument("--profiled", type=int, default=32)
    ap.add_argument("--model-dir", default=os.environ.get("RETRO_BENCH_MODEL_DIR", "/dev/shm"))
    ap.add_argument("--seed", type=int, default=1234)
    args = ap.parse_args()

    import torch

    from . import engine as E
    from . import gguf_writer as gw
    from . import synth

    if not torch.cuda.is_available():
        print("bench_shapes needs an MI355X: no HIP device is visible", file=sys.stderr)
        return 2
    if args.config == "mxfp4-scaled":
        out = {"kernels": {"ggml": "k_mxs (Q8_0 activation blocks)", "exact": "k_mxe (f32 activations as six hexadecimal digits)"},
               "weights": "pseudo-random, from HBM", "cases": []}
        for exact in (False, True):
            for what, n, k in (("gate_up", 2 * 128 * 768, 2048), ("down", 128 * 2048, 768)):
                for t in (1, 4, 8, 16):
                    us = E.kernel_mxfp4_scaled_time(n, k, t, True, 50, exact=exact)
                    nbytes = n * (k // 32) * 17
                    out["cases"].append({"arithmetic": "exact" if exact else "ggml", "matrix": what, "rows": n, "k": k, "tokens": t,
                                         "us": round(us, 2), "weight_bytes": nbytes, "tb_per_s": round(nbytes / us / 1e6, 3),
                                         "frac_of_8_tb_per_s": round(nbytes / us / 1e6 / 8.0, 3)})
        print(json.dumps(out))
        return 0
    rng = np.random.default_rng(args.seed)
    if args.config == "c4":
        shape, n_seq = synth.QWEN25_7B_Q8, 64
        lengths = rng.integers(256, 2048 + 1, n_seq)
    else:
        shape, n_seq = synth.QWEN3_30B_A3B, 128
        if args.config == "c5-q4km":
            shape = synth.scaled(shape, matrix_type=gw.GGML_Q4_K, v_type=gw.GGML_Q6_K, output_type=gw.GGML_Q6_K,
                                 expert_type=gw.GGML_Q4_K, expert_down_type=gw.GGML_Q6_K, finer_layers="more_bits",
                                 name="qwen3-30b-a3b-shape-q4_k_m")
        else:
            shape = synth.scaled(shape, expert_type=gw.GGML_MXFP4)
        lengths = np.exp(rng.uniform(np.log(64), np.log(2048), n_seq)).astype(np.int64)
    lengths = [int(n) for n in lengths]

    model_path = Path(args.model_dir) / ("retro-bench-%s-seed%d.gguf" % (shape.name, args.seed))
    if not model_path.exists():
        tmp = model_path.with_suffix(".tmp")
        synth.write_model(tmp, shape, seed=args.seed, device="cuda")
        os.replace(tmp, model_path)
    torch.cuda.empty_cache()

    n_ctx = sum((n + args.new + 1 + 31) // 32 * 32 for n in lengths)
    eng = E.Engine(model_path, E.EngineConfig(n_ctx=n_ctx, n_seq_max=n_seq, n_batch=512, n_ubatch=512))
    adapters = []
    if args.config == "c4":
        for i in range(8):
            a = Path(args.model_dir) / ("retro-bench-c4-lora-%d-seed%d.gguf" % (i, args.seed))
            if not a.exists():
                synth.write_lora_adapter(a, shape, rank=16, alpha=16.0, seed=args.seed + 100 + i, std_a=0.02, std_b=0.01)
            adapters.append(eng.adapter_load(a, 1.0))
    route = [int(rng.choice(adapters + [E.RETRO_STEP_ADAPTER_BASE])) if adapters else 0 for _ in range(n_seq)]

    out = E.StepOutput(512)
    greedy = E.SamplingParamsV2.greedy()
    last = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s, n in enumerate(lengths):
        prompt = rng.integers(0, shape.n_vocab, n).astype(np.int32)
        for at in range(0, n, 512):
            eng.step([E.StepRow(s, s, prompt[at:at + 512], at, sample=at + 512 >= n, sampling=greedy,
                                adapter=E.RowAdapter(route[s]))], out)
        last.append(out.row(0).token)
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0

    pos = list(lengths)
    plain = max(1, args.new - args.profiled)
    step_s = []
    prof = {}
    for it in range(args.new):
        if it == plain:
            eng.profile(2)
            eng.profile_read(reset=True)
        rows = [E.StepRow(s, s, [last[s]], pos[s], sample=True, sampling=greedy, adapter=E.RowAdapter(route[s]))
                for s in range(n_seq)]
        t0 = time.perf_counter()
        eng.step(rows, out)
        step_s.append(time.perf_counter() - t0)
        for s in range(n_seq):
            last[s] = out.row(s).token
            pos[s] += 1
    if args.new > plain:
        prof = eng.profile_read(reset=True)
    timed = step_s[2:plain] if plain > 4 else step_s[:plain]
    ms = 1e3 * float(np.mean(timed))
    n_prof = args.new - plain
    # the timed steps are the first `plain` ones: their mean context
    by = step_algorithmic_bytes(shape, synth, gw, n_seq, float(np.mean(lengths)) + (2 + plain) / 2)
    total_bytes = by["weights"] + by["experts"] + by["kv"]
    line = {
        "config": args.config, "model": shape.name, "sequences": n_seq,
        "prompt_tokens": int(sum(lengths)), "mean_context_during_decode": float(np.mean(lengths)) + args.new / 2,
        "prefill_tok_s": round(sum(lengths) / prefill_s, 1),
        "decode_ms_per_step": round(ms, 3), "decode_tok_s": round(n_seq / ms * 1e3, 1), "decode_steps_timed": len(timed),
        "algorithmic_bytes_per_step": by, "step_frac_of_hbm_roofline": round(total_bytes / 8e12 / (ms * 1e-3), 4),
        "adapters": len(adapters), "rows_routed_to_an_adapter": sum(1 for r in route if r > 0),
        "kernel_ms_per_step": {k: round(t / n_prof, 4) for k, (t, n) in sorted(prof.items(), key=lambda kv: -kv[1][0]) if n},
        "kernel_launches_per_step": {k: n // n_prof for k, (t, n) in prof.items() if n},
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
