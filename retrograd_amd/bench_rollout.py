"""GRPO-rollout style measurement on one MI355X: the trainer handle's generation
context behind the step scheduler, prompts that share a long prefix, several
sampled completions per prompt.

    python -m retrograd_amd.bench_rollout [--shape c3|small] [--prompts 32] [--samples 8]

The default is the rollout configuration of the benchmark set: the 8B-shape Q4_K
model, 32 prompts made of a 2048-token common prefix and a unique suffix of
32..512 tokens, 8 completions each (256 sequences decoded together), top-k 40 at
temperature 1 from per-sequence seeded generators. The common prefix is decoded
once and pinned first. Prints one JSON line: sampled tokens per second over
everything (prefix, suffix prefill and decode), and the prefix-cache counters
that say how much prefill the shared prefix saved.
This is a secondary figure; bench.py at the repository root measures the headline
decode step."""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--shape", default="c3", choices=["c3", "small"])
    ap.add_argument("--prompts", type=int, default=32)
    ap.add_argument("--samples", type=int, default=8)
    ap.add_argument("--prefix", type=int, default=2048)
    ap.add_argument("--max-new", type=int, default=128)
    ap.add_argument("--model-dir", default=os.environ.get("RETRO_BENCH_MODEL_DIR", "/dev/shm"))
    ap.add_argument("--seed", type=int, default=1234)
    args = ap.parse_args()

    import torch

    from . import engine as E
    from . import scheduler as S
    from . import synth
    from . import trainer as T

    if not torch.cuda.is_available():
        print("bench_rollout needs an MI355X: no HIP device is visible", file=sys.stderr)
        return 2
    if args.shape == "c3":
        shape, suffix_lo, suffix_hi = synth.LLAMA3_8B_Q4K, 32, 512
    else:
        shape, suffix_lo, suffix_hi = synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=4, n_vocab=32000,
                                                   name="llama3-8b-shape-q4_k-4layers"), 32, 512
    model_path = Path(args.model_dir) / ("retro-bench-%s-seed%d.gguf" % (shape.name, args.seed))
    if not model_path.exists():
        tmp = model_path.with_suffix(".tmp")
        synth.write_model(tmp, shape, seed=args.seed, device="cuda")
        os.replace(tmp, model_path)
    torch.cuda.empty_cache()

    n_seq = args.prompts * args.samples
    if n_seq > 256:
        print("at most 256 sequences decode together", file=sys.stderr)
        return 2
    per_seq = args.prefix + suffix_hi + args.max_new
    per_seq = (per_seq + 511) // 512 * 512
    tr = T.Trainer(model_path, T.TrainConfig(n_ctx=per_seq, n_batch=512, generation_concurrency=n_seq, generation_batch=512))
    sched = S.Scheduler.over_trainer(tr, S.SchedulerOptions(mode=S.CONTINUOUS, n_batch=512, queue_capacity=args.prompts,
                                                            event_capacity=args.max_new + 8, min_prefix_len=8,
                                                            swap_min_tokens=1 << 62))
    sched.initialize()
    rng = np.random.default_rng(args.seed)
    common = [int(t) for t in rng.integers(0, shape.n_vocab, args.prefix)]
    prompts = [common + [int(t) for t in rng.integers(0, shape.n_vocab, int(rng.integers(suffix_lo, suffix_hi + 1)))]
               for _ in range(args.prompts)]
    requests = [S.Request(p, [E.SamplingParamsV2(temperature=1.0, top_p=1.0, top_k=40, seed=1000 * i + j,
                                                 max_new_tokens=args.max_new) for j in range(args.samples)])
                for i, p in enumerate(prompts)]

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    # The common prefix is decoded once and pinned, the way a system prompt is: the wave below then finds it
    # in the prefix tree (requests admitted together do not share with each other, only with what has finished).
    warm = S.run_requests(sched, [S.Request(common, [E.SamplingParamsV2.greedy(max_new_tokens=1)])])
    if warm[0].error:
        print("the warm-up request failed: %s" % warm[0].error, file=sys.stderr)
        return 1
    pin = sched.pin_prefix(common)
    torch.cuda.synchronize()
    t_warm = time.perf_counter()
    outcomes = S.run_requests(sched, requests)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    sched.unpin(pin)
    errors = [o.error for o in outcomes if o.error]
    if errors:
        print("a request failed: %s" % errors[0], file=sys.stderr)
        return 1
    sampled = sum(len(c.tokens) for o in outcomes for c in o.completions)
    kv = sched.kv_stats()
    prompt_tokens = sum(len(p) for p in prompts)
    line = {
        "metric": "rollout tok/s, 8B-shape Q4_K, shared-prefix prompts x sampled completions (secondary figure)",
        "value": round(sampled / (t1 - t0), 1), "unit": "tok/s", "n_gpus": 1,
        "seconds": round(t1 - t0, 3), "seconds_of_the_common_prefix": round(t_warm - t0, 3),
        "config": {"workload": "%d prompts = %d-token common prefix + suffix U[%d,%d], %d completions each, top-k 40, "
                               "temperature 1, %d new tokens; trainer generation context behind the step scheduler"
                               % (args.prompts, args.prefix, suffix_lo, suffix_hi, args.samples, args.max_new),
                   "model": shape.name, "sequences": n_seq},
        "prefix_cache": {"hits": kv.hits, "misses": kv.misses, "prompt_cells": kv.prompt_cells,
                         "prefilled_cells": kv.prefilled_cells, "prompt_tokens_submitted": prompt_tokens,
                         "prefill_saved_frac": round(1 - kv.prefilled_cells / max(kv.prompt_cells, 1), 4)},
        "sampled_tokens": sampled, "data": "synthetic",
    }
    print(json.dumps(line))
    sched.close()
    tr.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
