#!/usr/bin/env python3
"""Headline benchmark: decode tok/s of the Llama-3-8B-shaped Q4_K ragged batch-64
workload on one MI355X, and that as a fraction of the HBM roofline.

A "step" is one call of the engine's step entry point over one decode batch:
one row per live sequence (64 rows, ragged contexts). Prints ONE JSON line.
`value` is sampled tokens per second over exactly --steps timed decode steps,
with all inputs resident in HBM. As in the reference's own serving benchmark
(src/bench/serving.rs:464-603) the decode phase is timed separately from
prefill: when a request finishes and a new one is admitted into its slot, the
new prompt is prefilled in its own (untimed, separately reported) steps before
the decode batch resumes with all 64 sequences live.

Workload (the second configuration of the benchmark set): 32 layers, hidden 4096, 32/8 heads of 128,
FFN 14336, vocab 128256, Q4_K matrices, f16 KV; 64 concurrent sequences,
prompt lengths log-uniform in [128, 4096], uniform random token ids, greedy
(top_k = 1), 256 new tokens each, a new request admitted whenever one finishes.
The 64 initial sequences start at staggered points of their 256-token budget so
the timed window is the steady state rather than a synchronized cohort.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--shape", default="c2", choices=["c2", "c2-q4km", "small"],
                    help="c2-q4km = the same workload on the type mix of a Q4_K_M file (a secondary figure); "
                         "small = a reduced shape for a quick functional run")
    ap.add_argument("--model-dir", default=os.environ.get("RETRO_BENCH_MODEL_DIR", "/dev/shm"))
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=16)
    ap.add_argument("--profile-all", action="store_true", help="also print a per-category kernel time breakdown to stderr")
    ap.add_argument("--stream-probe", type=int, default=0, metavar="MIB",
                    help="after the timed steps also launch the plain copy kernel over this many MiB (known traffic, "
                         "for scaling rocprofv3 memory counters)")
    ap.add_argument("--traffic-file", default=str(ROOT / "profiles" / "k_attention_c2_hbm_traffic.txt"),
                    help="text summary of the rocprofv3 --pmc runs; its traffic_bytes_per_launch line fills roofline.traffic")
    return ap.parse_args()


class Sequence:
    __slots__ = ("request", "slot", "prompt", "pos", "generated", "budget", "last_token")

    def __init__(self, request, slot, prompt, budget):
        self.request, self.slot, self.prompt, self.budget = request, slot, prompt, budget
        self.pos = 0            # positions resident in the KV
        self.generated = 0
        self.last_token = None  # sampled, not yet resident


class Workload:
    """Continuous batching over the engine: decode rows first, then prefill
    chunks inside the token budget (the order the reference's scheduler composes
    a step in, crates/retrograd-infer/src/scheduler.rs:933-1089)."""

    def __init__(self, eng, E, n_slots, n_batch, n_vocab, max_new, len_lo, len_hi, seed):
        self.eng, self.E = eng, E
        self.n_batch, self.n_vocab, self.max_new = n_batch, n_vocab, max_new
        self.len_lo, self.len_hi = len_lo, len_hi
        self.rng = np.random.default_rng(seed)
        self.next_request = 0
        self.seqs = [None] * n_slots
        self.out = E.StepOutput(n_batch)
        self.sampling = E.SamplingParamsV2.greedy()
        self.finished = 0

    def new_request(self, slot, budget=None):
        n = int(round(math.exp(self.rng.uniform(math.log(self.len_lo), math.log(self.len_hi)))))
        n = min(max(n, self.len_lo), self.len_hi)
        prompt = self.rng.integers(0, self.n_vocab, n).astype(np.int32)
        s = Sequence(self.next_request, slot, prompt, self.max_new if budget is None else budget)
        self.next_request += 1
        self.seqs[slot] = s
        return s

    def prefill_pending(self):
        return any(s is not None and s.last_token is None for s in self.seqs)

    def compose(self, phase):
        E = self.E
        rows, kinds = [], []
        budget = self.n_batch
        if phase == "decode":
            for s in self.seqs:
                if s is not None and s.last_token is not None:
                    rows.append(E.StepRow(s.request, s.slot, [s.last_token], s.pos, sample=True, sampling=self.sampling))
                    kinds.append(("decode", s))
            return rows, kinds
        for s in self.seqs:
            if s is None or s.last_token is not None or budget <= 0:
                continue
            remaining = len(s.prompt) - s.pos
            n = min(remaining, budget)
            last = n == remaining
            rows.append(E.StepRow(s.request, s.slot, s.prompt[s.pos:s.pos + n], s.pos, sample=last, sampling=self.sampling))
            kinds.append(("prefill", s, n))
            budget -= n
        return rows, kinds

    def step(self, phase):
        """Runs one step of `phase` ("decode" or "prefill"). Returns (sampled
        tokens, decode rows, attention cells read, tokens in the step, seconds)."""
        rows, kinds = self.compose(phase)
        t0 = time.perf_counter()
        self.eng.step(rows, self.out)     # synchronous: returns after the device finished
        dt = time.perf_counter() - t0
        sampled = decode_rows = cells = tokens = 0
        for i, kind in enumerate(kinds):
            s = kind[1]
            r = self.out.row(i)
            if kind[0] == "decode":
                s.pos += 1
                decode_rows += 1
                tokens += 1
                cells += s.pos
            else:
                s.pos += kind[2]
                tokens += kind[2]
                cells += s.pos
            if r.sampled:
                sampled += 1
                s.last_token = r.token
                s.generated += 1
                if s.generated >= s.budget:
                    self.eng.seq_rm(s.slot)
                    self.eng.request_free(s.request)
                    self.finished += 1
                    self.new_request(s.slot)
        return sampled, decode_rows, cells, tokens, dt


def read_traffic(path: str, workload: str):
    """HBM bytes per launch of the dominant kernel as measured with rocprofv3
    --pmc FETCH_SIZE / WRITE_SIZE (scaled by the copy kernel), from the text
    summary of those runs; None when there is no summary for this workload."""
    try:
        fields = {}
        for line in Path(path).read_text().splitlines():
            if "=" in line and not line.startswith("#"):
                k, v = line.split("=", 1)
                fields[k.strip()] = v.strip()
        if fields.get("workload") != workload:
            return None
        return float(fields["traffic_bytes_per_launch"])
    except (OSError, KeyError, ValueError):
        return None


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the decode step has no multi-GPU path in this build (--gpus must be 1)", file=sys.stderr)
        return 2

    import torch

    import oracle
    from retrograd_amd import engine as E
    from retrograd_amd import synth

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X: no HIP device is visible", file=sys.stderr)
        return 2

    if args.shape in ("c2", "c2-q4km"):
        shape = synth.LLAMA3_8B_Q4K if args.shape == "c2" else synth.LLAMA3_8B_Q4K_M
        n_slots, max_new, len_lo, len_hi, n_batch = 64, 256, 128, 4096, 512
    else:
        shape = synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=4, n_vocab=32000, name="llama3-8b-shape-q4_k-4layers")
        n_slots, max_new, len_lo, len_hi, n_batch = 64, 64, 64, 1024, 512
    n_ctx = n_slots * (len_hi + max_new)

    model_path = Path(args.model_dir) / ("retro-bench-%s-seed%d.gguf" % (shape.name, args.seed))
    if not model_path.exists():
        t0 = time.perf_counter()
        tmp = model_path.with_suffix(".tmp")
        synth.write_model(tmp, shape, seed=args.seed, device="cuda")
        os.replace(tmp, model_path)
        print("[bench] wrote %s (%.1f GB) in %.1fs" % (model_path, model_path.stat().st_size / 1e9, time.perf_counter() - t0), file=sys.stderr, flush=True)
    torch.cuda.empty_cache()

    t0 = time.perf_counter()
    eng = E.Engine(model_path, E.EngineConfig(n_ctx=n_ctx, n_seq_max=n_slots, n_batch=n_batch, n_ubatch=n_batch))
    print("[bench] engine ready in %.1fs" % (time.perf_counter() - t0), file=sys.stderr, flush=True)

    wl = Workload(eng, E, n_slots, n_batch, shape.n_vocab, max_new, len_lo, len_hi, args.seed)
    # initial cohort, staggered through its generation budget
    stagger = np.random.default_rng(args.seed + 1).integers(1, max_new + 1, n_slots)
    for slot in range(n_slots):
        wl.new_request(slot, budget=int(stagger[slot]))
    t0 = time.perf_counter()
    n_pre = 0
    while wl.prefill_pending():
        wl.step("prefill")
        n_pre += 1
        if n_pre % 50 == 0:
            print("[bench] initial prefill: %d steps" % n_pre, file=sys.stderr, flush=True)
    print("[bench] initial prefill of %d sequences: %d steps, %.1fs" % (n_slots, n_pre, time.perf_counter() - t0), file=sys.stderr, flush=True)

    def run_decode_steps(n, timed):
        """n decode steps; prompts of requests admitted on the way are prefilled in
        their own steps in between. Returns the totals of the decode steps and of
        the prefill steps."""
        dec = [0, 0, 0, 0, 0.0]
        pre = [0, 0.0, 0]
        done = 0
        while done < n:
            if wl.prefill_pending():
                if timed:
                    eng.profile(0)
                r = wl.step("prefill")
                pre[0] += r[3]
                pre[1] += r[4]
                pre[2] += 1
                continue
            if timed:
                eng.profile(2 if args.profile_all else 1)
            r = wl.step("decode")
            for i in range(5):
                dec[i] += r[i]
            done += 1
        return dec, pre

    run_decode_steps(args.warmup, False)
    eng.profile_read(reset=True)
    torch.cuda.synchronize()
    wall0 = time.perf_counter()
    (sampled, decode_rows, cells, tokens, elapsed), (pre_tokens, pre_seconds, pre_steps) = run_decode_steps(args.steps, True)
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    prof = eng.profile_read(reset=True)
    eng.profile(0)

    ms_per_step = elapsed / args.steps * 1e3
    tok_s = sampled / elapsed

    # ---- roofline of the dominant kernel (paged attention, one launch per layer)
    hp = shape
    kv_bytes_per_cell_layer = 2 * hp.n_head_kv * hp.head_dim * 2
    attn_ms, attn_launches = prof["attention"]
    algo_bytes_per_launch = kv_bytes_per_cell_layer * cells / args.steps
    attn_avg_s = attn_ms / max(attn_launches, 1) * 1e-3
    attn_gbs = algo_bytes_per_launch / attn_avg_s / 1e9 if attn_avg_s > 0 else 0.0

    # ---- whole-step roofline (north star): weights once + KV of every attended cell
    w_bytes = synth.streamed_weight_bytes(hp)       # every dense matrix once, at its stored type
    step_bytes = w_bytes + hp.n_layer * kv_bytes_per_cell_layer * (cells / args.steps)
    step_roof_tok_s = (sampled / args.steps) / (step_bytes / (HBM_PEAK_GBS * 1e9))

    result = {
        "metric": ("decode tok/s, 8B-shape Q4_K ragged batch 64; % of HBM roofline" if args.shape != "c2-q4km" else
                   "decode tok/s, 8B shape with the Q4_K_M type mix (Q6_K output, ffn_down and attn_v on half the layers), "
                   "ragged batch 64 (secondary figure)"),
        "value": round(tok_s, 1),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("q4_k" if args.shape != "c2-q4km" else "q4_k / q6_k") + " weights x f16 hi/lo activations, f32 accumulate, f16 KV",
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: %s, %d live sequences, prompts log-uniform [%d,%d], greedy, %d new tokens, continuous batching"
                        % (shape.name, n_slots, len_lo, len_hi, max_new),
            "n_batch": n_batch,
            "mean_decode_rows_per_step": round(decode_rows / args.steps, 2),
            "mean_tokens_per_step": round(tokens / args.steps, 2),
            "mean_kv_cells_attended_per_step": round(cells / args.steps, 1),
            "requests_finished_in_window": wl.finished,
            "timing": "sum of the %d decode steps' own durations; prefill of admitted requests runs between them, untimed" % args.steps,
            "prefill_between_decode_steps": {"steps": pre_steps, "tokens": pre_tokens,
                                             "tok_s": round(pre_tokens / pre_seconds, 1) if pre_seconds > 0 else None},
            "mixed_tok_s_including_prefill_time": round(sampled / wall, 1),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "k_attention<128, true> (paged split-KV attention of a decode step, one launch per layer)",
            "achieved": round(attn_gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(attn_gbs / HBM_PEAK_GBS, 4),
            "traffic": read_traffic(args.traffic_file, shape.name),
            "algorithmic_bytes_per_launch": round(algo_bytes_per_launch),
            "avg_launch_us": round(attn_avg_s * 1e6, 2),
            "launches_timed": attn_launches,
            "step": {
                "algorithmic_bytes_per_step": round(step_bytes),
                "roofline_tok_s": round(step_roof_tok_s, 1),
                "frac": round(tok_s / step_roof_tok_s, 4),
            },
        },
    }
    if args.stream_probe > 0:
        us = E.kernel_stream_time(args.stream_probe << 20, False, 3)
        print("[bench] copy kernel over %d MiB: %.1f us per launch" % (args.stream_probe, us), file=sys.stderr, flush=True)
    if args.profile_all:
        print("[bench] kernel time per step (ms): " + ", ".join(
            "%s=%.3f" % (k, v[0] / args.steps) for k, v in prof.items()), file=sys.stderr, flush=True)

    if not args.no_cpu_baseline:
        result["cpu_baseline"], result["parity_full_size"] = cpu_baseline(eng, E, oracle, wl, model_path, args.cpu_rows)
    else:
        result["cpu_baseline"] = None

    eng.close()
    print(json.dumps(result), flush=True)
    return 0


def cpu_baseline(eng, E, oracle, wl, model_path, n_rows):
    """Times the CPU oracle on one decode step over the first n_rows live
    sequences of the same workload (their KV imported from the engine's own
    snapshots), and compares its logits with the engine's for the same rows."""
    live = [s for s in wl.seqs if s is not None and s.last_token is not None][:n_rows]
    model = oracle.Model(model_path)
    ctx = oracle.Context(model, max(s.slot for s in live) + 1)
    t0 = time.perf_counter()
    for s in live:
        ctx.import_snapshot(s.slot, eng.seq_save(s.slot))
    print("[bench] cpu baseline: imported %d sequences in %.1fs" % (len(live), time.perf_counter() - t0), file=sys.stderr, flush=True)
    rows = [(s.slot, s.pos, [s.last_token], True) for s in live]
    t0 = time.perf_counter()
    want = ctx.step_rows(rows)
    cpu_s = time.perf_counter() - t0
    # a few more decode steps of the same rows (fed with the oracle's own greedy tokens), for about 10 s of CPU work
    cpu_steps = 1
    feed = [int(r.argmax()) for r in want]
    while cpu_s < 8.0 and cpu_steps < 8:
        t0 = time.perf_counter()
        more = ctx.step_rows([(s.slot, s.pos + cpu_steps, [feed[i]], True) for i, s in enumerate(live)])
        cpu_s += time.perf_counter() - t0
        feed = [int(r.argmax()) for r in more]
        cpu_steps += 1
    out = E.StepOutput(len(live))
    eng.step([E.StepRow(s.request, s.slot, [s.last_token], s.pos, sample=True, sampling=wl.sampling) for s in live], out)
    got = eng.debug_logits()
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    margins = np.sort(want, axis=1)
    margin = margins[:, -1] - margins[:, -2]
    same = [int(out.row(i).token) == int(want[i].argmax()) for i in range(len(live))]
    decided = [bool(m > 2 * 2e-2) for m in margin]
    parity = {
        "rows": len(live),
        "max_abs_logit_error": float(err.max()),
        "mean_abs_relative_error": float(err.mean() / np.abs(want).mean()),
        "greedy_tokens_equal": int(sum(same)),
        "greedy_tokens_equal_where_margin_exceeds_tolerance": "%d/%d" % (sum(s for s, d in zip(same, decided) if d), sum(decided)),
    }
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    base = {
        "value": round(len(live) * cpu_steps / cpu_s, 3),
        "unit": "tok/s",
        "cores": cores,
        "kind": "port",
        "sample": "%d consecutive decode steps of %d of the 64 live sequences (mean context %d), %.1fs of CPU work; KV imported from the engine"
                  % (cpu_steps, len(live), int(np.mean([s.pos for s in live])), cpu_s),
    }
    return base, parity


if __name__ == "__main__":
    sys.exit(main())
