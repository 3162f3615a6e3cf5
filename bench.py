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
                    help="text summary of the rocprofv3 --pmc runs of the attention kernel; its traffic_ratio line (HBM bytes "
                         "moved per algorithmic byte) is applied to this run's algorithmic bytes")
    ap.add_argument("--matmul-traffic-file", default=str(ROOT / "profiles" / "k_mm5_q4k_c2_hbm_traffic.txt"),
                    help="the same kind of summary for the tile matmul family")
    ap.add_argument("--activations", default="exact", choices=["exact", "ggml"],
                    help="arithmetic of the measured engine: exact (f16 hi/lo activations, the default and the one the "
                         "logit tolerances are shown on) or ggml (activations converted to Q8_K / Q8_0 as the reference's CPU path does)")
    ap.add_argument("--kv", default="f16", choices=["f16", "q8_0", "q4_0"],
                    help="storage of the KV cache; the headline is f16 as the workload names it, q8_0 and q4_0 are secondary configurations")
    ap.add_argument("--kernel-steps", type=int, default=8, help="decode steps timed per kernel category after the timed region")
    ap.add_argument("--attention-timeline", default="", metavar="FILE",
                    help="after the timed region, record the workgroup timeline of one decode attention launch and write a text summary")
    ap.add_argument("--no-scheduler-leg", action="store_true", help="skip the run of the same workload through the step scheduler")
    ap.add_argument("--scheduler-requests", type=int, default=128)
    ap.add_argument("--no-ggml-leg", action="store_true", help="skip the secondary measurement under the ggml arithmetic")
    ap.add_argument("--one-sequence", action="store_true",
                    help="measure only the single-sequence decode steps (512-token context) in the chosen arithmetic and "
                         "print their JSON: the workload of the small-batch kernel profiles")
    ap.add_argument("--single-token-matvec", action="store_true",
                    help="with --one-sequence in the exact arithmetic: the matrix-vector kernel with f32 rows instead of the tile kernels "
                         "(what RETRO_GEMV_EXACT=1 selects)")
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


def read_traffic_ratio(path: str, workload: str):
    """HBM bytes moved per algorithmic byte by the attention kernel, as measured with rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE (scaled by the copy kernel) on a run whose own algorithmic bytes the summary
    records beside the counters; None when there is no summary for this workload."""
    try:
        fields = {}
        for line in Path(path).read_text().splitlines():
            if "=" in line and not line.startswith("#"):
                k, v = line.split("=", 1)
                fields[k.strip()] = v.strip()
        if fields.get("workload") != workload:
            return None
        if "traffic_ratio" in fields:
            return float(fields["traffic_ratio"])
        return float(fields["traffic_bytes_per_launch"]) / float(fields["algorithmic_bytes_per_launch"])
    except (OSError, KeyError, ValueError, ZeroDivisionError):
        return None


def read_matmul_traffic(path: str, workload: str, algorithmic_bytes: float):
    """HBM bytes per launch of the tile matmul family: the ratio its own counter summary records (same two-run
    FETCH_SIZE / WRITE_SIZE method as the attention kernel's) times this run's algorithmic bytes; None without one."""
    ratio = read_traffic_ratio(path, workload)
    return round(ratio * algorithmic_bytes) if ratio else None


def matrix_bytes_by_category(shape, synth, gw):
    """Stored bytes of the matrices each matmul category of a decode step streams, per launch (one layer;
    the head once per step)."""
    cats = {"qkv": 0, "o_proj": 0, "gate_up": 0, "down": 0, "head": 0}
    for name, n_in, n_out, t in synth.matrix_types(shape):
        el, by = gw.BLOCK_GEOMETRY[synth.storage_type(t, n_in)]
        b = n_in // el * by * n_out
        if name == "output.weight":
            cats["head"] += b
        elif not name.startswith("blk.0."):
            continue
        elif "attn_q" in name or "attn_k" in name or "attn_v" in name:
            cats["qkv"] += b
        elif "attn_output" in name:
            cats["o_proj"] += b
        elif "ffn_gate" in name or "ffn_up" in name:
            cats["gate_up"] += b
        elif "ffn_down" in name:
            cats["down"] += b
    return cats


def measure_decode(args, eng, E, synth, gw, shape, geometry, profile_kernels):
    """Prefills the staggered initial cohort, then times args.steps decode steps (no profiling inside them), then,
    with profile_kernels, args.kernel_steps more decode steps with HIP events on the engine's stream around every
    kernel category. Returns the measurements and the workload (still live)."""
    import torch
    n_slots, max_new, len_lo, len_hi, n_batch = geometry
    wl = Workload(eng, E, n_slots, n_batch, shape.n_vocab, max_new, len_lo, len_hi, args.seed)
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

    def run_decode_steps(n, level):
        """n decode steps; prompts of requests admitted on the way are prefilled in their own steps in between
        (events off). Returns the totals of the decode steps and of the prefill steps."""
        dec = [0, 0, 0, 0, 0.0]
        pre = [0, 0.0, 0]
        done = 0
        while done < n:
            if wl.prefill_pending():
                eng.profile(0)
                r = wl.step("prefill")
                pre[0] += r[3]
                pre[1] += r[4]
                pre[2] += 1
                continue
            eng.profile(level)
            r = wl.step("decode")
            for i in range(5):
                dec[i] += r[i]
            done += 1
        eng.profile(0)
        return dec, pre

    run_decode_steps(args.warmup, 0)
    eng.profile_read(reset=True)
    finished0 = wl.finished
    torch.cuda.synchronize()
    wall0 = time.perf_counter()
    dec, pre = run_decode_steps(args.steps, 2 if args.profile_all else 0)        # the timed steps carry no event pairs
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    prof = eng.profile_read(reset=True)
    out = {"dec": dec, "pre": pre, "wall": wall, "prof": prof, "finished": wl.finished - finished0, "kernels": None}
    if profile_kernels and args.kernel_steps > 0:
        kdec, _ = run_decode_steps(args.kernel_steps, 2)
        out["kernels"] = (eng.profile_read(reset=True), kdec, args.kernel_steps)
    if profile_kernels and args.attention_timeline:
        eng.attention_timeline(True)
        run_decode_steps(3, 0)
        stamps = eng.attention_timeline_read()
        eng.attention_timeline(False)
        Path(args.attention_timeline).write_text(attention_timeline_summary(stamps))
    return out, wl


def attention_timeline_summary(stamps) -> str:
    """Text summary of one decode attention launch from the six values its workgroups leave (clock ticks of 10 ns at
    the start, after the prologue, when the first wave is done, when all waves are done, at the end; the row's pages)."""
    if len(stamps) == 0:
        return "no decode step took the one-launch attention\n"
    st = stamps.astype(np.int64)
    t0 = st[:, 0].min()
    us = lambda col: (st[:, col] - t0) / 100.0
    start, pro, first, allw, end, pages = us(0), us(1), us(2), us(3), us(4), st[:, 5]
    lines = ["workgroups %d, pages %d (16 KiB of K and V each: %.1f MB), launch span %.1f us (first start to last end): %.2f TB/s"
             % (len(st), pages.sum(), pages.sum() * 16384 / 1e6, end.max(), pages.sum() * 16384 / end.max() / 1e6),
             "per workgroup, mean: prologue %.2f us, pages streamed in %.2f us (%.3f us per page; the first wave is done after "
             "%.0f %% of that), merge and store %.2f us"
             % ((pro - start).mean(), (allw - pro).mean(), ((allw - pro) / pages).mean(),
                100.0 * ((first - pro) / np.maximum(allw - pro, 1e-9)).mean(), (end - allw).mean()),
             "", "time us | workgroups resident | of them streaming pages | started so far | finished so far"]
    for t in np.arange(0.0, end.max() + 5.0, 5.0):
        lines.append("%7.0f | %19d | %24d | %14d | %15d" % (t, ((start <= t) & (end > t)).sum(), ((pro <= t) & (allw > t)).sum(),
                                                              (start <= t).sum(), (end <= t).sum()))
    lines += ["", "workgroups by pages of their row: pages | count | mean start us | mean duration us | us per page"]
    edges = [0, 8, 16, 32, 48, 64, 96, 128, 1 << 30]
    for lo, hi in zip(edges[:-1], edges[1:]):
        sel = (pages > lo) & (pages <= hi)
        if sel.any():
            lines.append("%4d..%-4s | %5d | %13.1f | %16.1f | %.3f" % (lo + 1, hi if hi < (1 << 30) else "", sel.sum(), start[sel].mean(),
                                                                       (end - start)[sel].mean(), ((allw - pro)[sel] / pages[sel]).mean()))
    return "\n".join(lines) + "\n"


def scheduler_leg(args, eng, E, shape, geometry):
    """The same workload through the product's step scheduler in continuous mode (the policy of
    crates/retrograd-infer/src/scheduler.rs:933-1404: FIFO admission with cell reservations, decode rows first,
    prefill chunks of new requests inside the same steps): every request is submitted at once, the scheduler
    admits them as slots free up, and sampled tokens are counted over the whole run, prefill included."""
    import torch
    from retrograd_amd import scheduler as S
    n_slots, max_new, len_lo, len_hi, n_batch = geometry
    rng = np.random.default_rng(args.seed + 7)
    n_req = args.scheduler_requests
    sched = S.Scheduler.over_engine(eng, S.SchedulerOptions(mode=S.CONTINUOUS, n_batch=n_batch, queue_capacity=n_req,
                                                            event_capacity=max_new + 8, slow_client_timeout=60.0,
                                                            prefix_cache=True, min_prefix_len=8, swap_min_tokens=1 << 62))
    sched.initialize()
    prompts = []
    for _ in range(n_req):
        n = int(round(math.exp(rng.uniform(math.log(len_lo), math.log(len_hi)))))
        prompts.append(rng.integers(0, shape.n_vocab, min(max(n, len_lo), len_hi)).astype(np.int32))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    streams = [sched.submit(S.Request.single([int(t) for t in p], E.SamplingParamsV2.greedy(seed=i, max_new_tokens=max_new)))
               for i, p in enumerate(prompts)]
    steps = 0
    while not sched.is_idle():
        sched.pump()
        steps += 1
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    sampled = 0
    for s_ in streams:
        events = s_.drain()
        sampled += sum(1 for e in events if e.type == "Token")
        if any(e.type == "Error" for e in events):
            raise RuntimeError("a scheduled request failed")
    kv = sched.kv_stats()
    sched.close()
    return {
        "tok_s": round(sampled / seconds, 1), "seconds": round(seconds, 3), "steps": steps, "requests": n_req,
        "sampled_tokens": sampled, "prompt_tokens": int(sum(len(p) for p in prompts)),
        "mode": "continuous: decode rows and prefill chunks share steps of at most %d tokens; prefill time included" % n_batch,
        "kv_stats": {"hits": kv.hits, "misses": kv.misses, "prompt_cells": kv.prompt_cells, "prefilled_cells": kv.prefilled_cells,
                     "evictions": kv.evictions},
    }


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the decode step has no multi-GPU path in this build (--gpus must be 1)", file=sys.stderr)
        return 2

    import torch

    import oracle
    from retrograd_amd import engine as E
    from retrograd_amd import gguf_writer as gw
    from retrograd_amd import synth

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X: no HIP device is visible", file=sys.stderr)
        return 2

    if args.shape in ("c2", "c2-q4km"):
        shape = synth.LLAMA3_8B_Q4K if args.shape == "c2" else synth.LLAMA3_8B_Q4K_M
        geometry = (64, 256, 128, 4096, 512)
    else:
        shape = synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=4, n_vocab=32000, name="llama3-8b-shape-q4_k-4layers")
        geometry = (64, 64, 64, 1024, 512)
    n_slots, max_new, len_lo, len_hi, n_batch = geometry
    n_ctx = n_slots * (len_hi + max_new)

    model_path = Path(args.model_dir) / ("retro-bench-%s-seed%d.gguf" % (shape.name, args.seed))
    if not model_path.exists():
        t0 = time.perf_counter()
        tmp = model_path.with_suffix(".tmp")
        synth.write_model(tmp, shape, seed=args.seed, device="cuda")
        os.replace(tmp, model_path)
        print("[bench] wrote %s (%.1f GB) in %.1fs" % (model_path, model_path.stat().st_size / 1e9, time.perf_counter() - t0), file=sys.stderr, flush=True)
    torch.cuda.empty_cache()

    def new_engine(activations):
        os.environ["RETRO_ACTIVATIONS"] = activations
        t0 = time.perf_counter()
        eng = E.Engine(model_path, E.EngineConfig(n_ctx=n_ctx, n_seq_max=n_slots, n_batch=n_batch, n_ubatch=n_batch,
                                                  kv_dtype={"f16": E.KV_F16, "q8_0": E.KV_Q8_0, "q4_0": E.KV_Q4_0}[args.kv]))
        print("[bench] engine (%s arithmetic) ready in %.1fs" % (activations, time.perf_counter() - t0), file=sys.stderr, flush=True)
        return eng

    if args.one_sequence:
        eng = new_engine(args.activations)
        if args.single_token_matvec:
            eng.single_token_matvec(True)
        kvb = 2 * shape.n_head_kv * shape.head_dim * 2 * {"f16": 32, "q8_0": 17, "q4_0": 9}[args.kv] // 32
        leg = one_sequence_leg(eng, E, shape, n_slots, synth.streamed_weight_bytes(shape), kvb, steps=args.steps)
        eng.close()
        print(json.dumps({"metric": "single-sequence decode steps, %s" % shape.name, "activations": args.activations,
                          "single_token_matvec": bool(args.single_token_matvec), "kv_cache": args.kv, **leg}), flush=True)
        return 0
    eng = new_engine(args.activations)
    m, wl = measure_decode(args, eng, E, synth, gw, shape, geometry, profile_kernels=True)
    sampled, decode_rows, cells, tokens, elapsed = m["dec"]
    pre_tokens, pre_seconds, pre_steps = m["pre"]
    prof = m["prof"]

    ms_per_step = elapsed / args.steps * 1e3
    tok_s = sampled / elapsed

    hp = shape
    kv_bytes_per_cell_layer = 2 * hp.n_head_kv * hp.head_dim * 2       # K and V, f16
    if args.kv == "q8_0":
        kv_bytes_per_cell_layer = kv_bytes_per_cell_layer * 17 // 32      # 34 bytes per block of 32 values
    elif args.kv == "q4_0":
        kv_bytes_per_cell_layer = kv_bytes_per_cell_layer * 9 // 32       # 18 bytes per block of 32 values
    ratio = read_traffic_ratio(args.traffic_file, shape.name) if args.kv == "f16" else None      # measured on the f16 attention kernel

    # ---- whole-step roofline (north star): weights once + KV of every attended cell
    w_bytes = synth.streamed_weight_bytes(hp)       # every dense matrix once, at its stored type
    step_bytes = w_bytes + hp.n_layer * kv_bytes_per_cell_layer * (cells / args.steps)
    step_roof_tok_s = (sampled / args.steps) / (step_bytes / (HBM_PEAK_GBS * 1e9))

    # ---- every kernel family of the step, from the profiled steps after the timed region
    kernels = []
    mm_name = "k_mm5_q4k" if args.shape == "c2" else "k_mm5_q4k / k_mm2_q6k"
    if m["kernels"]:
        kprof, kdec, ksteps = m["kernels"]
        kcells = kdec[2] / ksteps
        cats = matrix_bytes_by_category(hp, synth, gw)
        fam_ms = fam_bytes = fam_launches = 0.0
        attn_name = ("k_attention_decode<128, 8> (rotation, KV store, attention and split merge of a pure decode step)"
                     if args.kv == "f16" else "k_attention<128, true, true> over a %s cache" % args.kv)
        rows = [(attn_name, "attention", kv_bytes_per_cell_layer * kcells)]
        rows += [("%s (%s)" % (mm_name, c), c, cats[c]) for c in ("qkv", "o_proj", "gate_up", "down")]
        for name, cat, by in rows:
            ms, n = kprof[cat]
            if n == 0:
                continue
            us = ms / n * 1e3
            kernels.append({"kernel": name, "launches_per_step": round(n / ksteps, 2), "algorithmic_bytes_per_launch": round(by),
                            "avg_launch_us": round(us, 2), "ms_per_step": round(ms / ksteps, 3),
                            "achieved_GBs": round(by / (us * 1e-6) / 1e9, 1), "frac": round(by / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)})
            if cat == "attention" and ratio:
                kernels[-1]["traffic_ratio"] = ratio
                kernels[-1]["traffic"] = round(ratio * by)
            if cat != "attention":
                fam_ms += ms; fam_bytes += by * n; fam_launches += n
        if fam_launches:
            us = fam_ms / fam_launches * 1e3
            kernels.append({"kernel": "%s, the layer matmuls together (furthest from its roof)" % mm_name,
                            "launches_per_step": round(fam_launches / ksteps, 2),
                            "algorithmic_bytes_per_launch": round(fam_bytes / fam_launches), "avg_launch_us": round(us, 2),
                            "ms_per_step": round(fam_ms / ksteps, 3),
                            "achieved_GBs": round(fam_bytes / fam_launches / (us * 1e-6) / 1e9, 1),
                            "frac": round(fam_bytes / fam_launches / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)})
        others = {c: round(kprof[c][0] / ksteps, 3) for c in ("norm", "rope", "combine", "head", "sample", "pack", "embed") if kprof[c][1]}
        kernels.append({"kernel": "latency-bound kernels, ms per step (events around each launch, which adds a few us to each)", **others})

    # The dominant kernel by time per step is the tile matmul (one kernel, four launches per layer and the head):
    # algorithmic bytes = the stored bytes of the matrices a step streams, duration = its launches' HIP events.
    dominant = {"kernel": None, "achieved": None, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": None, "traffic": None}
    if m["kernels"]:
        kprof, kdec, ksteps = m["kernels"]
        mm_ms = sum(kprof[c][0] for c in ("qkv", "o_proj", "gate_up", "down", "head"))
        mm_n = sum(kprof[c][1] for c in ("qkv", "o_proj", "gate_up", "down", "head"))
        at_ms = kprof["attention"][0]
        if mm_n and mm_ms >= at_ms:
            by = w_bytes * ksteps / mm_n
            us = mm_ms / mm_n * 1e3
            dominant = {
                "kernel": "%s (the tile matmul: qkv, attention output, gate/up + SwiGLU, down of every layer and the head; "
                          "%.3f ms of a step against %.3f ms of attention)" % (mm_name, mm_ms / ksteps, at_ms / ksteps),
                "achieved": round(by / (us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(by / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                "traffic": read_matmul_traffic(args.matmul_traffic_file, shape.name, by), "algorithmic_bytes_per_launch": round(by),
                "avg_launch_us": round(us, 2), "launches_timed": int(mm_n),
                "note": "average over the family's launches of %d profiled decode steps after the timed region (HIP events on the "
                        "engine's stream; an event pair adds a few us to each launch)" % ksteps,
            }
        else:
            n = kprof["attention"][1]
            by = kv_bytes_per_cell_layer * kdec[2] / ksteps
            us = at_ms / max(n, 1) * 1e3
            dominant = {"kernel": "k_attention (paged split-KV attention of a decode step, one launch per layer)",
                        "achieved": round(by / (us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": round(by / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4), "traffic": round(ratio * by) if ratio else None,
                        "algorithmic_bytes_per_launch": round(by), "avg_launch_us": round(us, 2), "launches_timed": int(n)}

    arithmetic = ("f16 hi/lo activations (about 22 bits)" if args.activations == "exact" else
                  "activations converted to Q8_K blocks as the reference's CPU path does (ggml arithmetic)")
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
        "dtype": ("q4_k" if args.shape != "c2-q4km" else "q4_k / q6_k") + " weights x " + arithmetic + ", f32 accumulate, " + ("f16 KV" if args.kv == "f16" else args.kv.upper() + " KV (a secondary configuration: the workload names an f16 cache)"),
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: %s, %d live sequences, prompts log-uniform [%d,%d], greedy, %d new tokens, continuous batching"
                        % (shape.name, n_slots, len_lo, len_hi, max_new),
            "n_batch": n_batch,
            "activations": args.activations,
            "kv_cache": args.kv,
            "mean_decode_rows_per_step": round(decode_rows / args.steps, 2),
            "mean_tokens_per_step": round(tokens / args.steps, 2),
            "mean_kv_cells_attended_per_step": round(cells / args.steps, 1),
            "requests_finished_in_window": m["finished"],
            "timing": "sum of the %d decode steps' own durations; prefill of admitted requests runs between them, untimed" % args.steps,
            "prefill_between_decode_steps": {"steps": pre_steps, "tokens": pre_tokens,
                                             "tok_s": round(pre_tokens / pre_seconds, 1) if pre_seconds > 0 else None},
            "mixed_tok_s_including_prefill_time": round(sampled / m["wall"], 1),
        },
        "roofline": {
            "bound": "hbm",
            **dominant,
            "step": {
                "algorithmic_bytes_per_step": round(step_bytes),
                "roofline_tok_s": round(step_roof_tok_s, 1),
                "frac": round(tok_s / step_roof_tok_s, 4),
            },
            "kernels": kernels,
        },
    }
    if args.stream_probe > 0:
        us = E.kernel_stream_time(args.stream_probe << 20, False, 3)
        print("[bench] copy kernel over %d MiB: %.1f us per launch" % (args.stream_probe, us), file=sys.stderr, flush=True)
    if args.profile_all:
        print("[bench] kernel time per step (ms): " + ", ".join(
            "%s=%.3f" % (k, v[0] / args.steps) for k, v in prof.items()), file=sys.stderr, flush=True)

    if not args.no_cpu_baseline:
        result["cpu_baseline"], result["parity_full_size"] = cpu_baseline(eng, E, oracle, wl, model_path, args.cpu_rows, args.activations, kv=args.kv)
    else:
        result["cpu_baseline"] = None

    if not args.no_scheduler_leg:
        for s_ in wl.seqs:                         # the hand-composed cohort gives its slots back
            if s_ is not None:
                eng.seq_rm(s_.slot)
                eng.request_free(s_.request)
        result["config"]["through_the_step_scheduler"] = scheduler_leg(args, eng, E, shape, geometry)
        result["config"]["one_sequence"] = {args.activations: one_sequence_leg(eng, E, shape, n_slots, w_bytes, kv_bytes_per_cell_layer)}
        if args.activations == "exact":
            # opt-in (RETRO_GEMV_EXACT=1): the matrix-vector kernel with f32 rows; a sequence decoded alone then differs
            # in the last bits from the same sequence inside a batch, so the tile kernels stay the default
            eng.single_token_matvec(True)
            result["config"]["one_sequence"]["exact_with_the_single_token_matvec_kernel"] = one_sequence_leg(eng, E, shape, n_slots, w_bytes, kv_bytes_per_cell_layer)
            eng.single_token_matvec(False)
        result["config"]["small_steps"] = [one_sequence_leg(eng, E, shape, n_slots, w_bytes, kv_bytes_per_cell_layer, n_seq=n) for n in (8, 32)]
    eng.close()
    del eng

    if not args.no_ggml_leg and args.activations == "exact":
        # secondary figure: the same timed loop with the activations converted as the reference's CPU path converts them
        eng = new_engine("ggml")
        m2, wl2 = measure_decode(args, eng, E, synth, gw, shape, geometry, profile_kernels=False)
        s2, _, c2, _, e2 = m2["dec"]
        b2 = w_bytes + hp.n_layer * kv_bytes_per_cell_layer * (c2 / args.steps)
        leg = {"value": round(s2 / e2, 1), "unit": "tok/s", "ms_per_step": round(e2 / args.steps * 1e3, 4),
               "step_frac_of_hbm_roofline": round((s2 / e2) / ((s2 / args.steps) / (b2 / (HBM_PEAK_GBS * 1e9))), 4),
               "arithmetic": "RETRO_ACTIVATIONS=ggml: Q8_K / Q8_0 activation conversion before every quantised matmul",
               "parity": "unpinned at this depth: a value within an ulp of a rounding boundary takes the neighbouring code in one of "
                         "two faithful implementations, and over 32 layers the two drift as far apart as the conversion moves the "
                         "logits in the first place, so the full-size comparison below cannot tell a correct kernel from a wrong one; "
                         "the kernels of this mode are checked per matmul against the oracle's codes and, on models of two layers "
                         "at the real widths, end to end (tests/test_gpu_fullsize.py)"}
        if not args.no_cpu_baseline:
            _, leg["parity_full_size_against_the_oracle_in_the_same_arithmetic"] = cpu_baseline(eng, E, oracle, wl2, model_path, args.cpu_rows, "ggml", time_it=False, kv=args.kv)
        for s_ in wl2.seqs:
            if s_ is not None:
                eng.seq_rm(s_.slot)
                eng.request_free(s_.request)
        leg["one_sequence"] = one_sequence_leg(eng, E, shape, n_slots, w_bytes, kv_bytes_per_cell_layer)
        result["ggml_arithmetic"] = leg
        eng.close()
    os.environ["RETRO_ACTIVATIONS"] = "exact"

    print(json.dumps(result), flush=True)
    return 0


def one_sequence_leg(eng, E, shape, n_slots, w_bytes, kv_bytes_per_cell_layer, context=512, steps=48, n_seq=1):
    """Decode steps of n_seq sequences (1 by default) at a fixed context on an engine whose slots are free again:
    the small-batch end of the same step, the ubatch grid of the reference's serving benchmark
    (src/bench/serving.rs:121-131 measures 1, 8 and 32 rows)."""
    for slot in range(n_slots):
        eng.seq_rm(slot)
    rng = np.random.default_rng(99)
    out = E.StepOutput(max(8, n_seq))
    greedy = E.SamplingParamsV2.greedy()
    request = 1 << 40
    prompts = [rng.integers(0, shape.n_vocab, context).astype(np.int32) for _ in range(n_seq)]
    tokens = []
    for i, prompt in enumerate(prompts):
        eng.step([E.StepRow(request + i, i, prompt, 0, sample=True, sampling=greedy)], out)
        tokens.append(out.row(0).token)
    pos, times = context, []
    for it in range(steps):
        t0 = time.perf_counter()
        eng.step([E.StepRow(request + i, i, [tokens[i]], pos, sample=True, sampling=greedy) for i in range(n_seq)], out)
        dt = time.perf_counter() - t0
        tokens, pos = [out.row(i).token for i in range(n_seq)], pos + 1
        if it >= 8:
            times.append(dt)
    for i in range(n_seq):
        eng.seq_rm(i)
        eng.request_free(request + i)
    sec = float(np.median(times))
    step_bytes = w_bytes + shape.n_layer * kv_bytes_per_cell_layer * n_seq * (context + steps // 2)
    return {"rows": n_seq, "context": context, "ms_per_step": round(sec * 1e3, 4), "tok_s": round(n_seq / sec, 1),
            "step_frac_of_hbm_roofline": round(step_bytes / (HBM_PEAK_GBS * 1e9) / sec, 4),
            "timing": "median of %d decode steps of %d row(s), host clock around each step" % (len(times), n_seq)}


def cpu_baseline(eng, E, oracle, wl, model_path, n_rows, activations="exact", time_it=True, kv="f16"):
    """Times the CPU oracle on one decode step over the first n_rows live
    sequences of the same workload (their KV imported from the engine's own
    snapshots), and compares its logits with the engine's for the same rows."""
    live = [s for s in wl.seqs if s is not None and s.last_token is not None][:n_rows]
    model = oracle.Model(model_path)
    ctx = oracle.Context(model, max(s.slot for s in live) + 1, activations=activations, kv=kv)
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
    while time_it and cpu_s < 8.0 and cpu_steps < 8:
        t0 = time.perf_counter()
        more = ctx.step_rows([(s.slot, s.pos + cpu_steps, [feed[i]], True) for i, s in enumerate(live)])
        cpu_s += time.perf_counter() - t0
        feed = [int(r.argmax()) for r in more]
        cpu_steps += 1
    # the engine decodes every live sequence in that step, as in the timed region (a full 64-token chunk takes
    # the decode kernels the headline is measured on); the rows the oracle computed come first
    taken = {id(s) for s in live}
    every = live + [s for s in wl.seqs if s is not None and s.last_token is not None and id(s) not in taken]
    out = E.StepOutput(len(every))
    eng.step([E.StepRow(s.request, s.slot, [s.last_token], s.pos, sample=True, sampling=wl.sampling) for s in every], out)
    got = eng.debug_logits()[:len(live)]
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    margins = np.sort(want, axis=1)
    margin = margins[:, -1] - margins[:, -2]
    same = [int(out.row(i).token) == int(want[i].argmax()) for i in range(len(live))]
    decided = [bool(m > 2 * 2e-2) for m in margin]
    parity = {
        "rows": len(live),
        "rows_in_the_engine_step": len(every),
        "max_abs_logit_error": float(err.max()),
        "mean_abs_relative_error": float(err.mean() / np.abs(want).mean()),
        "greedy_tokens_equal": int(sum(same)),
        "greedy_tokens_equal_where_margin_exceeds_tolerance": "%d/%d" % (sum(s for s, d in zip(same, decided) if d), sum(decided)),
        "against": "the CPU oracle in the %s arithmetic on the same KV and tokens. The oracle's forward pass is pinned against "
                   "Hugging Face transformers logits (tests/golden/hf_reference_logits.npz); the reference's own ggml build is "
                   "absent, so float-level parity with it is unpinned. The reference's CPU path converts activations to Q8_K "
                   "before every Q4_K matmul, which by the oracle moves logits 3.5-6 %% (mean-abs relative) away from the exact "
                   "product; the 2e-2 / 1e-3 tolerances are shown on the exact arithmetic." % activations,
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
