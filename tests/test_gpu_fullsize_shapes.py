"""Decode steps at the full shapes of the other configurations of the benchmark set, against the CPU oracle:

* multi-LoRA decode on the Qwen2.5-7B shape (28 layers, hidden 3584 = 14 super-blocks, 28 / 4 heads of 128, FFN 18944,
  vocabulary 152064, Q8_0, q/k/v biases) with eight rank-16 F16 adapters on q, k, v and the attention output, rows
  routed to different adapters and to the base (routing contract: reference
  crates/retrograd-ffi/runtime/src/retro_gen_core.cpp:2539-2564);
* the mixture of experts of the Qwen3-30B-A3B shape (48 layers, hidden 2048, 32 / 4 heads, 128 experts of width 768
  with top-8 routing, attention in Q8_0, experts in MXFP4), prefilled with enough tokens that the experts see ragged
  counts;
* the 8B shape's widths (hidden 4096, FFN 14336, vocabulary 128256) at two layers under the ggml activation arithmetic,
  where depth does not yet hide a wrong kernel behind the arithmetic's own drift: full 64-row steps (tile kernels) and
  one- and two-row steps (the integer matrix-vector kernel).

At these sizes the oracle cannot prefill in test time: it takes every sequence's KV from the engine's own snapshots and
computes one decode step (logits within 2e-2 max-abs / 1e-3 mean-abs relative in the exact arithmetic), and the
size-independent properties are checked bit for bit: a copied slot decodes like its source, a permuted batch like the
original. The split-K, row-group and expert-grouping index arithmetic of the kernels is what these shapes add to the
small models of test_gpu_lora.py and test_gpu_moe.py."""
import os
from pathlib import Path

import numpy as np
import pytest

import oracle
from engine_helpers import assert_logits_close, greedy, logit_errors
from retrograd_amd import engine as E
from retrograd_amd import gguf_writer as gw
from retrograd_amd import synth

pytestmark = pytest.mark.gpu


def _cached(tmp_path_factory, name, write):
    shm = Path("/dev/shm")
    base = shm if shm.is_dir() and os.access(shm, os.W_OK) else tmp_path_factory.mktemp("full_shapes")
    path = base / name
    if not path.exists():
        tmp = path.with_suffix(".tmp%d" % os.getpid())
        write(tmp)
        os.replace(tmp, path)
    return path


def _prefill(eng, slot, toks, adapter=None, chunk=512):
    out = E.StepOutput()
    for at in range(0, len(toks), chunk):
        done = at + chunk >= len(toks)
        kw = {"adapter": E.RowAdapter(adapter)} if adapter is not None else {}
        eng.step([E.StepRow(slot, slot, toks[at:at + chunk], at, sample=done, sampling=greedy(), **kw)], out)
    return out.row(0).token


def test_multi_lora_decode_at_the_full_qwen25_7b_shape(tmp_path_factory):
    shape = synth.QWEN25_7B_Q8
    print("full shape: %s with eight rank-16 adapters" % shape.name, flush=True)
    model = _cached(tmp_path_factory, "retro-bench-%s-seed1234.gguf" % shape.name,
                    lambda p: synth.write_model(p, shape, seed=1234, device="cuda"))
    files = [_cached(tmp_path_factory, "retro-bench-c4-lora-%d-seed1234.gguf" % i,
                     lambda p, i=i: synth.write_lora_adapter(p, shape, rank=16, alpha=16.0, seed=1234 + 100 + i, std_a=0.02, std_b=0.01))
             for i in range(8)]
    eng = E.Engine(model, E.EngineConfig(n_ctx=8 * 1536, n_seq_max=8, n_batch=512, n_ubatch=512))
    ids = [eng.adapter_load(f, 1.0) for f in files]
    assert ids == list(range(1, 9))
    rng = np.random.default_rng(11)
    lens = [300, 47, 700, 1200]
    route = [ids[0], E.RETRO_STEP_ADAPTER_BASE, ids[4], ids[7]]
    prompts = [rng.integers(0, shape.n_vocab, n).astype(np.int32) for n in lens]
    feed = [_prefill(eng, i, prompts[i], route[i]) for i in range(4)]
    print("prefilled", flush=True)

    # the oracle's context from the engine's snapshots of before the step
    m = oracle.Model(model)
    assert [m.load_adapter(f, 1.0) for f in files] == ids
    ctx = oracle.Context(m, 8)
    checked = (0, 1, 2)           # an adapter, the base, another adapter
    for s in checked:
        ctx.import_snapshot(s, eng.seq_save(s))
    for i in range(3):            # copies of three slots, to decode beside their sources
        eng.seq_cp(i, 4 + i)

    out = E.StepOutput()
    eng.step([E.StepRow(i, i, [feed[i]], lens[i], sample=True, sampling=greedy(), adapter=E.RowAdapter(route[i])) for i in range(4)], out)
    src = eng.debug_logits().copy()
    src_tok = [out.row(i).token for i in range(4)]
    want = ctx.step_rows([(s, lens[s], [feed[s]], True) for s in checked],
                         adapters=[route[s] if route[s] > 0 else -1 for s in checked])
    print("errors", logit_errors(src[list(checked)], want), flush=True)
    assert_logits_close(src[list(checked)], want)
    for row, s in enumerate(checked):
        srt = np.sort(want[row])[::-1]
        if srt[0] - srt[1] > 4e-2:
            assert src_tok[s] == int(want[row].argmax())
    # a row routed elsewhere gives other logits: the routing is not a no-op at this shape
    assert not np.array_equal(src[0], src[1])

    # the copies under their sources' adapters, in another order: bit for bit
    order = [2, 0, 1]
    eng.step([E.StepRow(10 + i, 4 + i, [feed[i]], lens[i], sample=True, sampling=greedy(), adapter=E.RowAdapter(route[i])) for i in order], out)
    got = eng.debug_logits()
    for at, i in enumerate(order):
        assert out.row(at).token == src_tok[i]
        assert np.array_equal(got[at], src[i]), "a copy decodes like its source, wherever its row stands"
    eng.close()


def test_mixture_of_experts_decode_at_the_full_qwen3_30b_a3b_shape(tmp_path_factory):
    shape = synth.scaled(synth.QWEN3_30B_A3B, expert_type=gw.GGML_MXFP4)
    print("full shape: %s, MXFP4 experts" % shape.name, flush=True)
    model = _cached(tmp_path_factory, "retro-bench-%s-seed1234.gguf" % shape.name,
                    lambda p: synth.write_model(p, shape, seed=1234, device="cuda"))
    eng = E.Engine(model, E.EngineConfig(n_ctx=8 * 512, n_seq_max=8, n_batch=512, n_ubatch=512))
    rng = np.random.default_rng(12)
    lens = [70, 25, 40, 33]
    prompts = [rng.integers(0, shape.n_vocab, n).astype(np.int32) for n in lens]
    out = E.StepOutput()
    # one ragged prefill step: 168 tokens over 128 experts with top-8 routing, about ten tokens per expert, unevenly
    eng.step([E.StepRow(i, i, prompts[i], 0, sample=True, sampling=greedy()) for i in range(4)], out)
    feed = [out.row(i).token for i in range(4)]
    print("prefilled", flush=True)

    m = oracle.Model(model)
    ctx = oracle.Context(m, 8)
    checked = (1, 3)
    for s in checked:
        ctx.import_snapshot(s, eng.seq_save(s))
    for i in range(3):
        eng.seq_cp(i, 4 + i)
    eng.step([E.StepRow(i, i, [feed[i]], lens[i], sample=True, sampling=greedy()) for i in range(4)], out)
    src = eng.debug_logits().copy()
    src_tok = [out.row(i).token for i in range(4)]
    want = ctx.step_rows([(s, lens[s], [feed[s]], True) for s in checked])
    print("errors", logit_errors(src[list(checked)], want), flush=True)
    assert_logits_close(src[list(checked)], want)
    for row, s in enumerate(checked):
        srt = np.sort(want[row])[::-1]
        if srt[0] - srt[1] > 4e-2:
            assert src_tok[s] == int(want[row].argmax())

    order = [1, 2, 0]
    eng.step([E.StepRow(10 + i, 4 + i, [feed[i]], lens[i], sample=True, sampling=greedy()) for i in order], out)
    got = eng.debug_logits()
    for at, i in enumerate(order):
        assert out.row(at).token == src_tok[i]
        assert np.array_equal(got[at], src[i]), "a copy decodes like its source, wherever its row stands"
    eng.close()


def test_ggml_arithmetic_at_the_real_widths_two_layers_deep(tmp_path_factory, monkeypatch):
    shape = synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, name="llama3-8b-widths-2-layers-q4_k")
    print("ggml arithmetic: %s" % shape.name, flush=True)
    model = _cached(tmp_path_factory, "retro-test-%s-seed77.gguf" % shape.name,
                    lambda p: synth.write_model(p, shape, seed=77, device="cuda"))
    monkeypatch.setenv("RETRO_ACTIVATIONS", "ggml")
    n_seq = 64
    eng = E.Engine(model, E.EngineConfig(n_ctx=n_seq * 128, n_seq_max=n_seq, n_batch=512, n_ubatch=512))
    rng = np.random.default_rng(13)
    lens = [int(n) for n in rng.integers(4, 40, n_seq)]
    prompts = [rng.integers(0, shape.n_vocab, n).astype(np.int32) for n in lens]
    out = E.StepOutput(n_seq)
    feed = [0] * n_seq
    for at in range(0, n_seq, 16):          # sixteen ragged rows per prefill step
        eng.step([E.StepRow(i, i, prompts[i], 0, sample=True, sampling=greedy()) for i in range(at, at + 16)], out)
        for j in range(16):
            feed[at + j] = out.row(j).token
    m = oracle.Model(model)
    ggml_ctx, exact_ctx = oracle.Context(m, n_seq, activations="ggml"), oracle.Context(m, n_seq, activations="exact")
    for s in range(n_seq):
        snap = eng.seq_save(s)
        ggml_ctx.import_snapshot(s, snap)
        exact_ctx.import_snapshot(s, snap)

    def compare(slots, what):
        rows = [(s, lens[s], [feed[s]], True) for s in slots]
        eng.step([E.StepRow(s, s, [feed[s]], lens[s], sample=True, sampling=greedy()) for s in slots], out)
        got = eng.debug_logits().copy()
        want = ggml_ctx.step_rows(rows)
        exact = exact_ctx.step_rows(rows)
        drift_max, drift = logit_errors(got, want)
        _, conversion = logit_errors(exact, want)
        print("%s: drift %.2e (max %.2e), conversion %.2e" % (what, drift, drift_max, conversion), flush=True)
        assert drift < 0.6 * conversion, (what, drift, conversion)
        for i in range(len(slots)):
            srt = np.sort(want[i])[::-1]
            if srt[0] - srt[1] > 4 * drift_max:
                assert out.row(i).token == int(want[i].argmax()), what
        for s in slots:                     # back to the prompt, in the engine and in both oracle contexts
            eng.seq_rm(s, lens[s], -1)
            ggml_ctx.seq_rm(s, lens[s], -1)
            exact_ctx.seq_rm(s, lens[s], -1)

    compare(list(range(n_seq)), "64 rows (tile kernels)")
    compare([5], "one row (integer matrix-vector kernel)")
    compare([9, 40], "two rows (integer matrix-vector kernel)")
    eng.close()


def test_single_row_steps_of_the_exact_arithmetic_at_the_real_widths(tmp_path_factory, monkeypatch):
    # A step of one token runs the matrix-vector kernel with f32 rows (RMSNorm, SwiGLU fused into its staging, the
    # output projection from the attention launch's planes): its logits against the oracle at the stated tolerances,
    # and against the tile kernels (RETRO_GEMV_EXACT=0) on the same KV; the fused steps launch no norm of their own.
    shape = synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, name="llama3-8b-widths-2-layers-q4_k")
    print("exact single-row steps: %s" % shape.name, flush=True)
    model = _cached(tmp_path_factory, "retro-test-%s-seed77.gguf" % shape.name,
                    lambda p: synth.write_model(p, shape, seed=77, device="cuda"))
    n_seq = 4
    rng = np.random.default_rng(21)
    lens = [int(n) for n in rng.integers(4, 40, n_seq)]
    prompts = [rng.integers(0, shape.n_vocab, n).astype(np.int32) for n in lens]
    m = oracle.Model(model)
    ctx = oracle.Context(m, n_seq, activations="exact")
    logits = {}
    for exact_kernel in (1, 0):
        monkeypatch.setenv("RETRO_GEMV_EXACT", str(exact_kernel))
        eng = E.Engine(model, E.EngineConfig(n_ctx=n_seq * 128, n_seq_max=n_seq, n_batch=512, n_ubatch=512))
        out = E.StepOutput(n_seq)
        eng.step([E.StepRow(i, i, prompts[i], 0, sample=True, sampling=greedy()) for i in range(n_seq)], out)
        feed = [out.row(i).token for i in range(n_seq)]
        if exact_kernel:
            for s in range(n_seq):
                ctx.import_snapshot(s, eng.seq_save(s))
        eng.profile(2)
        eng.profile_read()
        got = []
        for s in range(n_seq):
            eng.step([E.StepRow(s, s, [feed[s]], lens[s], sample=True, sampling=greedy())], out)
            got.append(eng.debug_logits()[0].copy())
        prof = eng.profile_read()
        eng.profile(0)
        # two layers: four norm launches per step on the tile kernels (the final norm counts with the head), none on the fused path
        assert prof["norm"][1] == (0 if exact_kernel else n_seq * 4), prof["norm"]
        logits[exact_kernel] = np.stack(got)
        eng.close()
    want = ctx.step_rows([(s, lens[s], [feed[s]], True) for s in range(n_seq)])
    assert_logits_close(logits[1], want)
    assert_logits_close(logits[0], want)
    mx, mr = logit_errors(logits[1], logits[0])
    print("matrix-vector kernel against the tile kernels: max %.2e, mean relative %.2e" % (mx, mr), flush=True)
    assert mx <= 2e-3 and mr <= 1e-4


@pytest.mark.parametrize("matrix_type", [gw.GGML_Q8_0, gw.GGML_Q4_K])
def test_a_gate_up_matrix_wider_than_the_chip_has_workgroups(tmp_path_factory, matrix_type):
    # FFN 18944 (the Qwen2.5-7B width) is 296 groups of 128 fused gate/up rows for 256 CUs: steps of 33 to 64 tokens
    # multiply the first 256 groups with the fused SiLU epilogue and the other 40 with K split over workgroups, a
    # small launch adding the slices. One layer at hidden 1024 against the oracle, at 64, 40 (split) and 20 rows
    # (one launch: smaller workgroups share a CU), and the hidden columns on either side of the seam by a copy.
    shape = synth.scaled(synth.QWEN25_7B_Q8, n_layer=1, n_embd=1024, n_head=8, n_head_kv=2, n_vocab=1024,
                         matrix_type=matrix_type, name="one-layer-ffn-18944-%d" % matrix_type)
    print("gate/up with left-over row groups: %s" % shape.name, flush=True)
    model = _cached(tmp_path_factory, "retro-test-%s-seed5.gguf" % shape.name,
                    lambda p: synth.write_model(p, shape, seed=5, device="cuda"))
    n_seq = 64
    eng = E.Engine(model, E.EngineConfig(n_ctx=n_seq * 64, n_seq_max=n_seq + 1, n_batch=512, n_ubatch=512))
    rng = np.random.default_rng(3)
    lens = [int(n) for n in rng.integers(2, 12, n_seq)]
    prompts = [rng.integers(0, shape.n_vocab, n).astype(np.int32) for n in lens]
    out = E.StepOutput(n_seq)
    m = oracle.Model(model)
    ctx = oracle.Context(m, n_seq + 1)
    eng.step([E.StepRow(i, i, prompts[i], 0, sample=True, sampling=greedy()) for i in range(n_seq)], out)
    ctx.step_rows([(i, 0, prompts[i], True) for i in range(n_seq)])
    feed = [out.row(i).token for i in range(n_seq)]
    for rows in (64, 40, 20):
        eng.step([E.StepRow(s, s, [feed[s]], lens[s], sample=True, sampling=greedy()) for s in range(rows)], out)
        got = eng.debug_logits().copy()
        want = ctx.step_rows([(s, lens[s], [feed[s]], True) for s in range(rows)])
        assert_logits_close(got, want)
        if rows == 64:
            eng.seq_cp(7, n_seq)
            eng.seq_rm(n_seq, lens[7], -1)
            eng.step([E.StepRow(n_seq, n_seq, [feed[7]], lens[7], sample=True, sampling=greedy())]
                     + [E.StepRow(s, s, [feed[s]], lens[s] + 1, sample=True, sampling=greedy()) for s in range(39)], out)
            again = eng.debug_logits()[0].copy()
            eng.seq_rm(n_seq)
            for s in range(39):
                eng.seq_rm(s, lens[s] + 1, -1)
            assert np.array_equal(again, got[7]), "a copy decodes like its source, wherever its row stands"
        for s in range(rows):
            eng.seq_rm(s, lens[s], -1)
            ctx.seq_rm(s, lens[s], -1)
    eng.close()


def test_the_left_over_gate_up_groups_under_the_ggml_arithmetic(tmp_path_factory, monkeypatch):
    # The same split with Q8_0 weights under the ggml arithmetic: the small launch that adds the slices also makes the
    # Q8_0 blocks of the down projection's rows. One layer deep the engine stays well inside the distance the
    # conversion itself moves the logits.
    shape = synth.scaled(synth.QWEN25_7B_Q8, n_layer=1, n_embd=1024, n_head=8, n_head_kv=2, n_vocab=1024,
                         matrix_type=gw.GGML_Q8_0, name="one-layer-ffn-18944-%d" % gw.GGML_Q8_0)
    print("gate/up with left-over row groups, ggml arithmetic: %s" % shape.name, flush=True)
    model = _cached(tmp_path_factory, "retro-test-%s-seed5.gguf" % shape.name,
                    lambda p: synth.write_model(p, shape, seed=5, device="cuda"))
    monkeypatch.setenv("RETRO_ACTIVATIONS", "ggml")
    n_seq = 48
    eng = E.Engine(model, E.EngineConfig(n_ctx=n_seq * 64, n_seq_max=n_seq, n_batch=512, n_ubatch=512))
    rng = np.random.default_rng(4)
    lens = [int(n) for n in rng.integers(2, 12, n_seq)]
    prompts = [rng.integers(0, shape.n_vocab, n).astype(np.int32) for n in lens]
    out = E.StepOutput(n_seq)
    eng.step([E.StepRow(i, i, prompts[i], 0, sample=True, sampling=greedy()) for i in range(n_seq)], out)
    feed = [out.row(i).token for i in range(n_seq)]
    m = oracle.Model(model)
    ggml_ctx, exact_ctx = oracle.Context(m, n_seq, activations="ggml"), oracle.Context(m, n_seq, activations="exact")
    for s in range(n_seq):
        snap = eng.seq_save(s)
        ggml_ctx.import_snapshot(s, snap)
        exact_ctx.import_snapshot(s, snap)
    rows = [(s, lens[s], [feed[s]], True) for s in range(n_seq)]
    eng.step([E.StepRow(s, s, [feed[s]], lens[s], sample=True, sampling=greedy()) for s in range(n_seq)], out)
    got = eng.debug_logits().copy()
    want, exact = ggml_ctx.step_rows(rows), exact_ctx.step_rows(rows)
    drift_max, drift = logit_errors(got, want)
    _, conversion = logit_errors(exact, want)
    print("drift %.2e (max %.2e), conversion %.2e" % (drift, drift_max, conversion), flush=True)
    assert drift < 0.6 * conversion, (drift, conversion)
    eng.close()

