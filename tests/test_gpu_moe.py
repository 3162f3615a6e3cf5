"""Mixture-of-experts layers on the GPU against the CPU oracle (qwen3moe:
softmax router, top-k experts with renormalised weights, SwiGLU experts;
MXFP4, Q8_0, Q4_K, Q5_K and Q6_K expert weights)."""
import numpy as np
import pytest

import oracle
from engine_helpers import assert_logits_close, greedy, logit_errors, run_both
from retrograd_amd import engine as E
from retrograd_amd import gguf_writer as gw
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

BASE = dict(n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64, n_vocab=1024, n_expert=16, n_expert_used=4,
            n_ff_exp=256)
SHAPES = {
    "mxfp4": synth.scaled(synth.QWEN3_30B_A3B, name="qwen3moe-small-mxfp4", **BASE),
    "q8_0": synth.scaled(synth.QWEN3_30B_A3B, name="qwen3moe-small-q8", expert_type=gw.GGML_Q8_0, **BASE),
    # the expert types of a Q4_K_M mixture-of-experts file
    "q4_k": synth.scaled(synth.QWEN3_30B_A3B, name="qwen3moe-small-q4k", expert_type=gw.GGML_Q4_K, **BASE),
    "q6_k": synth.scaled(synth.QWEN3_30B_A3B, name="qwen3moe-small-q6k", expert_type=gw.GGML_Q6_K, **BASE),
    "q5_k": synth.scaled(synth.QWEN3_30B_A3B, name="qwen3moe-small-q5k", expert_type=gw.GGML_Q5_K, **BASE),
    # the whole mix of such a file: Q4_K matrices and experts, Q6_K for attn_v, the experts' down projection and the head
    "q4_k_m": synth.scaled(synth.QWEN3_30B_A3B, name="qwen3moe-small-q4km", matrix_type=gw.GGML_Q4_K, v_type=gw.GGML_Q6_K,
                           output_type=gw.GGML_Q6_K, expert_type=gw.GGML_Q4_K, expert_down_type=gw.GGML_Q6_K, **BASE),
}


@pytest.mark.parametrize("key", list(SHAPES))
def test_moe_prefill_and_decode_match_the_oracle(tmp_path, key):
    shape = SHAPES[key]
    print("mixture of experts: %s" % shape.name, flush=True)
    path = tmp_path / "moe.gguf"
    synth.write_model(path, shape, seed=5, device="cpu", std=0.05)
    eng = E.Engine(path, E.EngineConfig(n_ctx=2048, n_seq_max=8, n_batch=256, n_ubatch=256))
    m = oracle.Model(path)
    ctx = oracle.Context(m, 8)
    rng = np.random.default_rng(2)
    lens = [7, 40, 65, 18, 3]                      # 133 tokens: experts see more than 32 tokens each
    prompts = [rng.integers(0, m.n_vocab, n) for n in lens]
    rows = [(i, i, p, 0, True) for i, p in enumerate(prompts)]
    out, got, want = run_both(eng, ctx, rows)
    assert_logits_close(got, want)
    pos = list(lens)
    for _ in range(3):
        feed = [int(want[i].argmax()) for i in range(len(lens))]
        rows = [(i, i, [feed[i]], pos[i], True) for i in range(len(lens))]
        out, got, want = run_both(eng, ctx, rows)
        assert_logits_close(got, want)
        pos = [p + 1 for p in pos]
    eng.close()


def test_mxfp4_experts_on_the_block_scaled_instruction(tmp_path, monkeypatch):
    """RETRO_MOE_SCALED=1: decode-sized steps multiply the MXFP4 experts on the block-scaled FP4 x FP8 matrix
    instruction (the stored codes and exponents as they are, the activations as hexadecimal digits); larger steps keep
    the tile kernels. Against the oracle, and against the default engine: close, and not the same bits, so the step did
    take the other path. An expert with more than 16 pairs (two groups of slots) and experts with none are among them."""
    shape = synth.scaled(synth.QWEN3_30B_A3B, name="qwen3moe-small-mxfp4-wide", n_layer=2, n_embd=512, n_head=8, n_head_kv=2,
                         head_dim=64, n_vocab=1024, n_expert=16, n_expert_used=4, n_ff_exp=768)
    print("mixture of experts on the block-scaled instruction: %s" % shape.name, flush=True)
    path = tmp_path / "moe.gguf"
    synth.write_model(path, shape, seed=6, device="cpu", std=0.05)
    cfg = E.EngineConfig(n_ctx=4096, n_seq_max=48, n_batch=256, n_ubatch=256)
    plain = E.Engine(path, cfg)
    monkeypatch.setenv("RETRO_MOE_SCALED", "1")
    scaled = E.Engine(path, cfg)
    m = oracle.Model(path)
    ctx = oracle.Context(m, 48)
    rng = np.random.default_rng(3)
    n_seq = 40                                     # 160 pairs over 16 experts: ten on average, some above 16
    lens = [int(n) for n in rng.integers(3, 30, n_seq)]
    prompts = [rng.integers(0, m.n_vocab, n) for n in lens]
    rows = [(i, i, p, 0, True) for i, p in enumerate(prompts)]
    out = E.StepOutput()
    for at in range(0, n_seq, 8):                  # prefill steps of more than 12 pairs per expert: the tile kernels
        for eng in (plain, scaled):
            eng.step([E.StepRow(r[0], r[1], r[2], r[3], sample=True, sampling=greedy()) for r in rows[at:at + 8]], out)
        ctx.step_rows([(r[1], r[3], r[2], r[4]) for r in rows[at:at + 8]])
    pos = list(lens)
    feed = [int(t) for t in rng.integers(0, m.n_vocab, n_seq)]
    differs = False
    for step in range(3):
        live = list(range(n_seq)) if step != 1 else [0, 5, 6]          # 160 pairs, then 12 (most experts idle), then 160
        steprows = [E.StepRow(i, i, [feed[i]], pos[i], sample=True, sampling=greedy()) for i in live]
        plain.step(steprows, out)
        a = plain.debug_logits().copy()
        scaled.step(steprows, out)
        b = scaled.debug_logits().copy()
        want = ctx.step_rows([(i, pos[i], [feed[i]], True) for i in live])
        assert_logits_close(a, want)
        assert_logits_close(b, want)
        mx, rel = logit_errors(b, a)
        print("step %d: scaled against tile kernels, max %.2e rel %.2e" % (step, mx, rel), flush=True)
        assert rel <= 2e-5
        differs = differs or not np.array_equal(a, b)
        for j, i in enumerate(live):
            feed[i] = int(want[j].argmax())
            pos[i] += 1
    assert differs
    plain.close()
    scaled.close()


@pytest.mark.parametrize("key", list(SHAPES))
def test_moe_under_the_ggml_arithmetic(tmp_path, key, monkeypatch):
    """RETRO_ACTIVATIONS=ggml: the router (F32) multiplies the rows as they are, the experts
    their Q8_0 conversion, the hidden rows are converted again for the down projection.
    End to end the product follows the oracle's ggml arithmetic as closely as rounding-boundary
    drift allows (tests/test_gpu_step.py explains the criterion): clearly closer than the
    plain product is."""
    shape = SHAPES[key]
    print("mixture of experts, ggml arithmetic: %s" % shape.name, flush=True)
    path = tmp_path / "moe.gguf"
    synth.write_model(path, shape, seed=5, device="cpu", std=0.05)
    monkeypatch.setenv("RETRO_ACTIVATIONS", "ggml")
    eng = E.Engine(path, E.EngineConfig(n_ctx=2048, n_seq_max=8, n_batch=256, n_ubatch=256))
    m = oracle.Model(path)
    rng = np.random.default_rng(2)
    lens = [7, 40, 65, 18, 3]
    prompts = [rng.integers(0, m.n_vocab, n) for n in lens]
    rows = [(i, i, p, 0, True) for i, p in enumerate(prompts)]
    out, got, want = run_both(eng, oracle.Context(m, 8, activations="ggml"), rows)
    exact = oracle.Context(m, 8, activations="exact").step_rows([(r[1], r[3], r[2], r[4]) for r in rows])
    (_, drift), (_, conversion) = logit_errors(got, want), logit_errors(exact, want)
    print("drift %.2e, conversion %.2e" % (drift, conversion), flush=True)
    assert drift < 0.6 * conversion, (drift, conversion)
    eng.close()
