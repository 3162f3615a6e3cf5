"""Per-row LoRA on the GPU against the CPU oracle: one step mixes rows decoded
under different adapters and under the base model (reference
crates/retrograd-ffi/runtime/src/retro_gen_core.cpp:2539-2564, tests/lora_rows.rs)."""
import numpy as np
import pytest

import oracle
from engine_helpers import assert_logits_close, greedy, logit_errors
from retrograd_amd import engine as E
from retrograd_amd import gguf_writer as gw
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

SHAPE = synth.scaled(synth.QWEN25_7B_Q8, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                     n_ff=1024, n_vocab=1024, name="qwen2-lora")


@pytest.fixture(scope="module")
def files(tmp_path_factory):
    d = tmp_path_factory.mktemp("lora")
    model = d / "m.gguf"
    synth.write_model(model, SHAPE, seed=77, device="cpu", std=0.05)
    a1, a2 = d / "a1.gguf", d / "a2.gguf"
    synth.write_lora_adapter(a1, SHAPE, rank=16, alpha=32.0, seed=1, std_a=0.1, std_b=0.1)
    synth.write_lora_adapter(a2, SHAPE, rank=8, alpha=8.0, seed=2, std_a=0.1, std_b=0.1,
                             targets=("attn_q", "attn_output"))
    # a target that is no matrix of a layer: never routed per row (reference retro_lora_train.h:2594-2596)
    ffn = d / "embd.gguf"
    w = gw.GGUFWriter()
    w.add("general.type", gw.T_STRING, "adapter")
    w.add("general.architecture", gw.T_STRING, SHAPE.arch)
    w.add("adapter.type", gw.T_STRING, "lora")
    w.add("adapter.lora.alpha", gw.T_FLOAT32, 4.0)
    rng = np.random.default_rng(5)
    w.add_tensor("token_embd.weight.lora_a", [SHAPE.n_embd, 4], gw.GGML_F32, rng.standard_normal((4, SHAPE.n_embd)).astype(np.float32).tobytes())
    w.add_tensor("token_embd.weight.lora_b", [4, SHAPE.n_vocab], gw.GGML_F32, rng.standard_normal((SHAPE.n_vocab, 4)).astype(np.float32).tobytes())
    w.write(ffn)
    return model, a1, a2, ffn


def test_rows_under_different_adapters_match_the_oracle(files):
    model, a1, a2, _ = files
    print("per-row LoRA: %s, ranks 16 and 8" % SHAPE.name, flush=True)
    eng = E.Engine(model, E.EngineConfig(n_ctx=1024, n_seq_max=4, n_batch=128, n_ubatch=128))
    m = oracle.Model(model)
    ctx = oracle.Context(m, 4)
    ids = [eng.adapter_load(a1, 1.0), eng.adapter_load(a2, 0.5)]
    oids = [m.load_adapter(a1, 1.0), m.load_adapter(a2, 0.5)]
    assert ids == oids == [1, 2]

    rng = np.random.default_rng(3)
    lens = [21, 9, 40, 13]
    prompts = [rng.integers(0, m.n_vocab, n) for n in lens]
    route = [ids[0], E.RETRO_STEP_ADAPTER_BASE, ids[1], 0]          # adapter 1, base, adapter 2, context (= base here)
    out = E.StepOutput()
    rows = [E.StepRow(i, i, prompts[i], 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(route[i])) for i in range(4)]
    eng.step(rows, out)
    got = eng.debug_logits()
    want = ctx.step_rows([(i, 0, prompts[i], True) for i in range(4)], adapters=[route[0], -1, route[2], -1])
    assert_logits_close(got, want)
    # the adapters do something: the same rows under the base model differ visibly
    base = oracle.Context(m, 4).step_rows([(i, 0, prompts[i], True) for i in range(4)])
    assert np.abs(want[0] - base[0]).max() > 5e-2 and np.abs(want[2] - base[2]).max() > 1e-2
    assert np.array_equal(want[1], base[1])

    pos = list(lens)
    for _ in range(3):       # decode steps (sliced matmuls at T = 4), teacher-forced with the oracle's tokens
        feed = [int(want[i].argmax()) for i in range(4)]
        rows = [E.StepRow(i, i, [feed[i]], pos[i], sample=True, sampling=greedy(), adapter=E.RowAdapter(route[i]))
                for i in range(4)]
        eng.step(rows, out)
        got = eng.debug_logits()
        want = ctx.step_rows([(i, pos[i], [feed[i]], True) for i in range(4)], adapters=[route[0], -1, route[2], -1])
        assert_logits_close(got, want)
        pos = [p + 1 for p in pos]

    info = eng.adapter_rows_info()
    E_, QD, KD = SHAPE.n_embd, SHAPE.n_head * SHAPE.head_dim, SHAPE.n_head_kv * SHAPE.head_dim
    el1 = SHAPE.n_layer * ((E_ + QD) + 2 * (E_ + KD) + (QD + E_))
    el2 = SHAPE.n_layer * ((E_ + QD) + (QD + E_))
    assert (info.n_adapters, info.max_rank) == (2, 16)
    assert info.stacked_bytes == (el1 + el2) * 16 * 4
    assert info.unpadded_bytes == el1 * 16 * 4 + el2 * 8 * 4
    eng.close()


FFN_TARGETS = ("attn_q", "ffn_gate", "ffn_up", "ffn_down")
# gate and up interleaved for the fused SwiGLU kernel (width a multiple of 64), and side by side on the generic kernels
FFN_SHAPES = {"interleaved": SHAPE, "side-by-side": synth.TINY_LLAMA}


@pytest.mark.parametrize("layout", list(FFN_SHAPES))
@pytest.mark.parametrize("activations", ["exact", "ggml"])
def test_adapters_on_the_feed_forward_matrices_match_the_oracle(tmp_path, layout, activations, monkeypatch):
    """Every true matrix of a layer may carry a pair (reference retro_lora.cpp:165-169): rows under an adapter with
    ffn_gate / ffn_up / ffn_down pairs, under an attention-only adapter and under the base share steps."""
    shape = FFN_SHAPES[layout]
    print("per-row LoRA on feed-forward matrices: %s, %s, %s arithmetic" % (shape.name, layout, activations), flush=True)
    if activations == "ggml":
        monkeypatch.setenv("RETRO_ACTIVATIONS", "ggml")
    model, ffn, attn = tmp_path / "m.gguf", tmp_path / "ffn.gguf", tmp_path / "attn.gguf"
    synth.write_model(model, shape, seed=31, device="cpu", std=0.05)
    synth.write_lora_adapter(ffn, shape, rank=4, alpha=8.0, seed=3, std_a=0.1, std_b=0.1, targets=FFN_TARGETS)
    synth.write_lora_adapter(attn, shape, rank=8, alpha=8.0, seed=4, std_a=0.1, std_b=0.1, targets=("attn_q", "attn_output"))
    eng = E.Engine(model, E.EngineConfig(n_ctx=1024, n_seq_max=4, n_batch=128, n_ubatch=128))
    m = oracle.Model(model)
    ctx = oracle.Context(m, 4, activations=activations)
    ids = [eng.adapter_load(ffn, 1.0), eng.adapter_load(attn, 0.5)]
    assert ids == [m.load_adapter(ffn, 1.0), m.load_adapter(attn, 0.5)]
    rng = np.random.default_rng(8)
    lens = [17, 33, 9, 66]           # 125 tokens: two 64-token chunks in the prefill step
    prompts = [rng.integers(0, m.n_vocab, n) for n in lens]
    route = [ids[0], ids[1], E.RETRO_STEP_ADAPTER_BASE, ids[0]]
    oroute = [ids[0], ids[1], -1, ids[0]]
    out = E.StepOutput()
    eng.step([E.StepRow(i, i, prompts[i], 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(route[i])) for i in range(4)], out)
    got = eng.debug_logits()
    want = ctx.step_rows([(i, 0, prompts[i], True) for i in range(4)], adapters=oroute)
    base = oracle.Context(m, 4, activations=activations).step_rows([(i, 0, prompts[i], True) for i in range(4)])
    assert np.abs(want[0] - base[0]).max() > 5e-2, "the feed-forward pairs do something"
    if activations == "exact":
        assert_logits_close(got, want)
    else:
        # two faithful implementations of the conversion drift apart by rounding ties; clearly nearer than the base model
        assert logit_errors(got, want)[1] < 0.3 * logit_errors(base, want)[1]
        eng.close()
        return
    pos = list(lens)
    for _ in range(3):
        feed = [int(want[i].argmax()) for i in range(4)]
        eng.step([E.StepRow(i, i, [feed[i]], pos[i], sample=True, sampling=greedy(), adapter=E.RowAdapter(route[i]))
                  for i in range(4)], out)
        got = eng.debug_logits()
        want = ctx.step_rows([(i, pos[i], [feed[i]], True) for i in range(4)], adapters=oroute)
        assert_logits_close(got, want)
        pos = [p + 1 for p in pos]
    # a step without a routed row goes back to the fused kernel: same logits as an engine that never loaded an adapter
    plain = E.Engine(model, E.EngineConfig(n_ctx=1024, n_seq_max=4, n_batch=128, n_ubatch=128))
    rows = lambda: [E.StepRow(9, 3, prompts[1], 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(E.RETRO_STEP_ADAPTER_BASE))]
    eng.seq_rm(3)
    eng.step(rows(), out)
    plain.step(rows(), out)
    assert np.array_equal(eng.debug_logits(), plain.debug_logits())
    info = eng.adapter_rows_info()
    E_, QD, F = shape.n_embd, shape.n_head * shape.head_dim, shape.n_ff
    el_ffn = shape.n_layer * ((E_ + QD) + 2 * (E_ + F) + (F + E_))
    el_attn = shape.n_layer * ((E_ + QD) + (QD + E_))
    assert info.stacked_bytes == (el_ffn + el_attn) * 8 * 4 and info.unpadded_bytes == el_ffn * 4 * 4 + el_attn * 8 * 4
    plain.close()
    eng.close()


def test_rows_under_adapters_with_the_ggml_arithmetic(files, monkeypatch):
    """RETRO_ACTIVATIONS=ggml: the base weights (Q8_0) multiply the Q8_0 conversion of a row,
    the F16 LoRA factors the same row rounded to f16 (and B the f16 rounding of A x), as
    ggml's CPU matmuls do. The criterion is the one of tests/test_gpu_step.py."""
    model, a1, a2, _ = files
    monkeypatch.setenv("RETRO_ACTIVATIONS", "ggml")
    eng = E.Engine(model, E.EngineConfig(n_ctx=1024, n_seq_max=4, n_batch=128, n_ubatch=128))
    m = oracle.Model(model)
    ids = [eng.adapter_load(a1, 1.0), eng.adapter_load(a2, 0.5)]
    assert [m.load_adapter(a1, 1.0), m.load_adapter(a2, 0.5)] == ids
    rng = np.random.default_rng(3)
    prompts = [rng.integers(0, m.n_vocab, n) for n in (21, 9, 40, 13)]
    route = [ids[0], E.RETRO_STEP_ADAPTER_BASE, ids[1], 0]
    out = E.StepOutput()
    eng.step([E.StepRow(i, i, prompts[i], 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(route[i])) for i in range(4)], out)
    got = eng.debug_logits()
    plan, adapters = [(i, 0, prompts[i], True) for i in range(4)], [route[0], -1, route[2], -1]
    want = oracle.Context(m, 4, activations="ggml").step_rows(plan, adapters=adapters)
    exact = oracle.Context(m, 4, activations="exact").step_rows(plan, adapters=adapters)
    (_, drift), (_, conversion) = logit_errors(got, want), logit_errors(exact, want)
    print("drift %.2e, conversion %.2e" % (drift, conversion), flush=True)
    assert drift < 0.6 * conversion, (drift, conversion)
    eng.close()


def test_the_context_adapter_and_per_row_adapters_share_a_step(files):
    """reference tests/lora_rows.rs:150-237: the context's own adapter is what rows with adapter 0
    follow, the others ignore it; every row of the mixed step matches the oracle's row under that
    adapter alone; unloading restacks; an empty routed set still bypasses the context adapter."""
    model, a1, a2, _ = files
    print("context adapter + per-row adapters", flush=True)
    eng = E.Engine(model, E.EngineConfig(n_ctx=1024, n_seq_max=4, n_batch=128, n_ubatch=128))
    m = oracle.Model(model)
    oid_a, oid_b = m.load_adapter(a1, 1.0), m.load_adapter(a2, 1.0)
    prompt = [int(t) for t in np.random.default_rng(4).integers(0, m.n_vocab, 23)]
    plan = [(i, 0, prompt, True) for i in range(4)]
    id_a, id_b = eng.adapter_load(a1, 1.0), eng.adapter_load(a2, 1.0)
    v0 = eng.weights_version()
    eng.load_lora(a2)                                 # the context's own adapter is b
    assert eng.active_adapter() == str(a2) and eng.weights_version() == v0 + 1
    out = E.StepOutput()
    route = [id_a, id_b, E.RETRO_STEP_ADAPTER_BASE, 0]
    eng.step([E.StepRow(i + 1, i, prompt, 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(route[i])) for i in range(4)], out)
    got = eng.debug_logits()
    want = oracle.Context(m, 4).step_rows(plan, adapters=[oid_a, oid_b, -1, oid_b])
    assert_logits_close(got, want)
    base = oracle.Context(m, 4).step_rows(plan)
    assert np.abs(want[0] - base[0]).max() > 5e-2, "the adapter must move the distribution, or the parity is vacuous"
    assert np.array_equal(got[1], got[3]), "a context row and a per-row b row are the same arithmetic"
    info = eng.adapter_rows_info()
    assert (info.n_adapters, info.max_rank) == (2, 16) and info.stacked_bytes > info.unpadded_bytes

    # unloading a restacks b alone; ids are not reused
    eng.adapter_unload(id_a)
    with pytest.raises(E.RuntimeFailure):
        eng.adapter_unload(id_a)
    for slot in range(4):
        eng.seq_rm(slot)
    eng.step([E.StepRow(5, 0, prompt, 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(id_b))], out)
    assert_logits_close(eng.debug_logits(), want[1:2])
    with pytest.raises(E.InvalidArgument):
        eng.step([E.StepRow(6, 1, prompt, 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(id_a))], out)

    # an empty routed set still bypasses the context adapter
    eng.adapter_unload(id_b)
    for slot in range(4):
        eng.seq_rm(slot)
    eng.step([E.StepRow(7 + i, i, prompt, 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(E.RETRO_STEP_ADAPTER_BASE))
              for i in range(4)], out)
    assert_logits_close(eng.debug_logits(), base)

    # named adapters: registered beside the others, one active; every switch is a weight change
    eng.load_lora_named("a", a1)
    assert eng.active_adapter() == str(a2), "registering does not activate"
    v1 = eng.weights_version()
    eng.activate_lora("a")
    assert eng.active_adapter() == "a" and eng.weights_version() == v1 + 1
    assert eng.memory().cells_used == 0, "a switch drops every resident cell"
    eng.step([E.StepRow(20, 0, prompt, 0, sample=True, sampling=greedy())], out)
    assert_logits_close(eng.debug_logits(), want[0:1])
    with pytest.raises(E.RuntimeFailure, match="no LoRA adapter registered under 'zzz'"):
        eng.activate_lora("zzz")
    eng.set_lora_enabled(False)
    assert eng.active_adapter() == ""
    eng.step([E.StepRow(21, 0, prompt, 0, sample=True, sampling=greedy())], out)
    assert_logits_close(eng.debug_logits(), base[0:1])
    with pytest.raises(E.RuntimeFailure, match="cannot enable LoRA: no adapter is active"):
        eng.set_lora_enabled(True)
    eng.close()


def test_the_scheduler_serves_a_named_adapter_through_the_engine(files):
    """A request that names an adapter (reference crates/retrograd-infer/tests/adapters.rs, there on the
    fake backend) is decoded under that context-wide adapter of the engine: the tokens are those of the
    same prompt under the same file as a per-row adapter, and the base model's afterwards."""
    from retrograd_amd import scheduler as S
    model, a1, _, _ = files
    print("scheduler: named adapter over the engine", flush=True)
    eng = E.Engine(model, E.EngineConfig(n_ctx=512, n_seq_max=4, n_batch=64, n_ubatch=64))
    sched = S.Scheduler.over_engine(eng, S.SchedulerOptions(mode=S.CONTINUOUS, n_batch=64, event_capacity=64))
    sched.initialize()
    sched.load_adapter("tuned", str(a1))
    prompt = [int(t) for t in np.random.default_rng(8).integers(0, SHAPE.n_vocab, 19)]

    def run(adapter):
        stream = sched.submit(S.Request(prompt, [E.SamplingParamsV2.greedy(max_new_tokens=4)], adapter=adapter))
        sched.run_until_idle()
        events = list(stream.drain())
        assert not [e for e in events if e.type == "Error"], events
        return [e.token for e in events if e.type == "Token"]

    tuned, plain = run("tuned"), run(None)
    assert eng.active_adapter() == ""
    sched.close()
    ref = E.Engine(model, E.EngineConfig(n_ctx=512, n_seq_max=4, n_batch=64, n_ubatch=64))
    rid = ref.adapter_load(a1, 1.0)
    out = E.StepOutput()

    def greedy_decode(adapter):
        ref.seq_rm(0)
        ref.step([E.StepRow(1, 0, prompt, 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(adapter))], out)
        toks = [out.row(0).token]
        for i in range(3):
            ref.step([E.StepRow(1, 0, [toks[-1]], len(prompt) + i, sample=True, sampling=greedy(), adapter=E.RowAdapter(adapter))], out)
            toks.append(out.row(0).token)
        return toks

    assert tuned == greedy_decode(rid) and plain == greedy_decode(E.RETRO_STEP_ADAPTER_BASE)
    assert tuned != plain
    eng.close()
    ref.close()


def test_adapter_errors_and_unload(files):
    model, a1, a2, ffn = files
    print("per-row LoRA: argument errors", flush=True)
    eng = E.Engine(model, E.EngineConfig(n_ctx=512, n_seq_max=2, n_batch=64, n_ubatch=64))
    out = E.StepOutput()
    toks = [1, 2, 3]
    with pytest.raises(E.InvalidArgument, match="is not a loaded per-row adapter"):
        eng.step([E.StepRow(0, 0, toks, 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(1))], out)
    with pytest.raises(E.RuntimeFailure, match="only the attention and dense feed-forward matrices"):
        eng.adapter_load(ffn)
    with pytest.raises(E.RuntimeFailure, match="failed to load LoRA adapter"):
        eng.adapter_load(model)
    aid = eng.adapter_load(a1)
    assert aid == 1, "a refused load does not consume an id"
    with pytest.raises(E.InvalidArgument, match="select different adapters"):
        eng.step([E.StepRow(0, 0, toks, 0, adapter=E.RowAdapter(aid)),
                  E.StepRow(1, 0, [4], 3, sample=True, sampling=greedy())], out)
    eng.step([E.StepRow(0, 0, toks, 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(aid))], out)
    eng.adapter_unload(aid)
    with pytest.raises(E.RuntimeFailure, match="no per-row adapter is loaded under id 1"):
        eng.adapter_unload(aid)
    with pytest.raises(E.InvalidArgument, match="is not a loaded per-row adapter"):
        eng.step([E.StepRow(0, 1, toks, 0, sample=True, sampling=greedy(), adapter=E.RowAdapter(aid))], out)
    assert eng.adapter_load(a2) == 2, "ids are never reused"
    assert eng.adapter_rows_info().n_adapters == 1
    eng.close()
