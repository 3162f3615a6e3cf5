"""The quantised KV caches (kv_dtype Q8_0 and Q4_0 of the engine configuration; reference
crates/retrograd-ffi/runtime/src/retro_engine.cpp:84-91 maps them to ggml's type_k / type_v) on the GPU against the
CPU oracle with the same cache type: K and V rows are stored as blocks of 32 along a head's row
(quantize_row_q8_0_ref / quantize_row_q4_0_ref), attention reads scale times code. The reference holds no vectors
for a quantised cache (its arithmetic is in the absent llama.cpp fork), so the oracle's treatment is pinned by the
row quantiser the reference's fixture digests pin (Q8_0), by the block decoder's known answer (Q4_0) and by the
float64 transformer (tests/test_oracle_model.py); against the reference itself it is parity unpinned."""
import numpy as np
import pytest

import oracle
from engine_helpers import assert_logits_close, greedy, logit_errors, run_both
from retrograd_amd import engine as E
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

SHAPES = {
    # head_dim 64, four query heads per kv head (the shared-instruction form of the attention kernel)
    "llama-hd64": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                               n_ff=1024, n_vocab=1024, name="llama-q4k-small"),
    # head_dim 128 as in the headline shape
    "llama-hd128": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=1024, n_head=8, n_head_kv=2, head_dim=128,
                                n_ff=2048, n_vocab=2048, name="llama-q4k-hd128"),
    # head_dim 32, seven query heads per kv head, biases, split-half rotation
    "qwen2-hd32": synth.scaled(synth.QWEN25_7B_Q8, n_layer=2, n_embd=512, n_head=14, n_head_kv=2, head_dim=32,
                               n_ff=1024, n_vocab=1024, name="qwen2-small"),
    # sixteen query heads on one kv head: the separate-operand form of the attention kernel
    "llama-g16": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=1024, n_head=16, n_head_kv=1, head_dim=64,
                              n_ff=1024, n_vocab=1024, name="llama-q4k-g16"),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    d = tmp_path_factory.mktemp("kv_q8")
    out = {}
    for i, (k, s) in enumerate(SHAPES.items()):
        out[k] = d / (k + ".gguf")
        synth.write_model(out[k], s, seed=300 + i, device="cpu", std=0.05)
    return out


KINDS = {"q8_0": (E.KV_Q8_0, 8, 17 / 32), "q4_0": (E.KV_Q4_0, 4, 9 / 32)}


def _pair(path, n_seq=6, n_ctx=2048, n_batch=256, activations="exact", kind="q8_0"):
    eng = E.Engine(path, E.EngineConfig(n_ctx=n_ctx, n_seq_max=n_seq, n_batch=n_batch, n_ubatch=n_batch, kv_dtype=KINDS[kind][0]))
    m = oracle.Model(path)
    return eng, oracle.Context(m, n_seq, activations=activations, kv=kind), m


@pytest.mark.parametrize("kind", list(KINDS))
@pytest.mark.parametrize("key", list(SHAPES))
def test_prefill_and_decode_over_a_q8_0_cache_match_the_oracle(models, key, kind):
    print(kind, "cache:", key, flush=True)
    bits = KINDS[kind][1]
    eng, ctx, m = _pair(models[key], kind=kind)
    rng = np.random.default_rng(5)
    lens = [5, 33, 70, 17]                       # partial pages, a page boundary, three pages
    prompts = [rng.integers(0, m.n_vocab, n) for n in lens]
    o, got, want = run_both(eng, ctx, [(i, i, p, 0, True) for i, p in enumerate(prompts)])
    assert_logits_close(got, want)
    # what the cache holds: the oracle's blocks, up to codes that sit on a rounding boundary of slightly different f32 rows
    shape = SHAPES[key]
    for layer, slot, pos, want_v in ((0, 1, 0, False), (0, 1, 32, True), (1, 2, 69, False), (1, 3, 16, True), (0, 0, 4, True)):
        mine = eng.debug_kv_q8(layer, slot, pos, want_v, shape.n_head_kv, shape.head_dim, bits)
        theirs = ctx.read_kv_values(layer, slot, pos, want_v)
        step = np.repeat(np.abs(theirs).reshape(-1, 32).max(axis=1) / (127 if bits == 8 else 8), 32)
        assert (np.abs(mine - theirs) <= 1.01 * step + 1e-7).all(), (layer, slot, pos, want_v)
        assert (mine == theirs).mean() > 0.9
    pos = list(lens)
    for _ in range(4):                           # decode steps, teacher-forced with the oracle's tokens
        feed = [int(want[i].argmax()) for i in range(4)]
        o, got, want = run_both(eng, ctx, [(i, i, [feed[i]], pos[i], True) for i in range(4)])
        assert_logits_close(got, want)
        pos = [p + 1 for p in pos]
    # the cache type matters: an f16 cache gives visibly different logits for the same tokens
    f16 = oracle.Context(m, 4).step_rows([(i, 0, prompts[i], True) for i in range(4)])
    q8 = oracle.Context(m, 4, kv=kind).step_rows([(i, 0, prompts[i], True) for i in range(4)])
    assert np.abs(f16 - q8).max() > 1e-4
    eng.close()


@pytest.mark.parametrize("kind", list(KINDS))
def test_long_rows_split_over_many_pages_and_items(models, kind):
    # 700 tokens: 22 pages, several work items per kv head, chunked prefill against one chunk in the oracle
    eng, ctx, m = _pair(models["llama-hd128"], n_seq=2, n_ctx=2048, n_batch=256, kind=kind)
    rng = np.random.default_rng(6)
    toks = rng.integers(0, m.n_vocab, 700)
    out = E.StepOutput()
    for at in range(0, 700, 256):
        eng.step([E.StepRow(0, 0, toks[at:at + 256], at, sample=at + 256 >= 700, sampling=greedy())], out)
    got = eng.debug_logits()
    want = ctx.step_rows([(0, 0, toks, True)])
    # A row that differs in its last bits between the two sides can take the neighbouring code where it sits on a
    # rounding boundary. A four-bit step is an eighth of the block's peak, so over 700 positions the few such codes
    # move the logits more than the f16 tolerances allow for: wider ones for Q4_0, still two orders below what the
    # cache type itself does to the logits.
    tol = dict(max_abs=5e-2, mean_rel=5e-3) if kind == "q4_0" else {}
    assert_logits_close(got, want, **tol)
    if kind == "q4_0":
        f16 = oracle.Context(m, 1).step_rows([(0, 0, toks, True)])
        assert logit_errors(f16, want)[1] > 20 * logit_errors(got, want)[1]
    o, got, want = run_both(eng, ctx, [(0, 0, [int(want[0].argmax())], 700, True)])
    assert_logits_close(got, want, **tol)
    eng.close()


@pytest.mark.parametrize("kind", list(KINDS))
def test_copies_and_snapshots_of_a_q8_0_cache_decode_like_their_source(models, kind):
    shape = SHAPES["llama-hd64"]
    bits = KINDS[kind][1]
    eng, ctx, m = _pair(models["llama-hd64"], n_seq=6, n_ctx=1024, n_batch=128, kind=kind)
    rng = np.random.default_rng(7)
    toks = rng.integers(0, m.n_vocab, 50)
    out = E.StepOutput()
    eng.step([E.StepRow.prefill(0, 0, toks[:45], 0)], out)
    ctx.step_rows([(0, 0, toks[:45], False)])
    eng.seq_cp(0, 1)              # whole copy: shares both pages
    eng.seq_cp(0, 2, 0, 40)       # partial copy [0, 40): page 1 is copied cell by cell
    ctx.seq_cp(0, 1)
    ctx.seq_cp(0, 2, 0, 40)
    snap = eng.seq_save(0)
    per_row = shape.n_head_kv * (shape.head_dim * bits // 16 + shape.head_dim // 32) * 2
    assert len(snap) == 24 + shape.n_layer * 2 * 45 * per_row
    eng.seq_load(3, snap)
    assert eng.seq_pos(3) == (0, 44)
    eng.step([E.StepRow.prefill(2, 2, toks[40:45], 40)], out)
    ctx.step_rows([(2, 40, toks[40:45], False)])
    rows = [(s, s, toks[45:], 45, True) for s in range(3)]      # the copy writes into a shared page: copy on write
    o, got, want = run_both(eng, ctx, rows)
    assert_logits_close(got, want)
    assert np.array_equal(got[0], got[1])
    eng.step([E.StepRow(3, 3, toks[45:], 45, sample=True, sampling=greedy())], out)
    assert np.array_equal(eng.debug_logits()[0], got[0]), "a restored snapshot decodes like its source, bit for bit"
    # a snapshot of the other cache type is refused
    f16 = E.Engine(models["llama-hd64"], E.EngineConfig(n_ctx=1024, n_seq_max=6, n_batch=128, n_ubatch=128))
    with pytest.raises(E.RuntimeFailure, match="snapshot was refused"):
        f16.seq_load(0, snap)
    assert abs(eng.memory().kv_bytes / f16.memory().kv_bytes - KINDS[kind][2]) < 1e-3     # 34 (18) bytes per 32 values against 64
    other = "q4_0" if kind == "q8_0" else "q8_0"
    third = E.Engine(models["llama-hd64"], E.EngineConfig(n_ctx=1024, n_seq_max=6, n_batch=128, n_ubatch=128, kv_dtype=KINDS[other][0]))
    with pytest.raises(E.RuntimeFailure, match="snapshot was refused"):
        third.seq_load(0, snap)
    third.close()
    f16.close()
    eng.close()


@pytest.mark.parametrize("kind", list(KINDS))
def test_the_ggml_arithmetic_converts_the_query_row_too(models, monkeypatch, kind):
    """ggml's CPU attention multiplies a Q8_0 K row with the query row converted to Q8_0 (the type's companion
    format); RETRO_ACTIVATIONS=ggml does the same over a Q8_0 cache. Criterion as in tests/test_gpu_step.py: the
    product follows the oracle's ggml logits more closely than the exact arithmetic does."""
    monkeypatch.setenv("RETRO_ACTIVATIONS", "ggml")
    eng, ctx, m = _pair(models["llama-hd64"], activations="ggml", kind=kind)
    rng = np.random.default_rng(8)
    prompts = [rng.integers(0, m.n_vocab, n) for n in (40, 21, 66)]
    o, got, want = run_both(eng, ctx, [(i, i, p, 0, True) for i, p in enumerate(prompts)])
    exact = oracle.Context(m, 3, kv=kind).step_rows([(i, 0, p, True) for i, p in enumerate(prompts)])
    assert logit_errors(got, want)[1] < 0.5 * logit_errors(exact, want)[1]
    eng.close()


def test_the_cache_type_this_library_does_not_hold_is_refused(models):
    with pytest.raises(E.EngineError, match="f32 KV cache is not implemented"):
        E.Engine(models["llama-hd64"], E.EngineConfig(n_ctx=256, n_seq_max=2, n_batch=64, n_ubatch=64, kv_dtype=E.KV_F32))


@pytest.mark.parametrize("kind", list(KINDS))
def test_a_trainers_quantised_generation_context_decodes_like_an_engine_with_the_same_cache(models, kind):
    """generation_kv_dtype = Q8_0 / Q4_0 (reference tests/engine_runtime.rs:218-238 compares a trainer's quantised
    generation context with an engine of the same kv_dtype bit for bit): tokens and log-probabilities of a greedy
    continuation."""
    from retrograd_amd import trainer as T
    tr = T.Trainer(models["llama-hd64"], T.TrainConfig(n_ctx=128, n_batch=128, generation_concurrency=2,
                                                       generation_kv_dtype={"q8_0": 1, "q4_0": 2}[kind]))
    eng = E.Engine(models["llama-hd64"], E.EngineConfig(n_ctx=256, n_seq_max=2, n_batch=128, n_ubatch=128, kv_dtype=KINDS[kind][0]))
    f16 = E.Engine(models["llama-hd64"], E.EngineConfig(n_ctx=256, n_seq_max=2, n_batch=128, n_ubatch=128))
    rng = np.random.default_rng(9)
    prompts = [rng.integers(0, 1024, n) for n in (40, 23)]

    def run(h):
        out = E.StepOutput()
        h.step([E.StepRow(i, i, prompts[i], 0, sample=True, sampling=greedy()) for i in range(2)], out)
        toks = [[r.token] for r in out.rows()]
        lps = [[np.float32(r.logprob).view(np.uint32)] for r in out.rows()]
        for step in range(5):
            h.step([E.StepRow(i, i, [toks[i][-1]], len(prompts[i]) + step, sample=True, sampling=greedy()) for i in range(2)], out)
            for i, r in enumerate(out.rows()):
                toks[i].append(r.token)
                lps[i].append(np.float32(r.logprob).view(np.uint32))
        return toks, lps
    a, b, c = run(tr), run(eng), run(f16)
    assert a == b
    assert c[1] != a[1], "an f16 cache gives other log-probabilities"
    assert abs(tr.memory().kv_bytes / f16.memory().kv_bytes - KINDS[kind][2]) < 1e-3
    with pytest.raises(E.EngineError, match="generation_kv_dtype must be"):
        T.Trainer(models["llama-hd64"], T.TrainConfig(n_ctx=128, n_batch=128, generation_concurrency=2, generation_kv_dtype=3))
    tr.close(); eng.close(); f16.close()
