"""The decode step on the GPU against the CPU oracle, through the C ABI.

Tolerances of the benchmark definition: logits within 2e-2 max-abs and 1e-3 mean-abs
relative error; packing, cells, slot ranges and greedy token ids bit-exact
(token ids are compared where the oracle's own top-1/top-2 margin exceeds the
logit tolerance - a margin below the tolerance is a tie no two float
implementations are required to break alike)."""
import numpy as np
import pytest

import oracle
from engine_helpers import assert_logits_close, greedy, logit_errors, run_both
from retrograd_amd import engine as E
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

SMALL = {
    "tiny-llama-q8": synth.TINY_LLAMA,
    "llama-q4k": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                              n_ff=1024, n_vocab=1024, name="llama-q4k-small"),
    "llama-q4k-hd128": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=1024, n_head=8, n_head_kv=2,
                                    head_dim=128, n_ff=2048, n_vocab=2048, name="llama-q4k-hd128"),
    "qwen2-q8": synth.scaled(synth.QWEN25_7B_Q8, n_layer=2, n_embd=512, n_head=14, n_head_kv=2, head_dim=32,
                             n_ff=1024, n_vocab=1024, name="qwen2-small"),
    # the type mix of a Q4_K_M file: output.weight, ffn_down and attn_v in Q6_K, the rest in Q4_K
    "llama-q4k-m": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                                n_ff=1024, n_vocab=1024, output_type=14, down_type=14, v_type=14, name="llama-q4k-m-small"),
    # every matrix in Q6_K: the fused qkv matrix and the interleaved gate/up matrix with its SwiGLU epilogue on Q6_K tiles
    "llama-q6k": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                              n_ff=1024, n_vocab=1024, matrix_type=14, name="llama-q6k-small"),
    # q and k joined in Q4_K, v on its own in Q6_K, with biases: two launches that leave their K-slices side by side
    "qwen2-q4k-m": synth.scaled(synth.QWEN25_7B_Q8, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                                n_ff=1024, n_vocab=1024, matrix_type=12, v_type=14, down_type=14, name="qwen2-q4k-m-small"),
    # wide enough (four super-blocks per row) for decode steps to split K: the q+k and v launches share their K-slices
    "llama-q4k-m-1024": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=1024, n_head=8, n_head_kv=2, head_dim=128,
                                     n_ff=2048, n_vocab=2048, output_type=14, down_type=14, v_type=14,
                                     name="llama-q4k-m-1024"),
    # the type mix of a Q5_K_M file: Q5_K matrices, Q6_K for output.weight, ffn_down and attn_v
    "llama-q5k-m": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=1024, n_head=8, n_head_kv=2, head_dim=128,
                                n_ff=2048, n_vocab=2048, matrix_type=13, output_type=14, down_type=14, v_type=14,
                                name="llama-q5k-m-1024"),
    # per-frequency rotation divisors (rope_freqs.weight, Llama 3.1's long-context rule) and linear scaling
    "llama-rope-freqs": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                                     n_ff=1024, n_vocab=1024, rope_freqs=True, rope_scaling_linear=2.0,
                                     name="llama-rope-freqs-small"),
    # yarn scaling: interpolated, mixed and kept frequencies, cosines and sines times 1 + 0.1 ln(factor)
    "llama-yarn": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                               n_ff=1024, n_vocab=1024, rope_base=10000.0, rope_scaling_yarn=4.0, rope_original_context=64,
                               name="llama-yarn-small"),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    d = tmp_path_factory.mktemp("gpu_models")
    out = {}
    for i, (k, s) in enumerate(SMALL.items()):
        p = d / (k + ".gguf")
        synth.write_model(p, s, seed=100 + i, device="cpu", std=0.05 if k != "tiny-llama-q8" else 0.02)
        out[k] = p
    return out


def _pair(path, n_seq=8, n_ctx=2048, n_batch=256):
    eng = E.Engine(path, E.EngineConfig(n_ctx=n_ctx, n_seq_max=n_seq, n_batch=n_batch, n_ubatch=n_batch))
    m = oracle.Model(path)
    return eng, oracle.Context(m, n_seq), m


@pytest.mark.parametrize("key", list(SMALL))
def test_prefill_and_decode_logits_match_oracle(models, key):
    print("model", key, flush=True)
    eng, ctx, m = _pair(models[key])
    rng = np.random.default_rng(1)
    lens = [5, 33, 64, 17]
    prompts = [rng.integers(0, m.n_vocab, n) for n in lens]
    rows = [(i, i, p, 0, True) for i, p in enumerate(prompts)]
    out, got, want = run_both(eng, ctx, rows)
    assert_logits_close(got, want)
    toks = [r.token for r in out.rows()]
    for i, t in enumerate(toks):
        srt = np.sort(want[i])[::-1]
        if srt[0] - srt[1] > 4e-2:
            assert t == int(want[i].argmax())
    # three decode steps, teacher-forced with the oracle's tokens
    pos = list(lens)
    for _ in range(3):
        feed = [int(want[i].argmax()) for i in range(4)]
        rows = [(i, i, [feed[i]], pos[i], True) for i in range(4)]
        out, got, want = run_both(eng, ctx, rows)
        assert_logits_close(got, want)
        pos = [p + 1 for p in pos]
    for i in range(4):
        assert eng.seq_pos(i) == ctx.seq_pos(i) == (0, pos[i] - 1)
    eng.close()


@pytest.mark.parametrize("key", list(SMALL))
def test_ggml_arithmetic_follows_the_oracle_as_closely_as_its_rounding_allows(models, key, monkeypatch):
    """RETRO_ACTIVATIONS=ggml: activations converted as ggml's CPU matmul does. Per matmul the
    product and the oracle agree to float rounding (test_gpu_kernels.py). Over a whole forward
    a value near a rounding boundary takes different codes on the two sides and every later
    conversion amplifies that, exactly as between the oracle and its float64 restatement
    (tests/test_oracle_model.py). The yardstick for "as close as rounding allows" is that
    restatement against itself with its matrices perturbed by 2e-5 relative, the size of an
    f32 accumulation error: the product must drift from the oracle no further than that,
    must be clearly closer to the ggml arithmetic than the plain product is, and must pick
    the same token wherever the margin exceeds the drift."""
    from ref_transformer import NumpyModel
    print("model", key, flush=True)
    monkeypatch.setenv("RETRO_ACTIVATIONS", "ggml")
    eng = E.Engine(models[key], E.EngineConfig(n_ctx=2048, n_seq_max=8, n_batch=256, n_ubatch=256))
    m = oracle.Model(models[key])
    ggml_ctx, exact_ctx = oracle.Context(m, 8, activations="ggml"), oracle.Context(m, 8, activations="exact")
    rng = np.random.default_rng(1)
    lens = [5, 33, 64, 17]
    prompts = [rng.integers(0, m.n_vocab, n) for n in lens]
    rows = [(i, i, p, 0, True) for i, p in enumerate(prompts)]
    out, got, want = run_both(eng, ggml_ctx, rows)
    exact = exact_ctx.step_rows([(r[1], r[3], r[2], r[4]) for r in rows])
    drift_max, drift = logit_errors(got, want)
    _, conversion = logit_errors(exact, want)
    clean, noisy = NumpyModel(models[key], activations="ggml"), NumpyModel(models[key], activations="ggml")
    noise = np.random.default_rng(7)
    for name in noisy.r.tensors:
        w = noisy.t(name)
        if w is not None and w.ndim >= 2:
            noisy.w[name] = w * (1 + 2e-5 * noise.standard_normal(w.shape))
    a = np.stack([clean.forward(p)[-1] for p in prompts])
    b = np.stack([noisy.forward(p)[-1] for p in prompts])
    _, yardstick = logit_errors(b, a)
    print("drift %.2e (max %.2e), yardstick %.2e, conversion %.2e" % (drift, drift_max, yardstick, conversion), flush=True)
    assert drift <= yardstick and drift < 0.6 * conversion, (drift, yardstick, conversion)
    for i, r in enumerate(out.rows()):
        srt = np.sort(want[i])[::-1]
        if srt[0] - srt[1] > 4 * drift_max:
            assert r.token == int(want[i].argmax())
    eng.close()


@pytest.mark.parametrize("key", ["llama-q4k", "llama-q4k-hd128", "llama-q4k-m-1024", "qwen2-q8", "tiny-llama-q8", "llama-q6k", "qwen2-q4k-m", "llama-q5k-m"])
def test_small_steps_under_the_ggml_arithmetic_take_the_integer_kernel(models, key, monkeypatch):
    """Steps of one or two tokens under RETRO_ACTIVATIONS=ggml multiply their Q4_K matrices by integer products of
    the stored codes with the rows' Q8_K codes (Q6_K matrices of the same model stay on the tile kernels), and where
    every consumer of a row is that kernel it makes the codes itself from the residual or gate/up rows, and the
    output projection of a single-token step merges the attention splits itself (the default; RETRO_GEMV_FUSE=0 keeps
    the producers' own launches). Against the oracle's ggml arithmetic such a step must
    drift no further than the same step through the tile kernels (RETRO_GEMV_MAX_T=0) does - all differ from it by
    float rounding that later conversions amplify - and the engines must stay as close to each other as either is
    to the oracle."""
    print("model", key, flush=True)
    monkeypatch.setenv("RETRO_ACTIVATIONS", "ggml")
    cfg = E.EngineConfig(n_ctx=2048, n_seq_max=8, n_batch=256, n_ubatch=256)
    m = oracle.Model(models[key])
    rng = np.random.default_rng(5)
    lens = [5, 33, 200, 17]         # slot 2: seven pages, two attention splits per kv head in a single-token step
    prompts = [rng.integers(0, m.n_vocab, n) for n in lens]
    plans = [[0, 1, 2, 3], [1, 3], [2], [0, 1, 3], [0], [0, 1, 2, 3], [2]]      # the slots of each decode step
    feeds = [[int(t) for t in rng.integers(0, m.n_vocab, len(p))] for p in plans]
    runs = {}
    for name, limit, fuse in (("integer", None, None), ("unfused", None, "0"), ("tiles", "0", None)):
        for var, value in (("RETRO_GEMV_MAX_T", limit), ("RETRO_GEMV_FUSE", fuse)):
            if value is None:
                monkeypatch.delenv(var, raising=False)
            else:
                monkeypatch.setenv(var, value)
        eng = E.Engine(models[key], cfg)
        ctx = oracle.Context(m, 8, activations="ggml")
        run_both(eng, ctx, [(i, i, p, 0, True) for i, p in enumerate(prompts)])
        pos = list(lens)
        steps = []
        for plan, feed in zip(plans, feeds):
            rows = [(s, s, [feed[j]], pos[s], True) for j, s in enumerate(plan)]
            _, got, want = run_both(eng, ctx, rows)
            steps.append((got.copy(), want.copy()))
            for s in plan:
                pos[s] += 1
        runs[name] = steps
        eng.close()
    for i, plan in enumerate(plans):
        (gi, want), (gt, want_t) = runs["integer"][i], runs["tiles"][i]
        assert np.array_equal(want, want_t)
        _, drift_i = logit_errors(gi, want)
        _, drift_t = logit_errors(gt, want)
        _, apart = logit_errors(gi, gt)
        gu, _ = runs["unfused"][i]
        _, drift_u = logit_errors(gu, want)
        _, apart_u = logit_errors(gi, gu)
        print("step of %d rows: integer %.2e, its producers unfused %.2e, tiles %.2e from the oracle; %.2e and %.2e apart"
              % (len(plan), drift_i, drift_u, drift_t, apart_u, apart), flush=True)
        assert drift_i <= 2 * drift_t + 1e-4 and apart <= 2 * max(drift_i, drift_t) + 1e-4, (i, drift_i, drift_t, apart)
        assert drift_u <= 2 * drift_t + 1e-4 and apart_u <= 2 * max(drift_i, drift_u) + 1e-4, (i, drift_u, apart_u)
        assert drift_i <= 5e-2


def test_packing_is_bit_exact_with_the_oracle(models):
    eng, ctx, m = _pair(models["llama-q4k"], n_seq=8, n_ctx=1024, n_batch=128)
    rng = np.random.default_rng(2)
    plan = [(3, 40, True), (0, 1, True), (7, 33, False), (5, 9, True)]   # slot, n, sample
    rows = [(i, s, rng.integers(0, m.n_vocab, n), 0, smp) for i, (s, n, smp) in enumerate(plan)]
    out = E.StepOutput()
    eng.step([E.StepRow(r[0], r[1], r[2], r[3], sample=r[4], sampling=greedy()) for r in rows], out)
    pk = eng.debug_pack(128, 128)
    want = oracle.pack_rows([(r[1], r[3], r[2], r[4]) for r in rows])
    assert np.array_equal(pk["token"], want["token"])
    assert np.array_equal(pk["pos"], want["pos"])
    assert np.array_equal(pk["seq"], want["seq"])
    assert np.array_equal(pk["out_index"] >= 0, want["output"].astype(bool))
    assert np.array_equal(pk["last_index"][:4], want["last_index"])
    assert list(pk["counts"][:2]) == [83, 3]
    # block table: lowest free page first, in row order; cells follow the table
    page = 32
    tables = np.stack([eng.debug_pages(s) for s in range(8)])
    assert list(tables[3][:2]) == [0, 1] and tables[0][0] == 2 and list(tables[7][:2]) == [3, 4] and tables[5][0] == 5
    cells = oracle.pack_cells(want["pos"], want["seq"], tables, page)
    assert np.array_equal(pk["cell"].astype(np.int64), cells)
    assert [r.sampled for r in out.rows()] == [True, True, False, True]
    eng.close()


def test_chunked_prefill_matches_one_shot(models):
    eng, ctx, m = _pair(models["llama-q4k-hd128"], n_batch=128)
    rng = np.random.default_rng(3)
    toks = rng.integers(0, m.n_vocab, 100)
    out = E.StepOutput()
    eng.step([E.StepRow(0, 0, toks, 0, sample=True, sampling=greedy())], out)
    one = eng.debug_logits().copy()
    eng.step([E.StepRow.prefill(1, 1, toks[:37], 0)], out)
    eng.step([E.StepRow.prefill(1, 1, toks[37:70], 37)], out)
    eng.step([E.StepRow(1, 1, toks[70:], 70, sample=True, sampling=greedy())], out)
    chunked = eng.debug_logits()
    want = ctx.step_rows([(0, 0, toks, True)])
    assert_logits_close(one, want)
    assert_logits_close(chunked, want)
    # K/V written by either schedule are the same f16 values as the oracle's
    for pos in (0, 36, 37, 99):
        for want_v in (False, True):
            a = eng.debug_kv(1, 0, pos, want_v, m.n_head_kv * m.head_dim).astype(np.float32)
            b = eng.debug_kv(1, 1, pos, want_v, m.n_head_kv * m.head_dim).astype(np.float32)
            c = ctx.read_kv(1, 0, pos, want_v).astype(np.float32)
            assert np.abs(a - c).max() <= 2e-2 * np.abs(c).max() + 1e-3
            assert np.abs(b - c).max() <= 2e-2 * np.abs(c).max() + 1e-3
    eng.close()


def test_seq_cp_seq_rm_and_snapshots(models):
    eng, ctx, m = _pair(models["llama-q4k"], n_seq=6, n_ctx=1024, n_batch=128)
    rng = np.random.default_rng(4)
    toks = rng.integers(0, m.n_vocab, 50)
    out = E.StepOutput()
    eng.step([E.StepRow.prefill(0, 0, toks[:45], 0)], out)
    ctx.step_rows([(0, 0, toks[:45], False)])
    eng.seq_cp(0, 1)              # whole copy: shares both pages
    eng.seq_cp(0, 2, 0, 40)       # partial copy [0, 40)
    ctx.seq_cp(0, 1)
    ctx.seq_cp(0, 2, 0, 40)
    assert eng.seq_pos(1) == (0, 44) and eng.seq_pos(2) == (0, 39)
    assert eng.memory().cells_used == 45 + 45 + 40     # counted once per slot that references them
    snap = eng.seq_save(0)
    assert len(snap) == eng.seq_save_len(0)
    eng.seq_load(3, snap)
    assert eng.seq_pos(3) == (0, 44)
    # continue all four: slot 2 first re-decodes positions 40..44
    eng.step([E.StepRow.prefill(2, 2, toks[40:45], 40)], out)
    ctx.step_rows([(2, 40, toks[40:45], False)])
    rows = [(s, s, toks[45:], 45, True) for s in range(3)]
    o, got, want = run_both(eng, ctx, rows)
    assert_logits_close(got, want)
    # copy == source bit for bit (same arithmetic on the same cells / same bytes)
    assert np.array_equal(got[0], got[1])
    eng.step([E.StepRow(3, 3, toks[45:], 45, sample=True, sampling=greedy())], out)
    restored = eng.debug_logits()
    assert_logits_close(restored, want[:1])
    # removal
    eng.seq_rm(1, 30, -1)
    assert eng.seq_pos(1) == (0, 29)
    eng.seq_rm(1)
    assert eng.seq_pos(1) == (-1, -1)
    with pytest.raises(E.RuntimeFailure):
        eng.seq_rm(0, 10, 20)      # a hole in the middle cannot be removed
    with pytest.raises(E.BufferTooSmall):
        eng.seq_save_into(0, 0, bytearray(16))
    eng.close()


def test_forks_inside_a_page_fit_the_pool_up_to_n_ctx_distinct_cells(models):
    # Eight slots share a 48-cell prefix that ends in the middle of a page and each decodes 58 cells of its
    # own: 48 + 8 x 58 = 512 = n_ctx distinct cells. Every fork pays a private copy of the half-filled page
    # and ends in a partial page, 25 pages in all where 512 cells would be 16.
    eng, ctx, m = _pair(models["tiny-llama-q8"], n_seq=8, n_ctx=512, n_batch=64)
    rng = np.random.default_rng(21)
    prefix = rng.integers(0, m.n_vocab, 48)
    out = E.StepOutput()
    eng.step([E.StepRow.prefill(0, 0, prefix, 0)], out)
    ctx.step_rows([(0, 0, prefix, False)])
    for s in range(1, 8):
        eng.seq_cp(0, s)
        ctx.seq_cp(0, s)
    tails = rng.integers(0, m.n_vocab, (8, 58))
    for at in range(0, 58, 8):
        rows = [(s, s, tails[s, at:at + 8], 48 + at, True) for s in range(8)]
        o, got, want = run_both(eng, ctx, rows)
        assert_logits_close(got, want)
    assert all(eng.seq_pos(s) == (0, 105) for s in range(8))
    eng.close()


def test_slot_reuse_after_removal(models):
    # A slot is emptied and refilled between two steps: its block-table entries
    # change twice (to "none", then to new pages) before the device sees them.
    eng, ctx, m = _pair(models["llama-q4k"], n_seq=4, n_ctx=512, n_batch=128)
    rng = np.random.default_rng(9)
    for cycle in range(4):
        n = int(rng.integers(20, 90))
        toks = rng.integers(0, m.n_vocab, n)
        slot = cycle % 2
        eng.seq_rm(slot)
        ctx.seq_rm(slot)
        o, got, want = run_both(eng, ctx, [(cycle, slot, toks, 0, True)])
        assert_logits_close(got, want)
        o, got, want = run_both(eng, ctx, [(cycle, slot, [int(want[0].argmax())], n, True)])
        assert_logits_close(got, want)
        eng.request_free(cycle)
    eng.close()


def test_step_argument_errors_are_reported_before_decoding(models):
    eng, ctx, m = _pair(models["tiny-llama-q8"], n_seq=4, n_ctx=256, n_batch=32)
    out = E.StepOutput()
    ok = lambda **kw: E.StepRow(kw.get("request", 0), kw.get("slot", 0), kw.get("tokens", [1, 2]), kw.get("pos0", 0),
                                sample=kw.get("sample", False), sampling=kw.get("sampling", greedy()),
                                n_top_logprobs=kw.get("n_top", 0), adapter=kw.get("adapter", E.RowAdapter()))
    cases = [
        ([ok(slot=4)], "slot is outside"),
        ([ok(tokens=[m.n_vocab])], "outside the vocabulary"),
        ([ok(pos0=255)], "positions exceed"),
        ([ok(tokens=list(range(33)))], "exceed the context's physical batch"),
        ([ok(request=0), ok(request=1, slot=0, pos0=1)], "overlap"),
        ([ok(request=-1, sample=True)], "request id"),
        ([ok(sample=True, sampling=E.SamplingParamsV2(temperature=0.0))], "temperature"),
        ([ok(sample=True, sampling=E.SamplingParamsV2(top_p=0.0))], "top_p"),
        ([ok(sample=True, sampling=E.SamplingParamsV2(min_p=1.5))], "min_p"),
        ([ok(adapter=E.RowAdapter.loaded(3))], "not a loaded per-row adapter"),
    ]
    for rows, needle in cases:
        with pytest.raises(E.InvalidArgument) as err:
            eng.step(rows, out)
        assert needle in str(err.value), (needle, str(err.value))
        assert eng.seq_pos(0) == (-1, -1)
    # a request id twice is caught on the caller side too (step.rs:412-505)
    with pytest.raises(E.InvalidArgument):
        eng.step([ok(request=5), ok(request=5, slot=1)], out)
    # capacity is a runtime condition, not an invalid argument
    eng.step([ok(tokens=list(range(1, 30)))], out)
    with pytest.raises(E.RuntimeFailure):
        eng.step([ok(pos0=10)], out)         # already resident
    eng.close()


def test_introspection_and_memory(models):
    path = models["tiny-llama-q8"]
    eng = E.Engine(path, E.EngineConfig(n_ctx=512, n_seq_max=4, n_batch=64, n_ubatch=64))
    assert eng.vocab_size() == 512 and eng.context_size() == 512 and eng.kv_unified()
    assert not eng.is_hybrid() and eng.weights_version() == 0
    mem = eng.memory()
    assert (mem.n_slots, mem.cells_total, mem.cells_used, mem.recurrent_bytes) == (4, 512, 0, 0)
    assert mem.kv_bytes > 0
    # FNV-1a over the path bytes, then the u64 payload size (retro_runtime.hpp:856-868)
    from gguf_reader import Reader
    r = Reader(path)
    from retrograd_amd import gguf_writer as gw
    size = sum(gw.tensor_nbytes(ne, t) for ne, t, _ in r.tensors.values())
    h = 14695981039346656037
    for b in str(path).encode() + size.to_bytes(8, "little"):
        h = ((h ^ b) * 1099511628211) & (2 ** 64 - 1)
    assert eng.model_fingerprint() == h
    assert eng.detokenize_bytes([5, 6]) == b"<t5><t6>"
    assert not eng.is_eog_token(2) and eng.eos_token() == -1
    part = E.Engine(path, E.EngineConfig(n_ctx=512, n_seq_max=4, n_batch=64, n_ubatch=64, kv_unified=False))
    assert part.context_size() == 128 and not part.kv_unified()
    part.close()
    eng.close()


def test_rope_frequency_factors_and_linear_scaling_change_the_rotation_as_in_the_oracle(tmp_path):
    """rope_freqs.weight (per-frequency divisors of the angle: ggml's rope, theta / ff) and rope.scaling.type =
    linear. The same weights with and without them: each engine follows its own oracle, and the two differ by far
    more than the tolerance, so an engine that ignored the factors would not pass. A scaling rule that is not
    implemented is refused at load."""
    base = synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64, n_ff=1024,
                        n_vocab=1024, name="rope-plain")
    with_f = synth.scaled(base, rope_freqs=True, rope_scaling_linear=2.0, name="rope-factors")
    paths = {}
    for key, shape in (("plain", base), ("factors", with_f)):
        paths[key] = tmp_path / (key + ".gguf")
        synth.write_model(paths[key], shape, seed=31, device="cpu", std=0.05)
    toks = np.random.default_rng(3).integers(0, 1024, 200)
    logits = {}
    for key, path in paths.items():
        eng, ctx, m = _pair(path, n_seq=2, n_ctx=1024)
        out, got, want = run_both(eng, ctx, [(1, 0, toks, 0, True)])
        assert_logits_close(got, want)
        logits[key] = got
        eng.close()
    mx, mr = logit_errors(logits["factors"], logits["plain"])
    print("the factors move the logits by %.3g (max), %.3g (mean, relative)" % (mx, mr), flush=True)
    assert mx > 0.2 and mr > 1e-2
    raw = bytearray(paths["factors"].read_bytes())
    at = raw.find(b"linear")
    assert at > 0
    raw[at:at + 6] = b"yarnxx"
    bad = tmp_path / "unknown-scaling.gguf"
    bad.write_bytes(bytes(raw))
    with pytest.raises(E.EngineError, match="not implemented"):
        E.Engine(bad, E.EngineConfig(n_ctx=256, n_seq_max=1, n_batch=64, n_ubatch=64))


@pytest.mark.parametrize("key", ["llama", "llama-rope-freqs", "llama-linear", "qwen2", "qwen3moe"])
def test_engine_reproduces_hugging_face_transformers_logits(tmp_path, key):
    """The engine against tests/golden/hf_reference_logits.npz (Hugging Face transformers in float64 over the
    dequantised weights of the same seeded file, K and V rounded to f16): every position's logits, through one
    step of 14 rows that each prefill a prefix of the prompt into a slot of their own."""
    import importlib.util
    from pathlib import Path
    here = Path(__file__).resolve().parent / "golden"
    spec = importlib.util.spec_from_file_location("hf_reference_logits", here / "hf_reference_logits.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    golden = np.load(here / "hf_reference_logits.npz")
    shape, seed, std = mod.CASES[key]
    path = tmp_path / (key + ".gguf")
    synth.write_model(path, shape, seed=seed, device="cpu", std=std)
    assert bytes(golden[key + ".sha256"]).hex() == mod.sha256(path)
    toks = [int(t) for t in golden[key + ".tokens"]]
    want = golden[key + ".logits"]
    print("hf fixture", key, flush=True)
    n = len(toks)
    eng = E.Engine(path, E.EngineConfig(n_ctx=n * 32, n_seq_max=n, n_batch=256, n_ubatch=256))
    out = E.StepOutput()
    eng.step([E.StepRow(i, i, toks[:i + 1], 0, sample=True, sampling=greedy()) for i in range(n)], out)
    got = eng.debug_logits()
    assert_logits_close(got, want)
    mx, mr = logit_errors(got, want)
    assert mr <= 1e-4, (mx, mr)       # far inside the tolerance: only f32 / f16-pair rounding separates the two
    for i, r in enumerate(out.rows()):
        srt = np.sort(want[i])[::-1]
        if srt[0] - srt[1] > 4e-2:
            assert r.token == int(want[i].argmax())
    eng.close()


def test_tokenization_through_the_abi_reproduces_sentencepiece_ids_and_round_trips(tmp_path):
    """retro_engine_tokenize / _text / _fragment over a model file whose vocabulary is the sentencepiece model of
    tests/golden/spm_reference_ids.json: the library's own ids for every text, the two-call size contract, and
    detokenize(tokenize(text)) == text."""
    import ctypes as C
    import json
    from pathlib import Path
    golden = json.loads((Path(__file__).resolve().parent / "golden" / "spm_reference_ids.json").read_text())
    vocab = {"tokens": [v[0] for v in golden["vocab"]], "scores": [v[1] for v in golden["vocab"]],
             "types": [v[2] for v in golden["vocab"]], "bos": golden["bos"], "eos": golden["eos"], "unk": golden["unk"]}
    shape = synth.scaled(synth.TINY_LLAMA, n_vocab=len(vocab["tokens"]), name="tiny-llama-spm")
    path = tmp_path / "spm.gguf"
    synth.write_model(path, shape, seed=5, device="cpu", vocab=vocab)
    eng = E.Engine(path, E.EngineConfig(n_ctx=256, n_seq_max=2, n_batch=64, n_ubatch=64))
    for c in golden["cases"]:
        assert eng.tokenize(c["text"], add_special=False, parse_special=False) == c["ids"], c["text"]
        assert eng.tokenize(c["text"], add_special=True, parse_special=False) == [golden["bos"]] + c["ids"]
        # round trip: the dummy prefix comes back as a leading space
        assert eng.detokenize_bytes(c["ids"]).decode() == " " + c["text"], c["text"]
    ids = eng.tokenize("<s>hello world</s>")                 # tokenize_text's flags: BOS added, special texts parsed
    assert ids[:2] == [golden["bos"], golden["bos"]] and ids[-1] == golden["eos"]
    # the size contract: no buffer -> count; too small -> -2 with the count; text required
    lib, n = eng._lib, C.c_size_t()
    assert lib.retro_engine_tokenize_text(eng._h, b"hello world", None, 0, C.byref(n)) == 0 and n.value == len(golden["cases"][0]["ids"]) + 1
    small = (C.c_int32 * 1)()
    assert lib.retro_engine_tokenize_fragment(eng._h, b"hello world", small, 1, C.byref(n)) == -2 and n.value == len(golden["cases"][0]["ids"])
    assert lib.retro_engine_tokenize_text(eng._h, b"", None, 0, C.byref(n)) == -1 and "text is required" in E.last_error()
    # the generated token ids of a greedy step detokenize and re-tokenize consistently with the vocabulary size
    out = E.StepOutput()
    eng.step([E.StepRow(0, 0, eng.tokenize("attention is all you need"), 0, sample=True, sampling=greedy())], out)
    assert 0 <= out.row(0).token < len(vocab["tokens"])
    eng.close()
    # the trainer handle's twins (retro_trainer_tokenize_text / _fragment / _with) answer from the same vocabulary
    from retrograd_amd import trainer as T
    tr = T.Trainer(path, T.TrainConfig(n_ctx=64, n_batch=64))
    for c in golden["cases"][:4]:
        assert tr.tokenize(c["text"], add_special=False, parse_special=False) == c["ids"], c["text"]
    assert tr._lib.retro_engine_tokenize_text(tr._h, b"hello world", None, 0, C.byref(n)) == 0 and n.value == len(golden["cases"][0]["ids"]) + 1
    assert tr._lib.retro_engine_tokenize_fragment(tr._h, b"hello world", small, 1, C.byref(n)) == -2
    tr.close()


@pytest.mark.gpu
@pytest.mark.parametrize("pre", ["llama-bpe", "qwen2", "gpt-2"])
def test_tokenization_of_a_byte_pair_vocabulary_reproduces_the_tokenizers_librarys_ids(tmp_path, pre):
    """A model file whose vocabulary is the byte-level byte-pair one of tests/golden/bpe_reference_ids.json
    (tokenizer.ggml.model = gpt2, with its merges and the name of its pre-tokeniser pattern): the library's own
    ids through retro_engine_tokenize, BOS by the kind's default, and detokenize(tokenize(text)) == text."""
    import json
    from pathlib import Path
    golden = json.loads((Path(__file__).resolve().parent / "golden" / "bpe_reference_ids.json").read_text())
    kind = next(k for k in golden["kinds"] if k["pre"] == pre)
    vocab = {"model": "gpt2", "pre": pre, "tokens": kind["tokens"], "merges": kind["merges"],
             "types": [3 if i in kind["control"] else 1 for i in range(len(kind["tokens"]))], "bos": 0, "eos": 1}
    shape = synth.scaled(synth.TINY_LLAMA, n_vocab=len(kind["tokens"]), name="tiny-llama-bpe-" + pre)
    path = tmp_path / "bpe.gguf"
    synth.write_model(path, shape, seed=6, device="cpu", vocab=vocab)
    eng = E.Engine(path, E.EngineConfig(n_ctx=256, n_seq_max=2, n_batch=64, n_ubatch=64))
    for c in kind["cases"]:
        special = "<|" in c["text"]
        assert eng.tokenize(c["text"], add_special=False, parse_special=special) == c["ids"], c["text"]
        assert eng.detokenize_bytes(c["ids"], unparse_special=True).decode() == c["text"], c["text"]
    hello = next(c["ids"] for c in kind["cases"] if c["text"] == "Hello world")
    assert eng.tokenize("Hello world") == ([0] if pre == "llama-bpe" else []) + hello
    assert b"".join(eng.token_piece(t) for t in hello) == b"Hello world"
    assert eng.token_piece(0) == b"" and eng.token_piece(0, special=True) == b"<|begin_of_text|>"
    with pytest.raises(E.EngineError, match="outside the vocabulary"):
        eng.token_piece(len(kind["tokens"]))
    out = E.StepOutput()
    eng.step([E.StepRow(0, 0, eng.tokenize("attention is all you need"), 0, sample=True, sampling=greedy())], out)
    assert 0 <= out.row(0).token < len(kind["tokens"])
    eng.close()
