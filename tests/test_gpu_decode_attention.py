"""The one-launch attention of pure decode steps (k_attention_decode: rotation, KV store, attention and split merge)
against the three launches it replaces (k_rope_store, k_attention, k_attention_combine; RETRO_FUSED_DECODE_ATTENTION=0)
on the same model and requests, and against the CPU oracle: llama's adjacent-pair rotation with heads of 128 and the
NeoX pairing with heads of 64 and q/k/v biases, per-head q / k RMSNorm (qwen3moe, heads of 64 and of 128, norm weights
away from one), sequences from one page to many (so that the eight waves of a
workgroup hold nothing, one page or several), a sequence whose beginning was removed, and steps of one row."""
import numpy as np
import pytest

import oracle
from engine_helpers import assert_logits_close, greedy, logit_errors
from retrograd_amd import engine as E
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

SHAPES = {
    "llama-hd128": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=1024, n_head=8, n_head_kv=2, head_dim=128,
                                n_ff=2048, n_vocab=2048, name="llama-q4k-hd128"),
    "qwen2-hd64": synth.scaled(synth.QWEN25_7B_Q8, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64,
                               n_ff=1024, n_vocab=1024, matrix_type=12, name="qwen2-q4k-hd64"),
    "qwen3moe-hd64": synth.scaled(synth.QWEN3_30B_A3B, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64, n_vocab=1024,
                                  n_expert=16, n_expert_used=4, n_ff_exp=256, norm_std=0.2, name="qwen3moe-qknorm-hd64"),
    "qwen3moe-hd128": synth.scaled(synth.QWEN3_30B_A3B, n_layer=2, n_embd=512, n_head=8, n_head_kv=4, head_dim=128, n_vocab=1024,
                                   n_expert=16, n_expert_used=4, n_ff_exp=256, norm_std=0.2, name="qwen3moe-qknorm-hd128"),
}


@pytest.mark.parametrize("key", list(SHAPES))
def test_one_launch_equals_three_and_the_oracle(key, tmp_path, monkeypatch):
    shape = SHAPES[key]
    print("decode attention:", shape.name, flush=True)
    path = tmp_path / "m.gguf"
    synth.write_model(path, shape, seed=31, device="cpu", std=0.05)
    cfg = E.EngineConfig(n_ctx=8 * 1024, n_seq_max=8, n_batch=256, n_ubatch=256)
    monkeypatch.setenv("RETRO_FUSED_DECODE_ATTENTION", "1")
    one = E.Engine(path, cfg)
    monkeypatch.setenv("RETRO_FUSED_DECODE_ATTENTION", "0")
    three = E.Engine(path, cfg)
    m = oracle.Model(path)
    ctx = oracle.Context(m, 8)
    rng = np.random.default_rng(4)
    lens = [1, 31, 32, 33, 250, 700, 95]          # positions 0 .. len - 1 resident before the decode steps
    prompts = [rng.integers(0, shape.n_vocab, n) for n in lens]
    out = E.StepOutput()
    for eng in (one, three):
        for i, p in enumerate(prompts):
            for at in range(0, len(p), 256):
                eng.step([E.StepRow(i, i, p[at:at + 256], at, sample=False, sampling=greedy())], out)
    for i, p in enumerate(prompts):
        ctx.step_rows([(i, 0, p, False)])
    # slot 5 loses its first 100 positions: its resident span starts inside a page
    for x in (one, three, ctx):
        x.seq_rm(5, 0, 100)
    pos = list(lens)
    feed = [int(t) for t in rng.integers(0, shape.n_vocab, len(lens))]
    for step in range(3):
        rows = list(range(len(lens))) if step != 1 else [4]          # all rows, one row, all rows
        got = {}
        for name, eng in (("one", one), ("three", three)):
            eng.step([E.StepRow(i, i, [feed[i]], pos[i], sample=True, sampling=greedy()) for i in rows], out)
            got[name] = (eng.debug_logits().copy(), [out.row(j).token for j in range(len(rows))])
        want = ctx.step_rows([(i, pos[i], [feed[i]], True) for i in rows])
        assert_logits_close(got["one"][0], want)
        assert_logits_close(got["three"][0], want)
        mx, rel = logit_errors(got["one"][0], got["three"][0])
        print("step %d: one launch against three, max %.2e rel %.2e" % (step, mx, rel), flush=True)
        assert rel <= 2e-5, (mx, rel)
        # the rows written into the cache are the same values
        kd = shape.n_head_kv * shape.head_dim
        for i in rows:
            for want_v in (False, True):
                a = one.debug_kv(1, i, pos[i], want_v, kd).astype(np.float32)
                b = three.debug_kv(1, i, pos[i], want_v, kd).astype(np.float32)
                bad = np.flatnonzero(~np.isclose(a, b, rtol=2e-3, atol=1e-4 * np.abs(b).max()))      # layer 1 sees layer 0's attention, equal to 1e-5
                assert bad.size == 0, (i, want_v, bad[:8], a[bad[:8]], b[bad[:8]])
        for j, i in enumerate(rows):
            srt = np.sort(want[j])[::-1]
            if srt[0] - srt[1] > 4e-2:
                assert got["one"][1][j] == int(want[j].argmax())
            feed[i] = int(want[j].argmax())
            pos[i] += 1
    one.close()
    three.close()


def test_the_timeline_records_every_workgroup_and_changes_nothing(tmp_path):
    shape = SHAPES["llama-hd128"]
    path = tmp_path / "m.gguf"
    synth.write_model(path, shape, seed=31, device="cpu", std=0.05)
    eng = E.Engine(path, E.EngineConfig(n_ctx=4 * 512, n_seq_max=4, n_batch=256, n_ubatch=256))
    rng = np.random.default_rng(5)
    lens = [40, 200, 7]
    out = E.StepOutput()
    for i, n in enumerate(lens):
        eng.step([E.StepRow(i, i, rng.integers(0, shape.n_vocab, n), 0, sample=False, sampling=greedy())], out)
    assert eng.attention_timeline_read().shape == (0, 6)
    rows = lambda extra: [E.StepRow(i, i, [5 + i], lens[i] + extra, sample=True, sampling=greedy()) for i in range(3)]
    eng.step(rows(0), out)
    plain = eng.debug_logits().copy()
    for i in range(3):
        eng.seq_rm(i, lens[i], -1)
    eng.attention_timeline(True)
    eng.step(rows(0), out)
    assert np.array_equal(eng.debug_logits(), plain)
    st = eng.attention_timeline_read().astype(np.int64)
    assert st.shape == (3 * shape.n_head_kv, 6)
    assert sorted(st[:, 5].tolist()) == sorted([n // 32 + 1 for n in lens] * shape.n_head_kv)        # pages per row
    assert (np.diff(st[:, :5], axis=1)[:, [0, 2, 3]] >= 0).all() and (st[:, 3] >= st[:, 1]).all()
    assert (st[:, 4] - st[:, 0]).max() < 100 * 1000          # a workgroup of this size ends within a millisecond
    eng.attention_timeline(False)
    assert eng.attention_timeline_read().shape == (0, 6)
    eng.close()


def test_the_longest_sequences_the_one_launch_takes_and_the_first_it_leaves(tmp_path, monkeypatch):
    """A workgroup's eight waves hold 64 page ids each: 512 pages, 16384 positions. A sequence decodes across that
    boundary - on the one launch up to it, on the three launches beyond - and equals an engine that never takes the
    one launch."""
    shape = SHAPES["qwen2-hd64"]
    path = tmp_path / "m.gguf"
    synth.write_model(path, shape, seed=32, device="cpu", std=0.05)
    cfg = E.EngineConfig(n_ctx=17 * 1024, n_seq_max=2, n_batch=512, n_ubatch=512)
    monkeypatch.setenv("RETRO_FUSED_DECODE_ATTENTION", "1")
    one = E.Engine(path, cfg)
    monkeypatch.setenv("RETRO_FUSED_DECODE_ATTENTION", "0")
    three = E.Engine(path, cfg)
    rng = np.random.default_rng(6)
    n0 = 16384 - 3
    prompt = rng.integers(0, shape.n_vocab, n0).astype(np.int32)
    out = E.StepOutput()
    for eng in (one, three):
        for at in range(0, n0, 512):
            eng.step([E.StepRow(0, 0, prompt[at:at + 512], at, sample=False, sampling=greedy())], out)
        eng.step([E.StepRow(1, 1, prompt[:40], 0, sample=False, sampling=greedy())], out)
    one.attention_timeline(True)
    tok = [7, 9]
    for step in range(6):          # positions 16381 .. 16386 of slot 0: the last three on the fallback
        got = []
        for eng in (one, three):
            eng.step([E.StepRow(0, 0, [tok[0]], n0 + step, sample=True, sampling=greedy()),
                      E.StepRow(1, 1, [tok[1]], 40 + step, sample=True, sampling=greedy())], out)
            got.append((eng.debug_logits().copy(), [out.row(0).token, out.row(1).token]))
        mx, rel = logit_errors(got[0][0], got[1][0])
        took_one_launch = len(one.attention_timeline_read()) > 0
        print("position %d: one launch %s, max %.2e rel %.2e" % (n0 + step, took_one_launch, mx, rel), flush=True)
        assert took_one_launch == (n0 + step + 1 <= 16384)
        assert rel <= 2e-5, (step, mx, rel)
        one.attention_timeline(False)          # forget the recorded launch, so that the next read tells this step's path
        one.attention_timeline(True)
        tok = got[1][1]
    one.close()
    three.close()
