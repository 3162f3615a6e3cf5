"""The decode step at the full shape of the headline configuration (Llama-3-8B shape, Q4_K,
32 layers, hidden 4096, 32 / 8 heads of 128, FFN 14336, vocabulary 128256), where the CPU
oracle cannot run a prefill in test time: size-independent properties (a copy decodes like
its source, a restored snapshot like the saved slot, a permuted batch like the original,
another chunking of the prompt like the first - bit for bit where the arithmetic is the same,
within the logit tolerances where the launch shapes differ), plus one decode step of two
sequences against the oracle, which takes their KV from the engine's own snapshots."""
import os
from pathlib import Path

import numpy as np
import pytest

import oracle
from engine_helpers import assert_logits_close, greedy
from retrograd_amd import engine as E
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

SHAPE = synth.LLAMA3_8B_Q4K


@pytest.fixture(scope="module")
def model_path(tmp_path_factory):
    # the benchmark's own model file when it is already there (4.6 GB, written on the GPU in seconds)
    shm = Path("/dev/shm")
    base = shm if shm.is_dir() and os.access(shm, os.W_OK) else tmp_path_factory.mktemp("full")
    path = base / ("retro-bench-%s-seed1234.gguf" % SHAPE.name)
    if not path.exists():
        tmp = path.with_suffix(".tmp%d" % os.getpid())
        synth.write_model(tmp, SHAPE, seed=1234, device="cuda")
        os.replace(tmp, path)
    return path


def test_full_shape_properties_and_one_step_against_the_oracle(model_path):
    print("full shape: %s" % SHAPE.name, flush=True)
    eng = E.Engine(model_path, E.EngineConfig(n_ctx=8 * 2560, n_seq_max=8, n_batch=512, n_ubatch=512))
    rng = np.random.default_rng(5)
    lens = [700, 1500, 47, 2100]
    prompts = [rng.integers(0, SHAPE.n_vocab, n).astype(np.int32) for n in lens]
    out = E.StepOutput()

    def prefill(slot, toks, chunk):
        last = None
        for at in range(0, len(toks), chunk):
            piece = toks[at:at + chunk]
            done = at + chunk >= len(toks)
            eng.step([E.StepRow(slot, slot, piece, at, sample=done, sampling=greedy())], out)
            if done:
                last = (out.row(0).token, eng.debug_logits()[0].copy())
        return last

    first = [prefill(i, prompts[i], 512) for i in range(4)]
    print("prefilled", flush=True)

    # another chunking of the same prompt: other launch shapes, the same logits within the tolerances
    tok_b, logits_b = prefill(4, prompts[0], 300)
    assert_logits_close(logits_b[None], first[0][1][None])
    margin = np.sort(first[0][1])[::-1]
    if margin[0] - margin[1] > 4e-2:
        assert tok_b == first[0][0]
    eng.seq_rm(4)

    # copies and a restored snapshot decode like their sources: slots 4..6 copy 0..2, slot 7 restores 3
    for i in range(3):
        eng.seq_cp(i, 4 + i)
    snap = eng.seq_save(3)
    eng.seq_load(7, snap)
    assert [eng.seq_pos(s) for s in range(4, 8)] == [(0, n - 1) for n in lens]
    feed = [t for t, _ in first]
    rows = [E.StepRow(i, i, [feed[i]], lens[i], sample=True, sampling=greedy()) for i in range(4)]
    eng.step(rows, out)
    src = eng.debug_logits().copy()
    src_tok = [out.row(i).token for i in range(4)]
    # ... in a permuted batch
    order = [2, 0, 3, 1]
    eng.step([E.StepRow(10 + i, 4 + i, [feed[i]], lens[i], sample=True, sampling=greedy()) for i in order], out)
    got = eng.debug_logits()
    for at, i in enumerate(order):
        assert out.row(at).token == src_tok[i]
        if i < 3:
            assert np.array_equal(got[at], src[i]), "a copy decodes like its source, wherever its row stands"
        else:
            assert np.array_equal(got[at], src[i]), "a restored snapshot decodes like the slot it was saved from"
    print("copies, snapshot, permutation", flush=True)

    # one decode step of two sequences against the oracle (KV from the engine's snapshots of before the step)
    m = oracle.Model(model_path)
    ctx = oracle.Context(m, 8)
    for s in (2, 0):
        eng.seq_rm(s, lens[s], -1)                     # back to the prompt
        ctx.import_snapshot(s, eng.seq_save(s))
    want = ctx.step_rows([(2, lens[2], [feed[2]], True), (0, lens[0], [feed[0]], True)])
    assert_logits_close(np.stack([src[2], src[0]]), want)
    for row, s in enumerate((2, 0)):
        srt = np.sort(want[row])[::-1]
        if srt[0] - srt[1] > 4e-2:
            assert src_tok[s] == int(want[row].argmax())
    eng.close()
