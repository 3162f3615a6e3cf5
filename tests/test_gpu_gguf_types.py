"""Model files in the block types without kernels of their own, against the CPU oracle through the C ABI: Q4_0,
Q5_0, IQ4_NL and Q3_K (rewritten as Q8_0 at load and multiplied on the Q8_0 tile kernels) and Q4_1, Q5_1, Q2_K,
IQ4_XS (decoded element by element by the generic kernel). Every matrix of the file, the token embedding and the
output matrix included, is of the type under test; the payload bytes are uniformly random, so every code, sub-block
scale and high bit occurs. Same tolerances as tests/test_gpu_step.py."""
import numpy as np
import pytest

import oracle
from engine_helpers import assert_logits_close, run_both
from retrograd_amd import engine as E
from retrograd_amd import gguf_writer as gw
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

TYPES = {"q4_0": gw.GGML_Q4_0, "q4_1": gw.GGML_Q4_1, "q5_0": gw.GGML_Q5_0, "q5_1": gw.GGML_Q5_1, "q2_k": gw.GGML_Q2_K,
         "q3_k": gw.GGML_Q3_K, "iq4_nl": gw.GGML_IQ4_NL, "iq4_xs": gw.GGML_IQ4_XS}


@pytest.mark.parametrize("name", list(TYPES))
def test_a_model_of_this_type_follows_the_oracle(tmp_path, name):
    print("type", name, flush=True)
    shape = synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=512, n_head=8, n_head_kv=2, head_dim=64, n_ff=1024,
                         n_vocab=1024, matrix_type=TYPES[name], name="llama-%s-small" % name)
    path = tmp_path / (name + ".gguf")
    synth.write_model(path, shape, seed=300 + TYPES[name], device="cpu", std=0.05)
    eng = E.Engine(path, E.EngineConfig(n_ctx=1024, n_seq_max=4, n_batch=128, n_ubatch=128))
    m = oracle.Model(path)
    ctx = oracle.Context(m, 4)
    rng = np.random.default_rng(2)
    lens = [7, 33, 64, 18]
    prompts = [rng.integers(0, m.n_vocab, n) for n in lens]
    out, got, want = run_both(eng, ctx, [(i, i, p, 0, True) for i, p in enumerate(prompts)])
    assert_logits_close(got, want)
    assert float(np.abs(want).max()) > 0.05          # the comparison is not one of zeros
    pos = list(lens)
    for _ in range(2):
        feed = [int(want[i].argmax()) for i in range(4)]
        out, got, want = run_both(eng, ctx, [(i, i, [feed[i]], pos[i], True) for i in range(4)])
        assert_logits_close(got, want)
        pos = [p + 1 for p in pos]
    # the fingerprint is over the file's own tensor sizes, whatever the loader made of them (retro_runtime.hpp:856-868)
    from gguf_reader import Reader
    size = sum(gw.tensor_nbytes(ne, t) for ne, t, _ in Reader(path).tensors.values())
    h = 14695981039346656037
    for b in str(path).encode() + size.to_bytes(8, "little"):
        h = ((h ^ b) * 1099511628211) & (2 ** 64 - 1)
    assert eng.model_fingerprint() == h
    eng.close()
