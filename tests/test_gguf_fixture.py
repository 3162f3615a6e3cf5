"""The reference pins its generated tiny fixtures by sha256
(reference tests/fixtures/TINY_*_FIXTURE.toml). Reproducing the digests with
this repository's GGUF writer, f16 rounding and the oracle's Q8_0 quantiser is
a known-answer test of all of them."""
import numpy as np
import pytest

import oracle
from golden import reference_tiny_fixtures as ref


@pytest.mark.parametrize("name", ["qwen2-f32", "qwen2-f16", "qwen2-q8_0", "olmoe-f32"])
def test_reference_fixture_digest(name, tmp_path):
    if name == "olmoe-f32":
        blob = ref.build_olmoe_f32()
    else:
        blob = ref.build_qwen2(name.split("-")[1], oracle.quantize_q8_0)
    assert ref.digest(blob) == ref.DIGESTS[name]


def test_oracle_reader_parses_the_reference_fixture(tmp_path):
    blob = ref.build_qwen2("q8_0", oracle.quantize_q8_0)
    path = tmp_path / "tiny-q8.gguf"
    path.write_bytes(blob)
    m = oracle.Model(path)
    assert (m.n_layer, m.n_embd, m.n_head, m.n_head_kv, m.head_dim, m.n_ff, m.n_vocab) == (4, 64, 4, 2, 16, 128, 260)
    assert m.rope_neox
    # The Q8_0 twin holds the f16-grid numbers up to the quantiser's step: one
    # decode over it is finite and has the biased-output shape.
    ctx = oracle.Context(m, 2)
    logits = ctx.step_rows([(0, 0, [1, 5, 9], True)])
    assert logits.shape == (1, 260) and np.isfinite(logits).all()


def test_synth_q8_0_matches_oracle_quantiser():
    import torch
    from retrograd_amd import synth
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(8, 256, generator=g) * 0.02).half().float()
    a = synth.quantize_q8_0(x).numpy().ravel()
    b = oracle.quantize_q8_0(x.numpy())
    # Same recipe (d = amax/127, round half away) up to float32-vs-double in the
    # scaled value: codes may differ by one on exact ties only.
    assert np.array_equal(a.reshape(-1, 34)[:, :2], b.reshape(-1, 34)[:, :2])
    diff = np.abs(a.reshape(-1, 34)[:, 2:].view(np.int8).astype(int) - b.reshape(-1, 34)[:, 2:].view(np.int8).astype(int))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.01
