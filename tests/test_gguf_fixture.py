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


def test_synthetic_type_mixes_follow_the_layer_rule_and_their_byte_count(tmp_path):
    """The Q4_K_M mix bench.py can run: which layers take the finer type, and that the bytes bench.py charges a
    decode step for are the bytes of the matrices the file holds."""
    from retrograd_amd import synth
    big = synth.LLAMA3_8B_Q4K_M
    finer = [l for l in range(big.n_layer) if synth.finer_layer(big, l)]
    # llama.cpp's rule for 32 layers: the first and the last eighth and every third layer between
    assert finer == [0, 1, 2, 3, 6, 9, 12, 15, 18, 21, 24, 27, 28, 29, 30, 31]
    assert synth.streamed_weight_bytes(synth.LLAMA3_8B_Q4K) == 3925868544 + 295501824
    assert synth.streamed_weight_bytes(big) == 4616331264
    small = synth.scaled(big, n_layer=8, n_embd=256, n_head=4, n_head_kv=2, head_dim=64, n_ff=512, n_vocab=512,
                         rope_freqs=True, name="q4km-small")
    path = tmp_path / "mix.gguf"
    synth.write_model(path, small, seed=3, device="cpu")
    from gguf_reader import Reader
    r = Reader(path)
    on_disk = 0
    for name, n_in, n_out, t in synth.matrix_types(small):
        ne, typ, data = r.raw(name)
        assert typ == t and list(ne) == [n_in, n_out], name
        on_disk += len(data)
    assert on_disk == synth.streamed_weight_bytes(small)
    for l in range(8):
        want = 14 if synth.finer_layer(small, l) else 12
        assert r.tensors["blk.%d.ffn_down.weight" % l][1] == want and r.tensors["blk.%d.attn_v.weight" % l][1] == want
        assert r.tensors["blk.%d.attn_q.weight" % l][1] == 12
    assert r.tensors["output.weight"][1] == 14
    assert r.tensors["rope_freqs.weight"][1] == 0 and list(r.tensors["rope_freqs.weight"][0]) == [32]
