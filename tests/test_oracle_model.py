"""Pins oracle/model.hpp (parity with the reference is unpinned at float level:
the reference holds no absolute logits of a causal model). Checks: an
independent float64 numpy transformer, chunked prefill == token-by-token,
permutation of batch rows, seq_cp copy == source, zero-padded LoRA rank is
exact, adapter delta against the dense formula."""
import numpy as np
import pytest

import oracle
from retrograd_amd import gguf_writer as gw
from retrograd_amd import synth
from ref_transformer import NumpyModel

SHAPES = {
    "llama-q8": synth.TINY_LLAMA,
    "llama-q4k": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=256, n_head=4, n_head_kv=2, head_dim=64,
                              n_ff=512, n_vocab=320, name="llama-q4k-small"),
    "qwen2-q8": synth.scaled(synth.QWEN25_7B_Q8, n_layer=2, n_embd=128, n_head=4, n_head_kv=2, head_dim=32,
                             n_ff=256, n_vocab=300, name="qwen2-small"),
    "qwen3moe": synth.scaled(synth.QWEN3_30B_A3B, n_layer=2, n_embd=128, n_head=4, n_head_kv=2, head_dim=64,
                             n_vocab=288, n_expert=8, n_expert_used=2, n_ff_exp=64, name="qwen3moe-small"),
    # the type mix of a Q4_K_M file: output.weight, ffn_down and attn_v in Q6_K
    "llama-q4k-m": synth.scaled(synth.LLAMA3_8B_Q4K, n_layer=2, n_embd=256, n_head=4, n_head_kv=2, head_dim=64,
                                n_ff=512, n_vocab=320, output_type=14, down_type=14, v_type=14, name="llama-q4k-m-small"),
    # per-frequency rotation divisors (rope_freqs.weight, Llama 3.1's long-context rule) and linear scaling
    "llama-rope-freqs": synth.scaled(synth.TINY_LLAMA, rope_freqs=True, rope_scaling_linear=2.0, rope_base=500000.0,
                                     name="tiny-llama-rope-freqs"),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    d = tmp_path_factory.mktemp("orc")
    out = {}
    for i, (k, s) in enumerate(SHAPES.items()):
        p = d / (k + ".gguf")
        synth.write_model(p, s, seed=10 + i, device="cpu", std=0.05)
        out[k] = p
    return out


@pytest.mark.parametrize("activations", ["exact", "ggml"])
@pytest.mark.parametrize("key", list(SHAPES))
def test_forward_matches_independent_float64_transformer(models, key, activations):
    m = oracle.Model(models[key])
    ctx = oracle.Context(m, 2, activations=activations)
    # Under the ggml arithmetic the activations entering a matmul are re-quantised (Q8_K / Q8_0).
    # A value within an ulp of a rounding boundary can take the neighbouring code in one of the
    # two implementations (f32 here, f64 there), which moves the logits by ~1e-3; about one
    # prompt in five has such a value somewhere (see the next test). In either arithmetic the
    # same happens, at the 1e-5 level, to a K or V value on a rounding boundary of the f16
    # cache. These prompts have neither.
    rng = np.random.default_rng(10 if key == "llama-q4k-m" else 6)
    toks = rng.integers(0, m.n_vocab, 12)
    p = {"token": toks, "pos": np.arange(12), "seq": np.zeros(12), "output": np.ones(12)}
    got = ctx.step(p["token"], p["pos"], p["seq"], p["output"])
    want = NumpyModel(models[key], activations=activations).forward(toks)
    assert got.shape == want.shape
    # float32 storage of activations between ops is the only difference.
    assert np.abs(got - want).max() < 2e-5 * max(1.0, np.abs(want).max())
    assert np.array_equal(got.argmax(-1), want.argmax(-1))


def test_what_the_ggml_activation_conversion_costs_and_how_it_drifts(models):
    """Two measurements that decide how the product is tested. (1) The reference's CPU
    arithmetic (activations converted to Q8_K before every Q4_K matmul) is percents of the
    logit scale away from the plain product, far outside a 1e-3 tolerance. (2) Two faithful
    implementations of that arithmetic agree to float rounding on most prompts and to no
    better than ~1e-3..1e-2 on the rest: a single activation on the other side of a rounding
    boundary is enough, and every later conversion amplifies the difference."""
    m = oracle.Model(models["llama-q4k"])
    nm = NumpyModel(models["llama-q4k"], activations="ggml")
    dist, drift = [], []
    for seed in range(5, 15):
        toks = np.random.default_rng(seed).integers(0, m.n_vocab, 12)
        pos, seq, out = np.arange(12), np.zeros(12), np.ones(12)
        ggml = oracle.Context(m, 1, activations="ggml").step(toks, pos, seq, out)
        exact = oracle.Context(m, 1, activations="exact").step(toks, pos, seq, out)
        dist.append(np.abs(ggml - exact).mean() / np.abs(exact).mean())
        drift.append(np.abs(ggml - nm.forward(toks)).max() / np.abs(exact).max())
    assert min(dist) > 1e-2, dist                      # (1): every prompt, an order of magnitude outside 1e-3
    clean = [d for d in drift if d < 1e-6]
    flipped = [d for d in drift if d >= 1e-6]
    assert clean and flipped, drift                    # (2): both kinds occur among ten prompts
    assert all(1e-4 < d < 5e-2 for d in flipped), drift


def test_chunked_prefill_equals_token_by_token(models):
    m = oracle.Model(models["llama-q4k"])
    rng = np.random.default_rng(6)
    toks = rng.integers(0, m.n_vocab, 17)
    a = oracle.Context(m, 2).step_rows([(0, 0, toks, True)])
    c = oracle.Context(m, 2)
    c.step_rows([(1, 0, toks[:5], False)])
    c.step_rows([(1, 5, toks[5:16], False)])
    b = c.step_rows([(1, 16, toks[16:], True)])
    assert np.array_equal(a, b)
    assert c.seq_pos(1) == (0, 16) and c.seq_pos(0) == (-1, -1)


def test_batch_row_permutation_and_slot_independence(models):
    m = oracle.Model(models["qwen2-q8"])
    rng = np.random.default_rng(7)
    prompts = [rng.integers(0, m.n_vocab, n) for n in (3, 9, 5)]
    c1 = oracle.Context(m, 4)
    a = c1.step_rows([(s, 0, p, True) for s, p in enumerate(prompts)])
    c2 = oracle.Context(m, 4)
    order = [2, 0, 1]
    b = c2.step_rows([(3 - s, 0, prompts[s], True) for s in order])
    assert np.array_equal(a[order], b)


def test_seq_cp_copy_continues_like_source(models):
    m = oracle.Model(models["llama-q8"])
    rng = np.random.default_rng(8)
    toks = rng.integers(0, m.n_vocab, 10)
    c = oracle.Context(m, 3)
    c.step_rows([(0, 0, toks[:9], False)])
    c.seq_cp(0, 1)            # whole copy
    c.seq_cp(0, 2, 0, 6)      # partial copy [0, 6)
    assert c.seq_pos(1) == (0, 8) and c.seq_pos(2) == (0, 5)
    c.step_rows([(2, 6, toks[6:9], False)])
    out = c.step_rows([(s, 9, toks[9:], True) for s in range(3)])
    assert np.array_equal(out[0], out[1]) and np.array_equal(out[0], out[2])
    c.seq_rm(1, 4, -1)
    assert c.seq_pos(1) == (0, 3)
    c.seq_rm(1)
    assert c.seq_pos(1) == (-1, -1)


@pytest.mark.parametrize("activations", ["exact", "ggml"])
def test_lora_delta_matches_dense_formula_and_rank_padding(models, tmp_path, activations):
    shape = SHAPES["qwen2-q8"]
    m = oracle.Model(models["qwen2-q8"])
    ad = tmp_path / "a.gguf"
    synth.write_lora_adapter(ad, shape, rank=4, alpha=8.0, seed=3, std_a=0.1, std_b=0.1,
                             targets=("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down"))
    aid = m.load_adapter(ad, 0.5)
    assert aid == 1
    rng = np.random.default_rng(9)
    toks = rng.integers(0, m.n_vocab, 6)
    c = oracle.Context(m, 2, activations=activations)
    got = c.step_rows([(0, 0, toks, True), (1, 0, toks, True)], adapters=[aid, -1])
    from gguf_reader import Reader
    r = Reader(ad)
    lora = {}
    for name in r.tensors:
        if name.endswith(".lora_a"):
            base = name[:-7]
            A = r.dense(name, oracle.decode_row)
            B = r.dense(base + ".lora_b", oracle.decode_row)
            lora[base] = (A, B, 0.5 * 8.0 / 4, r.tensors[name][1])
    nm = NumpyModel(models["qwen2-q8"], activations=activations)
    want_ad = nm.forward(toks, lora=lora)[-1]
    want_base = nm.forward(toks)[-1]
    assert np.abs(got[0] - want_ad).max() < 2e-5 * max(1.0, np.abs(want_ad).max())
    assert np.abs(got[1] - want_base).max() < 2e-5 * max(1.0, np.abs(want_base).max())
    assert np.abs(want_ad - want_base).max() > 1e-3   # the adapter does something


@pytest.mark.parametrize("activations", ["exact", "ggml"])
def test_a_q8_0_cache_holds_the_reference_quantisers_blocks_and_attention_reads_them(models, activations):
    """kv="q8_0": K and V rows are stored as quantize_row_q8_0_ref blocks (32 values along a head's row, f16
    scale) and attention reads scale times code; under the ggml arithmetic the query row is converted as well.
    Pinned by the fixture-pinned row quantiser (what is stored is a fixed point of it, on its grid) and by the
    float64 numpy transformer with its own numpy quantiser. Against the reference's ggml build: parity unpinned."""
    m = oracle.Model(models["qwen2-q8"])
    rng = np.random.default_rng(12)
    toks = rng.integers(0, m.n_vocab, 40)
    c = oracle.Context(m, 1, activations=activations, kv="q8_0")
    got = c.step_rows([(0, 0, toks, True)])[0]
    for layer, pos, want_v in ((0, 0, False), (0, 39, True), (1, 17, False), (1, 33, True)):
        row = c.read_kv_values(layer, 0, pos, want_v)
        blocks = np.frombuffer(oracle.quantize_q8_0(row), np.uint8).reshape(-1, 34)
        again = blocks[:, :2].copy().view(np.float16).astype(np.float32) * blocks[:, 2:].view(np.int8).astype(np.float32)
        assert np.array_equal(again.reshape(-1), row)
        assert np.abs(blocks[:, 2:].view(np.int8)).max(axis=1).min() == 127 or (row.reshape(-1, 32) == 0).all(axis=1).any()
    nm = NumpyModel(models["qwen2-q8"], activations=activations, kv="q8_0")
    want = nm.forward(toks)[-1]
    # a code on a rounding boundary may fall either way between the two (f32 against float64 rows): looser than the f16 comparison
    assert np.abs(got - want).max() < 2e-3 * max(1.0, np.abs(want).max())
    f16 = oracle.Context(m, 1, activations=activations).step_rows([(0, 0, toks, True)])[0]
    assert np.abs(f16 - got).max() > 20 * np.abs(got - want).max(), "the cache type moves the logits far more than the two disagree"


# ---- the forward pass against Hugging Face transformers ------------------------------------------------

def _hf_golden():
    import importlib.util
    from pathlib import Path
    here = Path(__file__).resolve().parent / "golden"
    spec = importlib.util.spec_from_file_location("hf_reference_logits", here / "hf_reference_logits.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)          # imports numpy and this repository's writer only; transformers stays unloaded
    return mod, np.load(here / "hf_reference_logits.npz")


@pytest.mark.parametrize("key", ["llama", "llama-rope-freqs", "llama-linear", "llama-yarn", "qwen2", "qwen3moe"])
def test_forward_reproduces_hugging_face_transformers_logits(tmp_path, key):
    """tests/golden/hf_reference_logits.npz holds logits of LlamaForCausalLM / Qwen2ForCausalLM /
    Qwen3MoeForCausalLM (float64, K and V rounded to f16 as the cache stores them) over the dequantised
    weights of the same seeded files. A wrong RoPE pairing or q/k row permutation, head mapping, bias,
    q/k-norm, norm weight, frequency divisor, router rule or expert layout moves these logits by the size of
    the logits themselves; the oracle (f32 between operations) must be within 1e-4 of their scale."""
    mod, golden = _hf_golden()
    shape, seed, std = mod.CASES[key]
    path = tmp_path / (key + ".gguf")
    synth.write_model(path, shape, seed=seed, device="cpu", std=std)
    assert bytes(golden[key + ".sha256"]).hex() == mod.sha256(path), \
        "the seeded model file differs from the one the fixture was made from: run tests/golden/hf_reference_logits.py again"
    toks = golden[key + ".tokens"]
    want = golden[key + ".logits"].astype(np.float64)
    m = oracle.Model(path)
    # all positions: the step returns one row per output token
    n = len(toks)
    got = oracle.Context(m, 1, activations="exact").step(toks, np.arange(n), np.zeros(n), np.ones(n))
    assert got.shape == want.shape
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 1e-4 * scale, (np.abs(got - want).max(), scale)
    assert np.abs(got - want).mean() <= 2e-5 * np.abs(want).mean()
    assert np.array_equal(got.argmax(-1), want.argmax(-1))


def test_lora_delta_reproduces_hugging_face_logits_with_the_adapter_merged(tmp_path):
    """scale * alpha / r * B (A x) on q, k, v, o, gate, up and down of a qwen2 file against the Hugging Face model whose dense
    matrices had scale * alpha / r * B A added."""
    mod, golden = _hf_golden()
    L = mod.LORA
    shape, seed, std = mod.CASES[L["case"]]
    path, ad = tmp_path / "m.gguf", tmp_path / "a.gguf"
    synth.write_model(path, shape, seed=seed, device="cpu", std=std)
    synth.write_lora_adapter(ad, shape, rank=L["rank"], alpha=L["alpha"], seed=L["seed"], std_a=L["std_a"], std_b=L["std_b"],
                             targets=L["targets"])
    assert bytes(golden[L["case"] + ".lora.sha256"]).hex() == mod.sha256(ad)
    toks = golden[L["case"] + ".tokens"]
    want = golden[L["case"] + ".lora.logits"].astype(np.float64)
    base = golden[L["case"] + ".logits"].astype(np.float64)
    m = oracle.Model(path)
    aid = m.load_adapter(ad, L["scale"])
    n = len(toks)
    got = oracle.Context(m, 1, activations="exact").step(toks, np.arange(n), np.zeros(n), np.ones(n), adapter_of=np.full(n, aid))
    # the adapter factors are stored as f16 and multiplied in f32: a little looser than the dense comparison
    assert np.abs(got - want).max() <= 2e-4 * np.abs(want).max(), np.abs(got - want).max()
    assert np.abs(want - base).mean() > 0.1


@pytest.mark.parametrize("activations", ["exact", "ggml"])
def test_a_q4_0_cache_holds_four_bit_blocks_and_attention_reads_them(models, activations):
    """kv="q4_0": K and V rows are stored as quantize_row_q4_0_ref blocks (32 values along a head's row; d = m / -8
    for the value m of largest magnitude, so m itself is stored exactly as code 0; the other codes 0..15) and
    attention reads d (code - 8). What is stored lies on that grid, and the logits follow the float64 numpy
    transformer with its own numpy quantiser. Against the reference's ggml build: parity unpinned."""
    m = oracle.Model(models["qwen2-q8"])
    rng = np.random.default_rng(13)
    toks = rng.integers(0, m.n_vocab, 40)
    c = oracle.Context(m, 1, activations=activations, kv="q4_0")
    got = c.step_rows([(0, 0, toks, True)])[0]
    f16c = oracle.Context(m, 1, activations=activations)
    f16 = f16c.step_rows([(0, 0, toks, True)])[0]
    for layer, pos, want_v in ((0, 0, False), (0, 39, True), (1, 17, False), (1, 33, True)):
        row = c.read_kv_values(layer, 0, pos, want_v).reshape(-1, 32)
        peak = row[np.arange(len(row)), np.abs(row).argmax(-1)]
        d = (peak / np.float32(-8.0)).astype(np.float32)
        codes = row / d[:, None] + 8
        assert np.array_equal(codes, np.rint(codes)) and codes.min() == 0 and codes.max() <= 15
        assert (codes.min(axis=1) == 0).all()
        if layer == 0:           # the first layer's rows come from the same inputs as the f16 cache's: within half a step of them
            plain = f16c.read_kv_values(layer, 0, pos, want_v).reshape(-1, 32)
            assert (np.abs(row - plain) <= 0.5001 * np.abs(d)[:, None] + 1e-3 * np.abs(plain)).all() or \
                   (np.abs(row - plain) <= 1.0001 * np.abs(d)[:, None]).all()
    nm = NumpyModel(models["qwen2-q8"], activations=activations, kv="q4_0")
    want = nm.forward(toks)[-1]
    # a code on a rounding boundary may fall either way between the two (f32 against float64 rows), and a four-bit step is coarse
    assert np.abs(got - want).max() < 2e-2 * max(1.0, np.abs(want).max())
    assert np.abs(f16 - got).max() > 5 * np.abs(got - want).max(), "the cache type moves the logits far more than the two disagree"
