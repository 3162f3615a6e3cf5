"""The MXFP4 products on the block-scaled FP4 x FP8 matrix instruction. In ggml's arithmetic: against the CPU oracle's matmul in that
arithmetic (Q8_0 activation blocks times the decoded MXFP4 rows, summed in f64), and bit for bit against integer
arithmetic where every product and sum is exact: activations whose blocks have amax 127 convert to themselves
(d = 1), so the result is the integer sum of code products times the weight blocks' powers of two."""
import numpy as np
import pytest
import torch

import oracle
from retrograd_amd import engine as E
from retrograd_amd import gguf_writer as gw
from retrograd_amd import synth

pytestmark = pytest.mark.gpu

DOUBLED = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.float64)   # reference quant.rs:61


def _random_rows(rng, n, k, e_lo=118, e_hi=136):
    raw = rng.integers(0, 256, (n, k // 32, 17), dtype=np.uint8)
    raw[..., 0] = rng.integers(e_lo, e_hi, (n, k // 32), dtype=np.uint8)
    return raw.reshape(n, -1)


def _decode(raw, n, k):
    blk = raw.reshape(n, k // 32, 17)
    d = np.exp2(blk[..., 0].astype(np.float64) - 128.0)[..., None]
    lo, hi = blk[..., 1:] & 15, blk[..., 1:] >> 4
    return (np.concatenate([DOUBLED[lo], DOUBLED[hi]], axis=-1) * d).reshape(n, k)


@pytest.mark.parametrize("n,k,t", [(64, 256, 1), (208, 768, 5), (1024, 2048, 16), (48, 4608, 3)])
def test_integer_activations_bit_for_bit(n, k, t):
    rng = np.random.default_rng(n + k + t)
    raw = _random_rows(rng, n, k, 124, 131)
    x = rng.integers(-127, 128, (t, k)).astype(np.float32)
    x.reshape(t, k // 32, 32)[:, :, 0] = 127.0          # every block converts with d = 1
    print("mxfp4 scaled, integers: n %d k %d t %d" % (n, k, t), flush=True)
    got = E.kernel_mxfp4_scaled(raw, n, k, x)
    want = x.astype(np.float64) @ _decode(raw, n, k).T
    assert np.abs(want).max() < 2 ** 24          # the sums are exact in f32 in any order
    assert np.array_equal(got, want.astype(np.float32))
    assert np.array_equal(got, oracle.matmul(gw.GGML_MXFP4, raw, n, k, x))


@pytest.mark.parametrize("n,k,t", [(256, 2048, 16), (2048, 768, 7), (160, 1024, 1)])
def test_against_the_oracle_matmul(n, k, t):
    g = torch.Generator().manual_seed(n + t)
    raw = synth.quantize_mxfp4(torch.randn(n, k, generator=g) * 0.03).numpy()
    x = (torch.randn(t, k, generator=g) * torch.rand(t, 1, generator=g) * 3).numpy()
    x[0, 32:64] = 0.0                                   # an all-zero block: d = 0, codes 0
    print("mxfp4 scaled, normal data: n %d k %d t %d" % (n, k, t), flush=True)
    got = E.kernel_mxfp4_scaled(raw, n, k, x)
    want = oracle.matmul(gw.GGML_MXFP4, raw, n, k, x)
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
    # the conversion is ggml's, not a no-op: the f32 product differs by far more than the tolerance
    exact = x.astype(np.float64) @ _decode(raw, n, k).T
    assert np.abs(exact - want).max() > 50 * 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("n,k,t", [(64, 256, 1), (224, 768, 5), (1024, 2048, 16), (96, 6400, 3), (32, 1792, 16)])
def test_exact_arithmetic_on_integers_bit_for_bit(n, k, t):
    """Integers below 2^19 in a block whose largest value is below 2^20 are six hexadecimal digits exactly, and every
    sum stays below 2^24 ulps of its result, so the product is the integer product."""
    rng = np.random.default_rng(n + k + t + 1)
    raw = _random_rows(rng, n, k, 126, 130)
    x = rng.integers(-2000, 2001, (t, k)).astype(np.float32)
    x[:, ::64] *= 64.0          # some blocks reach 2^17: their small members still have all their bits
    print("mxfp4 scaled, exact arithmetic, integers: n %d k %d t %d" % (n, k, t), flush=True)
    got = E.kernel_mxfp4_scaled(raw, n, k, x, exact=True)
    want = x.astype(np.float64) @ _decode(raw, n, k).T
    assert np.abs(want).max() < 2 ** 31
    assert np.abs(got - want).max() <= np.abs(want).max() * 2.0 ** -20          # f32 accumulation over the row
    small = rng.integers(-7, 8, (t, k)).astype(np.float32)          # sums below 2^24: exact in f32 in any order
    want = small.astype(np.float64) @ _decode(raw, n, k).T
    assert np.abs(want).max() < 2 ** 24
    assert np.array_equal(E.kernel_mxfp4_scaled(raw, n, k, small, exact=True), want.astype(np.float32))


@pytest.mark.parametrize("n,k,t", [(256, 2048, 16), (2048, 768, 7), (160, 1024, 1)])
def test_exact_arithmetic_against_the_oracle_matmul(n, k, t):
    g = torch.Generator().manual_seed(n + t + 7)
    raw = synth.quantize_mxfp4(torch.randn(n, k, generator=g) * 0.03).numpy()
    x = (torch.randn(t, k, generator=g) * torch.rand(t, 1, generator=g) * 3).numpy()
    x[0, 32:64] = 0.0                                   # an all-zero block
    x[-1, 64:96] *= 1e-6                                # a block of tiny values beside ordinary ones
    x[-1, 100] = 300.0                                  # a block with one large value: its neighbours keep 24 bits below it
    print("mxfp4 scaled, exact arithmetic: n %d k %d t %d" % (n, k, t), flush=True)
    got = E.kernel_mxfp4_scaled(raw, n, k, x, exact=True)
    want = x.astype(np.float64) @ _decode(raw, n, k).T
    assert np.abs(got - want).max() <= 2e-6 * np.abs(want).max()
    oracle.set_exact_activations(True)
    try:
        by_oracle = oracle.matmul(gw.GGML_MXFP4, raw, n, k, x)
    finally:
        oracle.set_exact_activations(False)
    assert np.abs(got - by_oracle).max() <= 2e-6 * np.abs(want).max()


def test_shapes_the_kernel_does_not_take_are_refused():
    raw = np.zeros((16, 17 * 8), np.uint8)
    x = np.zeros((17, 256), np.float32)
    with pytest.raises(E.EngineError):
        E.kernel_mxfp4_scaled(raw, 16, 256, x)           # 17 tokens
    with pytest.raises(E.EngineError):
        E.kernel_mxfp4_scaled(np.zeros((8, 17 * 8), np.uint8), 8, 256, x[:1])    # rows not in 16s
    with pytest.raises(E.EngineError):
        E.kernel_mxfp4_scaled(np.zeros((16, 17 * 4), np.uint8), 16, 128, np.zeros((1, 128), np.float32))   # columns not in 256s
    with pytest.raises(E.EngineError):
        E.kernel_mxfp4_scaled(np.zeros((16, 17 * 152), np.uint8), 16, 4864, np.zeros((1, 4864), np.float32))   # operands beyond LDS
    with pytest.raises(E.EngineError):
        E.kernel_mxfp4_scaled(raw, 16, 256, x[:1], exact=True)                                                 # rows not in 32s
