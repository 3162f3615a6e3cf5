"""Kernel-level parity on the GPU, through the C ABI of include/retro_kernels.h.

Reference values come from the CPU oracle's block decoders: the same stored
bytes decoded on the host, multiplied in float64 with the f32 activations (the
kernels carry them as f16 hi/lo pairs, about 22 bits) or, under the ggml
arithmetic, with the activations as ggml's CPU matmul converts them for that
weight type (Q8_K / Q8_0 codes times their scale, f16 or bf16 rounding; the
oracle's activation_row). Both sides convert the same f32 inputs, so the
codes are identical. The products are accumulated in f32: 2e-5 of the output
scale covers that."""
import numpy as np
import pytest
import torch

import oracle
from retrograd_amd import engine as E
from retrograd_amd import gguf_writer as gw
from retrograd_amd import synth

pytestmark = pytest.mark.gpu


def _weights(t, n, k, seed):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(n, k, generator=g) * 0.05
    raw = synth.encode(w, t)
    raw = np.ascontiguousarray(raw).view(np.uint8).reshape(n, -1)
    dense = np.stack([oracle.decode_row(t, raw[i], k) for i in range(n)]).astype(np.float64)
    return raw, dense


def _ref(t, dense, x, ggml):
    """ggml: the rows as ggml's CPU matmul converts them for this weight type; else the f32 values."""
    seen = np.stack([oracle.activation_row(t, row) for row in x]) if ggml else x
    return seen.astype(np.float64) @ dense.T


@pytest.mark.parametrize("ggml", [False, True])
@pytest.mark.parametrize("t", [gw.GGML_Q4_K, gw.GGML_Q8_0])
@pytest.mark.parametrize("n,k,T", [(16, 256, 1), (48, 512, 7), (64, 1024, 16), (256, 4096, 33),
                                   (4096, 2048, 64), (160, 768, 100), (2064, 256, 3), (96, 1024, 24), (512, 4096, 48)])
def test_tile_matmul_matches_decoded_blocks(t, n, k, T, ggml):
    print("case", t, n, k, T, ggml, flush=True)
    raw, dense = _weights(t, n, k, seed=n + k + T)
    x = np.random.default_rng(T).standard_normal((T, k)).astype(np.float32)
    want = _ref(t, dense, x, ggml)
    scale = np.abs(want).max()
    for mode in (1, 2):      # register-only tiles, LDS-staged tiles
        got = E.kernel_matmul(t, raw, n, k, x, use_tiles=mode, ggml_activations=ggml)
        assert np.abs(got - want).max() <= 2e-5 * scale + 1e-6, mode
    gen = E.kernel_matmul(t, raw, n, k, x, use_tiles=False, ggml_activations=ggml)
    assert np.abs(gen - want).max() <= 2e-5 * scale + 1e-6


@pytest.mark.parametrize("ggml", [False, True])
@pytest.mark.parametrize("t", [gw.GGML_Q6_K, gw.GGML_Q5_K])
@pytest.mark.parametrize("n,k,T", [(16, 256, 1), (48, 512, 7), (64, 1024, 16), (256, 4096, 33), (4096, 2048, 64),
                                   (160, 768, 100), (2064, 256, 3), (96, 1024, 24), (512, 4096, 48), (1024, 14336, 5)])
def test_q6k_and_q5k_tile_matmul_matches_decoded_blocks(t, n, k, T, ggml):
    # Q6_K and Q5_K have LDS-staged tiles only (the types of Q4_K_M / Q5_K_M files beside Q4_K)
    print("case", t, n, k, T, ggml, flush=True)
    raw, dense = _weights(t, n, k, seed=n + k + T)
    x = np.random.default_rng(T).standard_normal((T, k)).astype(np.float32)
    want = _ref(t, dense, x, ggml)
    scale = np.abs(want).max()
    got = E.kernel_matmul(t, raw, n, k, x, use_tiles=2, ggml_activations=ggml)
    assert np.abs(got - want).max() <= 2e-5 * scale + 1e-6
    with pytest.raises(E.EngineError):
        E.kernel_matmul(t, raw, n, k, x, use_tiles=1)       # no register-only variant
    gen = E.kernel_matmul(t, raw, n, k, x, use_tiles=False, ggml_activations=ggml)
    assert np.abs(gen - want).max() <= 2e-5 * scale + 1e-6


@pytest.mark.parametrize("ggml", [False, True])
@pytest.mark.parametrize("t,k", [(gw.GGML_F16, 344), (gw.GGML_F32, 100), (gw.GGML_Q8_0, 128),
                                 (gw.GGML_MXFP4, 96), (gw.GGML_Q4_K, 256), (gw.GGML_BF16, 64), (gw.GGML_Q6_K, 512),
                                 (gw.GGML_Q5_K, 512)])
def test_generic_matmul_every_storage_type(t, k, ggml):
    print("case", t, k, ggml, flush=True)
    n, T = 37, 11
    if t == gw.GGML_BF16:
        g = torch.Generator().manual_seed(1)
        w = (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16)
        raw = w.view(torch.int16).numpy().view(np.uint8).reshape(n, -1)
        dense = w.float().numpy().astype(np.float64)
    else:
        raw, dense = _weights(t, n, k, seed=k)
    x = np.random.default_rng(2).standard_normal((T, k)).astype(np.float32)
    want = _ref(t, dense, x, ggml)
    got = E.kernel_matmul(t, raw, n, k, x, use_tiles=False, ggml_activations=ggml)
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max() + 1e-6
    if ggml and t in (gw.GGML_F16, gw.GGML_BF16, gw.GGML_Q8_0, gw.GGML_Q4_K, gw.GGML_MXFP4, gw.GGML_Q6_K, gw.GGML_Q5_K):
        assert np.abs(want - _ref(t, dense, x, False)).max() > 1e-4 * np.abs(want).max()     # the conversion is visible


@pytest.mark.parametrize("ggml", [False, True])
@pytest.mark.parametrize("n,k,T", [(128, 2048, 128), (5, 512, 9), (130, 2304, 33), (7, 4104, 17), (16, 8, 64), (33, 1024, 512)])
def test_f32_rows_over_many_tokens(n, k, T, ggml):
    # F32 matrices (the expert router) over more than eight tokens have a kernel of their own: a workgroup per four
    # features and eight tokens. Ragged feature and token counts, rows shorter and longer than its four k-chunks;
    # up to eight tokens the generic kernel still runs and must give the same numbers to rounding.
    print("case", n, k, T, ggml, flush=True)
    rng = np.random.default_rng(n + k + T)
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    raw = w.view(np.uint8).reshape(n, -1)
    x = rng.standard_normal((T, k)).astype(np.float32)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    scale = np.abs(want).max()
    bias = rng.standard_normal(n).astype(np.float32)
    got = E.kernel_matmul(gw.GGML_F32, raw, n, k, x, use_tiles=False, ggml_activations=ggml, bias=bias)
    assert np.abs(got - (want + bias)).max() <= 2e-5 * scale + 1e-6
    y0 = rng.standard_normal((T, n)).astype(np.float32)
    got = E.kernel_matmul(gw.GGML_F32, raw, n, k, x, use_tiles=False, ggml_activations=ggml, accumulate_into=y0)
    assert np.abs(got - (want + y0)).max() <= 3e-5 * scale + 1e-6
    few = E.kernel_matmul(gw.GGML_F32, raw, n, k, x[:8], use_tiles=False, ggml_activations=ggml)
    many = E.kernel_matmul(gw.GGML_F32, raw, n, k, x, use_tiles=False, ggml_activations=ggml)
    assert np.abs(few - many[:8]).max() <= 2e-6 * scale + 1e-7


def test_matmul_bias_and_accumulate():
    t, n, k, T = gw.GGML_Q4_K, 64, 512, 20
    raw, dense = _weights(t, n, k, seed=5)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((T, k)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    y0 = rng.standard_normal((T, n)).astype(np.float32)
    want = _ref(t, dense, x, False)
    for tiles in (2, 1, 0):
        got = E.kernel_matmul(t, raw, n, k, x, use_tiles=tiles, bias=bias)
        assert np.abs(got - (want + bias)).max() <= 3e-5 * np.abs(want).max()
        got = E.kernel_matmul(t, raw, n, k, x, use_tiles=tiles, accumulate_into=y0)
        assert np.abs(got - (want + y0)).max() <= 3e-5 * np.abs(want).max()


def test_tile_matmul_exact_on_integer_data():
    # Small-integer activations and weights whose products and sums are exact
    # in f32: the tile kernel must be bit-exact, which catches any misplaced
    # nibble, scale or min.
    rng = np.random.default_rng(7)
    n, k, T = 32, 512, 16
    blocks = rng.integers(0, 256, (n, k // 256, 144), dtype=np.uint8)
    blocks[..., 0:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    blocks[..., 2:4] = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)
    raw = blocks.reshape(n, -1)
    dense = np.stack([oracle.decode_row(gw.GGML_Q4_K, raw[i], k) for i in range(n)]).astype(np.float64)
    # an extreme of magnitude 127 in every block makes the integers their own Q8_K / Q8_0 codes (scale 1)
    x = rng.integers(-4, 5, (T, k)).astype(np.float32)
    x[:, ::32] = rng.choice([-127.0, 127.0], (T, k // 32))
    assert np.array_equal(np.stack([oracle.activation_row(gw.GGML_Q4_K, r) for r in x]), x)
    assert np.array_equal(np.stack([oracle.activation_row(gw.GGML_Q8_0, r) for r in x]), x)
    want = x.astype(np.float64) @ dense.T
    for mode in (1, 2):
        for ggml in (False, True):
            got = E.kernel_matmul(gw.GGML_Q4_K, raw, n, k, x, use_tiles=mode, ggml_activations=ggml)
            assert np.array_equal(got.astype(np.float64), want), (mode, ggml)
    q8 = rng.integers(0, 256, (n, k // 32, 34), dtype=np.uint8)
    q8[..., 0:2] = np.frombuffer(np.float16(0.125).tobytes(), np.uint8)
    raw = q8.reshape(n, -1)
    dense = np.stack([oracle.decode_row(gw.GGML_Q8_0, raw[i], k) for i in range(n)]).astype(np.float64)
    want = x.astype(np.float64) @ dense.T
    for mode in (1, 2):
        for ggml in (False, True):
            got = E.kernel_matmul(gw.GGML_Q8_0, raw, n, k, x, use_tiles=mode, ggml_activations=ggml)
            assert np.array_equal(got.astype(np.float64), want), (mode, ggml)


@pytest.mark.parametrize("n,k,T", [(16, 256, 1), (48, 512, 2), (2064, 256, 2), (64, 1024, 1), (256, 4096, 1), (32, 8192, 2),
                                   (128, 14336, 2), (4096, 4096, 2), (1024, 14336, 1), (320, 16384, 2), (16, 8448, 1),
                                   (64, 18944, 2), (48, 24576, 1), (112, 3584, 2)])
@pytest.mark.parametrize("t", [gw.GGML_Q4_K, gw.GGML_Q8_0, gw.GGML_Q6_K, gw.GGML_Q5_K])
def test_integer_matvec_matches_decoded_blocks(t, n, k, T):
    # The kernel of very small steps under the ggml arithmetic: integer products of the stored codes with the
    # Q8_K codes of the rows. Its sums are those of the converted values times the decoded weights, so the
    # reference of the tile kernels is its reference too.
    print("case", t, n, k, T, flush=True)
    raw, dense = _weights(t, n, k, seed=n + k + T)
    rng = np.random.default_rng(T + k)
    x = rng.standard_normal((T, k)).astype(np.float32)
    x[0, :256] = 0.0                                    # blocks of zeros: scale 0, codes 0
    want = _ref(t, dense, x, True)
    scale = np.abs(want).max()
    got = E.kernel_matmul(t, raw, n, k, x, use_tiles=2, ggml_activations=True, integer=True)
    assert np.abs(got - want).max() <= 2e-5 * scale + 1e-6
    tiles = E.kernel_matmul(t, raw, n, k, x, use_tiles=2, ggml_activations=True)
    assert np.abs(got - tiles).max() <= 2e-5 * scale + 1e-6
    bias = rng.standard_normal(n).astype(np.float32)
    y0 = rng.standard_normal((T, n)).astype(np.float32)
    got = E.kernel_matmul(t, raw, n, k, x, use_tiles=2, ggml_activations=True, integer=True, bias=bias)
    assert np.abs(got - (want + bias)).max() <= 3e-5 * scale + 1e-6
    got = E.kernel_matmul(t, raw, n, k, x, use_tiles=2, ggml_activations=True, integer=True, accumulate_into=y0)
    assert np.abs(got - (want + y0)).max() <= 3e-5 * scale + 1e-6


def test_integer_matvec_exact_on_integer_data_and_refusals():
    # Random bytes in every position of the tile (every code, scale and min), dyadic d and dmin, activations
    # that are their own Q8_K codes: every product and sum is exact in i32 and f32, so a misplaced nibble,
    # scale, min or activation byte shows as a wrong bit.
    rng = np.random.default_rng(17)
    n, k = 48, 768
    blocks = rng.integers(0, 256, (n, k // 256, 144), dtype=np.uint8)
    blocks[..., 0:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    blocks[..., 2:4] = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)
    raw = blocks.reshape(n, -1)
    dense = np.stack([oracle.decode_row(gw.GGML_Q4_K, raw[i], k) for i in range(n)]).astype(np.float64)
    for T in (1, 2):
        x = rng.integers(-4, 5, (T, k)).astype(np.float32)
        x[:, ::32] = rng.choice([-127.0, 127.0], (T, k // 32))
        assert np.array_equal(np.stack([oracle.activation_row(gw.GGML_Q4_K, r) for r in x]), x)
        want = x.astype(np.float64) @ dense.T
        got = E.kernel_matmul(gw.GGML_Q4_K, raw, n, k, x, use_tiles=2, ggml_activations=True, integer=True)
        assert np.array_equal(got.astype(np.float64), want), T
    # one activation at a time: element e alone is non-zero, which places every byte of the code order
    for e in (0, 1, 2, 3, 4, 5, 6, 7, 8, 31, 32, 100, 255, 256, 767):
        one = np.zeros((1, k), np.float32)
        one[0, e] = -127.0
        got = E.kernel_matmul(gw.GGML_Q4_K, raw, n, k, one, use_tiles=2, ggml_activations=True, integer=True)
        assert np.array_equal(got[0].astype(np.float64), -127.0 * dense[:, e]), e
    # Q8_0: every byte value as a weight code (-128 included), d = 0.125, the same self-coding activations
    q8 = rng.integers(0, 256, (n, k // 32, 34), dtype=np.uint8)
    q8[..., 0:2] = np.frombuffer(np.float16(0.125).tobytes(), np.uint8)
    raw8 = q8.reshape(n, -1)
    dense8 = np.stack([oracle.decode_row(gw.GGML_Q8_0, raw8[i], k) for i in range(n)]).astype(np.float64)
    for T in (1, 2):
        x = rng.integers(-4, 5, (T, k)).astype(np.float32)
        x[:, ::32] = rng.choice([-127.0, 127.0], (T, k // 32))
        assert np.array_equal(np.stack([oracle.activation_row(gw.GGML_Q8_0, r) for r in x]), x)
        got = E.kernel_matmul(gw.GGML_Q8_0, raw8, n, k, x, use_tiles=2, ggml_activations=True, integer=True)
        assert np.array_equal(got.astype(np.float64), x.astype(np.float64) @ dense8.T), T
    for e in (0, 1, 3, 4, 7, 8, 31, 32, 33, 255, 256, 767):
        one = np.zeros((1, k), np.float32)
        one[0, e] = 127.0
        got = E.kernel_matmul(gw.GGML_Q8_0, raw8, n, k, one, use_tiles=2, ggml_activations=True, integer=True)
        assert np.array_equal(got[0].astype(np.float64), 127.0 * dense8[:, e]), e
    x = rng.standard_normal((3, k)).astype(np.float32)
    with pytest.raises(E.EngineError, match="at most 2 tokens"):
        E.kernel_matmul(gw.GGML_Q4_K, raw, n, k, x, use_tiles=2, ggml_activations=True, integer=True)
    with pytest.raises(E.EngineError, match="at most 2 tokens"):
        E.kernel_matmul(gw.GGML_Q4_K, raw, n, k, x[:1], use_tiles=2, integer=True)      # the exact arithmetic has no codes
    # Q5_K: the same with a fifth bit per code (blocks of 176 bytes: d, dmin, scales, 32 bytes of fifth bits, nibbles)
    b5 = rng.integers(0, 256, (n, k // 256, 176), dtype=np.uint8)
    b5[..., 0:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    b5[..., 2:4] = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)
    raw5 = b5.reshape(n, -1)
    dense5 = np.stack([oracle.decode_row(gw.GGML_Q5_K, raw5[i], k) for i in range(n)]).astype(np.float64)
    for T in (1, 2):
        x = rng.integers(-4, 5, (T, k)).astype(np.float32)
        x[:, ::32] = rng.choice([-127.0, 127.0], (T, k // 32))
        got = E.kernel_matmul(gw.GGML_Q5_K, raw5, n, k, x, use_tiles=2, ggml_activations=True, integer=True)
        assert np.array_equal(got.astype(np.float64), x.astype(np.float64) @ dense5.T), T
    for e in (0, 1, 2, 3, 4, 5, 6, 7, 8, 31, 32, 39, 64, 100, 255, 256, 767):
        one = np.zeros((1, k), np.float32)
        one[0, e] = -127.0
        got = E.kernel_matmul(gw.GGML_Q5_K, raw5, n, k, one, use_tiles=2, ggml_activations=True, integer=True)
        assert np.array_equal(got[0].astype(np.float64), -127.0 * dense5[:, e]), e
    with pytest.raises(E.EngineError, match="takes Q8_K or Q8_0 conversions"):      # an F16 matrix has none
        E.kernel_matmul(gw.GGML_F16, np.zeros((16, 512), np.uint8), 16, 256, x[:1, :256], use_tiles=0, ggml_activations=True, integer=True)


def test_integer_matvec_q6k_exact_for_every_code_and_scale():
    # Random bytes: every six-bit code and every i8 scale (-128 and 127 included) in every position of the tile, d = 1,
    # activations that are their own Q8_K codes: all integer, so the result is bit-exact or a bit is misplaced.
    rng = np.random.default_rng(29)
    n, k = 48, 768
    blocks = rng.integers(0, 256, (n, k // 256, 210), dtype=np.uint8)
    blocks[..., 208:210] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blocks[0, 0, 192:208] = np.array([-128, 127, -127, 126, -1, 0, 1, 15, 16, -16, -15, 17, -17, 112, -113, 64], np.int8).view(np.uint8)
    raw = blocks.reshape(n, -1)
    dense = np.stack([oracle.decode_row(gw.GGML_Q6_K, raw[i], k) for i in range(n)]).astype(np.float64)
    for T in (1, 2):
        x = rng.integers(-2, 3, (T, k)).astype(np.float32)
        x[:, ::32] = rng.choice([-127.0, 127.0], (T, k // 32))
        assert np.array_equal(np.stack([oracle.activation_row(gw.GGML_Q6_K, r) for r in x]), x)
        want = x.astype(np.float64) @ dense.T
        assert ((np.abs(x).astype(np.float64) @ np.abs(dense).T) <= 2.0 ** 24).all()
        got = E.kernel_matmul(gw.GGML_Q6_K, raw, n, k, x, use_tiles=2, ggml_activations=True, integer=True)
        assert np.array_equal(got.astype(np.float64), want), T
    for e in (0, 1, 2, 3, 4, 5, 6, 7, 8, 15, 16, 31, 32, 63, 64, 95, 96, 127, 128, 200, 255, 256, 767):
        one = np.zeros((1, k), np.float32)
        one[0, e] = -127.0
        got = E.kernel_matmul(gw.GGML_Q6_K, raw, n, k, one, use_tiles=2, ggml_activations=True, integer=True)
        assert np.array_equal(got[0].astype(np.float64), -127.0 * dense[:, e]), e


@pytest.mark.parametrize("t", [gw.GGML_Q4_K, gw.GGML_Q8_0, gw.GGML_Q6_K, gw.GGML_Q5_K])
@pytest.mark.parametrize("kind", [1, 2])
@pytest.mark.parametrize("n,k,T", [(64, 4096, 1), (64, 4096, 2), (32, 512, 1), (48, 1024, 2), (32, 14336, 1), (16, 14336, 2),
                                   (16, 8448, 2), (32, 2048, 1), (32, 3584, 1), (16, 18944, 1), (16, 256, 1), (16, 256, 2), (32, 768, 2)])
def test_integer_matvec_with_its_producer_fused(t, kind, n, k, T):
    # The Q8_K blocks made by the kernel itself while it stages them (RMSNorm of residual rows, or SwiGLU of a gate/up
    # product) against the producer's own launch followed by the kernel, and against the CPU: the norm / SiLU in
    # float64, the conversion by the oracle, the decoded weights. A row of 4096 is normalised in the very order the
    # standalone kernel uses, so there the two paths agree bit for bit; elsewhere the sum of squares is added in
    # another order and a code on a rounding boundary may differ.
    print("case", t, kind, n, k, T, flush=True)
    raw, dense = _weights(t, n, k, seed=n + k + T + kind)
    rng = np.random.default_rng(k + T)
    eps = 1e-5
    if kind == 1:
        x = (rng.standard_normal((T, k)) * 3.0).astype(np.float32)
        w = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
        fused, unfused = E.kernel_gemv_fused(1, t, raw, n, k, x, norm_w=w, eps=eps)
        x64 = x.astype(np.float64)
        rows = x64 / np.sqrt((x64 * x64).mean(-1, keepdims=True) + eps) * w
    else:
        group = 64 if k % 64 == 0 else 0
        gu = rng.standard_normal((T, 2 * k)).astype(np.float32)
        fused, unfused = E.kernel_gemv_fused(2, t, raw, n, k, gu, group=group)
        g64 = gu.astype(np.float64).reshape(T, k // 64, 2, 64)
        rows = (g64[:, :, 0] / (1 + np.exp(-g64[:, :, 0])) * g64[:, :, 1]).reshape(T, k)
    want = _ref(t, dense, rows.astype(np.float32), True)
    scale = np.abs(want).max()
    # a code that flips moves one product by d_x * |w|: allow a few of them on top of the float rounding
    flip = np.abs(rows).max() / 127.0 * np.abs(dense).max()
    assert np.abs(unfused - want).max() <= 2e-5 * scale + 8 * flip
    assert np.abs(fused - want).max() <= 2e-5 * scale + 8 * flip
    if kind == 2 or k == 4096:
        assert np.array_equal(fused, unfused)
    else:
        assert np.abs(fused - unfused).max() <= 8 * flip + 1e-6


@pytest.mark.parametrize("t", [gw.GGML_Q4_K, gw.GGML_Q8_0, gw.GGML_Q6_K, gw.GGML_Q5_K])
@pytest.mark.parametrize("kind", [11, 12])
@pytest.mark.parametrize("n,k", [(64, 4096), (32, 512), (48, 1024), (32, 14336), (16, 8448), (32, 2048), (32, 3584), (16, 18944), (16, 256),
                                 (32, 768), (16, 24576)])
def test_exact_matvec_with_its_producer_fused(t, kind, n, k):
    # The exact arithmetic's single-token kernel: f32 rows times the decoded weights, the row made by the kernel itself
    # (RMSNorm of a residual row, SwiGLU of a gate/up product) or read back from the hi / lo planes the producer's own
    # launch leaves, against the float64 product of the decoded weights with the float64 norm / SiLU. The fused row
    # keeps all of f32; the planes keep 22 bits of every value.
    print("case", t, kind, n, k, flush=True)
    raw, dense = _weights(t, n, k, seed=n + k + kind)
    rng = np.random.default_rng(k + kind)
    eps = 1e-5
    if kind == 11:
        x = (rng.standard_normal((1, k)) * 3.0).astype(np.float32)
        w = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
        fused, unfused = E.kernel_gemv_fused(11, t, raw, n, k, x, norm_w=w, eps=eps)
        x64 = x.astype(np.float64)
        rows = x64 / np.sqrt((x64 * x64).mean(-1, keepdims=True) + eps) * w
    else:
        group = 64 if k % 64 == 0 else 0
        gu = rng.standard_normal((1, 2 * k)).astype(np.float32)
        fused, unfused = E.kernel_gemv_fused(12, t, raw, n, k, gu, group=group)
        g64 = gu.astype(np.float64).reshape(1, k // 64, 2, 64)
        rows = (g64[:, :, 0] / (1 + np.exp(-g64[:, :, 0])) * g64[:, :, 1]).reshape(1, k)
    want = rows @ dense.astype(np.float64).T
    # what f32 products and sums of k terms may lose, against the sum of the terms' magnitudes
    bound = 4e-7 * (np.abs(rows) @ np.abs(dense).astype(np.float64).T) + 1e-6
    assert (np.abs(fused - want) <= 8 * bound).all(), float(np.abs(fused - want).max())
    assert (np.abs(unfused - want) <= 8 * bound).all(), float(np.abs(unfused - want).max())
    scale = np.abs(want).max()
    assert np.abs(fused - want).max() <= 2e-5 * scale and np.abs(unfused - want).max() <= 2e-5 * scale


def test_exact_matvec_places_every_code():
    # One non-zero activation at a time: the product is that column of the decoded weights, bit for bit (a single
    # product per row, nothing to round) - every position of a tile, every sub-block scale and offset.
    rng = np.random.default_rng(5)
    for t in (gw.GGML_Q4_K, gw.GGML_Q5_K, gw.GGML_Q6_K, gw.GGML_Q8_0):
        n, k = 32, 768
        raw, dense = _weights(t, n, k, seed=int(t) + 3)
        w = np.ones(k, np.float32)
        for e in list(range(0, 40)) + [63, 64, 127, 128, 255, 256, 300, 511, 512, 767] + [int(v) for v in rng.integers(0, k, 8)]:
            gu = np.zeros((1, 2 * k), np.float32)
            # SwiGLU of (gate, up) = (big, u): silu(40) = 40 to f32 precision, so the staged value is 40 * u
            blk, off = divmod(e, 64)
            gu[0, blk * 128 + off] = 40.0
            gu[0, blk * 128 + 64 + off] = 0.025
            fused, unfused = E.kernel_gemv_fused(12, t, raw, n, k, gu, group=64)
            v = np.float32(np.float32(40.0) / (np.float32(1.0) + np.exp(np.float32(-40.0)))) * np.float32(0.025)
            want = (np.float64(v) * dense[:, e].astype(np.float64))
            assert np.abs(fused[0] - want).max() <= 1e-6 * np.abs(want).max() + 1e-12, (t, e)


def test_q6k_tiles_are_exact_for_every_code_and_scale():
    # Random bytes: every six-bit code, every i8 scale (-128 and 127 included, whose products with a code
    # are not all f16 numbers) in every position of the tile. With d = 1 and small-integer activations all
    # products and sums are exact in f32, so the result is bit-exact or a bit is misplaced.
    rng = np.random.default_rng(11)
    n, k, T = 48, 768, 16
    blocks = rng.integers(0, 256, (n, k // 256, 210), dtype=np.uint8)
    blocks[..., 208:210] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blocks[0, 0, 192:208] = np.array([-128, 127, -127, 126, -1, 0, 1, 15, 16, -16, -15, 17, -17, 112, -113, 64], np.int8).view(np.uint8)
    raw = blocks.reshape(n, -1)
    dense = np.stack([oracle.decode_row(gw.GGML_Q6_K, raw[i], k) for i in range(n)]).astype(np.float64)
    x = rng.integers(-2, 3, (T, k)).astype(np.float32)
    x[:, ::32] = rng.choice([-127.0, 127.0], (T, k // 32))
    assert np.array_equal(np.stack([oracle.activation_row(gw.GGML_Q6_K, r) for r in x]), x)
    want = x.astype(np.float64) @ dense.T
    assert ((np.abs(x).astype(np.float64) @ np.abs(dense).T) <= 2.0 ** 24).all()
    for ggml in (False, True):
        got = E.kernel_matmul(gw.GGML_Q6_K, raw, n, k, x, use_tiles=2, ggml_activations=ggml)
        assert np.array_equal(got.astype(np.float64), want), ggml
    # one code at a time: element e of row r alone is non-zero
    for e in (0, 1, 7, 8, 15, 16, 31, 32, 63, 64, 95, 96, 127, 128, 200, 255):
        one = np.zeros((1, 256), np.float32)
        one[0, e] = 1.0
        got = E.kernel_matmul(gw.GGML_Q6_K, raw[:16, :210].copy(), 16, 256, one, use_tiles=2)
        assert np.array_equal(got[0].astype(np.float64), dense[:16, e]), e


def test_q5k_tiles_are_exact_for_every_code_scale_and_min():
    # Random bytes: every five-bit code, six-bit scale and min in every tile position; d = dmin = 1 and
    # small-integer activations keep every product and sum exact in f32.
    rng = np.random.default_rng(13)
    n, k, T = 48, 768, 16
    blocks = rng.integers(0, 256, (n, k // 256, 176), dtype=np.uint8)
    blocks[..., 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blocks[..., 2:4] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    raw = blocks.reshape(n, -1)
    dense = np.stack([oracle.decode_row(gw.GGML_Q5_K, raw[i], k) for i in range(n)]).astype(np.float64)
    x = rng.integers(-2, 3, (T, k)).astype(np.float32)
    x[:, ::32] = rng.choice([-127.0, 127.0], (T, k // 32))
    assert np.array_equal(np.stack([oracle.activation_row(gw.GGML_Q5_K, r) for r in x]), x)
    want = x.astype(np.float64) @ dense.T
    assert ((np.abs(x).astype(np.float64) @ np.abs(dense).T) <= 2.0 ** 24).all()
    for ggml in (False, True):
        got = E.kernel_matmul(gw.GGML_Q5_K, raw, n, k, x, use_tiles=2, ggml_activations=ggml)
        assert np.array_equal(got.astype(np.float64), want), ggml
    for e in (0, 1, 4, 7, 8, 15, 16, 31, 32, 63, 64, 95, 96, 127, 128, 200, 255):
        one = np.zeros((1, 256), np.float32)
        one[0, e] = 1.0
        got = E.kernel_matmul(gw.GGML_Q5_K, raw[:16, :176].copy(), 16, 256, one, use_tiles=2)
        assert np.array_equal(got[0].astype(np.float64), dense[:16, e]), e


@pytest.mark.parametrize("t", [gw.GGML_Q4_K, gw.GGML_Q8_0, gw.GGML_Q6_K, gw.GGML_Q5_K])
def test_split_k_matmul_is_deterministic_and_exact(t):
    # 4096 x 4096 at 64 tokens splits K across workgroups; the reduction order
    # is fixed, so two runs agree bit for bit, and both match the decoded blocks.
    n, k, T = 4096, 4096, 64
    raw, dense = _weights(t, n, k, seed=77)
    x = np.random.default_rng(5).standard_normal((T, k)).astype(np.float32)
    want = _ref(t, dense, x, False)
    a = E.kernel_matmul(t, raw, n, k, x, use_tiles=2)
    b = E.kernel_matmul(t, raw, n, k, x, use_tiles=2)
    assert np.array_equal(a, b)
    assert np.abs(a - want).max() <= 2e-5 * np.abs(want).max()
    y0 = np.random.default_rng(6).standard_normal((T, n)).astype(np.float32)
    c = E.kernel_matmul(t, raw, n, k, x, use_tiles=2, accumulate_into=y0)
    assert np.abs(c - (want + y0)).max() <= 3e-5 * np.abs(want).max()


@pytest.mark.parametrize("t", [gw.GGML_Q4_K, gw.GGML_Q8_0, gw.GGML_Q6_K, gw.GGML_Q5_K])
@pytest.mark.parametrize("T", [65, 100, 128, 192])
def test_split_k_matmul_over_several_token_chunks(t, T):
    # 2048 rows are 16 row groups: at two or three 64-token chunks K is still split across workgroups, every
    # slice holding all the chunks' rows; the slices are added in slice order.
    print("case", t, T, flush=True)
    n, k = 2048, 4096
    raw, dense = _weights(t, n, k, seed=31 + T)
    x = np.random.default_rng(T).standard_normal((T, k)).astype(np.float32)
    want = _ref(t, dense, x, False)
    a = E.kernel_matmul(t, raw, n, k, x, use_tiles=2)
    b = E.kernel_matmul(t, raw, n, k, x, use_tiles=2)
    assert np.array_equal(a, b)
    assert np.abs(a - want).max() <= 2e-5 * np.abs(want).max()
    y0 = np.random.default_rng(6).standard_normal((T, n)).astype(np.float32)
    c = E.kernel_matmul(t, raw, n, k, x, use_tiles=2, accumulate_into=y0)
    assert np.abs(c - (want + y0)).max() <= 3e-5 * np.abs(want).max()


def test_sample_prepare_matches_numpy():
    rng = np.random.default_rng(11)
    V = 5003
    logits = (rng.standard_normal((6, V)) * 3).astype(np.float32)
    logits[2, 100] = logits[2, 4000] = logits[2].max() + 1.0      # tie for the maximum: lowest id wins
    logits[3, :50] = 2.5                                           # ties inside the top-k
    k = [0, 1, 5, 64, 40, 8]
    argmax, mx, se, ids, vals = E.kernel_sample_prepare(logits, k)
    for r in range(6):
        row = logits[r]
        assert argmax[r] == int(np.flatnonzero(row == row.max())[0])
        assert mx[r] == row.max()
        ref = np.exp(row.astype(np.float64) - float(row.max())).sum()
        assert abs(se[r] - ref) <= 1e-12 * ref
        order = np.lexsort((np.arange(V), -row.astype(np.float64)))[:k[r]]
        assert list(ids[r, :k[r]]) == list(order)
        assert np.array_equal(vals[r, :k[r]], row[order])


@pytest.mark.parametrize("n_rows", [1, 5, 64])
def test_sample_prepare_in_slices_matches_numpy(n_rows):
    # rows that ask for at most one candidate over a large vocabulary take the sliced scan
    rng = np.random.default_rng(13)
    V = 20011                                                      # no multiple of the slice granularity
    logits = (rng.standard_normal((n_rows, V)) * 3).astype(np.float32)
    logits[0, 17] = logits[0, 19000] = logits[0].max() + 1.0      # the maximum twice, in different slices: lowest id wins
    if n_rows > 2:
        logits[2, -1] = logits[2].max() + 2.0                      # ... and in the very last position
    k = [r % 2 for r in range(n_rows)]
    argmax, mx, se, ids, vals = E.kernel_sample_prepare(logits, k)
    for r in range(n_rows):
        row = logits[r]
        assert argmax[r] == int(np.flatnonzero(row == row.max())[0])
        assert mx[r] == row.max()
        ref = np.exp(row.astype(np.float64) - float(row.max())).sum()
        assert abs(se[r] - ref) <= 1e-12 * ref
        if k[r]:
            assert ids[r, 0] == argmax[r] and vals[r, 0] == row.max()
