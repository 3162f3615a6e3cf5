"""Pins oracle/quant.hpp: the known answers the reference's own decoder tests
hold (reference crates/rir-core/src/quant.rs:534-581), exhaustive f16 against
numpy, and a brute-force per-element Q4_K / MXFP4 decoder written from the
addressing the reference's generated mat-vec spells out
(generated/rir/mul_mat_vec_q4_K/cpu.rs:52-120: d@0, dmin@2, scales@4..16,
qs@16..144)."""
import numpy as np
import pytest

import oracle
from retrograd_amd import gguf_writer as gw


def test_half_conversion_known_answers():
    # quant.rs:534-541
    h = np.array([0x3C00, 0xBC00, 0x0000, 0x0001, 0x0400, 0x7BFF], np.uint16)
    want = np.array([1.0, -1.0, 0.0, 2.0 ** -24, 2.0 ** -14, 65504.0], np.float32)
    assert np.array_equal(oracle.half_to_float(h), want)


def test_half_to_float_exhaustive_against_numpy():
    h = np.arange(65536, dtype=np.uint16)
    got = oracle.half_to_float(h)
    want = h.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_float_to_half_against_numpy_rounding():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 5, 200000).astype(np.float32),
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32),            # every half is a fixed point
        np.array([65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -24 * 1.5, 0.0, -0.0], np.float32),
    ])
    x = x[np.isfinite(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.float_to_half(x), want)
    # halfway cases between adjacent halves round to even
    h = np.arange(0x0001, 0x7BFE, 7, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = (lo + hi) / 2
    want = np.where(h % 2 == 0, h, h + 1).astype(np.uint16)
    assert np.array_equal(oracle.double_to_half(mid), want)


def test_e8m0_half_scale_known_answers():
    # quant.rs:545-553
    assert oracle.e8m0_half(127) == 0.5
    assert oracle.e8m0_half(128) == 1.0
    assert oracle.e8m0_half(129) == 2.0
    assert np.float32(oracle.e8m0_half(1)).view(np.uint32) == 0x00400000
    assert np.float32(oracle.e8m0_half(0)).view(np.uint32) == 0x00200000


def test_q8_0_decodes_scale_times_byte():
    # quant.rs:557-568
    blk = bytearray(34)
    blk[0:2] = (0x3C00).to_bytes(2, "little")
    for j in range(32):
        blk[2 + j] = (j - 16) & 0xFF
    v = oracle.decode_row(gw.GGML_Q8_0, bytes(blk), 32)
    assert np.array_equal(v, np.arange(-16, 16, dtype=np.float32))


def _f16(b, off):
    return np.frombuffer(bytes(b[off:off + 2]), np.float16)[0].astype(np.float32)


def _q4k_brute(block: bytes) -> np.ndarray:
    """One element at a time: element e lives in 64-element group g = e // 64;
    within it the first 32 are low nibbles, the last 32 high nibbles of the
    same 32 bytes; sub-block j = e // 32 picks the 6-bit scale/min."""
    d, dmin = _f16(block, 0), _f16(block, 2)
    sc = block[4:16]
    qs = block[16:144]
    out = np.zeros(256, np.float32)
    for e in range(256):
        j = e // 32
        if j < 4:
            s, m = sc[j] & 63, sc[j + 4] & 63
        else:
            s = (sc[j + 4] & 0x0F) | ((sc[j - 4] >> 6) << 4)
            m = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4)
        byte = qs[(e // 64) * 32 + e % 32]
        q = (byte >> 4) if (e % 64) >= 32 else (byte & 0x0F)
        out[e] = np.float32(np.float32(d * np.float32(s)) * np.float32(q)) - np.float32(dmin * np.float32(m))
    return out


def test_q4_k_against_bruteforce_addressing():
    rng = np.random.default_rng(1)
    for _ in range(20):
        blk = bytearray(rng.integers(0, 256, 144, dtype=np.uint8).tobytes())
        blk[0:2] = (0x2400).to_bytes(2, "little")   # pinned finite scales, as quant.rs:206-212
        blk[2:4] = (0x2000).to_bytes(2, "little")
        got = oracle.decode_row(gw.GGML_Q4_K, bytes(blk), 256)
        assert np.array_equal(got, _q4k_brute(bytes(blk)))


def test_q4_k_single_nibble_lands_on_one_element():
    # A lone nibble set in qs must light exactly one element: catches swapped
    # halves and wrong group strides.
    for byte_index in (0, 31, 32, 95, 127):
        for high in (False, True):
            blk = bytearray(144)
            blk[0:2] = (0x3C00).to_bytes(2, "little")      # d = 1
            for j in range(4):
                blk[4 + j] = 1                              # scales of sub-blocks 0..3 = 1
                blk[12 + j] = 1                             # low nibble: scales of sub-blocks 4..7 = 1
            blk[16 + byte_index] = 0x50 if high else 0x05
            v = oracle.decode_row(gw.GGML_Q4_K, bytes(blk), 256)
            e = (byte_index // 32) * 64 + (32 if high else 0) + byte_index % 32
            want = np.zeros(256, np.float32)
            want[e] = 5.0
            assert np.array_equal(v, want), (byte_index, high)


def test_mxfp4_nibble_halves_and_table():
    table = [0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12]   # doubled E2M1, quant.rs:61
    blk = bytearray(17)
    blk[0] = 128                                    # half-scale 1.0
    for j in range(16):
        blk[1 + j] = j | ((15 - j) << 4)
    v = oracle.decode_row(gw.GGML_MXFP4, bytes(blk), 32)
    want = np.array([table[j] for j in range(16)] + [table[15 - j] for j in range(16)], np.float32)
    assert np.array_equal(v, want)
    blk[0] = 127
    assert np.array_equal(oracle.decode_row(gw.GGML_MXFP4, bytes(blk), 32), want * 0.5)


def test_partial_block_is_refused():
    with pytest.raises(oracle.OracleError):
        oracle.row_bytes(gw.GGML_Q4_K, 128)
    assert oracle.row_bytes(gw.GGML_Q4_K, 4096) == 16 * 144
    assert oracle.row_bytes(gw.GGML_Q8_0, 4096) == 128 * 34
    assert oracle.row_bytes(gw.GGML_MXFP4, 64) == 34


def test_synthetic_quantisers_round_trip_close():
    # Not a parity statement: only that the synthetic-model quantisers write
    # blocks that decode near their input (valid scales, right packing).
    import torch
    from retrograd_amd import synth
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4, 512, generator=g) * 0.02
    for t, tol in ((gw.GGML_Q8_0, 0.01), (gw.GGML_Q4_K, 0.12), (gw.GGML_MXFP4, 0.3)):
        raw = synth.encode(x, t)
        for r in range(4):
            y = oracle.decode_row(t, raw[r], 512)
            err = np.abs(y - x[r].numpy()).max() / np.abs(x[r].numpy()).max()
            assert err < tol, (t, err)


# ---- the activations of a matmul as ggml's CPU path sees them -------------------------

Q8_K_WEIGHT, Q8_0_WEIGHT = 12, 8          # Q4_K and Q8_0 weights: Q8_K and Q8_0 activations


def test_q8_k_activations_hand_computed():
    # ggml quantize_row_q8_K_ref: the first value of largest magnitude maps to -127
    x = np.zeros(256, np.float32)
    x[:5] = [1.0, -2.0, 0.5, 2.0, 62.5 / 63.5]
    got = oracle.activation_row(Q8_K_WEIGHT, x)
    iscale = np.float32(-127.0) / np.float32(-2.0)           # 63.5
    d = np.float32(1.0) / iscale
    # 63.5 ties to the even 64; 31.75 -> 32; the opposite extreme reaches +127 (the cap); 62.5 ties to the even 62
    want = np.array([64, -127, 32, 127, 62], np.float32) * d
    assert np.array_equal(got[:5], want)
    assert not got[5:].any()
    # the sign of the scale follows the FIRST extreme; the values it stands for are the same
    y = x.copy()
    y[1], y[3] = 2.0, -2.0
    got2 = oracle.activation_row(Q8_K_WEIGHT, y)
    assert np.array_equal(got2[[1, 3]], [2.0, -2.0]) and np.array_equal(got2[[0, 2, 4]], got[[0, 2, 4]])
    # an all-zero block stays zero, blocks are independent
    z = np.zeros(512, np.float32)
    z[256:261] = x[:5] * 3
    got3 = oracle.activation_row(Q8_K_WEIGHT, z)
    assert not got3[:256].any() and np.allclose(got3[256:261], want * 3, rtol=1e-6)


def test_q8_0_activations_are_the_fixture_pinned_quantiser():
    # the Q8_0 row quantiser that reproduces the reference's fixture digests, decoded again
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(32 * 64) * 2).astype(np.float32)
    x[:32] = 0
    via_blocks = oracle.decode_row(8, oracle.quantize_q8_0(x), x.size)
    assert np.array_equal(oracle.activation_row(Q8_0_WEIGHT, x), via_blocks)
    assert np.array_equal(oracle.activation_row(39, x), via_blocks)        # MXFP4 weights take Q8_0 activations too
    # half away from zero: 2.5 -> 3 with scale 1 (amax 127)
    v = np.zeros(32, np.float32)
    v[:4] = [127.0, 2.5, -2.5, 1.4]
    assert np.array_equal(oracle.activation_row(Q8_0_WEIGHT, v)[:4], [127.0, 3.0, -3.0, 1.0])


def test_activation_conversion_against_the_numpy_restatement():
    from ref_transformer import ggml_activations
    rng = np.random.default_rng(0)
    for wt in (0, 1, 8, 12, 30, 39):
        for i in range(60):
            x = (rng.standard_normal(512) * rng.choice([1e-3, 1.0, 50.0])).astype(np.float32)
            if i % 7 == 0:
                x[rng.integers(0, 512, 300)] = 0
            assert np.array_equal(oracle.activation_row(wt, x).astype(np.float64), ggml_activations(x, wt)), (wt, i)
    x = rng.standard_normal(64).astype(np.float32)
    assert np.array_equal(oracle.activation_row(0, x), x)                   # F32 weights: untouched
    assert np.array_equal(oracle.activation_row(1, x), x.astype(np.float16).astype(np.float32))


def test_matmul_on_grid_activations_is_the_plain_product():
    # integers with an extreme of 127 in every block are their own codes (scale 1): nothing is lost
    rng = np.random.default_rng(1)
    k, n = 512, 24
    x = rng.integers(-127, 128, (3, k)).astype(np.float32)
    x[:, ::32] = 127
    for wt in (8, 12):
        w = (rng.standard_normal((n, k)) * 0.1).astype(np.float32)
        raw = synth_quantise(wt, w)
        dense = np.stack([oracle.decode_row(wt, raw[i], k) for i in range(n)]).astype(np.float64)
        got = oracle.matmul(wt, raw, n, k, x)
        assert np.abs(got - x.astype(np.float64) @ dense.T).max() < 1e-4
    # and off the grid the product is that of the converted activations
    xf = rng.standard_normal((3, k)).astype(np.float32)
    conv = np.stack([oracle.activation_row(12, r) for r in xf]).astype(np.float64)
    got = oracle.matmul(12, raw, n, k, xf)
    assert np.abs(got - conv @ dense.T).max() < 1e-5
    assert np.abs(got - xf.astype(np.float64) @ dense.T).max() > 1e-3


def synth_quantise(wt, w):
    import torch
    from retrograd_amd import synth
    return np.asarray(synth.encode(torch.from_numpy(w), wt)).reshape(w.shape[0], -1)


# ---- Q6_K (the finer type of a Q4_K_M file: output.weight, half of ffn_down and attn_v) -----------

def _q6_k_by_the_block_loops(blk):
    """One 210-byte block decoded by the loop structure the reference spells out
    (crates/rir-core/src/quant.rs:444-464): two halves of 128, 32 positions each feeding four outputs."""
    ql, qh, sc = blk[0:128], blk[128:192], blk[192:208].view(np.int8)
    d = np.float32(blk[208:210].view(np.float16)[0])
    y = np.zeros(256, np.float32)
    for n in (0, 128):
        a, h, s = ql[n // 2:], qh[n // 4:], sc[n // 16:]
        for l in range(32):
            i = l // 16
            q1 = ((int(a[l]) & 0xF) | ((int(h[l]) & 3) << 4)) - 32
            q2 = ((int(a[l + 32]) & 0xF) | (((int(h[l]) >> 2) & 3) << 4)) - 32
            q3 = ((int(a[l]) >> 4) | (((int(h[l]) >> 4) & 3) << 4)) - 32
            q4 = ((int(a[l + 32]) >> 4) | (((int(h[l]) >> 6) & 3) << 4)) - 32
            y[n + l] = d * np.float32(s[i]) * np.float32(q1)
            y[n + l + 32] = d * np.float32(s[i + 2]) * np.float32(q2)
            y[n + l + 64] = d * np.float32(s[i + 4]) * np.float32(q3)
            y[n + l + 96] = d * np.float32(s[i + 6]) * np.float32(q4)
    return y


def test_q6_k_against_the_block_loops_and_single_codes():
    Q6_K = 14
    assert oracle.row_bytes(Q6_K, 512) == 2 * 210
    rng = np.random.default_rng(11)
    raw = rng.integers(0, 256, 2 * 210, dtype=np.uint8)
    for b in range(2):
        raw[b * 210 + 208:b * 210 + 210] = np.frombuffer(np.float16(0.03125 * (b + 1)).tobytes(), np.uint8)
    got = oracle.decode_row(Q6_K, raw, 512)
    want = np.concatenate([_q6_k_by_the_block_loops(raw[b * 210:(b + 1) * 210]) for b in range(2)])
    assert np.array_equal(got, want)
    # one code, one element: all codes 32 (value 0) except element e, scales 1, d 1
    for e in (0, 17, 33, 95, 127, 128, 200, 255):
        blk = np.zeros(210, np.uint8)
        blk[128:192] = 0xAA                      # top bits 2 everywhere: codes 32 -> 0
        blk[192:208] = 1
        blk[208:210] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
        assert not oracle.decode_row(Q6_K, blk, 256).any()
        half, g, l = e // 128, (e % 128) // 32, e % 32
        # code 63 (value 31): nibble 15, top bits 3
        blk[64 * half + l + 32 * (g & 1)] |= 0xF0 if g >= 2 else 0x0F
        blk[128 + 32 * half + l] |= 3 << (2 * g)
        y = oracle.decode_row(Q6_K, blk, 256)
        assert y[e] == 31.0 and np.count_nonzero(y) == 1, e
    # the synthetic quantiser writes blocks that decode near their input
    import torch
    from retrograd_amd import synth
    x = torch.randn(3, 512, generator=torch.Generator().manual_seed(4)) * 0.05
    enc = synth.encode(x, Q6_K)
    for r in range(3):
        y = oracle.decode_row(Q6_K, enc[r], 512)
        assert np.abs(y - x[r].numpy()).max() < 0.04 * np.abs(x[r].numpy()).max()
    # Q6_K weights take Q8_K activations
    v = rng.standard_normal(256).astype(np.float32)
    assert np.array_equal(oracle.activation_row(Q6_K, v), oracle.activation_row(12, v))


# ---- Q5_K (the main type of a Q5_K_M file) --------------------------------------------------------

def _q5_k_by_the_block_loops(blk):
    """One 176-byte block decoded by the loop structure the reference spells out
    (crates/rir-core/src/quant.rs:418-442): four groups of 64, two running bit masks for the fifth bit."""
    d, dmin = np.float32(blk[0:2].view(np.float16)[0]), np.float32(blk[2:4].view(np.float16)[0])
    scales, qh, qs = blk[4:16], blk[16:48], blk[48:176]

    def scale_min(j):
        if j < 4:
            return int(scales[j]) & 63, int(scales[j + 4]) & 63
        return (int(scales[j + 4]) & 0xF) | ((int(scales[j - 4]) >> 6) << 4), (int(scales[j + 4]) >> 4) | ((int(scales[j]) >> 6) << 4)

    y = np.zeros(256, np.float32)
    u1, u2, o = 1, 2, 0
    for g in range(4):
        ql = qs[32 * g:]
        sc1, m1 = scale_min(2 * g)
        sc2, m2 = scale_min(2 * g + 1)
        d1, mm1 = d * np.float32(sc1), dmin * np.float32(m1)
        d2, mm2 = d * np.float32(sc2), dmin * np.float32(m2)
        for l in range(32):
            h1 = 16 if int(qh[l]) & u1 else 0
            h2 = 16 if int(qh[l]) & u2 else 0
            y[o + l] = d1 * np.float32((int(ql[l]) & 0xF) + h1) - mm1
            y[o + 32 + l] = d2 * np.float32((int(ql[l]) >> 4) + h2) - mm2
        o += 64
        u1 <<= 2
        u2 <<= 2
    return y


def test_q5_k_against_the_block_loops_and_single_codes():
    Q5_K = 13
    assert oracle.row_bytes(Q5_K, 512) == 2 * 176
    rng = np.random.default_rng(12)
    raw = rng.integers(0, 256, 2 * 176, dtype=np.uint8)
    for b in range(2):
        raw[b * 176:b * 176 + 2] = np.frombuffer(np.float16(0.03125 * (b + 1)).tobytes(), np.uint8)
        raw[b * 176 + 2:b * 176 + 4] = np.frombuffer(np.float16(0.015625 * (b + 1)).tobytes(), np.uint8)
    got = oracle.decode_row(Q5_K, raw, 512)
    want = np.concatenate([_q5_k_by_the_block_loops(raw[b * 176:(b + 1) * 176]) for b in range(2)])
    assert np.array_equal(got, want)
    # one code, one element: d = 1, dmin = 0, every scale 1 (the six-bit fields of sub-blocks 0-3 in bytes 4-7,
    # of 4-7 in the low nibbles of bytes 12-15), all codes 0 except element e, which gets 31
    for e in (0, 17, 31, 32, 63, 64, 100, 127, 128, 200, 255):
        blk = np.zeros(176, np.uint8)
        blk[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
        blk[4:8] = 1
        blk[12:16] = 1
        assert not oracle.decode_row(Q5_K, blk, 256).any()
        s, l = e // 32, e % 32
        blk[48 + 32 * (s // 2) + l] |= 0xF0 if s & 1 else 0x0F
        blk[16 + l] |= 1 << s
        y = oracle.decode_row(Q5_K, blk, 256)
        assert y[e] == 31.0 and np.count_nonzero(y) == 1, e
    # the same bytes without the fifth bits are the Q4_K block with the same header and nibbles
    blk5 = rng.integers(0, 256, 176, dtype=np.uint8)
    blk5[16:48] = 0
    blk4 = np.concatenate([blk5[0:16], blk5[48:176]])
    assert np.array_equal(oracle.decode_row(Q5_K, blk5, 256), oracle.decode_row(12, blk4, 256))
    # the synthetic quantiser writes blocks that decode near their input
    import torch
    from retrograd_amd import synth
    x = torch.randn(3, 512, generator=torch.Generator().manual_seed(4)) * 0.05
    enc = synth.encode(x, Q5_K)
    for r in range(3):
        y = oracle.decode_row(Q5_K, enc[r], 512)
        assert np.abs(y - x[r].numpy()).max() < 0.05 * np.abs(x[r].numpy()).max()
    # Q5_K weights take Q8_K activations
    v = rng.standard_normal(256).astype(np.float32)
    assert np.array_equal(oracle.activation_row(Q5_K, v), oracle.activation_row(12, v))


# ---- the legacy and i-quant types (quant.rs:236-306, 327-396, 465-480) ------------------------------
# Each against a per-element closed form in numpy (element e -> byte, shift and scale index, derived from the
# layouts, where the oracle follows the reference's running loops), on random blocks with finite scales; the
# reference's own Q4_0 known answer; and single codes placed on single elements.

_IQ4NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float32)


def _h(blk, off):
    return np.float32(blk[off:off + 2].view(np.float16)[0])


def _closed_form(wt, blk):
    e = np.arange(256 if wt in (10, 11, 23) else 32)
    u = blk.astype(np.int64)
    if wt in (2, 20, 3, 6, 7):                                   # blocks of 32: element e is a nibble of byte e % 16
        head = {2: 2, 20: 2, 3: 4, 6: 6, 7: 8}[wt]
        nib = (u[head + e % 16] >> (4 * (e // 16))) & 15
        if wt in (6, 7):
            qh = int.from_bytes(bytes(blk[head - 4:head]), "little")
            nib = nib | (((qh >> e) & 1) << 4)                   # the fifth bit of element e is bit e of qh
        d = _h(blk, 0)
        if wt == 2:
            return d * (nib - 8).astype(np.float32)
        if wt == 20:
            return d * _IQ4NL[nib]
        if wt == 6:
            return d * (nib - 16).astype(np.float32)
        return d * nib.astype(np.float32) + _h(blk, 2)            # Q4_1, Q5_1
    if wt == 10:                                                 # Q2_K: scales[16] | qs[64] | d | dmin
        q = (u[16 + (e >> 7) * 32 + (e & 31)] >> (2 * ((e >> 5) & 3))) & 3
        sc = u[e >> 4]
        dl = _h(blk, 80) * (sc & 15).astype(np.float32)
        ml = _h(blk, 82) * (sc >> 4).astype(np.float32)
        return dl * q.astype(np.float32) - ml
    if wt == 11:                                                 # Q3_K: hmask[32] | qs[64] | scales[12] | d
        q = (u[32 + (e >> 7) * 32 + (e & 31)] >> (2 * ((e >> 5) & 3))) & 3
        high = (u[e & 31] >> (e >> 5)) & 1
        i = e >> 4                                               # scale i: four bits from scales[i % 8], two from scales[8 + i % 4]
        s = ((u[96 + i % 8] >> (4 * (i // 8))) & 15) | (((u[104 + i % 4] >> (2 * (i // 4))) & 3) << 4)
        dl = _h(blk, 108) * (s - 32).astype(np.float32)
        return dl * (q - 4 * (1 - high)).astype(np.float32)
    if wt == 23:                                                 # IQ4_XS: d | scales_h | scales_l[4] | qs[128]
        ib = e >> 5
        nib = (u[8 + 16 * ib + e % 16] >> (4 * ((e >> 4) & 1))) & 15
        sh = int(u[2]) | (int(u[3]) << 8)
        ls = ((u[4 + ib // 2] >> (4 * (ib % 2))) & 15) | (((sh >> (2 * ib)) & 3) << 4)
        return (_h(blk, 0) * (ls - 32).astype(np.float32)) * _IQ4NL[nib]
    raise AssertionError(wt)


_LEGACY = {2: (32, 18, [0]), 3: (32, 20, [0, 2]), 6: (32, 22, [0]), 7: (32, 24, [0, 2]), 20: (32, 18, [0]),
           10: (256, 84, [80, 82]), 11: (256, 110, [108]), 23: (256, 136, [0])}


def _random_blocks(wt, n_blocks, rng):
    el, nb, scale_at = _LEGACY[wt]
    raw = rng.integers(0, 256, (n_blocks, nb), dtype=np.uint8)
    for off in scale_at:                                         # finite f16 scales of mixed sign and magnitude
        raw[:, off:off + 2] = (rng.standard_normal(n_blocks) * 0.05).astype(np.float16).view(np.uint8).reshape(n_blocks, 2)
    return raw


@pytest.mark.parametrize("wt", sorted(_LEGACY), ids=["q4_0", "q4_1", "q5_0", "q5_1", "q2_k", "q3_k", "iq4_nl", "iq4_xs"])
def test_legacy_and_iquant_types_against_the_closed_form(wt):
    el, nb, _ = _LEGACY[wt]
    rng = np.random.default_rng(wt)
    raw = _random_blocks(wt, 24, rng)
    got = oracle.decode_row(wt, raw.reshape(-1), 24 * el).reshape(24, el)
    for b in range(24):
        np.testing.assert_array_equal(got[b], _closed_form(wt, raw[b]).astype(np.float32))
    with pytest.raises(oracle.OracleError):
        oracle.row_bytes(wt, el - 1)
    assert oracle.row_bytes(wt, 3 * el) == 3 * nb


def test_q4_0_known_answer_of_the_reference():
    """crates/rir-core/src/quant.rs:572-581: d = 1, every byte 0x81 -> low nibbles (first half) 1 - 8, high 8 - 8."""
    blk = np.zeros(18, np.uint8)
    blk[0:2] = np.array([0x3c00], np.uint16).view(np.uint8)
    blk[2:] = 0x81
    v = oracle.decode_row(2, blk, 32)
    assert (v[:16] == -7.0).all() and (v[16:] == 0.0).all()


def test_single_codes_of_the_super_block_types_land_on_single_elements():
    one = np.array([0x3c00], np.uint16).view(np.uint8)
    # Q2_K: all sub-block scales 1 (no mins), one 2-bit code 3 at element 100 = second 32 of the first half, l = 4
    blk = np.zeros(84, np.uint8)
    blk[0:16] = 0x01
    blk[80:82] = one
    blk[16 + 4] = 3 << 6
    v = oracle.decode_row(10, blk, 256)
    assert v[100] == 3.0 and np.count_nonzero(v) == 1
    # Q3_K: every scale 33 (d * 1), all high bits set (no -4): one code 2 at element 200 = half 1, j = 2, position 8
    blk = np.zeros(110, np.uint8)
    blk[0:32] = 0xff
    blk[96:104] = 0x11                                          # low four bits 1 of all sixteen scales
    blk[104:108] = 0xaa                                         # high two bits 2 -> 33
    blk[108:110] = one
    blk[32 + 32 + 8] = 2 << 4
    v = oracle.decode_row(11, blk, 256)
    assert v[200] == 2.0 and np.count_nonzero(v) == 1
    # ... and with its high bit clear the same element reads 2 - 4
    blk[8] &= ~np.uint8(1 << 6)
    assert oracle.decode_row(11, blk, 256)[200] == -2.0
    # IQ4_XS: sub-block 5 with scale 33, the others 32 (zero): code 15 (113) at element 5 * 32 + 16 + 3
    blk = np.zeros(136, np.uint8)
    blk[0:2] = one
    blk[2:4] = np.array([0xaaaa], np.uint16).view(np.uint8)     # high bits 2 everywhere -> 32 + low
    blk[4 + 2] = 1 << 4                                         # low nibble of sub-block 5
    blk[8:] = 0x88                                              # code 8 everywhere: value 1 where the scale is not zero
    blk[8 + 16 * 5 + 3] = 0xf8
    v = oracle.decode_row(23, blk, 256)
    assert v[5 * 32 + 16 + 3] == 113.0 and (np.delete(v[160:192], 19) == 1.0).all() and np.count_nonzero(v) == 32
