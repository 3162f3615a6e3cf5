"""The block types a model file may hold besides the ones with kernels of their own (reference
crates/rir-core/src/quant.rs:223-310, 327-396, 465-480 decodes them all): Q4_0, Q5_0, IQ4_NL and Q3_K are rewritten
as Q8_0 rows when a model is loaded (retrograd_amd/csrc/transcode.hpp) - this file checks on the CPU that the
rewritten rows decode, under Q8_0's rule, to exactly the values the oracle's decoder of the original type gives."""
import subprocess
from pathlib import Path

import numpy as np
import pytest

import oracle
from retrograd_amd import gguf_writer as gw

ROOT = Path(__file__).resolve().parent.parent
GEOM = {gw.GGML_Q4_0: (32, 18, [0]), gw.GGML_Q5_0: (32, 22, [0]), gw.GGML_IQ4_NL: (32, 18, [0]), gw.GGML_Q3_K: (256, 110, [108])}


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
    d = tmp_path_factory.mktemp("transcode_unit")
    exe = d / "transcode_unit"
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-o", str(exe), str(ROOT / "tests/cpp/transcode_unit.cpp")], check=True)
    return exe, d


def _rewrite(harness, wt, raw, n):
    exe, d = harness
    (d / "in.bin").write_bytes(raw.tobytes())
    r = subprocess.run([str(exe), str(wt), str(n), str(d / "in.bin"), str(d / "out.bin")], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout
    return np.frombuffer((d / "out.bin").read_bytes(), np.uint8)


@pytest.mark.parametrize("wt", sorted(GEOM), ids=["q4_0", "q5_0", "q3_k", "iq4_nl"])
def test_rows_rewritten_as_q8_0_decode_to_the_same_values(harness, wt):
    el, nb, scale_at = GEOM[wt]
    rng = np.random.default_rng(wt)
    n_blocks = 96
    raw = rng.integers(0, 256, (n_blocks, nb), dtype=np.uint8)
    for off in scale_at:
        raw[:, off:off + 2] = (rng.standard_normal(n_blocks) * 0.05).astype(np.float16).view(np.uint8).reshape(n_blocks, 2)
    if wt == gw.GGML_Q3_K:
        # the one code Q8_0 cannot hold as it is: scale 0 (-32) times -4 = 128. Block 0 holds it in its first 32
        # elements and -124 = 31 * -4 in its second 32, block 1 nothing but 128s.
        raw[0, 96:108] = 0
        raw[0, 96 + 1] = 0x0f                    # scale 1's low nibble 15 ...
        raw[0, 104 + 1] |= 0x03                  # ... and high bits 3: 63 - 32 = 31, elements 16..31
        raw[0, 96 + 2] = 0x0f                    # scales 2 and 3 (elements 32..63) 31 as well
        raw[0, 104 + 2] |= 0x03
        raw[0, 96 + 3] = 0x0f
        raw[0, 104 + 3] |= 0x03
        raw[0, 0:32] = 0                         # no high bits: every code is q - 4
        raw[0, 32:96] = 0                        # q = 0
        raw[1, 0:108] = 0
    n = n_blocks * el
    q8 = _rewrite(harness, wt, raw.reshape(-1), n)
    assert q8.size == n // 32 * 34
    want = oracle.decode_row(wt, raw.reshape(-1), n)
    got = oracle.decode_row(gw.GGML_Q8_0, q8, n)
    np.testing.assert_array_equal(got, want)
    if wt == gw.GGML_Q3_K:
        d0 = float(raw[0, 108:110].view(np.float16)[0])
        assert want[0] == np.float32(d0) * 128 and want[40] == np.float32(d0) * -124
        codes = q8.reshape(-1, 34)[:, 2:].view(np.int8)
        assert (codes[0] == -128).sum() == 16 and codes[1, 0] == -124 and (codes[8] == -128).all()


def test_a_type_with_a_min_term_is_not_rewritten(harness):
    exe, d = harness
    (d / "in.bin").write_bytes(bytes(20))
    r = subprocess.run([str(exe), str(gw.GGML_Q4_1), "32", str(d / "in.bin"), str(d / "out.bin")], capture_output=True, text=True)
    assert r.returncode == 1 and "no exact Q8_0 form" in r.stdout
