"""The engine's GGUF container reader refuses malformed files with an error instead of crashing the host:
alignment zero or no power of two, tensor offsets that would wrap, entry counts larger than the file,
dimensions that are zero, negative or overflow. CPU only (the reader is a header; tests/cpp/gguf_unit.cpp)."""
import struct
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def _s(text: str) -> bytes:
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def _file(n_tensors=1, n_kv=1, alignment=32, ne=(64, 2), offset=0, ttype=0, payload=None, claim_tensors=None, claim_kv=None):
    out = struct.pack("<IIQQ", 0x46554747, 3, n_tensors if claim_tensors is None else claim_tensors,
                      n_kv if claim_kv is None else claim_kv)
    for _ in range(n_kv):
        out += _s("general.alignment") + struct.pack("<Ii", 5, alignment)      # an i32 value
    for i in range(n_tensors):
        out += _s("t%d" % i) + struct.pack("<I", len(ne))
        for d in ne:
            out += struct.pack("<q", d)
        out += struct.pack("<IQ", ttype, offset)
    a = alignment if alignment > 0 and alignment & (alignment - 1) == 0 else 32
    out += b"\0" * (-len(out) % a)
    n = 1
    for d in ne:
        n *= max(d, 0)
    out += payload if payload is not None else b"\0" * min(4 * n, 1 << 16)
    return out


@pytest.fixture(scope="module")
def reader(tmp_path_factory):
    exe = tmp_path_factory.mktemp("gguf_unit") / "gguf_unit"
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-o", str(exe), str(ROOT / "tests/cpp/gguf_unit.cpp")], check=True)
    return exe


def _run(reader, tmp_path, data: bytes):
    p = tmp_path / "case.gguf"
    p.write_bytes(data)
    r = subprocess.run([str(reader), str(p)], capture_output=True, text=True, timeout=30)
    return r.returncode, r.stdout.strip()


def test_a_well_formed_file_is_read(reader, tmp_path):
    code, out = _run(reader, tmp_path, _file())
    assert (code, out) == (0, "ok 1 tensors, 512 bytes")


CASES = [
    ("alignment zero", dict(alignment=0), "alignment"),
    ("alignment negative", dict(alignment=-32), "alignment"),
    ("alignment no power of two", dict(alignment=48), "alignment"),
    ("offset wraps", dict(offset=(1 << 64) - 16), "runs past the file"),
    ("offset past the end", dict(offset=1 << 40), "runs past the file"),
    ("payload shorter than the shape", dict(payload=b"\0" * 100), "runs past the file"),
    ("tensor count larger than the file", dict(claim_tensors=1 << 60), "more entries than the file"),
    ("key count larger than the file", dict(claim_kv=1 << 60), "more entries than the file"),
    ("zero dimension", dict(ne=(0, 2)), "not positive"),
    ("negative dimension", dict(ne=(-64, 2)), "not positive"),
    ("dimensions overflow", dict(ne=(1 << 31, 1 << 31, 1 << 31)), "larger than any file"),
    ("row no whole blocks", dict(ne=(48, 2), ttype=8), "whole blocks"),
    ("truncated", dict(cut=40), "truncated"),
]


@pytest.mark.parametrize("name, how, needle", CASES, ids=[c[0].replace(" ", "-") for c in CASES])
def test_malformed_files_are_refused_with_an_error(reader, tmp_path, name, how, needle):
    how = dict(how)
    cut = how.pop("cut", None)
    data = _file(**how)
    code, out = _run(reader, tmp_path, data if cut is None else data[:cut])
    assert code == 1 and out.startswith("refused:") and needle in out, (name, code, out)
