"""GGUF v3 container writer (no gguf-py dependency).

The byte layout is the one the reference's fixture generators produce
(reference scripts/gen-tiny-fixture.py:265-374): magic "GGUF", version 3,
tensor count, kv count (all little endian); typed key/values; a tensor table
of (name, n_dims, ne[], ggml type, offset into the data section); the header
padded to `general.alignment` and every tensor payload padded to it as well.
Tensor payloads may be `bytes`, numpy arrays or zero-argument callables that
return either, so multi-gigabyte synthetic models stream to disk one tensor at
a time.
"""

from __future__ import annotations

import struct
from typing import Callable, Iterable, Sequence, Union

import numpy as np

GGUF_MAGIC = 0x46554747
GGUF_VERSION = 3
DEFAULT_ALIGNMENT = 32

# GGUF metadata value types
T_UINT8, T_INT8, T_UINT16, T_INT16, T_UINT32, T_INT32, T_FLOAT32, T_BOOL, T_STRING, T_ARRAY = range(10)
T_UINT64, T_INT64, T_FLOAT64 = 10, 11, 12

# ggml tensor types used by the decode step
GGML_F32, GGML_F16, GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_BF16, GGML_MXFP4 = 0, 1, 8, 12, 13, 14, 30, 39
# ... and the types a model file may also hold: rewritten as Q8_0 at load or decoded element by element
GGML_Q4_0, GGML_Q4_1, GGML_Q5_0, GGML_Q5_1, GGML_Q2_K, GGML_Q3_K, GGML_IQ4_NL, GGML_IQ4_XS = 2, 3, 6, 7, 10, 11, 20, 23
BLOCK_GEOMETRY = {  # type -> (elements per block, bytes per block)
    GGML_F32: (1, 4), GGML_F16: (1, 2), GGML_BF16: (1, 2),
    GGML_Q8_0: (32, 34), GGML_MXFP4: (32, 17), GGML_Q4_K: (256, 144), GGML_Q5_K: (256, 176), GGML_Q6_K: (256, 210),
    GGML_Q4_0: (32, 18), GGML_Q4_1: (32, 20), GGML_Q5_0: (32, 22), GGML_Q5_1: (32, 24), GGML_IQ4_NL: (32, 18),
    GGML_Q2_K: (256, 84), GGML_Q3_K: (256, 110), GGML_IQ4_XS: (256, 136),
}

_SCALAR_FMT = {
    T_UINT8: "<B", T_INT8: "<b", T_UINT16: "<H", T_INT16: "<h", T_UINT32: "<I", T_INT32: "<i",
    T_FLOAT32: "<f", T_BOOL: "<?", T_UINT64: "<Q", T_INT64: "<q", T_FLOAT64: "<d",
}

Payload = Union[bytes, np.ndarray, Callable[[], Union[bytes, np.ndarray]]]


def _string(value: str) -> bytes:
    raw = value.encode("utf-8")
    return struct.pack("<Q", len(raw)) + raw


def encode_value(value_type: int, value, elem_type: int | None = None) -> bytes:
    """Payload bytes of one metadata value (without key and type tag)."""
    if value_type == T_STRING:
        return _string(value)
    if value_type == T_ARRAY:
        assert elem_type is not None
        out = bytearray(struct.pack("<IQ", elem_type, len(value)))
        if elem_type == T_STRING:
            for item in value:
                out += _string(item)
        else:
            out += struct.pack("<%d%s" % (len(value), _SCALAR_FMT[elem_type][1]), *value)
        return bytes(out)
    return struct.pack(_SCALAR_FMT[value_type], value)


def tensor_nbytes(ne: Sequence[int], ggml_type: int) -> int:
    elems, nbytes = BLOCK_GEOMETRY[ggml_type]
    count = 1
    for dim in ne:
        count *= dim
    assert ne[0] % elems == 0, "row length must be a multiple of the block size"
    return count // elems * nbytes


class GGUFWriter:
    def __init__(self, alignment: int = DEFAULT_ALIGNMENT) -> None:
        self.alignment = alignment
        self._kv: list[tuple[str, int, bytes]] = []
        self._tensors: list[tuple[str, list[int], int, Payload, int]] = []

    def add(self, key: str, value_type: int, value, elem_type: int | None = None) -> None:
        self._kv.append((key, value_type, encode_value(value_type, value, elem_type)))

    def add_tensor(self, name: str, ne: Iterable[int], ggml_type: int, payload: Payload,
                   nbytes: int | None = None) -> None:
        ne = [int(d) for d in ne]
        if nbytes is None:
            nbytes = tensor_nbytes(ne, ggml_type)
        self._tensors.append((name, ne, ggml_type, payload, nbytes))

    def header_bytes(self) -> bytes:
        out = bytearray(struct.pack("<IIQQ", GGUF_MAGIC, GGUF_VERSION, len(self._tensors), len(self._kv)))
        for key, value_type, payload in self._kv:
            out += _string(key) + struct.pack("<I", value_type) + payload
        offset = 0
        a = self.alignment
        for name, ne, ggml_type, _, nbytes in self._tensors:
            out += _string(name) + struct.pack("<I", len(ne))
            for dim in ne:
                out += struct.pack("<Q", dim)
            out += struct.pack("<IQ", ggml_type, offset)
            offset += (nbytes + a - 1) // a * a
        out += b"\0" * ((-len(out)) % a)
        return bytes(out)

    def write(self, path) -> int:
        """Streams the file to `path`; returns the bytes written."""
        a = self.alignment
        total = 0
        with open(path, "wb") as fh:
            header = self.header_bytes()
            fh.write(header)
            total += len(header)
            for name, _, _, payload, nbytes in self._tensors:
                data = payload() if callable(payload) else payload
                if isinstance(data, np.ndarray):
                    data = np.ascontiguousarray(data)
                    assert data.nbytes == nbytes, (name, data.nbytes, nbytes)
                    data.tofile(fh)
                else:
                    assert len(data) == nbytes, (name, len(data), nbytes)
                    fh.write(data)
                pad = (-nbytes) % a
                if pad:
                    fh.write(b"\0" * pad)
                total += nbytes + pad
        return total

    def to_bytes(self) -> bytes:
        parts = [self.header_bytes()]
        for _, _, _, payload, nbytes in self._tensors:
            data = payload() if callable(payload) else payload
            if isinstance(data, np.ndarray):
                data = np.ascontiguousarray(data).tobytes()
            assert len(data) == nbytes
            parts.append(data + b"\0" * ((-nbytes) % self.alignment))
        return b"".join(parts)
