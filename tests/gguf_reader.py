"""A small pure-Python GGUF reader used only by tests (a third, independent
parse of the container next to the oracle's and the engine's)."""
import struct

import numpy as np

from retrograd_amd import gguf_writer as gw

_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}


class Reader:
    def __init__(self, path):
        self.buf = memoryview(open(path, "rb").read())
        self.pos = 0
        magic, version, n_tensors, n_kv = self._unpack("<IIQQ")
        assert magic == gw.GGUF_MAGIC and version == 3
        self.kv = {}
        for _ in range(n_kv):
            key = self._str()
            (t,) = self._unpack("<I")
            self.kv[key] = self._value(t)
        self.tensors = {}
        for _ in range(n_tensors):
            name = self._str()
            (nd,) = self._unpack("<I")
            ne = list(self._unpack("<%dQ" % nd))
            t, off = self._unpack("<IQ")
            self.tensors[name] = (ne, t, off)
        a = self.kv.get("general.alignment", 32)
        self.data0 = (self.pos + a - 1) // a * a

    def _unpack(self, fmt):
        out = struct.unpack_from(fmt, self.buf, self.pos)
        self.pos += struct.calcsize(fmt)
        return out

    def _str(self):
        (n,) = self._unpack("<Q")
        s = bytes(self.buf[self.pos:self.pos + n]).decode()
        self.pos += n
        return s

    def _value(self, t):
        if t == 8:
            return self._str()
        if t == 9:
            et, n = self._unpack("<IQ")
            return [self._value(et) for _ in range(n)]
        return self._unpack(_SCALARS[t])[0]

    def raw(self, name):
        ne, t, off = self.tensors[name]
        n = gw.tensor_nbytes(ne, t)
        return ne, t, np.frombuffer(self.buf[self.data0 + off:self.data0 + off + n], np.uint8)

    def dense(self, name, decode_row):
        """float64 array shaped [..., ne[1], ne[0]] decoded row by row."""
        ne, t, raw = self.raw(name)
        rows = int(np.prod(ne[1:])) if len(ne) > 1 else 1
        rb = raw.size // rows
        out = np.stack([decode_row(t, raw[r * rb:(r + 1) * rb], ne[0]) for r in range(rows)]).astype(np.float64)
        return out.reshape(list(reversed(ne)))
