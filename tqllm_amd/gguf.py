"""GGUF expert-bank ingestion, host side: the Python mirror of include/tqmoe_gguf.hpp (the reference's reader and expert
slicer: src/core/gguf.hpp:71-91, gguf.cpp:116-200). A 3-D tensor [cols, rows, n_experts] is, byte for byte, the stacked
block stream [n_experts * rows][cols] that ExpertBank loads; one expert is a contiguous span of it."""
import struct

import numpy as np

# weights per block, bytes per block (gguf.cpp:116-152)
BLOCK_LAYOUT = {0: (1, 4), 1: (1, 2), 30: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 10: (256, 84), 11: (256, 110),
                12: (256, 144), 13: (256, 176), 14: (256, 210), 16: (256, 66), 17: (256, 74), 18: (256, 98), 19: (256, 50), 20: (32, 18),
                21: (256, 110), 22: (256, 82), 23: (256, 136), 323: (128, 76)}
_SCALAR = {0: "B", 1: "b", 2: "H", 3: "h", 4: "I", 5: "i", 6: "f", 7: "?", 10: "Q", 11: "q", 12: "d"}


class GgufError(RuntimeError):
    pass


class GgufTensor:
    def __init__(self, type, ne, offset, bytes):
        self.type, self.ne, self.offset, self.bytes = type, list(ne), offset, bytes


def gguf_block_layout(type):
    """(weights per block, bytes per block) or None for a type this reader cannot size."""
    return BLOCK_LAYOUT.get(type)


def gguf_expert_count(t):
    return t.ne[2] if len(t.ne) == 3 else 0


def gguf_expert_geometry(t, name):
    """(experts, cols, rows, bytes of one expert) of a 3-D expert tensor [cols, rows, experts], or GgufError: not 3-D, an empty
    expert axis, a type without a block layout, rows that do not end on a block boundary (a row is what the loaders read),
    a size past 64 bits, or a byte count other than the one recorded when the file was opened."""
    if len(t.ne) != 3:
        raise GgufError("%s: expected a 3-D tensor [cols, rows, experts], found %d dimension(s)" % (name, len(t.ne)))
    cols, rows, experts = t.ne
    if experts == 0:
        raise GgufError("%s: the expert axis is empty" % name)
    layout = gguf_block_layout(t.type)
    if layout is None:
        raise GgufError("%s: GGUF type %d has no block layout here" % (name, t.type))
    block_elems, block_bytes = layout
    if cols == 0 or rows == 0:
        raise GgufError("%s: an expert matrix of %d x %d holds nothing" % (name, rows, cols))
    if cols % block_elems:
        raise GgufError("%s: rows of %d weights do not end on the %d-weight blocks of type %d" % (name, cols, block_elems, t.type))
    each = cols // block_elems * block_bytes * rows
    if each * experts >= 1 << 64:
        raise GgufError("%s: tensor size overflows 64 bits" % name)
    if each * experts != t.bytes:
        raise GgufError("%s: %d experts of %d bytes make %d bytes, the file records %d" % (name, experts, each, each * experts, t.bytes))
    return experts, cols, rows, each


def gguf_expert_slice(t, idx, name):
    """Expert idx of a 3-D expert tensor as a 2-D tensor view of its own (gguf_expert_slice of src/core/gguf.hpp:77-91 in role).
    Fails closed: a wrong slice would silently read a neighbouring expert."""
    experts, cols, rows, each = gguf_expert_geometry(t, name)
    if not 0 <= idx < experts:
        raise GgufError("%s: expert %d requested, the tensor holds %d" % (name, idx, experts))
    return GgufTensor(t.type, [cols, rows], t.offset + idx * each, each)


class GgufFile:
    """Header, alignment and tensor table of a GGUF v2 / v3 file; tensor bytes are memory-mapped on demand."""

    def __init__(self, path):
        self.path = path
        self.alignment = 32
        self.tensors = {}
        with open(path, "rb") as f:
            self._f = f
            if f.read(4) != b"GGUF":
                raise GgufError("%s: not a GGUF file" % path)
            self.version = self._get("I")
            if self.version not in (2, 3):
                raise GgufError("%s: unsupported GGUF version %d" % (path, self.version))
            n_tensors, n_kv = self._get("Q"), self._get("Q")
            for _ in range(n_kv):
                key = self._str()
                v = self._value(self._get("I"))
                if key == "general.alignment" and isinstance(v, int) and v:
                    self.alignment = v
            infos = []
            for _ in range(n_tensors):
                name = self._str()
                nd = self._get("I")
                if nd > 4:
                    raise GgufError("%s: tensor %s has %d dimensions" % (path, name, nd))
                ne = [self._get("Q") for _ in range(nd)]
                infos.append((name, ne, self._get("I"), self._get("Q")))
            at = f.tell()
            self.data_offset = (at + self.alignment - 1) // self.alignment * self.alignment
            f.seek(0, 2)
            size = f.tell()
        del self._f
        for name, ne, type, rel in infos:
            n = int(np.prod(ne, dtype=np.uint64)) if ne else 1
            layout = gguf_block_layout(type)
            nbytes = 0
            if layout:
                if n % layout[0]:
                    raise GgufError("GGUF tensor %s: %d elements is not a multiple of the %d-element block of type %d" % (name, n, layout[0], type))
                nbytes = n // layout[0] * layout[1]
            if self.data_offset + rel + nbytes > size:
                raise GgufError("GGUF tensor %s runs past the end of %s" % (name, path))
            self.tensors[name] = GgufTensor(type, ne, self.data_offset + rel, nbytes)

    def _get(self, fmt):
        n = struct.calcsize("<" + fmt)
        b = self._f.read(n)
        if len(b) != n:
            raise GgufError("%s: truncated GGUF header" % self.path)
        return struct.unpack("<" + fmt, b)[0]

    def _str(self):
        n = self._get("Q")
        if n > 1 << 24:
            raise GgufError("%s: implausible string length in GGUF header" % self.path)
        return self._f.read(n).decode("utf-8", "replace")

    def _value(self, type):
        if type == 8:
            return self._str()
        if type == 9:
            et, n = self._get("I"), self._get("Q")
            return [self._value(et) for _ in range(n)]
        if type not in _SCALAR:
            raise GgufError("%s: unknown GGUF metadata type %d" % (self.path, type))
        return self._get(_SCALAR[type])

    def read(self, t):
        """The bytes of a tensor or of a slice, as a read-only uint8 array over the mapped file."""
        return np.memmap(self.path, dtype=np.uint8, mode="r", offset=t.offset, shape=(t.bytes,))

    def expert_bank(self, name):
        """(type, experts, rows, cols, bytes) of a whole 3-D expert tensor: what ExpertBank needs."""
        if name not in self.tensors:
            raise GgufError("%s: no tensor %s" % (self.path, name))
        t = self.tensors[name]
        gguf_expert_slice(t, 0, name)
        return t.type, t.ne[2], t.ne[1], t.ne[0], self.read(t)
