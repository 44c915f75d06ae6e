"""Read side of the `.jlm` container: header, tensor table, and where a packed
tensor's three planes (QS, D, SC) sit, including one expert's sheet of a bank.

Follows /root/reference/format/jlm/format.go:95-132,210-245 (header),
codec.go:9-14 (table record), schema.go:25-58 (type codes) and
read.go:447-469 (expert sheet = entry offsets + x * ExpPageSize).  Only what the
matmul path needs is here: no pager, no writer, no vocabulary or config.
"""
import gzip
import struct
from dataclasses import dataclass

import numpy as np

from . import quant

MAGIC = b"JITLLM\0\0"
HEADER_BYTES = 192

# container type code -> ggml type number, for the packed types this path serves
TYPE_TO_QUANT = {4: quant.Q8_0, 6: quant.Q4_K, 8: quant.Q6_K, 11: quant.MXFP4}
TYPE_NAMES = {1: "F32", 2: "F16", 3: "Q4", 4: "Q8", 5: "Q3S", 6: "Q4S", 7: "Q5S", 8: "Q6S",
              9: "BF16", 10: "Q5", 11: "MX4"}


@dataclass
class Entry:
    role: int
    block: int
    index: int
    type: int
    dims: tuple
    qs_off: int
    d_off: int
    sc_off: int
    name: str

    @property
    def k(self):
        return self.dims[0]

    @property
    def rows(self):
        return self.dims[1] if len(self.dims) > 1 else 1

    @property
    def sheets(self):
        return self.dims[2] if len(self.dims) > 2 else 1


class File:
    """A container held in memory (bytes)."""

    def __init__(self, data):
        self.data = data
        if len(data) < HEADER_BYTES or data[:8] != MAGIC:
            raise ValueError("jlm: not a container")
        u32 = lambda o: struct.unpack_from("<I", data, o)[0]
        u64 = lambda o: struct.unpack_from("<Q", data, o)[0]
        self.version = u32(8)
        self.page_size, self.n_blocks, self.n_tensors = u64(16), u32(24), u32(28)
        self.tab_off, self.tab_len = u64(48), u64(56)
        self.data_off, self.dense_off, self.dense_len = u64(64), u64(72), u64(80)
        self.n_exp_pages, self.exp_data_off, self.exp_page_size = u32(172), u64(176), u64(184)
        if self.tab_off + self.tab_len > len(data):
            raise ValueError("jlm: table runs past the file")
        self.entries = self._table(data[self.tab_off:self.tab_off + self.tab_len])

    @classmethod
    def open(cls, path):
        opener = gzip.open if str(path).endswith(".gz") else open
        with opener(path, "rb") as f:
            return cls(f.read())

    def _table(self, b):
        out, o = [], 0
        while o < len(b):
            if len(b) - o < 12:
                raise ValueError("jlm: table: trailing bytes")
            role, block, index, typ, ndim = struct.unpack_from("<HiiBB", b, o)
            o += 12
            if ndim == 0 or ndim > 4:
                raise ValueError(f"jlm: {ndim} dimensions")
            dims = struct.unpack_from(f"<{ndim}Q", b, o)
            o += 8 * ndim
            qs_off, d_off, sc_off, nlen = struct.unpack_from("<QQQH", b, o)
            o += 26
            name = b[o:o + nlen].decode("utf-8", "replace")
            o += nlen
            out.append(Entry(role, block, index, typ, dims, qs_off, d_off, sc_off, name))
        return out

    def planes(self, e, sheet=0):
        """(qs, d, sc) u32 arrays of a packed entry; `sheet` picks one expert of a bank.

        A bank is `sheets` independently packed tensors of e.rows rows; expert x's
        planes are the entry's offsets moved on by x * exp_page_size."""
        t = TYPE_TO_QUANT.get(e.type)
        if t is None:
            raise ValueError(f"jlm: {TYPE_NAMES.get(e.type, e.type)} is not a packed type of this path")
        if not 0 <= sheet < e.sheets:
            raise ValueError(f"jlm: sheet {sheet} of {e.sheets}")
        nq, nd, nsc = quant.packed_words(t, e.rows, e.k)
        x0 = sheet * self.exp_page_size if e.sheets > 1 else 0

        def cut(off, n):
            off += x0
            if off + 4 * n > len(self.data):
                raise ValueError("jlm: span runs past the file")
            return np.frombuffer(self.data, np.uint32, n, off)
        return t, cut(e.qs_off, nq), cut(e.d_off, nd), cut(e.sc_off, nsc)
