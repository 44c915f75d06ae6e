"""Regenerates the GGUF-layout source bytes the v29.jlm.gz fixture was written from.

The fixture is a container the reference's own writer produced from a synthetic
model (/root/reference/format/jlm/migrateold_test.go:17-77).  Its source bytes
come from Go's math/rand/v2 PCG(26, 30), drawn in tensor order; the generator
(PCG-DXSM, a published algorithm in Go's standard library) is restated here so
the test can re-pack the Q4_K tensors and compare planes byte for byte.  The
restatement checks itself: output_norm's stored values are drawn after the
first 1,136 draws and must match.
"""
import numpy as np

M64 = (1 << 64) - 1
M128 = (1 << 128) - 1
_MUL = (2549297995355413924 << 64) | 4865540595714422341
_INC = (6364136223846793005 << 64) | 1442695040888963407


class PCG:
    def __init__(self, seed1, seed2):
        self.s = (seed1 << 64) | seed2

    def uint64(self):
        self.s = (self.s * _MUL + _INC) & M128
        hi, lo = self.s >> 64, self.s & M64
        hi ^= hi >> 32
        hi = (hi * 0xda942042e4dd58b5) & M64
        hi ^= hi >> 48
        hi = (hi * (lo | 1)) & M64
        return hi

    def uint32(self):
        return self.uint64() >> 32

    def intn(self, n):
        if n & (n - 1) == 0:
            return self.uint64() & (n - 1)
        prod = self.uint64() * n
        hi, lo = prod >> 64, prod & M64
        if lo < n:
            thresh = ((1 << 64) - n) % n
            while lo < thresh:
                prod = self.uint64() * n
                hi, lo = prod >> 64, prod & M64
        return hi


def source_tensors():
    """[(name, block, kind, payload)] in the order the fixture's writer drew them.

    kind is 'q4k', 'q5k' or 'f32'; a bank's payload is its sheets back to back,
    16 rows of k = 256 each."""
    k, n_exp = 256, 4
    rng = PCG(26, 30)

    def ks(rows, block_b):
        b = bytearray(rows * k // 256 * block_b)
        for i in range(0, len(b), block_b):
            for j in range(4, block_b):
                b[i + j] = rng.uint32() & 0xFF
            d = 0x2c00 + rng.intn(0x400)
            dm = 0x2400 + rng.intn(0x400)
            b[i], b[i + 1], b[i + 2], b[i + 3] = d & 0xFF, d >> 8, dm & 0xFF, dm >> 8
        return np.frombuffer(bytes(b), np.uint8)

    def f32(n):
        return np.array([np.float32(1) + np.float32(rng.intn(100)) / np.float32(1000)
                         for _ in range(n)], np.float32)

    out = [("token_embd", -1, "q4k", ks(8, 144)), ("output_norm", -1, "f32", f32(k))]
    for b in range(2):
        out.append(("attn_norm", b, "f32", f32(k)))
        out.append(("attn_q", b, "q5k", ks(16, 176)))
        out.append(("attn_k", b, "q4k", ks(16, 144)))
        out.append(("exp_gate_bank", b, "q4k", ks(16 * n_exp, 144)))
        out.append(("exp_down_bank", b, "q5k", ks(16 * n_exp, 176)))
    return out
