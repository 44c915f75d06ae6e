"""Seeded synthetic weights and activations for tests and benchmarks.

The reference ships no Q4_K, Q6_K or MXFP4 weight quantizer (its tests use
random bytes with planted scales, real models arrive pre-quantized), so the
quantizers here are this package's own: deterministic, vectorised numpy,
ggml-shaped (per-sub-block scale/min, 6-bit or int8 sub-scales, f16 super
scale) without ggml's iterative refinement.  Only Q8_0 follows a recipe the
reference holds (/root/reference/convert/vision.go:155-186).  Matmul parity is
always measured on the quantized bytes, so the quantizer's choices do not
enter it.
"""
import numpy as np

from . import quant

_F16_SWEEP = np.array([0x3C00, 0x3800, 0x4000, 0x3400, 0x4200, 0x2E00, 0x3E00, 0x4400,
                       0x0001, 0x0200, 0x03FF, 0x0400, 0x1000, 0x7BFF, 0x5000, 0x0801], np.uint16)
_E8M0_SWEEP = np.array([127, 128, 126, 129, 104, 108, 113, 114, 120, 135, 143, 131], np.uint8)
_SCALE_OFFS = {quant.Q8_0: (0,), quant.Q4_K: (0, 2), quant.Q6_K: (208,)}
# e2m1 magnitudes doubled (the reference's MXFP4Values), codes 0..7; 8..15 negate
_MX_VALUES = np.array([0, 1, 2, 3, 4, 6, 8, 12], np.float32)


def _round_half_away(p):
    """math.Round: nearest integer, halves away from zero."""
    p = np.asarray(p, np.float64)
    return np.trunc(p + np.copysign(0.5, p))


def normal_weights(rows, k, seed=0, sigma=0.02):
    """f32 [rows][k] ~ N(0, sigma)."""
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((rows, k), np.float32) * np.float32(sigma)).astype(np.float32)


def activations(n, seed=1):
    """f32 [n] ~ N(0, 1)."""
    return np.random.default_rng(seed).standard_normal(n, np.float32)


def quantize_q8_0(w):
    """Q8_0 blocks of w [rows][k]: d = amax/127 stored as f16, codes rounded from the
    unrounded d (/root/reference/convert/vision.go:161-186)."""
    rows, k = w.shape
    x = w.reshape(rows, k // 32, 32).astype(np.float32)
    amax = np.abs(x).max(axis=2)
    d = (amax / np.float32(127)).astype(np.float32)
    inv = np.where(d != 0, np.float32(1) / np.where(d != 0, d, 1), 0).astype(np.float32)
    q = _round_half_away((x * inv[..., None]).astype(np.float32)).astype(np.int8)
    out = np.empty((rows, k // 32, 34), np.uint8)
    out[..., 0:2] = d.astype(np.float16).view(np.uint8).reshape(rows, k // 32, 2)
    out[..., 2:] = q.view(np.uint8)
    return out.reshape(-1)


def _pack_scales_k4(sc, m):
    """Sixteen 6-bit fields -> the 12 bytes of a Q4_K block (inverse of scaleMinK4,
    /root/reference/format/quant/dequant.go:360-365).  sc, m: [..., 8] uint8 < 64."""
    out = np.zeros(sc.shape[:-1] + (12,), np.uint8)
    for j in range(4):
        out[..., j] = (sc[..., j] & 63) | ((sc[..., j + 4] >> 4) << 6)
        out[..., j + 4] = (m[..., j] & 63) | ((m[..., j + 4] >> 4) << 6)
        out[..., j + 8] = (sc[..., j + 4] & 0xF) | ((m[..., j + 4] & 0xF) << 4)
    return out


def quantize_q4_k(w):
    """Q4_K super-blocks of w [rows][k] (k % 256 == 0), value = d*sc*q - dmin*m."""
    rows, k = w.shape
    nsb = k // 256
    x = w.reshape(rows, nsb, 8, 32).astype(np.float32)
    lo = np.minimum(x.min(axis=3), 0)
    hi = np.maximum(x.max(axis=3), 0)
    scale = (hi - lo) / np.float32(15)
    minv = -lo
    d = (scale.max(axis=2) / np.float32(63)).astype(np.float16)
    dmin = (minv.max(axis=2) / np.float32(63)).astype(np.float16)
    df, dmf = d.astype(np.float32), dmin.astype(np.float32)
    sc = np.where(df[..., None] > 0, _round_half_away(scale / np.where(df > 0, df, 1)[..., None]), 0)
    m = np.where(dmf[..., None] > 0, _round_half_away(minv / np.where(dmf > 0, dmf, 1)[..., None]), 0)
    sc = np.clip(sc, 0, 63).astype(np.uint8)
    m = np.clip(m, 0, 63).astype(np.uint8)
    deff = df[..., None] * sc.astype(np.float32)
    meff = dmf[..., None] * m.astype(np.float32)
    q = np.where(deff[..., None] > 0,
                 _round_half_away((x + meff[..., None]) / np.where(deff > 0, deff, 1)[..., None]), 0)
    q = np.clip(q, 0, 15).astype(np.uint8)
    out = np.empty((rows, nsb, 144), np.uint8)
    out[..., 0:2] = d.view(np.uint8).reshape(rows, nsb, 2)
    out[..., 2:4] = dmin.view(np.uint8).reshape(rows, nsb, 2)
    out[..., 4:16] = _pack_scales_k4(sc, m)
    # group g of 64: low nibbles = sub-block 2g, high nibbles = sub-block 2g+1
    qg = q.reshape(rows, nsb, 4, 2, 32)
    out[..., 16:] = (qg[:, :, :, 0, :] | (qg[:, :, :, 1, :] << 4)).reshape(rows, nsb, 128)
    return out.reshape(-1)


def quantize_q6_k(w):
    """Q6_K super-blocks of w [rows][k]: value = d*sc*(q-32), sc int8 per 16, q 0..63."""
    rows, k = w.shape
    nsb = k // 256
    x = w.reshape(rows, nsb, 16, 16).astype(np.float32)
    idx = np.abs(x).argmax(axis=3)
    mx = np.take_along_axis(x, idx[..., None], axis=3)[..., 0]  # signed extreme of each 16
    scale = mx / np.float32(-32)
    d = (np.abs(scale).max(axis=2) / np.float32(127)).astype(np.float16)
    df = d.astype(np.float32)
    sc = np.where(df[..., None] > 0, _round_half_away(scale / np.where(df > 0, df, 1)[..., None]), 0)
    sc = np.clip(sc, -128, 127).astype(np.int8)
    seff = df[..., None] * sc.astype(np.float32)
    q = np.where(seff[..., None] != 0,
                 _round_half_away(x / np.where(seff != 0, seff, 1)[..., None]), 0)
    q = (np.clip(q, -32, 31) + 32).astype(np.uint8).reshape(rows, nsb, 256)
    out = np.zeros((rows, nsb, 210), np.uint8)
    # element e of half n (128 each): l = e % 32, quarter j = e // 32
    for n in range(2):
        h = q[..., n * 128:(n + 1) * 128].reshape(rows, nsb, 4, 32)
        ql = out[..., n * 64:(n + 1) * 64]
        qh = out[..., 128 + n * 32:128 + (n + 1) * 32]
        ql[..., 0:32] = (h[..., 0, :] & 0xF) | ((h[..., 2, :] & 0xF) << 4)
        ql[..., 32:64] = (h[..., 1, :] & 0xF) | ((h[..., 3, :] & 0xF) << 4)
        qh[...] = ((h[..., 0, :] >> 4) | ((h[..., 1, :] >> 4) << 2) | ((h[..., 2, :] >> 4) << 4)
                   | ((h[..., 3, :] >> 4) << 6))
    out[..., 192:208] = sc.view(np.uint8)
    out[..., 208:210] = d.view(np.uint8).reshape(rows, nsb, 2)
    return out.reshape(-1)


def quantize_mxfp4(w):
    """MXFP4 blocks of w [rows][k]: E8M0 exponent e = floor(log2(amax)) - 2 + 127 so
    the largest element lands within the e2m1 range, then the nearest code;
    value = doubled_e2m1[code] * 2^(e-128)."""
    rows, k = w.shape
    x = w.reshape(rows, k // 32, 32).astype(np.float32)
    amax = np.abs(x).max(axis=2)
    e = np.where(amax > 0, np.floor(np.log2(np.where(amax > 0, amax, 1))) - 2 + 127, 0)
    e = np.clip(e, 0, 254).astype(np.int32)
    d = np.ldexp(np.float32(1), e - 128).astype(np.float32)
    t = np.abs(x) / d[..., None]
    code = np.abs(t[..., None] - _MX_VALUES).argmin(axis=-1).astype(np.uint8)
    code = np.where((x < 0) & (code != 0), code | 8, code).astype(np.uint8)
    out = np.empty((rows, k // 32, 17), np.uint8)
    out[..., 0] = e.astype(np.uint8)
    out[..., 1:] = code[..., :16] | (code[..., 16:] << 4)
    return out.reshape(-1)


QUANTIZERS = {quant.Q8_0: quantize_q8_0, quant.Q4_K: quantize_q4_k,
              quant.Q6_K: quantize_q6_k, quant.MXFP4: quantize_mxfp4}


def quantized_weights(t, rows, k, seed=0, sigma=0.02, chunk=2048):
    """GGUF row-major bytes of a [rows][k] N(0, sigma) matrix quantized to type t.

    Generated chunk rows at a time so a large matrix never holds more than a
    slice in f32; the stream of random numbers is the same for any chunk."""
    rng = np.random.default_rng(seed)
    rb = quant.row_bytes(t, k)
    out = np.empty(rows * rb, np.uint8)
    for r0 in range(0, rows, chunk):
        n = min(chunk, rows - r0)
        w = rng.standard_normal((n, k), np.float32) * np.float32(sigma)
        out[r0 * rb:(r0 + n) * rb] = QUANTIZERS[t](w)
    return out


def plant_scales(t, src, seed=0):
    """Overwrites every block's scale fields with finite values from a sweep that
    reaches the extremes (subnormal, smallest normal, largest finite f16; a spread
    of E8M0 exponents), so random bytes are valid weights
    (/root/reference/format/quant/types.go:145-216)."""
    src = np.asarray(src, np.uint8)
    bb = quant.block_bytes(t)
    nblk = src.size // bb
    blocks = src[:nblk * bb].reshape(nblk, bb)
    i = np.arange(nblk)
    if t == quant.MXFP4:
        blocks[:, 0] = _E8M0_SWEEP[(i + seed) % len(_E8M0_SWEEP)]
        return src
    offs = _SCALE_OFFS[t]
    for oi, o in enumerate(offs):
        h = _F16_SWEEP[(i * len(offs) + oi + seed) % len(_F16_SWEEP)]
        blocks[:, o] = h & 0xFF
        blocks[:, o + 1] = h >> 8
    return src


def random_weights(t, rows, k, seed=0):
    """Random bytes with planted scales: the reference's own recipe for kernel tests
    (/root/reference/engine/nn/packed_test.go:72-85)."""
    rng = np.random.default_rng(seed)
    src = rng.integers(0, 256, rows * quant.row_bytes(t, k), dtype=np.uint8)
    return plant_scales(t, src, seed)
