"""GPU parity of the MXFP4 x bf16 matmul against the reference's dequantize + f32 matmul,
through the C ABI.  Dequantized MXFP4 weights and bf16 activations are exact operands
of the bf16 matrix cores, so the only difference from an f64 evaluation of
Dequant32(W) . x is f32 summation order: the bar is rel-L2 <= 1e-3 as stated, and the
test also holds NMSE <= 1e-10."""
import numpy as np
import pytest

import oracle
from conftest import nmse, rel_l2
from jitllm_amd import quant, synth

pytestmark = pytest.mark.gpu


def to_bf16(x):
    """Round f32 to bf16 (nearest even); returns the uint16 bit patterns and the f32 values."""
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r, (r.astype(np.uint32) << 16).view(np.float32)


@pytest.mark.parametrize("shape", [(1, 2880, 2880), (3, 100, 512), (8, 130, 96), (64, 2880, 2880),
                                   (130, 200, 224), (1024, 2880, 2880), (9, 129, 2880), (17, 33, 160),
                                   (48, 16, 2880), (33, 300, 64), (1, 100, 512), (1, 131, 4192), (1, 37, 8192)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("weights", ["normal", "planted"])
@pytest.mark.parametrize("rows", [0, 96, 128], ids=["auto", "tile96", "tile128"])
def test_mxfp4_bf16_matmul_vs_dequant_f32(dev, devbuf, shape, weights, rows):
    """rows = rows per workgroup tile of the tiled GEMM (the library picks per shape; both are
    held to the bar); auto also takes 9..64 tokens to the few-token kernel (16-row
    workgroups, K split over wavefronts; a last group of fewer than four blocks and ragged
    rows are among the shapes) and one token to the kernel that keeps the activation in
    registers (one, two and three blocks a lane; k = 8192 is past it and runs the general one)."""
    ntok, nrows, k = shape
    dev.set_tuning(mxfp4__rows=rows)
    if weights == "planted" and ntok * nrows * k > 3e8:
        pytest.skip("the full-size case runs once, on quantized N(0, 0.02) weights")
    t = quant.MXFP4
    w = (synth.quantized_weights(t, nrows, k, seed=ntok) if weights == "normal"
         else synth.random_weights(t, nrows, k, seed=ntok))
    xb, xf = to_bf16(np.stack([synth.activations(k, seed=7 + i) for i in range(ntok)]))
    wd = oracle.dequant(t, w, nrows * k).reshape(nrows, k).astype(np.float64)
    want = xf.astype(np.float64) @ wd.T
    dw, dx = devbuf(w), devbuf(xb)
    out = devbuf(shape=(ntok * nrows + 8,), dtype=np.float32, fill=np.float32(2e30))
    for call in range(2):
        assert dev.matmul_mxfp4_bf16_dev(out.ptr, dw.ptr, dx.ptr, nrows, k, ntok)
        dev.synchronize()
        got = out.get()
        assert np.all(got[ntok * nrows:] == np.float32(2e30))
        got = got[:ntok * nrows].reshape(ntok, nrows)
        assert nmse(got, want) <= 1e-10, f"call {call}: NMSE {nmse(got, want):.3e}"
        assert rel_l2(got, want) <= 1e-3
    dev.set_tuning(mxfp4__rows=0)


def test_mxfp4_declines_what_it_cannot_serve(dev, devbuf):
    w = devbuf(synth.random_weights(quant.MXFP4, 4, 64, seed=1))
    x = devbuf(np.zeros(64, np.uint16))
    out = devbuf(shape=(4,), dtype=np.float32)
    assert dev.matmul_mxfp4_bf16_dev(out.ptr, w.ptr, x.ptr, 4, 48, 1) is False   # k not whole blocks


def test_mxfp4_k_split_forms_agree(dev, devbuf):
    """A small grid is widened along K (partial sums per split, added in order); every
    split count gives the same matrix up to f32 summation order."""
    ntok, nrows, k = 40, 300, 1504   # 1504 = 11.75 K stages: a short last stage
    t = quant.MXFP4
    w = synth.quantized_weights(t, nrows, k, seed=3)
    xb, xf = to_bf16(np.stack([synth.activations(k, seed=70 + i) for i in range(ntok)]))
    want = xf.astype(np.float64) @ oracle.dequant(t, w, nrows * k).reshape(nrows, k).astype(np.float64).T
    dw, dx = devbuf(w), devbuf(xb)
    for split in (1, 2, 3, 5, 8, 0):
        dev.set_tuning(mxfp4__split=split)
        out = devbuf(shape=(ntok, nrows), dtype=np.float32, fill=np.float32(-5e30))
        assert dev.matmul_mxfp4_bf16_dev(out.ptr, dw.ptr, dx.ptr, nrows, k, ntok)
        dev.synchronize()
        assert nmse(out.get(), want) <= 1e-10, f"split {split}"
    dev.set_tuning(mxfp4__split=0)


# ------------------------------------------------------------------ packed planes
def _exponent_spread(w, seed):
    """Give the blocks of GGUF MXFP4 bytes exponents from the whole storable range (2..254
    keeps every block packable; the matmul tests keep them near 127 so sums stay finite)."""
    w = w.copy()
    rng = np.random.default_rng(seed)
    w[0::17] = rng.integers(2, 255, w[0::17].size, dtype=np.uint8)
    return w


@pytest.mark.parametrize("shape", [(1, 32), (3, 64), (4, 96), (5, 2880), (130, 224), (257, 512), (2880, 2880)],
                         ids=lambda s: "x".join(map(str, s)))
def test_mxfp4_device_pack_is_the_reference_packer_byte_for_byte(dev, devbuf, shape):
    """/root/reference/jit/gpu/kernels/pack.go:52-199 with e8m0Store (:395) and DSlots 4 (:543-575):
    the device planes equal the CPU restatement's, ragged row counts (a last D word of one to
    three rows) and every storable exponent included, and unpacking gives the GGUF bytes back."""
    nrows, k = shape
    t = quant.MXFP4
    w = _exponent_spread(synth.random_weights(t, nrows, k, seed=nrows + k), seed=k)
    want_qs, want_d, _ = oracle.pack_weights(t, w, nrows, k)
    nq, nd, nsc = dev.packed_words(t, nrows, k)
    assert (nq, nd, nsc) == (want_qs.size, want_d.size, 0) == oracle.packed_words(t, nrows, k)
    dw = devbuf(w)
    qs = devbuf(shape=(nq + 4,), dtype=np.uint32, fill=np.uint32(0xA5A5A5A5))
    d = devbuf(shape=(nd + 4,), dtype=np.uint32, fill=np.uint32(0xA5A5A5A5))
    assert dev.pack_weights_dev(t, dw.ptr, nrows, k, qs.ptr, d.ptr, None)
    got_qs, got_d = qs.get(), d.get()
    assert np.array_equal(got_qs[:nq], want_qs) and np.all(got_qs[nq:] == 0xA5A5A5A5)
    assert np.array_equal(got_d[:nd], want_d) and np.all(got_d[nd:] == 0xA5A5A5A5)
    # back to GGUF blocks, whole and as a row range
    from jitllm_amd.device import Packed
    back = devbuf(shape=(w.size + 17,), dtype=np.uint8, fill=np.uint8(0xEE))
    assert dev.unpack_weights_dev(t, Packed(qs.ptr, d.ptr, None, 0, nrows), nrows, k, back.ptr)
    got = back.get()
    assert np.array_equal(got[:w.size], w) and np.all(got[w.size:] == 0xEE)
    if nrows >= 5:
        r0, n = nrows // 3 + 1, nrows - nrows // 3 - 2
        rb = k // 32 * 17
        assert dev.unpack_weights_dev(t, Packed(qs.ptr, d.ptr, None, r0, nrows), n, k, back.ptr)
        assert np.array_equal(back.get()[:n * rb], w[r0 * rb:(r0 + n) * rb])


def test_mxfp4_device_pack_refuses_what_the_reference_refuses(dev, devbuf):
    """/root/reference/jit/gpu/kernels/pack.go:407-420, /root/reference/internal/oracle/packed_test.go:220-247:
    exponents 0, 1 and 255 pass only on a block of +-0 codes; the device and the CPU restatement
    agree case by case."""
    t = quant.MXFP4
    nrows, k = 3, 1024
    base = np.zeros(17 * 32 * nrows, np.uint8)
    base[0::17] = 127
    base[1::17] = 0x21
    nq, nd, _ = dev.packed_words(t, nrows, k)
    qs, d = devbuf(shape=(nq,), dtype=np.uint32), devbuf(shape=(nd,), dtype=np.uint32)

    def both(w):
        try:
            oracle.pack_weights(t, w, nrows, k)
            want = True
        except ValueError:
            want = False
        got = dev.pack_weights_dev(t, devbuf(w).ptr, nrows, k, qs.ptr, d.ptr, None)
        assert got is want
        return got

    assert both(base)
    for e in (0, 1, 255):
        for blk in (3, 32 + 7, 17 * 32 * nrows // 17 - 1):     # first row, second row, last block
            bad = base.copy()
            bad[17 * blk] = e
            assert not both(bad)                   # the block still holds 0x21 codes
            bad[17 * blk + 1:17 * blk + 17] = 0
            assert both(bad)                       # all-zero codes pass at any exponent
            bad[17 * blk + 5] = 0x88
            assert both(bad)                       # -0 codes are still zero
            bad[17 * blk + 16] = 0x10
            assert not both(bad)
    assert both(base)                              # a refusal leaves nothing behind


@pytest.mark.parametrize("shape", [(1, 2880, 2880), (1, 5760, 2880), (2, 100, 512), (8, 130, 96), (5, 64, 32),
                                   (7, 257, 544), (64, 2880, 2880), (9, 129, 160), (130, 200, 224), (1024, 2880, 2880),
                                   (300, 70, 96)],
                         ids=lambda s: "x".join(map(str, s)))
def test_mxfp4_packed_matmul_vs_dequant_f32(dev, devbuf, shape):
    """Planes written by the device packer, read by the plane kernel (up to 8 tokens) or restored
    and fed to the matrix-core forms: the same bar as the GGUF-row path, and for more than 8
    tokens the same bits, since the restored rows are the GGUF rows."""
    from jitllm_amd.device import Packed
    ntok, nrows, k = shape
    t = quant.MXFP4
    w = synth.quantized_weights(t, nrows, k, seed=ntok + 11)
    xb, xf = to_bf16(np.stack([synth.activations(k, seed=40 + i) for i in range(ntok)]))
    want = xf.astype(np.float64) @ oracle.dequant(t, w, nrows * k).reshape(nrows, k).astype(np.float64).T
    nq, nd, _ = dev.packed_words(t, nrows, k)
    dw, dx = devbuf(w), devbuf(xb)
    qs, d = devbuf(shape=(nq,), dtype=np.uint32), devbuf(shape=(nd,), dtype=np.uint32)
    assert dev.pack_weights_dev(t, dw.ptr, nrows, k, qs.ptr, d.ptr, None)
    out = devbuf(shape=(ntok * nrows + 8,), dtype=np.float32, fill=np.float32(2e30))
    # mxfp4.planes: up to 8 tokens 64 / 32 / 16 = rows a workgroup of the plane matvec; more tokens
    # 3 = the plane GEMM whatever the grid; 2 = restore rows first (the GGUF path's bits)
    forms = (0, 64, 32, 16, 2) if ntok <= 8 else (0, 3, 2)
    got_by_form = {}
    for form in forms:
        dev.set_tuning(mxfp4__planes=form)
        out.put(np.full(ntok * nrows + 8, np.float32(2e30)))
        n0 = dev.launch_count()
        assert dev.matmul_mxfp4_packed_bf16_dev(out.ptr, Packed(qs.ptr, d.ptr, None, 0, nrows), dx.ptr, nrows, k, ntok)
        dev.synchronize()
        if ntok <= 8 and form != 2:
            assert dev.launch_count() - n0 == 1
        if form == 3:
            assert dev.launch_count() - n0 == 2      # prep + the plane GEMM, nothing restored
        got = out.get()
        assert np.all(got[ntok * nrows:] == np.float32(2e30))
        got = got[:ntok * nrows].reshape(ntok, nrows)
        assert nmse(got, want) <= 1e-10 and rel_l2(got, want) <= 1e-3, f"form {form}: NMSE {nmse(got, want):.3e}"
        got_by_form[form] = got
    dev.set_tuning(mxfp4__planes=0)
    if ntok > 8:
        ref = devbuf(shape=(ntok, nrows), dtype=np.float32)
        assert dev.matmul_mxfp4_bf16_dev(ref.ptr, dw.ptr, dx.ptr, nrows, k, ntok)
        dev.synchronize()
        assert np.array_equal(ref.get(), got_by_form[2])
    # a row range of the planes: rows r0 .. r0+n of the same buffer
    if nrows >= 100:
        r0, n = 37, nrows - 70
        out.put(np.full(ntok * nrows + 8, np.float32(2e30)))
        assert dev.matmul_mxfp4_packed_bf16_dev(out.ptr, Packed(qs.ptr, d.ptr, None, r0, nrows), dx.ptr, n, k, ntok)
        dev.synchronize()
        got = out.get()
        assert np.all(got[ntok * n:] == np.float32(2e30))
        assert nmse(got[:ntok * n].reshape(ntok, n), want[:, r0:r0 + n]) <= 1e-10


def test_mxfp4_packed_matmul_every_exponent_one_token(dev, devbuf):
    """The plane reader's scale is the stored byte plus one as an f32 exponent: blocks at both ends
    of the storable range (2 and 254) against the f64 evaluation of the dequantized rows."""
    from jitllm_amd.device import Packed
    t = quant.MXFP4
    nrows, k = 67, 64
    w = synth.random_weights(t, nrows, k, seed=5)
    w[0::17] = np.resize(np.array([2, 3, 64, 127, 128, 200], np.uint8), w[0::17].size)
    x = np.zeros(k, np.float32)
    x[::3] = 1.0
    x[1::3] = -0.5
    xb, xf = to_bf16(x[None, :])
    wd = oracle.dequant(t, w, nrows * k).reshape(nrows, k).astype(np.float64)
    want = (xf.astype(np.float64) @ wd.T).astype(np.float32)
    nq, nd, _ = dev.packed_words(t, nrows, k)
    qs, d = devbuf(shape=(nq,), dtype=np.uint32), devbuf(shape=(nd,), dtype=np.uint32)
    assert dev.pack_weights_dev(t, devbuf(w).ptr, nrows, k, qs.ptr, d.ptr, None)
    out = devbuf(shape=(nrows,), dtype=np.float32)
    assert dev.matmul_mxfp4_packed_bf16_dev(out.ptr, Packed(qs.ptr, d.ptr, None, 0, nrows), devbuf(xb).ptr, nrows, k, 1)
    dev.synchronize()
    got = out.get()
    assert np.all(np.isfinite(want)) and np.allclose(got, want, rtol=2e-6, atol=0)


# ------------------------------------------------------------------ block-scaled form (opt-in)
def mx_fp8_activations(xf):
    """The opt-in form's activation quantizer restated in numpy: per token and block of 32 a
    power-of-two scale that puts the block's largest magnitude in [224, 448], values rounded to
    fp8 e4m3 (three mantissa bits, subnormals below 2^-6), nearest even.  Returns the values
    the matrix instruction multiplies, as f64."""
    x = xf.astype(np.float64).reshape(xf.shape[0], -1, 32)
    amax = np.abs(x).max(axis=2, keepdims=True)
    m, ex = np.frexp(amax)                       # amax = m * 2^ex, m in [0.5, 1)
    e = ex - 1 - 8 + (2 * m > 1.75)              # floor(log2 amax) - 8, one more above 1.75 * 2^floor
    scale = np.where(amax > 0, np.exp2(e.astype(np.float64)), 1.0)
    v = x / scale
    _, vex = np.frexp(np.abs(v))
    step = np.exp2(np.maximum(vex - 1, -6) - 3.0)
    q = np.round(v / step) * step                # numpy rounds halves to even
    assert np.abs(q).max() <= 448
    return (q * scale).reshape(xf.shape)


@pytest.mark.parametrize("shape", [(1, 64, 64), (40, 130, 96), (128, 128, 2880), (130, 300, 160), (1024, 2880, 2880)],
                         ids=lambda s: "x".join(map(str, s)))
def test_mxfp4_scaled_form_is_exact_over_its_own_quantizer_and_reports_its_loss(dev, devbuf, shape):
    """`mxfp4.scaled` = 1 (never the default): the planes' e2m1 codes and E8M0 exponents go into
    v_mfma_scale_f32_32x32x64_f8f6f4 as they are, the activations as MX fp8.  Against the f64
    product of the dequantized weights with the SAME fp8 activations the result differs by the
    instruction's own accumulation (it sums a block's 32 products in less than f32: measured
    NMSE ~1e-10, bar 1e-8, which still pins the operand layout and the scale bytes: one
    misplaced element or exponent gives 1e-3 or more);
    against the bf16 activations the loss is the quantizer's, a few percent rel-L2, stated here
    and in the benchmark beside the form's time."""
    from jitllm_amd.device import Packed
    ntok, nrows, k = shape
    t = quant.MXFP4
    w = synth.quantized_weights(t, nrows, k, seed=ntok + 3)
    xb, xf = to_bf16(np.stack([synth.activations(k, seed=90 + i) for i in range(ntok)]))
    wd = oracle.dequant(t, w, nrows * k).reshape(nrows, k).astype(np.float64)
    want_q = mx_fp8_activations(xf) @ wd.T
    want = xf.astype(np.float64) @ wd.T
    nq, nd, _ = dev.packed_words(t, nrows, k)
    qs, d = devbuf(shape=(nq,), dtype=np.uint32), devbuf(shape=(nd,), dtype=np.uint32)
    assert dev.pack_weights_dev(t, devbuf(w).ptr, nrows, k, qs.ptr, d.ptr, None)
    out = devbuf(shape=(ntok * nrows + 8,), dtype=np.float32, fill=np.float32(2e30))
    dev.set_tuning(mxfp4__scaled=1)
    try:
        assert dev.matmul_mxfp4_packed_bf16_dev(out.ptr, Packed(qs.ptr, d.ptr, None, 0, nrows), devbuf(xb).ptr, nrows, k, ntok)
        dev.synchronize()
    finally:
        dev.set_tuning(mxfp4__scaled=0)
    got = out.get()
    assert np.all(got[ntok * nrows:] == np.float32(2e30))
    got = got[:ntok * nrows].reshape(ntok, nrows)
    assert nmse(got, want_q) <= 1e-8, f"NMSE {nmse(got, want_q):.3e} against its own quantizer"
    loss = rel_l2(got, want)
    print(f"block-scaled form {shape}: rel-L2 {loss:.3e} against bf16 activations")
    assert 1e-3 < loss <= 5e-2


@pytest.mark.parametrize("tuning", [{}, {"mxfp4__planes": 2}, {"mxfp4__scaled": 1}], ids=["auto", "restore", "scaled"])
def test_mxfp4_packed_reserve_shape_leaves_nothing_to_allocate(dev, devbuf, tuning):
    """jl_reserve_shape walks the packed MXFP4 call's own launch path (fragments of the plane GEMM,
    restored rows, the block-scaled form's fp8 fragments): afterwards the call itself allocates
    nothing, for shapes that grow on the one before."""
    from jitllm_amd.device import Packed
    from jitllm_amd.hipmem import mem_info
    t = quant.MXFP4
    dev.set_tuning(**tuning)
    try:
        for ntok, nrows, k in [(200, 640, 1024), (520, 1100, 2048), (48, 300, 4096)]:
            w = synth.quantized_weights(t, nrows, k, seed=ntok)
            xb, xf = to_bf16(np.stack([synth.activations(k, seed=3 + i) for i in range(ntok)]))
            nq, nd, _ = dev.packed_words(t, nrows, k)
            qs, d = devbuf(shape=(nq,), dtype=np.uint32), devbuf(shape=(nd,), dtype=np.uint32)
            assert dev.pack_weights_dev(t, devbuf(w).ptr, nrows, k, qs.ptr, d.ptr, None)
            dx = devbuf(xb)
            out = devbuf(shape=(ntok, nrows), dtype=np.float32)
            assert dev.reserve_shape(t, nrows, k, ntok, packed=True)
            dev.synchronize()
            free_before, _ = mem_info()
            assert dev.matmul_mxfp4_packed_bf16_dev(out.ptr, Packed(qs.ptr, d.ptr, None, 0, nrows), dx.ptr, nrows, k, ntok)
            dev.synchronize()
            assert mem_info()[0] == free_before, f"{ntok} x {k} -> {nrows}: the call allocated"
            want = xf.astype(np.float64) @ oracle.dequant(t, w, nrows * k).reshape(nrows, k).astype(np.float64).T
            assert rel_l2(out.get(), want) <= (5e-2 if tuning.get("mxfp4__scaled") else 1e-3)
    finally:
        dev.set_tuning(**{k_: 0 for k_ in tuning})
