"""GPU parity of the packed-plane path (the reference's device weight layout) against
the CPU oracle, through the C ABI.

Bars:
  * device pack (kernels.PackWeightsInto, /root/reference/jit/gpu/kernels/pack.go:52-199):
    byte for byte the oracle's planes, which the reference-written v29 container pins
    for Q4_K; the inverse permutation restores the GGUF bytes exactly
  * matvec / matmul over planes vs the f64 evaluation of the same int8 activations:
    NMSE <= 1e-10 (/root/reference/engine/nn/packed_test.go:140-147), rel-L2 <= 1e-3
  * planes of the reference-written container (tests/golden/v29.jlm.gz) fed straight to
    the kernel, expert sheets included
"""
import gzip
import os

import numpy as np
import pytest

import oracle
from conftest import GOLDEN, nmse, rel_l2
from jitllm_amd import jlm, quant, synth
from jitllm_amd.device import Packed

pytestmark = pytest.mark.gpu

TYPES = [quant.Q4_K, quant.Q8_0, quant.Q6_K]


def _window(t):
    return 256 if t in quant.K_QUANTS else 32


def _like_for_like(t, w, x, nrows, k, window):
    q, a_s, _ = oracle.quantize_act(x, window)
    return oracle.matvec_q8act_f64(t, w, q, a_s, nrows, k)


def _dev_planes(devbuf, qs, d, sc, row=0, stride=None):
    qd, dd = devbuf(qs), devbuf(d)
    sd = devbuf(sc) if sc is not None and sc.size else None
    p = Packed(qd.ptr, dd.ptr, sd.ptr if sd else None, row, stride)
    p.keep = (qd, dd, sd)
    return p


@pytest.mark.parametrize("t", TYPES)
@pytest.mark.parametrize("shape", [(1, 256), (9, 512), (300, 512), (257, 1024), (64, 4096)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_pack_on_device_is_byte_exact(dev, devbuf, t, shape):
    nrows, k = shape
    src = synth.random_weights(t, nrows, k, seed=nrows * 7 + k)
    wq, wd, wsc = oracle.pack_weights(t, src, nrows, k)
    assert dev.packed_words(t, nrows, k) == (wq.size, wd.size, wsc.size)
    sd = devbuf(src)
    qs = devbuf(shape=(wq.size,), dtype=np.uint32, fill=0xDEADBEEF)
    d = devbuf(shape=(wd.size,), dtype=np.uint32, fill=0xDEADBEEF)
    sc = devbuf(shape=(max(wsc.size, 1),), dtype=np.uint32, fill=0xDEADBEEF)
    assert dev.pack_weights_dev(t, sd.ptr, nrows, k, qs.ptr, d.ptr, sc.ptr if wsc.size else None)
    dev.synchronize()
    assert np.array_equal(qs.get(), wq)
    assert np.array_equal(d.get(), wd)
    if wsc.size:
        assert np.array_equal(sc.get(), wsc)
    if t in (quant.Q4_K, quant.Q6_K, quant.Q8_0):
        back = devbuf(shape=(src.size + 4,), dtype=np.uint8, fill=0x5A)
        assert dev.unpack_weights_dev(t, Packed(qs.ptr, d.ptr, sc.ptr if wsc.size else None, 0, nrows), nrows, k, back.ptr)
        dev.synchronize()
        assert np.array_equal(back.get()[:src.size], src)
        assert np.all(back.get()[src.size:] == 0x5A), "wrote past the rows"
        if nrows > 4:     # a row range inside the planes
            lo, n = nrows // 3, nrows // 2
            rb = quant.row_bytes(t, k)
            part = devbuf(shape=(n * rb,), dtype=np.uint8, fill=0x5A)
            assert dev.unpack_weights_dev(t, Packed(qs.ptr, d.ptr, sc.ptr if wsc.size else None, lo, nrows), n, k, part.ptr)
            dev.synchronize()
            assert np.array_equal(part.get(), src[lo * rb:(lo + n) * rb])


def test_packed_words_closed_form(dev):
    """kernels.PackedWords (/root/reference/jit/gpu/kernels/pack.go:580-621) against the oracle's."""
    for t in TYPES:
        for nrows, k in [(1, 256), (7, 512), (300, 4096), (4096, 14336)]:
            assert dev.packed_words(t, nrows, k) == tuple(oracle.packed_words(t, nrows, k))
    assert dev.packed_words(quant.Q4_K, 8, 288) is None
    assert dev.packed_words(quant.Q8_0, 8, 288) is not None


SHAPES = [(1, 256), (9, 512), (300, 512), (37, 1024), (64, 2048), (1000, 4096), (129, 14336), (4096, 768)]


@pytest.mark.parametrize("t", TYPES)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("weights", ["normal", "planted"])
def test_matvec_packed_vs_oracle(dev, devbuf, t, shape, weights):
    nrows, k = shape
    window = _window(t)
    dev.SetActWindow(window)
    if weights == "normal":
        w = synth.quantized_weights(t, nrows, k, seed=nrows + k)
    else:
        w = synth.random_weights(t, nrows, k, seed=nrows)
    x = synth.activations(k, seed=k)
    want = _like_for_like(t, w, x, nrows, k, window)
    p = _dev_planes(devbuf, *oracle.pack_weights(t, w, nrows, k), stride=nrows)
    xd = devbuf(x)
    for rw in (0, 16, 32, 64):
        dev.set_tuning(packed__rw=rw)
        out = devbuf(shape=(nrows + 8,), dtype=np.float32, fill=np.float32(7e30))
        assert dev.matvec_packed_dev(out.ptr, t, p, xd.ptr, nrows, k)
        dev.synchronize()
        got = out.get()
        assert np.all(got[nrows:] == np.float32(7e30)), "wrote past nrows"
        e = nmse(got[:nrows], want)
        assert e <= 1e-10, f"rw={rw}: NMSE {e:.3e} vs like-for-like f64"
        assert rel_l2(got[:nrows], want) <= 1e-3
    dev.set_tuning(packed__rw=0)
    if weights == "normal" and nrows >= 64:
        ref32 = oracle.matvec_packed_rows(t, *oracle.pack_weights(t, w, nrows, k), x, nrows, k)
        assert nmse(got[:nrows], ref32) <= 1e-3, "vs the f32-activation plane reader"
    dev.SetActWindow(32)


@pytest.mark.parametrize("t", TYPES)
def test_matvec_packed_window_32_and_block_shapes(dev, devbuf, t):
    """The 32 window (one scale per block) and every workgroup size give the same rows."""
    nrows, k = 203, 2304 if t == quant.Q8_0 else 2048
    if t == quant.Q8_0:
        k = 2304 + 32   # not a whole 256-element chunk: the last chunk is short
    dev.SetActWindow(32)
    w = synth.random_weights(t, nrows, k, seed=11)
    x = synth.activations(k, seed=12)
    want = _like_for_like(t, w, x, nrows, k, 32)
    p = _dev_planes(devbuf, *oracle.pack_weights(t, w, nrows, k), stride=nrows)
    xd = devbuf(x)
    for block in (64, 192, 512, 1024):
        for rw in (16, 32, 64):
            dev.set_tuning(packed__rw=rw, packed__block=block)
            out = devbuf(shape=(nrows,), dtype=np.float32, fill=np.float32(-3e33))
            assert dev.matvec_packed_dev(out.ptr, t, p, xd.ptr, nrows, k)
            dev.synchronize()
            e = nmse(out.get(), want)
            assert e <= 1e-10, f"block={block} rw={rw}: {e:.3e}"
    dev.set_tuning(packed__rw=0, packed__block=0)


@pytest.mark.parametrize("t", TYPES)
def test_matvec_packed_row_range_of_a_larger_buffer(dev, devbuf, t):
    """nn.Packed.Row / Stride: a matrix that is rows 40..140 of planes holding 203 rows."""
    stride, k, row, nrows = 203, 1024, 41, 100
    window = _window(t)
    dev.SetActWindow(window)
    w = synth.random_weights(t, stride, k, seed=21)
    x = synth.activations(k, seed=22)
    want = _like_for_like(t, w, x, stride, k, window)[row:row + nrows]
    p = _dev_planes(devbuf, *oracle.pack_weights(t, w, stride, k), row=row, stride=stride)
    xd = devbuf(x)
    out = devbuf(shape=(nrows,), dtype=np.float32, fill=np.float32(5e30))
    assert dev.matvec_packed_dev(out.ptr, t, p, xd.ptr, nrows, k)
    dev.synchronize()
    assert nmse(out.get(), want) <= 1e-10
    # rows outside the buffer are a contract violation, not a decline
    from jitllm_amd.device import DeviceError
    with pytest.raises(DeviceError):
        dev.matvec_packed_dev(out.ptr, t, Packed(p.qs, p.d, p.sc, stride - 10, stride), xd.ptr, nrows, k)
    dev.SetActWindow(32)


@pytest.mark.parametrize("t", TYPES)
@pytest.mark.parametrize("form", ["multi", "gather", "gather_act"])
def test_matvec_packed_multi_over_expert_sheets(dev, devbuf, t, form):
    """MatVecPackedMulti / Gather / GatherAct (/root/reference/engine/nn/packedmulti.go:24,84,93)
    over the sheets of an expert bank packed as ONE set of planes: every matrix has the bank's
    plane pointers and row0 = expert * rows, the addressing of an expert page
    (/root/reference/engine/nn/device.go:70-80).  One launch; each matrix is the packed matvec."""
    n_expert, nrows, k, window = 6, 90, 1024, _window(t)
    experts = [4, 0, 5, 2]
    dev.SetActWindow(window)
    bank = synth.random_weights(t, n_expert * nrows, k, seed=31)
    planes = _dev_planes(devbuf, *oracle.pack_weights(t, bank, n_expert * nrows, k), stride=n_expert * nrows)
    m = len(experts)
    xs = np.stack([synth.activations(k, seed=60 + j) for j in range(m)])
    ups = np.stack([synth.activations(k, seed=80 + j) for j in range(m)])
    if form == "multi":
        xs = np.repeat(xs[:1], m, axis=0)
    xd, ud = devbuf(xs), devbuf(ups)
    outs = [devbuf(shape=(nrows + 2,), dtype=np.float32, fill=np.float32(9e30)) for _ in range(m)]
    rb = quant.row_bytes(t, k)
    for rw in (0, 16, 64):
        dev.set_tuning(packed__rw=rw)
        assert dev.matvec_packed_multi_dev([o.ptr for o in outs], t, [(planes.qs, planes.d, planes.sc)] * m,
                                           [e * nrows for e in experts], n_expert * nrows, xd.ptr,
                                           0 if form == "multi" else k, ud.ptr if form == "gather_act" else None,
                                           nrows, k)
        dev.synchronize()
        for j, e in enumerate(experts):
            w = bank[e * nrows * rb:(e + 1) * nrows * rb]
            got = outs[j].get()
            assert np.all(got[nrows:] == np.float32(9e30))
            if form == "gather_act":
                g = xs[j].astype(np.float64)
                h = (g / (1 + np.exp(-g)) * ups[j].astype(np.float64)).astype(np.float32)
                assert rel_l2(got[:nrows], _like_for_like(t, w, h, nrows, k, window)) <= 1e-3
            else:
                assert nmse(got[:nrows], _like_for_like(t, w, xs[j], nrows, k, window)) <= 1e-10
    # the residual add rides on matrix 0 alone: resid += alpha * out[0], nothing else moves
    dev.set_tuning(packed__rw=0)
    resid0 = synth.activations(nrows + 2, seed=77)
    resid = devbuf(resid0)
    alpha = np.float32(-0.625)
    assert dev.matvec_packed_multi_dev([o.ptr for o in outs], t, [(planes.qs, planes.d, planes.sc)] * m,
                                       [e * nrows for e in experts], n_expert * nrows, xd.ptr,
                                       0 if form == "multi" else k, ud.ptr if form == "gather_act" else None,
                                       nrows, k, resid=resid.ptr, alpha=float(alpha))
    dev.synchronize()
    y0 = outs[0].get()[:nrows]
    want_r = resid0.copy()
    want_r[:nrows] = (resid0[:nrows] + (alpha * y0).astype(np.float32)).astype(np.float32)
    assert np.array_equal(resid.get(), want_r)
    dev.SetActWindow(32)


@pytest.mark.parametrize("t,k,window", [(quant.Q8_0, 1056, 32), (quant.Q4_K, 4096, 256), (quant.Q6_K, 5120, 32)])
def test_matvec_packed_multi_with_rmsnorm_in_front(dev, devbuf, t, k, window):
    """RMSNorm folded into the packed kernels' quantizer (the reference's RMSNormQuantRows,
    /root/reference/jit/gpu/kernels/elem.go:252-267): the normed vector the device writes
    must be the oracle's RMSNorm32 up to the order of the f64 sum (one f32 ulp at most,
    normally none), and every matrix's result the packed matvec of THAT vector.  Together
    with a gated activation the call is declined."""
    dev.SetActWindow(window)
    m, nrows = 3, 150
    ws = [synth.quantized_weights(t, nrows, k, seed=40 + j) for j in range(m)]
    pls = [_dev_planes(devbuf, *oracle.pack_weights(t, w, nrows, k), stride=nrows) for w in ws]
    x = synth.activations(k, seed=5) * np.float32(2.5)
    nw = (1 + 0.1 * np.random.default_rng(3).standard_normal(k)).astype(np.float32)
    eps = 1e-6
    xd, nwd = devbuf(x), devbuf(nw)
    dn = devbuf(shape=(k + 4,), dtype=np.float32, fill=np.float32(-3e30))
    outs = [devbuf(shape=(nrows,), dtype=np.float32, fill=np.float32(9e30)) for _ in range(m)]
    tri = [(p.qs, p.d, p.sc) for p in pls]
    for rw in (0, 16, 64):
        dev.set_tuning(packed__rw=rw)
        assert dev.matvec_packed_multi_dev([o.ptr for o in outs], t, tri, [0] * m, nrows, xd.ptr, 0, None, nrows, k,
                                           norm_w=nwd.ptr, norm_eps=eps, norm_out=dn.ptr)
        dev.synchronize()
        normed = dn.get()
        assert np.all(normed[k:] == np.float32(-3e30))
        normed = normed[:k]
        want_n = oracle.rmsnorm32(x, nw, eps)
        ulp = np.abs(normed.view(np.int32).astype(np.int64) - want_n.view(np.int32).astype(np.int64))
        assert ulp.max() <= 1 and np.mean(ulp != 0) <= 0.01
        for w, o in zip(ws, outs):
            assert nmse(o.get(), _like_for_like(t, w, normed, nrows, k, window)) <= 1e-10
            assert rel_l2(o.get(), _like_for_like(t, w, want_n, nrows, k, window)) <= 1e-3
    dev.set_tuning(packed__rw=0)
    assert dev.matvec_packed_multi_dev([o.ptr for o in outs], t, tri, [0] * m, nrows, xd.ptr, 0, xd.ptr, nrows, k,
                                       norm_w=nwd.ptr, norm_eps=eps) is False
    dev.SetActWindow(32)


@pytest.mark.parametrize("t", TYPES)
def test_matvec_packed_split_equals_fused(dev, devbuf, t):
    """Quantizer kernel + packed matvec over its output == the fused kernel, bit for bit."""
    nrows, k, window = 200, 4096, _window(t)
    dev.SetActWindow(window)
    w = synth.quantized_weights(t, nrows, k, seed=9)
    x = synth.activations(k, seed=10)
    p = _dev_planes(devbuf, *oracle.pack_weights(t, w, nrows, k), stride=nrows)
    xd = devbuf(x)
    q = devbuf(shape=(k,), dtype=np.int8)
    a_s = devbuf(shape=(k // 32,), dtype=np.float32)
    s16 = devbuf(shape=(k // 16,), dtype=np.float32)
    o1 = devbuf(shape=(nrows,), dtype=np.float32, fill=1.0)
    o2 = devbuf(shape=(nrows,), dtype=np.float32, fill=2.0)
    assert dev.quantize_act_dev(xd.ptr, 1, k, q.ptr, a_s.ptr, s16.ptr)
    assert dev.matvec_packed_q8_dev(o1.ptr, t, p, q.ptr, a_s.ptr, s16.ptr, nrows, k)
    assert dev.matvec_packed_dev(o2.ptr, t, p, xd.ptr, nrows, k)
    dev.synchronize()
    assert np.array_equal(o1.get().view(np.uint32), o2.get().view(np.uint32))
    dev.SetActWindow(32)


def _container():
    return jlm.File(gzip.open(os.path.join(GOLDEN, "v29.jlm.gz")).read())


def test_container_planes_fed_to_the_kernel(dev, devbuf):
    """Q4_K planes written by the reference's own converter (format/jlm/testdata/old/v29.jlm.gz),
    expert sheets included, go to the kernel as they lie in the file."""
    f = _container()
    dev.SetActWindow(256)
    seen = 0
    for e in f.entries:
        if jlm.TYPE_TO_QUANT.get(e.type) != quant.Q4_K:
            continue
        for sheet in range(e.sheets):
            _, qs, d, sc = f.planes(e, sheet)
            rows, k = e.rows, e.k
            x = synth.activations(k, seed=100 + seen)
            want = oracle.matvec_packed_rows(quant.Q4_K, qs, d, sc, x, rows, k)
            p = _dev_planes(devbuf, np.ascontiguousarray(qs), np.ascontiguousarray(d),
                            np.ascontiguousarray(sc), stride=rows)
            xd = devbuf(x)
            out = devbuf(shape=(rows,), dtype=np.float32, fill=np.float32(1e30))
            assert dev.matvec_packed_dev(out.ptr, quant.Q4_K, p, xd.ptr, rows, k)
            dev.synchronize()
            # the plane reader multiplies f32 activations; the kernel quantizes them
            assert nmse(out.get(), want) <= 2e-3, e.name
            # like for like: dequantize the planes row by row and evaluate in f64
            q8, a_s, _ = oracle.quantize_act(x, 256)
            deq = np.stack([oracle.row_packed(quant.Q4_K, qs, d, sc, r, rows, k) for r in range(rows)])
            xa = (q8.astype(np.float64).reshape(-1, 32) * a_s.astype(np.float64)[:, None]).reshape(-1)
            assert nmse(out.get(), deq.astype(np.float64) @ xa) <= 1e-10, e.name
            seen += 1
    assert seen >= 3
    dev.SetActWindow(32)


@pytest.mark.parametrize("t", TYPES)
@pytest.mark.parametrize("ntok", [1, 3, 16, 130])
def test_matmul_packed_vs_oracle(dev, devbuf, t, ntok):
    """JIT.MatMulPacked: every token quantized on its own; the GEMM form (Q4_K, 256 window,
    enough tokens) and the per-token form give the like-for-like values."""
    nrows, k = 300, 1024
    window = _window(t)
    dev.SetActWindow(window)
    w = synth.quantized_weights(t, nrows, k, seed=31)
    x = synth.activations(ntok * k, seed=32).reshape(ntok, k)
    want = oracle.matmul_q8act_f64(t, w, x, nrows, k, ntok, window)
    p = _dev_planes(devbuf, *oracle.pack_weights(t, w, nrows, k), stride=nrows)
    xd = devbuf(x)
    out = devbuf(shape=(ntok, nrows), dtype=np.float32, fill=np.float32(3e30))
    assert dev.matmul_packed_dev(out.ptr, t, p, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    got = out.get()
    assert nmse(got, want) <= 1e-10
    assert rel_l2(got, want) <= 1e-3
    dev.SetActWindow(32)


def test_matmul_packed_q6k_planes_window32(dev, devbuf):
    """Q6_K planes in a model whose window is 32 (a Q8_0 tensor beside them): unpacked into rows,
    then the window-32 matrix kernel; a row range of a larger plane set."""
    t, nrows, k, ntok, stride, row0 = quant.Q6_K, 200, 1024, 40, 300, 60
    dev.SetActWindow(32)
    w = synth.random_weights(t, stride, k, seed=5)
    rb = quant.row_bytes(t, k)
    x = synth.activations(ntok * k, seed=6).reshape(ntok, k)
    want = oracle.matmul_q8act_f64(t, w[row0 * rb:(row0 + nrows) * rb], x, nrows, k, ntok, 32)
    p = _dev_planes(devbuf, *oracle.pack_weights(t, w, stride, k), row=row0, stride=stride)
    xd = devbuf(x)
    out = devbuf(shape=(ntok, nrows), dtype=np.float32, fill=np.float32(3e30))
    n0 = dev.launch_count()
    assert dev.matmul_packed_dev(out.ptr, t, p, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    assert dev.launch_count() - n0 <= 5
    assert nmse(out.get(), want) <= 1e-10


def test_packed_host_pointer_seam(dev):
    """JIT.MatVecPacked / MatMulPacked over host planes: residency keyed on the QS pointer."""
    t, nrows, k = quant.Q4_K, 96, 1024
    dev.SetActWindow(256)
    w = synth.quantized_weights(t, nrows, k, seed=1)
    qs, d, sc = oracle.pack_weights(t, w, nrows, k)
    p = Packed(qs, d, sc, 0, nrows)
    x = synth.activations(k, seed=2)
    out = np.full(nrows, np.float32(9e9))
    assert dev.MatVecPacked(out, t, p, x, nrows, k) is True
    assert nmse(out, _like_for_like(t, w, x, nrows, k, 256)) <= 1e-10
    x3 = synth.activations(3 * k, seed=4).reshape(3, k)
    out3 = np.full((3, nrows), np.float32(9e9))
    assert dev.MatMulPacked(out3, t, p, x3, nrows, k, 3) is True
    assert nmse(out3, oracle.matmul_q8act_f64(t, w, x3, nrows, k, 3, 256)) <= 1e-10
    # a sub-range of the same resident planes
    sub = Packed(qs, d, sc, 16, nrows)
    out16 = np.full(32, np.float32(9e9))
    assert dev.MatVecPacked(out16, t, sub, x, 32, k) is True
    assert nmse(out16, _like_for_like(t, w, x, nrows, k, 256)[16:48]) <= 1e-10
    dev.ForgetPacked(p)
    # declines: a type with no planes here, k that is not whole super-blocks
    assert dev.MatVecPacked(out, quant.MXFP4, p, x, nrows, k) is False
    assert dev.MatVecPacked(out, t, p, x, nrows, k - 32) is False
    dev.SetActWindow(32)


@pytest.mark.parametrize("t", TYPES)
def test_grouped_operators_over_host_planes(dev, devbuf, t):
    """JIT.MatVecPackedMulti / Gather / GatherAct over host memory
    (/root/reference/engine/nn/packedmulti.go:24,84,93): a bank's sheets as row ranges of one set of
    planes, twenty matrices (two launches of at most sixteen), against the oracle and, bit for bit,
    against the device-pointer form; what the reference declines is declined."""
    from jitllm_amd import _lib
    n_expert, nrows, k, window = 7, 90, 1024, _window(t)
    experts = [4, 0, 5, 2, 6, 1, 3, 3, 0, 6, 2, 2, 5, 1, 4, 0, 6, 3, 1, 5]
    m = len(experts)
    dev.SetActWindow(window)
    bank = synth.random_weights(t, n_expert * nrows, k, seed=131)
    qs, d, sc = oracle.pack_weights(t, bank, n_expert * nrows, k)
    sc = sc if sc is not None and sc.size else None
    ps = [Packed(qs, d, sc, e * nrows, n_expert * nrows) for e in experts]
    xstride = k + 64
    xs = synth.activations(m * xstride, seed=61).reshape(m, xstride)
    ups = synth.activations(m * xstride, seed=62).reshape(m, xstride)
    rb = quant.row_bytes(t, k)
    sheet = lambda e: bank[e * nrows * rb:(e + 1) * nrows * rb]
    planes_d = _dev_planes(devbuf, qs, d, sc, stride=n_expert * nrows)
    xd, ud = devbuf(xs), devbuf(ups)

    def dev_form(js, xstride_, up):
        outs = [devbuf(shape=(nrows,), dtype=np.float32, fill=np.float32(9e30)) for _ in js]
        assert dev.matvec_packed_multi_dev([o.ptr for o in outs], t, [(planes_d.qs, planes_d.d, planes_d.sc)] * len(js),
                                           [experts[j] * nrows for j in js], n_expert * nrows,
                                           xd.ptr + js[0] * xstride_ * 4, xstride_, (ud.ptr + js[0] * xstride_ * 4) if up else None,
                                           nrows, k)
        dev.synchronize()
        return [o.get() for o in outs]

    x0 = xs[0].copy()
    # Multi: one shared activation
    outs = [np.full(nrows + 3, np.float32(7e30)) for _ in range(m)]
    assert dev.MatVecPackedMulti(outs, t, ps, xs[0], nrows, k) is True
    same = dev_form(list(range(16)), 0, False)
    for j, e in enumerate(experts):
        assert np.all(outs[j][nrows:] == np.float32(7e30)), "wrote past nrows"
        assert nmse(outs[j][:nrows], _like_for_like(t, sheet(e), xs[0][:k], nrows, k, window)) <= 1e-10
        if j < 16:
            assert np.array_equal(outs[j][:nrows].view(np.uint32), same[j].view(np.uint32))
    # Gather: an activation a matrix, at a stride
    outs = [np.full(nrows, np.float32(7e30)) for _ in range(m)]
    assert dev.MatVecPackedGather(outs, t, ps, xs.reshape(-1), xstride, nrows, k) is True
    same = dev_form(list(range(16)), xstride, False) + dev_form(list(range(16, m)), xstride, False)
    for j, e in enumerate(experts):
        assert nmse(outs[j], _like_for_like(t, sheet(e), xs[j][:k], nrows, k, window)) <= 1e-10
        assert np.array_equal(outs[j].view(np.uint32), same[j].view(np.uint32))
    # GatherAct: silu(x_j) * up_j, x left as it was
    keep = xs.copy()
    outs = [np.full(nrows, np.float32(7e30)) for _ in range(m)]
    assert dev.MatVecPackedGatherAct(outs, t, ps, xs.reshape(-1), ups.reshape(-1), _lib.ACT_SILU, xstride, nrows, k) is True
    assert np.array_equal(xs, keep)
    same = dev_form(list(range(16)), xstride, True) + dev_form(list(range(16, m)), xstride, True)
    for j, e in enumerate(experts):
        g = xs[j][:k].astype(np.float64)
        h = (g / (1 + np.exp(-g)) * ups[j][:k].astype(np.float64)).astype(np.float32)
        assert rel_l2(outs[j], _like_for_like(t, sheet(e), h, nrows, k, window)) <= 1e-3
        assert np.array_equal(outs[j].view(np.uint32), same[j].view(np.uint32))
    # one allocation for the bank: every matrix has the same QS pointer
    assert dev.resident_count() >= 1
    # declines, as the reference's: one matrix, another activation, a stride shorter than k, k off the grid
    one = [np.zeros(nrows, np.float32)]
    assert dev.MatVecPackedMulti(one, t, ps[:1], x0, nrows, k) is False
    assert dev.MatVecPackedGatherAct(outs, t, ps, xs.reshape(-1), ups.reshape(-1), 1, xstride, nrows, k) is False
    assert dev.MatVecPackedGather(outs, t, ps, xs.reshape(-1), k - 32, nrows, k) is False
    assert dev.MatVecPackedMulti(outs, t, ps, xs[0], nrows, k - 16) is False
    dev.ForgetPacked(ps[0])
    dev.SetActWindow(32)


def test_group_operator_over_host_planes(dev, devbuf):
    """JIT.MatVecPackedGroup over host memory (/root/reference/engine/nn/packedgroup.go:18-51): a
    block's q, k and v of different types and row counts on one activation; its gate and up (one
    type, one shape: one launch); a down projection on silu(x) * up with the residual riding on
    it.  Every matrix is the packed matvec of that matrix (TestGroupMatchesMatVec), bit for bit."""
    from jitllm_amd import _lib
    from jitllm_amd.device import MVGroup
    k, window = 2048, 256
    dev.SetActWindow(window)
    specs = [(quant.Q4_K, 512), (quant.Q4_K, 128), (quant.Q6_K, 128)]
    ws = [synth.quantized_weights(t, r, k, seed=70 + i) for i, (t, r) in enumerate(specs)]
    packs = []
    for (t, r), w in zip(specs, ws):
        qs, d, sc = oracle.pack_weights(t, w, r, k)
        packs.append(Packed(qs, d, sc if sc is not None and sc.size else None, 0, 0))   # stride 0: rows
    x = synth.activations(k, seed=9)
    n0 = dev.launch_count()
    outs = [np.full(r, np.float32(7e30)) for _, r in specs]
    g = MVGroup(outs, [t for t, _ in specs], packs, [r for _, r in specs], x, k)
    assert dev.MatVecPackedGroup(g) is True
    assert dev.launch_count() - n0 == 3       # three types / shapes: three launches
    for (t, r), w, o, p in zip(specs, ws, outs, packs):
        assert nmse(o, _like_for_like(t, w, x, r, k, window)) <= 1e-10
        single = np.zeros(r, np.float32)
        assert dev.MatVecPacked(single, t, Packed(p.qs, p.d, p.sc, 0, r), x, r, k) is True
        assert np.array_equal(single.view(np.uint32), o.view(np.uint32))
    # gate and up: one launch
    n0 = dev.launch_count()
    gu = [np.zeros(512, np.float32), np.zeros(512, np.float32)]
    w2 = synth.quantized_weights(quant.Q4_K, 512, k, seed=90)
    q2 = oracle.pack_weights(quant.Q4_K, w2, 512, k)
    p2 = Packed(q2[0], q2[1], q2[2], 0, 512)
    assert dev.MatVecPackedGroup(MVGroup(gu, [quant.Q4_K] * 2, [packs[0], p2], [512, 512], x, k)) is True
    assert dev.launch_count() - n0 == 1
    assert np.array_equal(gu[0].view(np.uint32), outs[0].view(np.uint32))
    assert nmse(gu[1], _like_for_like(quant.Q4_K, w2, x, 512, k, window)) <= 1e-10
    # a down projection: silu(x) * up in front, the residual on matrix 0
    up = synth.activations(k, seed=10)
    resid0 = synth.activations(512, seed=11)
    resid = resid0.copy()
    keep = x.copy()
    y = [np.zeros(512, np.float32)]
    assert dev.MatVecPackedGroup(MVGroup(y, [quant.Q4_K], [packs[0]], [512], x, k, ActUp=up, Act=_lib.ACT_SILU,
                                         Resid=resid, Alpha=0.5)) is True
    assert np.array_equal(x, keep)
    gx = x.astype(np.float64)
    h = (gx / (1 + np.exp(-gx)) * up.astype(np.float64)).astype(np.float32)
    assert rel_l2(y[0], _like_for_like(quant.Q4_K, ws[0], h, 512, k, window)) <= 1e-3
    assert np.array_equal(resid, (resid0 + (np.float32(0.5) * y[0]).astype(np.float32)).astype(np.float32))
    # nothing runs unless every matrix can: the second matrix's type has no planes
    before = [o.copy() for o in outs]
    bad = MVGroup(outs, [quant.Q4_K, quant.MXFP4, quant.Q6_K], packs, [r for _, r in specs], x, k)
    n0 = dev.launch_count()
    assert dev.MatVecPackedGroup(bad) is False
    assert dev.launch_count() == n0 and all(np.array_equal(a, b) for a, b in zip(before, outs))
    assert dev.MatVecPackedGroup(MVGroup(y, [quant.Q4_K], [packs[0]], [512], x, k, ActUp=up, Act=1)) is False
    for p in packs + [p2]:
        dev.ForgetPacked(p)
    dev.SetActWindow(32)


@pytest.mark.parametrize("shape", [(130, 300, 1024, 0, 300), (512, 260, 2048, 90, 400), (256, 700, 512, 0, 700),
                                   (96, 150, 2816, 37, 200), (200, 33000, 256, 0, 33000)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("form", [0, 1, 2], ids=["auto", "tile128x64", "tile256x128"])
def test_matmul_packed_q4k_reads_planes_where_they_lie(dev, devbuf, shape, form):
    """JIT.MatMulPacked (/root/reference/engine/nn/packedmm.go:23-139) never re-lays weights per
    call: the tiled GEMM forms read the QS / D / SC planes directly (their own activation prep in
    the planes' K order), with no row-restoring launch in front.  A row range inside a larger plane
    set (an expert's sheet inside its bank), a K split (few tokens, 11 super-blocks), the split of
    a grid between the two tiles (33000 rows); against the oracle, and bit for bit against the
    GEMM over the same weights as GGUF rows (the same integers, the same f32 epilogue)."""
    ntok, nrows, k, row0, stride = shape
    t = quant.Q4_K
    dev.SetActWindow(256)
    w = synth.random_weights(t, stride, k, seed=ntok + nrows)
    rb = quant.row_bytes(t, k)
    wsub = w[row0 * rb:(row0 + nrows) * rb]
    x = np.stack([synth.activations(k, seed=700 + i) * np.float32(1 + i % 3) for i in range(ntok)])
    x[ntok // 2] = 0
    p = _dev_planes(devbuf, *oracle.pack_weights(t, w, stride, k), row=row0, stride=stride)
    xd, wd = devbuf(x), devbuf(np.ascontiguousarray(wsub))
    dev.set_tuning(gemm__form=form)
    out = devbuf(shape=(ntok * nrows + 16,), dtype=np.float32, fill=np.float32(3e30))
    ref = devbuf(shape=(ntok * nrows + 16,), dtype=np.float32, fill=np.float32(3e30))
    n0 = dev.launch_count()
    assert dev.matmul_packed_dev(out.ptr, t, p, xd.ptr, nrows, k, ntok)
    launches = dev.launch_count() - n0
    assert dev.matmul_dev(ref.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    dev.set_tuning(gemm__form=0)
    got, same = out.get(), ref.get()
    assert np.all(got[ntok * nrows:] == np.float32(3e30)), "wrote past the output"
    got = got[:ntok * nrows].reshape(ntok, nrows)
    assert np.all(np.abs(got) < 1e30), "elements left unwritten"
    if nrows <= 1000:
        want = oracle.matmul_q8act_f64(t, wsub, x, nrows, k, ntok, 256)
    else:   # the oracle on a sample of rows: first, last, and around the tiles' boundary
        rows = np.unique(np.concatenate([np.arange(0, 40), np.arange(nrows - 40, nrows),
                                         np.arange(32768 - 20, 32768 + 20)]))
        want = oracle.matmul_q8act_f64(t, np.concatenate([wsub[r * rb:(r + 1) * rb] for r in rows]), x, len(rows), k,
                                       ntok, 256)
        got = got[:, rows]
    assert nmse(got, want) <= 1e-10
    assert np.all(got[ntok // 2] == 0)
    # no launch restores rows: prep + one or two tile kernels (+ the slab sum of a K split)
    assert launches <= 3, launches
    few32 = form == 0 and ntok > 64 and 2 * ((nrows + 31) // 32) * ((ntok + 63) // 64) <= 3 * 256
    if not few32 and form != 0:   # the same form on both sides: the same bits
        assert np.array_equal(out.get()[:ntok * nrows].view(np.uint32), same[:ntok * nrows].view(np.uint32))
    else:
        assert nmse(out.get()[:ntok * nrows], same[:ntok * nrows].astype(np.float64)) <= 1e-12
    dev.SetActWindow(32)
