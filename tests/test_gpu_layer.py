"""GPU tests of the block seam through the C ABI: a block's feed-forward weights handed over
once (nn.LayerDevice.PrepLayer, /root/reference/engine/nn/device.go:1096-1131) and the block run
by handle.  The bar: prepared once, run twice, both runs equal, bit for bit, to the pointer-form
entry points on the same operands (which the other GPU tests hold to the oracle); one case is
held to the oracle directly."""
import numpy as np
import pytest

import oracle
from conftest import rel_l2
from jitllm_amd import _lib, quant, synth

pytestmark = pytest.mark.gpu


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def _bank(t, n_expert, nrows, k, seed):
    return np.concatenate([synth.quantized_weights(t, nrows, k, seed=seed + e) for e in range(n_expert)])


def _planes(t, w, nrows, k):
    qs, d, sc = oracle.pack_weights(t, w, nrows, k)
    return qs, d, (sc if sc is not None and sc.size else None)


def _dev_planes(devbuf, pl):
    bufs = [None if p is None else devbuf(p) for p in pl]
    return bufs, tuple(None if b is None else b.ptr for b in bufs)


def silu(g):
    g = g.astype(np.float64)
    return g / (1 + np.exp(-g))


@pytest.mark.parametrize("packed", [False, True], ids=["rows", "planes"])
@pytest.mark.parametrize("t,down_t,normed", [(quant.Q8_0, quant.Q6_K, True), (quant.Q4_K, quant.Q4_K, False)])
def test_dense_block_one_row_by_handle_equals_the_two_launches(dev, devbuf, packed, t, down_t, normed):
    """One row of a dense block is the decode pair: gate and up in one launch (the norm riding in
    front), down over silu(gate) * up with the residual add riding on it."""
    E, F, window = 1024, 2816 if t == quant.Q8_0 else 2048, 32
    dev.SetActWindow(window)
    gate, up = synth.quantized_weights(t, F, E, seed=1), synth.quantized_weights(t, F, E, seed=2)
    down = synth.quantized_weights(down_t, E, F, seed=3)
    nw = (1 + 0.1 * np.random.default_rng(4).standard_normal(E)).astype(np.float32) if normed else None
    eps = 1e-5
    h = synth.activations(E, seed=5)
    resid0 = synth.activations(E, seed=6)
    hd = devbuf(h)
    # the pointer form
    g, u, y = (devbuf(shape=(n,), dtype=np.float32, fill=0) for n in (F, F, E))
    want = devbuf(resid0)
    nwd = None if nw is None else devbuf(nw)
    if packed:
        pg, pu, pd = _planes(t, gate, F, E), _planes(t, up, F, E), _planes(down_t, down, E, F)
        (kg, dg), (ku, du), (kd, dd) = (_dev_planes(devbuf, p) for p in (pg, pu, pd))
        assert dev.matvec_packed_multi_dev([g.ptr, u.ptr], t, [dg, du], [0, 0], F, hd.ptr, 0, None, F, E,
                                           norm_w=None if nwd is None else nwd.ptr, norm_eps=eps)
        assert dev.matvec_packed_multi_dev([y.ptr], down_t, [dd], [0], E, g.ptr, 0, u.ptr, E, F, resid=want.ptr,
                                           alpha=1.0)
    else:
        wg, wu, wd = devbuf(gate), devbuf(up), devbuf(down)
        assert dev.matvec_group_dev([g.ptr, u.ptr], [t, t], [wg.ptr, wu.ptr], [F, F], hd.ptr, E,
                                    norm_w=None if nwd is None else nwd.ptr, norm_eps=eps)
        assert dev.matvec_group_dev([y.ptr], [down_t], [wd.ptr], [E], g.ptr, F, act_up=u.ptr, resid=want.ptr,
                                    alpha=1.0)
    dev.synchronize()
    want_h = want.get()
    # by handle: prepared once, run twice
    before = dev.Layers()
    if packed:
        assert dev.PrepLayer(3, _lib.LAYER_DENSE, t, E, F, pg, pu, pd, down_type=down_t, norm_w=nw, norm_eps=eps)
    else:
        assert dev.PrepLayer(3, _lib.LAYER_DENSE, t, E, F, gate, up, down, down_type=down_t, norm_w=nw, norm_eps=eps)
    assert dev.Layers() == before + 1
    try:
        for _ in range(2):
            got = devbuf(resid0)
            n0 = dev.launch_count()
            assert dev.layer_ffn_dev(3, hd.ptr, got.ptr, 1)
            assert dev.launch_count() == n0 + 2
            dev.synchronize()
            assert np.array_equal(_bits(got.get()), _bits(want_h))
        # and the values are the block's: the oracle's matvecs chained in f64
        x = h if nw is None else oracle.rmsnorm32(h, nw, eps)
        gg = oracle.matvec_q8act_f64(t, gate, *oracle.quantize_act(x, window)[:2], F, E)
        uu = oracle.matvec_q8act_f64(t, up, *oracle.quantize_act(x, window)[:2], F, E)
        act = (silu(gg.astype(np.float32)) * uu.astype(np.float32).astype(np.float64)).astype(np.float32)
        yy = oracle.matvec_q8act_f64(down_t, down, *oracle.quantize_act(act, window)[:2], E, F)
        assert rel_l2(want_h - resid0, yy) <= 2e-3
    finally:
        dev.ReleaseLayers(3, 4)
    assert dev.Layers() == before
    with pytest.raises(Exception, match="not prepared"):
        dev.layer_ffn_dev(3, hd.ptr, want.ptr, 1)


@pytest.mark.parametrize("packed", [False, True], ids=["rows", "planes"])
def test_dense_block_many_rows_by_handle_is_a_mixture_of_one(dev, devbuf, packed):
    """More rows of a dense block run the mixture's grouped kernels with one expert that every
    row selects with weight 1; a block with a norm in front runs its rows one at a time."""
    E, F, n, t, window = 1024, 1536, 37, quant.Q4_K, 256
    dev.SetActWindow(window)
    gate, up, down = (synth.quantized_weights(t, r, k, seed=s) for r, k, s in ((F, E, 11), (F, E, 12), (E, F, 13)))
    h = np.stack([synth.activations(E, seed=20 + i) for i in range(n)])
    resid0 = np.stack([synth.activations(E, seed=70 + i) for i in range(n)])
    hd, want = devbuf(h), devbuf(resid0)
    sel = devbuf(np.zeros((n, 2), np.uint32))
    wt = devbuf(np.ones((n, 1), np.float32))
    if packed:
        pl = [_planes(t, w, r, k) for w, r, k in ((gate, F, E), (up, F, E), (down, E, F))]
        keep = [_dev_planes(devbuf, p) for p in pl]
        banks = [dev.packed_bank(ptrs[0], ptrs[1], ptrs[2], 0, r) for (_, ptrs), r in zip(keep, (F, F, E))]
        assert dev.moe_ffn_packed_dev(want.ptr, t, banks[0], banks[1], banks[2], hd.ptr, sel.ptr, 2, wt.ptr, n, 1, 1, F, E)
        assert dev.PrepLayer(0, _lib.LAYER_DENSE, t, E, F, *pl)
    else:
        wg, wu, wd = devbuf(gate), devbuf(up), devbuf(down)
        assert dev.moe_ffn_dev(want.ptr, t, wg.ptr, wu.ptr, wd.ptr, hd.ptr, sel.ptr, 2, wt.ptr, n, 1, 1, F, E)
        assert dev.PrepLayer(0, _lib.LAYER_DENSE, t, E, F, gate, up, down)
    dev.synchronize()
    want_h = want.get()
    try:
        for rows in (n, 5):     # the second run smaller: the fills cover what the run reads
            got = devbuf(resid0)
            assert dev.layer_ffn_dev(0, hd.ptr, got.ptr, rows)
            dev.synchronize()
            out = got.get()
            assert np.array_equal(_bits(out[:rows]), _bits(want_h[:rows]))
            assert np.array_equal(_bits(out[rows:]), _bits(resid0[rows:]))
    finally:
        dev.ReleaseLayers(0, 1)
        dev.SetActWindow(32)


def test_dense_block_with_a_norm_runs_its_rows_one_at_a_time(dev, devbuf):
    E, F, n, t, window = 512, 1024, 3, quant.Q6_K, 32
    dev.SetActWindow(window)
    gate, up, down = (synth.quantized_weights(t, r, k, seed=s) for r, k, s in ((F, E, 31), (F, E, 32), (E, F, 33)))
    nw = (1 + 0.1 * np.random.default_rng(34).standard_normal(E)).astype(np.float32)
    h = np.stack([synth.activations(E, seed=40 + i) for i in range(n)])
    resid0 = np.stack([synth.activations(E, seed=50 + i) for i in range(n)])
    hd, nwd = devbuf(h), devbuf(nw)
    wg, wu, wd = devbuf(gate), devbuf(up), devbuf(down)
    g, u, y = (devbuf(shape=(m,), dtype=np.float32, fill=0) for m in (F, F, E))
    want = devbuf(resid0)
    for r in range(n):
        assert dev.matvec_group_dev([g.ptr, u.ptr], [t, t], [wg.ptr, wu.ptr], [F, F], hd.ptr + r * E * 4, E,
                                    norm_w=nwd.ptr, norm_eps=1e-6)
        assert dev.matvec_group_dev([y.ptr], [t], [wd.ptr], [E], g.ptr, F, act_up=u.ptr, resid=want.ptr + r * E * 4,
                                    alpha=1.0)
    dev.synchronize()
    assert dev.PrepLayer(1, _lib.LAYER_DENSE, t, E, F, gate, up, down, norm_w=nw, norm_eps=1e-6)
    try:
        got = devbuf(resid0)
        n0 = dev.launch_count()
        assert dev.layer_ffn_dev(1, hd.ptr, got.ptr, n)
        assert dev.launch_count() == n0 + 2 * n
        dev.synchronize()
        assert np.array_equal(_bits(got.get()), _bits(want.get()))
    finally:
        dev.ReleaseLayers(0, 8)


@pytest.mark.parametrize("packed", [False, True], ids=["rows", "planes"])
@pytest.mark.parametrize("n", [1, 19])
def test_mixture_block_by_handle_routes_and_runs_like_the_three_calls(dev, devbuf, packed, n):
    """Router product, softmax + top-k, routed feed-forward: the three pointer-form calls
    (/root/reference/engine/model/moe.go:752-820) behind one handle."""
    E, F, n_expert, k_used, t, window = 512, 768, 8, 2, quant.Q4_K, 256
    dev.SetActWindow(window)
    gate, up, down = _bank(t, n_expert, F, E, 100), _bank(t, n_expert, F, E, 200), _bank(t, n_expert, E, F, 300)
    router = (np.random.default_rng(7).standard_normal((n_expert, E)) * 0.1).astype(np.float32)
    h = np.stack([synth.activations(E, seed=400 + i) for i in range(n)])
    resid0 = np.stack([synth.activations(E, seed=500 + i) for i in range(n)])
    hd, rd, want = devbuf(h), devbuf(router), devbuf(resid0)
    logits = devbuf(shape=(n, n_expert), dtype=np.float32, fill=0)
    sel = devbuf(shape=(n, k_used + 1), dtype=np.uint32, fill=0)
    wt = devbuf(shape=(n, k_used), dtype=np.float32, fill=0)
    assert dev.moe_logits_dev(logits.ptr, 0, rd.ptr, hd.ptr, n_expert, E, n)
    assert dev.moe_route_dev(logits.ptr, n, n_expert, k_used, sel.ptr, k_used + 1, wt.ptr)
    if packed:
        pl = [_planes(t, w, n_expert * r, k) for w, r, k in ((gate, F, E), (up, F, E), (down, E, F))]
        keep = [_dev_planes(devbuf, p) for p in pl]
        banks = [dev.packed_bank(ptrs[0], ptrs[1], ptrs[2], 0, n_expert * r) for (_, ptrs), r in zip(keep, (F, F, E))]
        assert dev.moe_ffn_packed_dev(want.ptr, t, banks[0], banks[1], banks[2], hd.ptr, sel.ptr, k_used + 1, wt.ptr, n,
                                      k_used, n_expert, F, E)
        assert dev.PrepLayer(5, _lib.LAYER_MOE, t, E, F, *pl, n_expert=n_expert, k_used=k_used, router=router)
    else:
        wg, wu, wd = devbuf(gate), devbuf(up), devbuf(down)
        assert dev.moe_ffn_dev(want.ptr, t, wg.ptr, wu.ptr, wd.ptr, hd.ptr, sel.ptr, k_used + 1, wt.ptr, n, k_used,
                               n_expert, F, E)
        assert dev.PrepLayer(5, _lib.LAYER_MOE, t, E, F, gate, up, down, n_expert=n_expert, k_used=k_used, router=router)
    dev.synchronize()
    want_h = want.get()
    assert not np.array_equal(want_h, resid0)
    try:
        for _ in range(2):
            got = devbuf(resid0)
            assert dev.layer_ffn_dev(5, hd.ptr, got.ptr, n)
            dev.synchronize()
            assert np.array_equal(_bits(got.get()), _bits(want_h))
    finally:
        dev.ReleaseLayers(5, 6)
        dev.SetActWindow(32)


def test_prep_layer_declines_what_has_no_kernel_and_replaces_a_block(dev, devbuf):
    E, F, t = 256, 512, quant.Q8_0
    gate, up, down = (synth.quantized_weights(t, r, k, seed=s) for r, k, s in ((F, E, 1), (F, E, 2), (E, F, 3)))
    before = dev.Layers()
    assert dev.PrepLayer(9, _lib.LAYER_DENSE, 99, E, F, gate, up, down) is False      # an unknown type
    assert dev.PrepLayer(9, _lib.LAYER_DENSE, quant.Q4_K, 96, F, gate, up, down) is False   # k not a multiple of 256
    assert dev.Layers() == before
    with pytest.raises(Exception):
        dev.PrepLayer(9, _lib.LAYER_MOE, t, E, F, gate, up, down, n_expert=4, k_used=2)   # no router
    assert dev.PrepLayer(9, _lib.LAYER_DENSE, t, E, F, gate, up, down)
    assert dev.PrepLayer(9, _lib.LAYER_DENSE, t, E, F, gate, up, down)     # again: replaced, not leaked
    assert dev.Layers() == before + 1
    dev.ReleaseLayers(0, 100)
    assert dev.Layers() == 0


def test_config2_block_by_handle_at_full_size(dev, devbuf):
    """The baseline's dense block at its own sizes -- gate and up Q8_0 14336 x 4096, down Q6_K
    4096 x 14336, RMSNorm in front, activation window 32 -- prepared from host memory and run by
    handle: the bits of the two pointer-form launches, whose kernels the full-size matvec tests hold
    to the oracle, and the block's value on a sample of rows recomputed in f64."""
    E, F, window, eps = 4096, 14336, 32, 1e-5
    dev.SetActWindow(window)
    gate, up = synth.quantized_weights(quant.Q8_0, F, E, seed=0), synth.quantized_weights(quant.Q8_0, F, E, seed=1)
    down = synth.quantized_weights(quant.Q6_K, E, F, seed=2)
    nw = (1 + 0.1 * np.random.default_rng(3).standard_normal(E)).astype(np.float32)
    h, resid0 = synth.activations(E, seed=4), synth.activations(E, seed=5)
    hd, nwd = devbuf(h), devbuf(nw)
    wg, wu, wd = devbuf(gate), devbuf(up), devbuf(down)
    g, u, y = (devbuf(shape=(n,), dtype=np.float32, fill=0) for n in (F, F, E))
    want = devbuf(resid0)
    assert dev.matvec_group_dev([g.ptr, u.ptr], [quant.Q8_0] * 2, [wg.ptr, wu.ptr], [F, F], hd.ptr, E, norm_w=nwd.ptr,
                                norm_eps=eps)
    assert dev.matvec_group_dev([y.ptr], [quant.Q6_K], [wd.ptr], [E], g.ptr, F, act_up=u.ptr, resid=want.ptr, alpha=1.0)
    dev.synchronize()
    for b in (wg, wu, wd):
        b.free()
    assert dev.PrepLayer(2, _lib.LAYER_DENSE, quant.Q8_0, E, F, gate, up, down, down_type=quant.Q6_K, norm_w=nw,
                         norm_eps=eps)
    try:
        for _ in range(2):
            got = devbuf(resid0)
            assert dev.layer_ffn_dev(2, hd.ptr, got.ptr, 1)
            dev.synchronize()
            assert np.array_equal(_bits(got.get()), _bits(want.get()))
    finally:
        dev.ReleaseLayers(2, 3)
    # the value itself, on the device's own gate and up (so a moved int8 of the gated activation
    # cannot hide an error): rows spread over the matrix
    gg, uu = g.get(), u.get()
    act = (silu(gg) * uu.astype(np.float64)).astype(np.float32)
    q, a_s, _ = oracle.quantize_act(act, window)
    rows = np.unique(np.linspace(0, E - 1, 96).astype(int))
    nb = F // 256 * 210
    sample = np.concatenate([down[r * nb:(r + 1) * nb] for r in rows])
    yy = oracle.matvec_q8act_f64(quant.Q6_K, sample, q, a_s, len(rows), F)
    assert rel_l2((want.get() - resid0)[rows], yy) <= 2e-3


def test_config4_mixture_block_by_handle_at_full_size(dev, devbuf):
    """The baseline's mixture block at its own sizes -- 128 experts of 768 x 2048 / 2048 x 768 Q4_K,
    64 rows routed top-8 -- prepared from host memory (340 MB, one allocation) and run by handle:
    the bits of the pointer-form calls, which the mixture tests hold to the oracle."""
    t, n_expert, k_used, F, E, rows = quant.Q4_K, 128, 8, 768, 2048, 64
    dev.SetActWindow(256)
    gate, up, down = _bank(t, n_expert, F, E, 1000), _bank(t, n_expert, F, E, 2000), _bank(t, n_expert, E, F, 3000)
    rng = np.random.default_rng(9)
    router = (rng.standard_normal((n_expert, E)) / np.sqrt(E)).astype(np.float32)
    h = rng.standard_normal((rows, E)).astype(np.float32)
    resid0 = rng.standard_normal((rows, E)).astype(np.float32)
    hd, rd = devbuf(h), devbuf(router)
    wg, wu, wd = devbuf(gate), devbuf(up), devbuf(down)
    try:
        # (a row count of its own each: seven rows are under two columns an expert and run another
        # kernel form, with another order of f32 sums, than sixty-four)
        want = {}
        for n in (rows, 7):
            want[n] = devbuf(resid0)
            assert dev.moe_block_dev(want[n].ptr, t, wg.ptr, wu.ptr, wd.ptr, rd.ptr, hd.ptr, n, k_used, n_expert, F, E)
        dev.synchronize()
        for b in (wg, wu, wd):
            b.free()
        assert dev.PrepLayer(4, _lib.LAYER_MOE, t, E, F, gate, up, down, n_expert=n_expert, k_used=k_used, router=router)
        for n in (rows, 7):
            got = devbuf(resid0)
            assert dev.layer_ffn_dev(4, hd.ptr, got.ptr, n)
            dev.synchronize()
            out = got.get()
            assert np.array_equal(_bits(out), _bits(want[n].get()))
            assert np.array_equal(_bits(out[n:]), _bits(resid0[n:]))
            assert not np.array_equal(out[:n], resid0[:n])
    finally:
        dev.ReleaseLayers(0, 8)
        dev.SetActWindow(32)
