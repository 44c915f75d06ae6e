"""GPU parity of the grouped decode matvecs (several matrices, one launch) against the
oracle, through the C ABI.  Each matrix of a group is the decode matvec on it: the bar is
the matvec's, NMSE <= 1e-10 against the f64 evaluation of the same int8 activations; the
gated form (silu(x) * up inside the quantizer) is held to rel-L2 <= 1e-3 because exp()
differs from numpy's in its last bits and can move an int8."""
import numpy as np
import pytest

import oracle
from conftest import nmse, rel_l2
from jitllm_amd import quant, synth

pytestmark = pytest.mark.gpu


def _want(t, w, x, nrows, k, window):
    q, a_s, _ = oracle.quantize_act(x, window)
    return oracle.matvec_q8act_f64(t, w, q, a_s, nrows, k)


def silu(g):
    g = g.astype(np.float64)
    return g / (1 + np.exp(-g))


def test_group_qkv_mixed_types_one_activation(dev, devbuf):
    """MatVecPackedGroup (/root/reference/engine/nn/packedgroup.go:13-51): q, k, v of a block."""
    k, window = 2048, 32
    dev.SetActWindow(window)
    spec = [(quant.Q4_K, 520), (quant.Q4_K, 128), (quant.Q6_K, 130), (quant.Q8_0, 7)]
    ws = [synth.quantized_weights(t, r, k, seed=i + 1) for i, (t, r) in enumerate(spec)]
    x = synth.activations(k, seed=9)
    dws, dx = [devbuf(w) for w in ws], devbuf(x)
    outs = [devbuf(shape=(r + 4,), dtype=np.float32, fill=np.float32(6e30)) for _, r in spec]
    before = dev.launch_count()
    assert dev.matvec_group_dev([o.ptr for o in outs], [t for t, _ in spec], [w.ptr for w in dws],
                                [r for _, r in spec], dx.ptr, k)
    # three formats, one launch (the reference's MatVecSegments,
    # /root/reference/jit/gpu/kernels/matvec.go:1411-1431)
    assert dev.launch_count() == before + 1
    dev.synchronize()
    for (t, r), w, o in zip(spec, ws, outs):
        got = o.get()
        assert np.all(got[r:] == np.float32(6e30)), "wrote past the matrix's rows"
        assert nmse(got[:r], _want(t, w, x, r, k, window)) <= 1e-10


@pytest.mark.parametrize("k,window", [(2048, 32), (4096, 256), (5120, 32)])
def test_group_with_rmsnorm_in_front(dev, devbuf, k, window):
    """RMSNorm folded into the group's quantizer (the reference's RMSNormQuantRows,
    /root/reference/jit/gpu/kernels/elem.go:252-267): the normed vector must equal the
    oracle's RMSNorm32 up to the order of the f64 sum (one f32 ulp at most, normally none),
    and the matvecs must be the matvecs of THAT vector -- checked on the vector the device
    wrote, so a moved int8 cannot hide an error."""
    dev.SetActWindow(window)
    types = (quant.Q4_K, quant.Q4_K, quant.Q6_K) if window == 32 else (quant.Q4_K, quant.Q4_K, quant.Q4_K)
    spec = list(zip(types, (300, 64, 130)))
    ws = [synth.quantized_weights(t, r, k, seed=i + 20) for i, (t, r) in enumerate(spec)]
    x = synth.activations(k, seed=31) * np.float32(3.5)
    nw = (1 + 0.1 * np.random.default_rng(8).standard_normal(k)).astype(np.float32)
    eps = 1e-5
    dws, dx, dnw = [devbuf(w) for w in ws], devbuf(x), devbuf(nw)
    dn = devbuf(shape=(k + 4,), dtype=np.float32, fill=np.float32(-3e30))
    outs = [devbuf(shape=(r,), dtype=np.float32, fill=np.float32(6e30)) for _, r in spec]
    for call in range(2):
        assert dev.matvec_group_dev([o.ptr for o in outs], [t for t, _ in spec], [w.ptr for w in dws],
                                    [r for _, r in spec], dx.ptr, k, norm_w=dnw.ptr, norm_eps=eps, norm_out=dn.ptr)
        dev.synchronize()
        normed = dn.get()
        assert np.all(normed[k:] == np.float32(-3e30))
        normed = normed[:k]
        want_n = oracle.rmsnorm32(x, nw, eps)
        ulp = np.abs(normed.view(np.int32).astype(np.int64) - want_n.view(np.int32).astype(np.int64))
        assert ulp.max() <= 1 and np.mean(ulp != 0) <= 0.01
        for (t, r), w, o in zip(spec, ws, outs):
            assert nmse(o.get(), _want(t, w, normed, r, k, window)) <= 1e-10
            assert rel_l2(o.get(), _want(t, w, want_n, r, k, window)) <= 1e-3
    dev.SetActWindow(32)


@pytest.mark.parametrize("t_d,n_ffn,window", [(quant.Q6_K, 14336, 32), (quant.Q8_0, 9216, 32), (quant.Q4_K, 11008 // 256 * 256, 256)],
                         ids=["q6_k_14336", "q8_0_9216", "q4_k_10752"])
def test_group_long_gated_activation_quantized_once(dev, devbuf, t_d, n_ffn, window):
    """A gated down projection with a long activation (three float4 groups a thread and more, each
    thread's groups loaded together ahead of its weights): silu(gate) * up formed by every
    workgroup (one launch, the default) and formed and quantized once by the quantizer kernel with
    the matvec staging the int8 copy (two launches, matvec.act_split = 1).  Both against the
    oracle, and bit for bit against each other; the residual add rides on either."""
    n_embd = 200
    dev.SetActWindow(window)
    wdn = synth.quantized_weights(t_d, n_embd, n_ffn, seed=3)
    gh = synth.activations(n_ffn, seed=6) * np.float32(2.0)
    uh = synth.activations(n_ffn, seed=7)
    h = (silu(gh) * uh.astype(np.float64)).astype(np.float32)
    want = _want(t_d, wdn, h, n_embd, n_ffn, window)
    dwd, g, u = devbuf(wdn), devbuf(gh), devbuf(uh)
    resid0 = synth.activations(n_embd, seed=5)
    got = {}
    for split, launches in ((0, 1), (1, 2)):
        dev.set_tuning(act_split=split)
        resid = devbuf(resid0)
        y = devbuf(shape=(n_embd + 4,), dtype=np.float32, fill=np.float32(5e30))
        before = dev.launch_count()
        assert dev.matvec_group_dev([y.ptr], [t_d], [dwd.ptr], [n_embd], g.ptr, n_ffn, act_up=u.ptr,
                                    resid=resid.ptr, alpha=0.5)
        assert dev.launch_count() == before + launches
        dev.synchronize()
        yh = y.get()
        assert np.all(yh[n_embd:] == np.float32(5e30))
        got[split] = yh[:n_embd]
        assert rel_l2(got[split], want) <= 1e-3
        assert np.array_equal(resid.get(), (resid0 + (np.float32(0.5) * got[split]).astype(np.float32)).astype(np.float32))
        assert np.array_equal(g.get(), gh), "the activation operand must be left as it was"
    dev.set_tuning(act_split=0)
    assert np.array_equal(got[0].view(np.uint32), got[1].view(np.uint32)), "quantized once != quantized by every workgroup"
    dev.SetActWindow(32)


def test_group_gate_up_then_gated_down_with_residual(dev, devbuf):
    """A gated feed-forward block as two groups: (gate, up) sharing x, then down over
    silu(gate) * up with the residual add riding on the launch."""
    n_embd, n_ffn, window = 1024, 2816, 32
    dev.SetActWindow(window)
    t_gu, t_d = quant.Q8_0, quant.Q6_K
    wg = synth.quantized_weights(t_gu, n_ffn, n_embd, seed=1)
    wu = synth.quantized_weights(t_gu, n_ffn, n_embd, seed=2)
    wdn = synth.quantized_weights(t_d, n_embd, n_ffn, seed=3)
    x = synth.activations(n_embd, seed=4)
    dwg, dwu, dwd, dx = devbuf(wg), devbuf(wu), devbuf(wdn), devbuf(x)
    g = devbuf(shape=(n_ffn,), dtype=np.float32, fill=0)
    u = devbuf(shape=(n_ffn,), dtype=np.float32, fill=0)
    assert dev.matvec_group_dev([g.ptr, u.ptr], [t_gu, t_gu], [dwg.ptr, dwu.ptr], [n_ffn, n_ffn], dx.ptr, n_embd)
    dev.synchronize()
    gh, uh = g.get(), u.get()
    assert nmse(gh, _want(t_gu, wg, x, n_ffn, n_embd, window)) <= 1e-10
    assert nmse(uh, _want(t_gu, wu, x, n_ffn, n_embd, window)) <= 1e-10
    resid0 = synth.activations(n_embd, seed=5)
    resid = devbuf(resid0)
    y = devbuf(shape=(n_embd,), dtype=np.float32, fill=0)
    alpha = np.float32(0.75)
    assert dev.matvec_group_dev([y.ptr], [t_d], [dwd.ptr], [n_embd], g.ptr, n_ffn, act_up=u.ptr,
                                resid=resid.ptr, alpha=float(alpha))
    dev.synchronize()
    yh = y.get()
    h = (silu(gh) * uh.astype(np.float64)).astype(np.float32)
    assert rel_l2(yh, _want(t_d, wdn, h, n_embd, n_ffn, window)) <= 1e-3
    assert np.array_equal(resid.get(), (resid0 + (alpha * yh).astype(np.float32)).astype(np.float32))
    assert np.array_equal(g.get(), gh), "the activation operand must be left as it was"
    dev.SetActWindow(32)


@pytest.mark.parametrize("t", [quant.Q4_K, quant.Q8_0, quant.Q6_K])
def test_multi_and_gather(dev, devbuf, t):
    """MatVecPackedMulti (one activation, a mixture's gate and up at decode) and
    MatVecPackedGather / GatherAct (each matrix its own activation at a stride)."""
    m, nrows, k = 16, 96, 1024
    window = 256 if t in quant.K_QUANTS else 32
    dev.SetActWindow(window)
    ws = [synth.quantized_weights(t, nrows, k, seed=10 + i) for i in range(m)]
    dws = [devbuf(w) for w in ws]
    x = synth.activations(k, seed=1)
    dx = devbuf(x)
    outs = [devbuf(shape=(nrows,), dtype=np.float32, fill=np.float32(1e30)) for _ in range(m)]
    assert dev.matvec_gather_dev([o.ptr for o in outs], t, [w.ptr for w in dws], dx.ptr, 0, None, nrows, k)
    dev.synchronize()
    for w, o in zip(ws, outs):
        assert nmse(o.get(), _want(t, w, x, nrows, k, window)) <= 1e-10
    # each matrix its own activation, stride k + 64 elements
    stride = k + 64
    xs = np.stack([np.concatenate([synth.activations(k, seed=30 + j), np.full(64, np.float32(9e9))]) for j in range(m)])
    ups = np.stack([np.concatenate([synth.activations(k, seed=60 + j), np.full(64, np.float32(9e9))]) for j in range(m)])
    dxs, dups = devbuf(xs), devbuf(ups)
    assert dev.matvec_gather_dev([o.ptr for o in outs[:8]], t, [w.ptr for w in dws[:8]], dxs.ptr, stride, None,
                                 nrows, k)
    dev.synchronize()
    for j in range(8):
        assert nmse(outs[j].get(), _want(t, ws[j], xs[j, :k], nrows, k, window)) <= 1e-10
    assert dev.matvec_gather_dev([o.ptr for o in outs[:8]], t, [w.ptr for w in dws[:8]], dxs.ptr, stride, dups.ptr,
                                 nrows, k)
    dev.synchronize()
    for j in range(8):
        h = (silu(xs[j, :k]) * ups[j, :k].astype(np.float64)).astype(np.float32)
        assert rel_l2(outs[j].get(), _want(t, ws[j], h, nrows, k, window)) <= 1e-3
    # more than sixteen matrices is a decline, not an error
    many = [outs[0].ptr] * 17
    assert dev.matvec_gather_dev(many, t, [dws[0].ptr] * 17, dx.ptr, 0, None, nrows, k) is False
    dev.SetActWindow(32)


@pytest.mark.parametrize("layout", ["rows", "packed"])
def test_shared_expert_add_gated_by_a_device_logit(dev, devbuf, layout):
    """A shared expert's contribution (/root/reference/engine/model/moe.go:401-497): the gate
    logit is a one-row router product on the device, the down projection adds
    scale * sigmoid(logit) * out into the residual on its own launch, sigma in f64 narrowed
    once (/root/reference/internal/oracle/moe.go:361-370).  The matvec is the plain matvec
    (checked on the out it wrote), the add is exact f32 arithmetic on that out."""
    n_embd, n_ffn, window, t = 1024, 512, 32, quant.Q8_0
    dev.SetActWindow(window)
    w = synth.quantized_weights(t, n_embd, n_ffn, seed=3)
    h = synth.activations(n_ffn, seed=4)
    xin = synth.activations(n_embd, seed=5)
    shr = (np.random.default_rng(6).standard_normal(n_embd) * 0.05).astype(np.float32)
    resid0 = synth.activations(n_embd, seed=7)
    hd, xd, shd, resid = devbuf(h), devbuf(xin), devbuf(shr), devbuf(resid0)
    logit = devbuf(shape=(1,), dtype=np.float32, fill=0)
    y = devbuf(shape=(n_embd,), dtype=np.float32, fill=0)
    assert dev.moe_logits_dev(logit.ptr, 0, shd.ptr, xd.ptr, 1, n_embd, 1)
    scale = np.float32(0.75)
    if layout == "rows":
        wd = devbuf(w)
        assert dev.matvec_group_dev([y.ptr], [t], [wd.ptr], [n_embd], hd.ptr, n_ffn, resid=resid.ptr,
                                    alpha=float(scale), resid_gate=logit.ptr)
    else:
        qs, d, sc = oracle.pack_weights(t, w, n_embd, n_ffn)
        pq, pd = devbuf(qs), devbuf(d)
        assert dev.matvec_packed_multi_dev([y.ptr], t, [(pq.ptr, pd.ptr, None)], [0], n_embd, hd.ptr, 0, None,
                                           n_embd, n_ffn, resid=resid.ptr, alpha=float(scale), resid_gate=logit.ptr)
    dev.synchronize()
    lg = logit.get()[0]
    assert lg.view(np.uint32) == oracle.router_logits(shr, xin, 1, n_embd)[0, 0].view(np.uint32)
    yh = y.get()
    assert nmse(yh, _want(t, w, h, n_embd, n_ffn, window)) <= 1e-10
    sig = np.float32(1.0 / (1.0 + np.exp(-np.float64(lg))))
    wgt = np.float32(scale * sig)
    want = (resid0 + (wgt * yh).astype(np.float32)).astype(np.float32)
    got = resid.get()
    # the device's f64 exp may differ from numpy's in its last bit, which can move the f32 weight by one ulp
    assert np.max(np.abs(got - want)) <= 2.0 ** -22 * np.max(np.abs(yh))
    dev.SetActWindow(32)
