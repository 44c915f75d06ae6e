"""GPU parity of the decode matvec path against the CPU oracle, through the C ABI.

Bars (the reference's own, /root/reference/jit/cpu/matvec_test.go:15-18,
jit/gpu/backend/matvec_test.go:16-21, engine/nn/packed_test.go:140-147):
  * activation quantizer and dequantizer: bit-exact (integer / byte work)
  * matvec vs the f64 evaluation of the SAME int8 activations: NMSE <= 1e-10,
    and rel-L2 <= 1e-3 (the stated tolerance) follows from it
  * matvec vs the f32-activation oracle: NMSE <= 1e-3
"""
import json
import os

import numpy as np
import pytest

import oracle
from conftest import GOLDEN, nmse, rel_l2
from jitllm_amd import quant, synth

pytestmark = pytest.mark.gpu

TYPES = [quant.Q4_K, quant.Q8_0, quant.Q6_K]


def boundary_activations(rng, k, window):
    """Values within two ulps of a rounding boundary (n + 0.5) * d, the inputs on which
    a quantizer one ulp off moves an int8 (/root/reference/jit/gpu/backend/quantbits_test.go:56-80)."""
    x = np.zeros(k, np.float32)
    for w in range(0, k, window):
        amax = np.float32(np.exp(rng.random() * 16 - 8))
        x[w] = amax if rng.integers(2) == 0 else -amax
        inv = np.float32(1) / (amax / np.float32(127))
        for i in range(w + 1, min(w + window, k)):
            n = float(1 + rng.integers(125))
            if rng.integers(2) == 0:
                n = -n
            v = np.float32((n + np.copysign(0.5, n)) / float(inv))
            bits = int(v.view(np.uint32)) + int(rng.integers(5)) - 2
            x[i] = np.uint32(bits).view(np.float32)
    return x


@pytest.mark.parametrize("window", [32, 256])
@pytest.mark.parametrize("k", [32, 288, 4096, 14336])
def test_quantizer_bit_exact(dev, devbuf, window, k):
    rng = np.random.default_rng(k + window)
    dev.SetActWindow(window)
    cases = [rng.standard_normal(k).astype(np.float32),
             boundary_activations(rng, k, window),
             np.zeros(k, np.float32)]
    cases[0][: min(k, 64)] *= 1e-30  # tiny values, subnormal scales
    x = np.stack(cases)
    ntok = x.shape[0]
    xd = devbuf(x)
    q = devbuf(shape=(ntok, k), dtype=np.int8, fill=77)
    a_s = devbuf(shape=(ntok, k // 32), dtype=np.float32, fill=-1)
    s16 = devbuf(shape=(ntok, k // 16), dtype=np.float32, fill=-1)
    assert dev.quantize_act_dev(xd.ptr, ntok, k, q.ptr, a_s.ptr, s16.ptr)
    dev.synchronize()
    gq, ga, gs = q.get(), a_s.get(), s16.get()
    for t in range(ntok):
        wq, wa, ws = oracle.quantize_act(x[t], window)
        assert np.array_equal(gq[t], wq), f"token {t}: {np.sum(gq[t] != wq)} int8 differ"
        assert np.array_equal(ga[t].view(np.uint32), wa.view(np.uint32))
        assert np.array_equal(gs[t], ws)
    dev.SetActWindow(32)


def _golden_cases():
    out = []
    for name, t in [("q4_k_tiny", quant.Q4_K), ("q6_k_tiny", quant.Q6_K), ("q8_0_gemma", quant.Q8_0),
                    ("q8_0_minilm", quant.Q8_0), ("q8_0_stories", quant.Q8_0)]:
        src = np.fromfile(os.path.join(GOLDEN, name + ".in"), np.uint8)
        want = np.fromfile(os.path.join(GOLDEN, name + ".f32"), np.uint32)
        out.append((name, t, src, want))
    j = json.load(open(os.path.join(GOLDEN, "mxfp4.json")))
    out.append(("mxfp4", quant.MXFP4, np.frombuffer(bytes.fromhex(j["blocks"]), np.uint8).copy(),
                np.array(j["bits"], np.uint32)))
    return out


@pytest.mark.parametrize("case", _golden_cases(), ids=lambda c: c[0])
def test_dequant_matches_golden_bits(dev, devbuf, case):
    """libggml / gguf-py vectors held by the reference's tests, uint32 equality."""
    _, t, src, want = case
    sd = devbuf(src)
    out = devbuf(shape=(want.size,), dtype=np.float32, fill=123.0)
    assert dev.dequant_dev(t, sd.ptr, out.ptr, want.size)
    dev.synchronize()
    got = out.get().view(np.uint32)
    assert np.array_equal(got, want), f"{np.sum(got != want)} of {want.size} bit patterns differ"


@pytest.mark.parametrize("t", TYPES + [quant.MXFP4])
def test_dequant_planted_scales_bit_exact(dev, devbuf, t):
    """Random bytes with planted extreme scales (subnormal .. largest finite f16)."""
    k, rows = 1024, 33
    src = synth.random_weights(t, rows, k, seed=5)
    want = oracle.dequant(t, src, rows * k).view(np.uint32)
    sd = devbuf(src)
    out = devbuf(shape=(rows * k,), dtype=np.float32, fill=1.0)
    assert dev.dequant_dev(t, sd.ptr, out.ptr, rows * k)
    dev.synchronize()
    assert np.array_equal(out.get().view(np.uint32), want)


def _like_for_like(t, w, x, nrows, k, window):
    q, a_s, _ = oracle.quantize_act(x, window)
    return oracle.matvec_q8act_f64(t, w, q, a_s, nrows, k)


SHAPES = [(1, 256), (37, 512), (300, 1024), (64, 2048), (1000, 4096), (129, 14336)]


@pytest.mark.parametrize("t", TYPES)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("weights", ["normal", "planted"])
def test_matvec_fused_vs_oracle(dev, devbuf, t, shape, weights):
    nrows, k = shape
    window = 256 if t in quant.K_QUANTS else 32
    dev.SetActWindow(window)
    if weights == "normal":
        w = synth.quantized_weights(t, nrows, k, seed=nrows + k)
    else:
        w = synth.random_weights(t, nrows, k, seed=nrows)
    x = synth.activations(k, seed=k)
    want = _like_for_like(t, w, x, nrows, k, window)
    wd, xd = devbuf(w), devbuf(x)
    out = devbuf(shape=(nrows + 8,), dtype=np.float32, fill=np.float32(7e30))  # poisoned
    for call in range(2):  # a second call into the same buffer
        assert dev.matvec_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k)
        dev.synchronize()
        got = out.get()
        assert np.all(got[nrows:] == np.float32(7e30)), "wrote past nrows"
        e = nmse(got[:nrows], want)
        assert e <= 1e-10, f"call {call}: NMSE {e:.3e} vs like-for-like f64"
        assert rel_l2(got[:nrows], want) <= 1e-3
    if weights == "normal" and nrows >= 64:  # a statistical bar: needs rows to average over
        ref32 = oracle.matvec_f64(t, w, x, nrows, k)
        assert nmse(got[:nrows], ref32) <= 1e-3, "vs f32-activation oracle"
    dev.SetActWindow(32)


@pytest.mark.parametrize("t", TYPES)
def test_matvec_every_kernel_shape(dev, devbuf, t):
    """Each (rows per wavefront, workgroup, grid) variant computes the same rows."""
    window = 32
    dev.SetActWindow(window)
    for nrows, k in [(75, 2048), (530, 4096), (70, 8192)]:
        w = synth.random_weights(t, nrows, k, seed=k)
        x = synth.activations(k, seed=3)
        want = _like_for_like(t, w, x, nrows, k, window)
        wd, xd = devbuf(w), devbuf(x)
        for rpw in (1, 2, 4):
            for block in (64, 256, 512, 1024):
                for grid in (0, 1, 3):
                    dev.set_tuning(rpw=rpw, block=block, grid=grid)
                    out = devbuf(shape=(nrows,), dtype=np.float32, fill=np.float32(-3e33))
                    assert dev.matvec_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k)
                    dev.synchronize()
                    e = nmse(out.get(), want)
                    assert e <= 1e-10, f"{nrows}x{k} rpw={rpw} block={block} grid={grid}: {e:.3e}"
    dev.set_tuning(rpw=0, block=0, grid=0)


@pytest.mark.parametrize("shape", [(300, 1024), (129, 14336), (70, 4160), (37, 96), (16 * 256 + 40, 2176)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_matvec_q8_0_both_row_forms(dev, devbuf, shape):
    """Q8_0 rows in both forms of the kernel: two blocks a lane-slot with every load 4-byte
    aligned (the library's pick when the rows are 4-byte aligned and hold an even number of
    blocks: here every k but 96 and every base but the odd one) and one block a slot
    (tuning matvec.q8pair = 2, also what a base that is only 2-byte aligned falls back to).
    Each against the oracle, both windows, planted scales, every rows-per-wavefront variant."""
    nrows, k = shape
    t = quant.Q8_0
    w = synth.random_weights(t, nrows, k, seed=nrows + k)
    x = synth.activations(k, seed=k + 1)
    wd, xd = devbuf(w), devbuf(x)
    shifted = devbuf(shape=(w.size + 16,), dtype=np.uint8, fill=0)     # the same bytes two bytes further on
    shifted.put(np.concatenate([np.zeros(2, np.uint8), w, np.zeros(14, np.uint8)]))
    for window in (32, 256):
        dev.SetActWindow(window)
        want = _like_for_like(t, w, x, nrows, k, window)
        for pair, base, rpw in [(0, wd.ptr, 0), (2, wd.ptr, 0), (0, shifted.ptr + 2, 0), (0, wd.ptr, 2), (0, wd.ptr, 4)]:
            dev.set_tuning(q8pair=pair, rpw=rpw)
            out = devbuf(shape=(nrows + 8,), dtype=np.float32, fill=np.float32(7e30))
            assert dev.matvec_dev(out.ptr, t, base, xd.ptr, nrows, k)
            dev.synchronize()
            got = out.get()
            assert np.all(got[nrows:] == np.float32(7e30)), "wrote past nrows"
            e = nmse(got[:nrows], want)
            assert e <= 1e-10, f"window {window} q8pair={pair} rpw={rpw} base%4={base % 4}: NMSE {e:.3e}"
            out.free()
    dev.set_tuning(q8pair=0, rpw=0)
    dev.SetActWindow(32)


@pytest.mark.parametrize("t", TYPES)
def test_matvec_split_equals_fused(dev, devbuf, t):
    """Quantizer kernel + matvec over its output == the fused kernel, bit for bit."""
    nrows, k, window = 200, 4096, 32
    dev.SetActWindow(window)
    w = synth.quantized_weights(t, nrows, k, seed=9)
    x = synth.activations(k, seed=10)
    wd, xd = devbuf(w), devbuf(x)
    q = devbuf(shape=(k,), dtype=np.int8)
    a_s = devbuf(shape=(k // 32,), dtype=np.float32)
    s16 = devbuf(shape=(k // 16,), dtype=np.float32)
    o1 = devbuf(shape=(nrows,), dtype=np.float32, fill=1.0)
    o2 = devbuf(shape=(nrows,), dtype=np.float32, fill=2.0)
    assert dev.quantize_act_dev(xd.ptr, 1, k, q.ptr, a_s.ptr, s16.ptr)
    assert dev.matvec_q8_dev(o1.ptr, t, wd.ptr, q.ptr, a_s.ptr, s16.ptr, nrows, k)
    assert dev.matvec_dev(o2.ptr, t, wd.ptr, xd.ptr, nrows, k)
    dev.synchronize()
    assert np.array_equal(o1.get().view(np.uint32), o2.get().view(np.uint32))


def test_device_seam_host_pointers(dev):
    """nn.Device.MatVec over host memory: served, residency keyed on the pointer, Forget,
    and declines for what it cannot serve."""
    nrows, k, t = 96, 1024, quant.Q4_K
    dev.SetActWindow(256)
    w = synth.quantized_weights(t, nrows, k, seed=1)
    x = synth.activations(k, seed=2)
    want = _like_for_like(t, w, x, nrows, k, 256)
    out = np.full(nrows, np.float32(9e9))
    assert dev.MatVec(out, t, w, x, nrows, k) is True
    assert nmse(out, want) <= 1e-10
    # a second offer of the same pointer reuses the device copy; new activations
    x2 = synth.activations(k, seed=3)
    assert dev.MatVec(out, t, w, x2, nrows, k) is True
    assert nmse(out, _like_for_like(t, w, x2, nrows, k, 256)) <= 1e-10
    # the bytes change under the same pointer: Forget, then the new bytes are used
    w[:] = synth.quantized_weights(t, nrows, k, seed=4)
    dev.Forget(w)
    assert dev.MatVec(out, t, w, x2, nrows, k) is True
    assert nmse(out, _like_for_like(t, w, x2, nrows, k, 256)) <= 1e-10
    dev.Forget(w)
    # batched: x [ntok][k] -> out [ntok][nrows], each token quantized on its own
    ntok = 3
    xs = np.stack([synth.activations(k, seed=20 + i) for i in range(ntok)])
    outs = np.zeros((ntok, nrows), np.float32)
    assert dev.MatMul(outs, t, w, xs, nrows, k, ntok) is True
    for i in range(ntok):
        assert nmse(outs[i], _like_for_like(t, w, xs[i], nrows, k, 256)) <= 1e-10
    dev.Forget(w)
    # declines: an unknown type and a k that is not whole blocks
    assert dev.MatVec(out, 2, w, x, nrows, k) is False          # Q4_0: not served
    assert dev.MatVec(out, t, w, x, nrows, k - 32) is False
    dev.SetActWindow(32)


def test_forget_frees_at_once_when_the_context_is_free(dev):
    """Forget applies at once when no call holds the context (the reference's TryLock branch,
    /root/reference/jit/gpu/tier/forget.go:38-49): the device copy of a forgotten buffer is
    gone -- free device memory is back -- before any other call is made."""
    from jitllm_amd.hipmem import mem_info
    nrows, k, t = 8192, 4096, quant.Q8_0                  # 35 MB of weights
    dev.SetActWindow(32)
    w = synth.random_weights(t, nrows, k, seed=5)
    x = synth.activations(k, seed=6)
    out = np.zeros(nrows, np.float32)
    dev.synchronize()
    free0, _ = mem_info()
    assert dev.MatVec(out, t, w, x, nrows, k) is True
    free1, _ = mem_info()
    assert free0 - free1 >= w.nbytes, "the weights are not resident after the first call"
    dev.Forget(w)
    free2, _ = mem_info()
    assert free2 - free1 >= w.nbytes, "Forget left the device copy allocated"
    assert dev.resident_count() == 0


def test_reserve_shape_on_one_thread_does_not_switch_off_another_threads_launches(dev, devbuf):
    """jl_reserve_shape walks a launch path with launching switched off.  That state belongs to
    the call, not to the context: a matvec another thread enqueues meanwhile on the same
    context must still be launched.  One thread reserves shapes in a loop, the other runs
    matvecs into a poisoned buffer and checks every one."""
    import threading
    nrows, k, t, window = 300, 1024, quant.Q4_K, 256
    dev.SetActWindow(window)
    w = synth.quantized_weights(t, nrows, k, seed=2)
    x = synth.activations(k, seed=3)
    want = _like_for_like(t, w, x, nrows, k, window)
    wd, xd = devbuf(w), devbuf(x)
    out = devbuf(shape=(nrows,), dtype=np.float32, fill=np.float32(7e30))
    stop = threading.Event()
    errors = []

    def reserver():
        i = 0
        while not stop.is_set():
            try:
                assert dev.reserve_shape(t, 512 + 64 * (i % 5), 4096, 128 + (i % 7))
            except Exception as e:      # noqa: BLE001 - reported by the main thread
                errors.append(e)
                return
            i += 1

    th = threading.Thread(target=reserver)
    th.start()
    try:
        for _ in range(300):
            out.put(np.full(nrows, np.float32(7e30)))
            before = dev.launch_count()
            assert dev.matvec_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k)
            dev.synchronize()
            got = out.get()
            assert np.all(np.abs(got) < 1e30), "a matvec was swallowed by another thread's dry run"
            assert nmse(got, want) <= 1e-10
    finally:
        stop.set()
        th.join(30)
    assert not errors, errors
    dev.SetActWindow(32)
