"""Seeded sweeps over shapes the fixed cases do not name: whichever kernel form the library
picks for a shape (decode matvec over rows or planes, per-token loop, few-token kernels,
tiled GEMMs with and without a K split, MXFP4 forms) must meet the same like-for-like bar,
NMSE <= 1e-10 against the f64 evaluation of the same int8 activations (MXFP4: of the same
bf16 activations), and write nothing past its output."""
import numpy as np
import pytest

import oracle
from conftest import nmse
from jitllm_amd import quant, synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(4))
def test_q4k_matmul_any_token_count(dev, devbuf, seed):
    """Q4_K, window 256, library's own choice of form: token counts on both sides of every
    threshold (3, 16/17, 64/65, 128/129, 192/193), ragged rows, K from one super-block up."""
    rng = np.random.default_rng(100 + seed)
    dev.SetActWindow(256)
    for ntok in rng.permutation([1, 2, 3, 7, 16, 17, 33, 64, 65, 100, 128, 129, 192, 193, 260])[:6]:
        ntok = int(ntok)
        nrows = int(rng.integers(1, 400))
        k = 256 * int(rng.integers(1, 9))
        w = synth.random_weights(quant.Q4_K, nrows, k, seed=seed * 97 + ntok) if rng.random() < 0.5 \
            else synth.quantized_weights(quant.Q4_K, nrows, k, seed=seed * 97 + ntok)
        x = (rng.standard_normal((ntok, k)) * rng.choice([1e-3, 1.0, 40.0])).astype(np.float32)
        wd, xd = devbuf(w), devbuf(x)
        out = devbuf(shape=(ntok * nrows + 3,), dtype=np.float32, fill=np.float32(5e30))
        assert dev.matmul_dev(out.ptr, quant.Q4_K, wd.ptr, xd.ptr, nrows, k, ntok)
        dev.synchronize()
        got = out.get()
        assert np.all(got[ntok * nrows:] == np.float32(5e30)), (ntok, nrows, k)
        want = oracle.matmul_q8act_f64(quant.Q4_K, w, x, nrows, k, ntok, 256)
        assert nmse(got[:ntok * nrows].reshape(ntok, nrows), want) <= 1e-10, (ntok, nrows, k)
    dev.SetActWindow(32)


@pytest.mark.parametrize("seed", range(3))
def test_decode_matvec_rows_and_planes(dev, devbuf, seed):
    """Every type, both windows where the type allows, rows and packed planes."""
    rng = np.random.default_rng(200 + seed)
    for _ in range(6):
        t = [quant.Q4_K, quant.Q6_K, quant.Q8_0][int(rng.integers(0, 3))]
        window = 32 if t == quant.Q8_0 else int(rng.choice([32, 256]))
        nrows = int(rng.integers(1, 700))
        k = 256 * int(rng.integers(1, 20)) if t != quant.Q8_0 else 32 * int(rng.integers(1, 150))
        dev.SetActWindow(window)
        w = synth.random_weights(t, nrows, k, seed=int(rng.integers(1 << 30)))
        x = (rng.standard_normal(k) * rng.choice([1e-2, 1.0, 100.0])).astype(np.float32)
        q, a_s, _ = oracle.quantize_act(x, window)
        want = oracle.matvec_q8act_f64(t, w, q, a_s, nrows, k)
        wd, xd = devbuf(w), devbuf(x)
        out = devbuf(shape=(nrows + 2,), dtype=np.float32, fill=np.float32(5e30))
        assert dev.matvec_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k)
        dev.synchronize()
        got = out.get()
        assert np.all(got[nrows:] == np.float32(5e30)) and nmse(got[:nrows], want) <= 1e-10, (t, nrows, k, window)
        qs, d, sc = oracle.pack_weights(t, w, nrows, k)
        pq, pd = devbuf(qs), devbuf(d)
        ps = devbuf(sc) if sc.size else None
        from jitllm_amd.device import Packed
        out2 = devbuf(shape=(nrows + 2,), dtype=np.float32, fill=np.float32(5e30))
        assert dev.matvec_packed_dev(out2.ptr, t, Packed(pq.ptr, pd.ptr, ps.ptr if ps else None, 0, nrows), xd.ptr, nrows, k)
        dev.synchronize()
        got2 = out2.get()
        assert np.all(got2[nrows:] == np.float32(5e30)) and nmse(got2[:nrows], want) <= 1e-10, (t, nrows, k, window)
    dev.SetActWindow(32)


@pytest.mark.parametrize("seed", range(2))
def test_mxfp4_any_token_count(dev, devbuf, seed):
    rng = np.random.default_rng(300 + seed)
    for ntok in rng.permutation([1, 8, 9, 16, 17, 40, 64, 65, 130])[:5]:
        ntok = int(ntok)
        nrows = int(rng.integers(1, 300))
        k = 32 * int(rng.integers(1, 40))
        if k % 8:
            continue
        w = synth.random_weights(quant.MXFP4, nrows, k, seed=seed * 31 + ntok)
        xf32 = rng.standard_normal((ntok, k)).astype(np.float32)
        u = xf32.view(np.uint32).astype(np.uint64)
        xb = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
        xv = (xb.astype(np.uint32) << 16).view(np.float32)
        wdq = oracle.dequant(quant.MXFP4, w, nrows * k).reshape(nrows, k).astype(np.float64)
        want = xv.astype(np.float64) @ wdq.T
        if not np.all(np.isfinite(want)) or np.abs(want).max() > 1e30:
            continue   # planted exponents can overflow f32 in the sum: not a parity question
        dw, dx = devbuf(w), devbuf(xb)
        out = devbuf(shape=(ntok * nrows + 3,), dtype=np.float32, fill=np.float32(2e30))
        assert dev.matmul_mxfp4_bf16_dev(out.ptr, dw.ptr, dx.ptr, nrows, k, ntok)
        dev.synchronize()
        got = out.get()
        assert np.all(got[ntok * nrows:] == np.float32(2e30)), (ntok, nrows, k)
        assert nmse(got[:ntok * nrows].reshape(ntok, nrows), want) <= 1e-10, (ntok, nrows, k)


@pytest.mark.parametrize("seed", range(4))
def test_q6k_q8_0_matmul_any_token_count(dev, devbuf, seed):
    """Q6_K with either activation window, Q8_0 and Q4_K with the window of 32, library's own
    choice of form (per-token loop, grouped dot-product kernel, 128-token tiles with and
    without a K split): token counts on both sides of every threshold, ragged rows, K of one
    stage up, K that is no multiple of 256 for Q8_0."""
    rng = np.random.default_rng(300 + seed)
    for ntok in rng.permutation([1, 2, 3, 8, 9, 17, 33, 64, 100, 128, 129, 260])[:6]:
        ntok = int(ntok)
        t, window = [(quant.Q6_K, 256), (quant.Q6_K, 32), (quant.Q8_0, 32), (quant.Q4_K, 32)][int(rng.integers(0, 4))]
        nrows = int(rng.integers(1, 400))
        k = 256 * int(rng.integers(1, 9)) if t != quant.Q8_0 else 128 * int(rng.integers(1, 17))
        dev.SetActWindow(window)
        w = synth.random_weights(t, nrows, k, seed=seed * 89 + ntok) if rng.random() < 0.5 \
            else synth.quantized_weights(t, nrows, k, seed=seed * 89 + ntok)
        x = (rng.standard_normal((ntok, k)) * rng.choice([1e-3, 1.0, 40.0])).astype(np.float32)
        wd, xd = devbuf(w), devbuf(x)
        out = devbuf(shape=(ntok * nrows + 3,), dtype=np.float32, fill=np.float32(5e30))
        assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
        dev.synchronize()
        got = out.get()
        assert np.all(got[ntok * nrows:] == np.float32(5e30)), (t, window, ntok, nrows, k)
        want = oracle.matmul_q8act_f64(t, w, x, nrows, k, ntok, window)
        assert nmse(got[:ntok * nrows].reshape(ntok, nrows), want) <= 1e-10, (t, window, ntok, nrows, k)
    dev.SetActWindow(32)
