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
                                   (48, 16, 2880), (33, 300, 64)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("weights", ["normal", "planted"])
@pytest.mark.parametrize("rows", [0, 96, 128], ids=["auto", "tile96", "tile128"])
def test_mxfp4_bf16_matmul_vs_dequant_f32(dev, devbuf, shape, weights, rows):
    """rows = rows per workgroup tile of the tiled GEMM (the library picks per shape; both are
    held to the bar); auto also takes 9..64 tokens to the few-token kernel (16-row
    workgroups, K split over wavefronts; a last group of fewer than four blocks and ragged
    rows are among the shapes)."""
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
