"""GPU parity of the Q4_K prefill GEMM against the CPU oracle, through the C ABI.

Bar: NMSE <= 1e-10 (hence rel-L2 <= 1e-5, inside the stated 1e-3) against the f64
evaluation of the SAME per-token int8 activations -- the reference's own bar for a
batched path (/root/reference/engine/nn/packedgemm_test.go:145-164) -- and the
GEMM's token t must equal the decode matvec of token t to the same bar
(/root/reference/engine/nn/packedmm_test.go:15-19)."""
import numpy as np
import pytest

import oracle
from conftest import nmse, rel_l2
from jitllm_amd import quant, synth

pytestmark = pytest.mark.gpu


def _oracle_matmul(t, w, x, nrows, k, ntok, window):
    return oracle.matmul_q8act_f64(t, w, x, nrows, k, ntok, window)


@pytest.mark.parametrize("shape", [(16, 128, 256), (130, 200, 512), (8, 37, 1024), (512, 300, 1024),
                                   (129, 129, 4096)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("weights", ["normal", "planted"])
@pytest.mark.parametrize("form", [1, 2, 3], ids=["tile128x64", "tile256x128", "two_pass"])
def test_gemm_q4k_vs_oracle(dev, devbuf, shape, weights, form):
    """Every form of the kernel: weights dequantized inside the matrix kernel on 128 x 64 and
    on 256 x 128 tiles, and weights expanded once per call into f16 fragments."""
    ntok, nrows, k = shape
    t = quant.Q4_K
    dev.SetActWindow(256)
    dev.set_tuning(gemm__form=form)
    w = (synth.quantized_weights(t, nrows, k, seed=ntok) if weights == "normal"
         else synth.random_weights(t, nrows, k, seed=ntok))
    x = np.stack([synth.activations(k, seed=100 + i) * np.float32(1 + i % 7) for i in range(ntok)])
    x[ntok // 2] = 0                       # an all-zero token: scale 0, inverse 0
    want = _oracle_matmul(t, w, x, nrows, k, ntok, 256)
    wd, xd = devbuf(w), devbuf(x)
    out = devbuf(shape=(ntok * nrows + 16,), dtype=np.float32, fill=np.float32(3e30))
    for call in range(2):
        assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
        dev.synchronize()
        got = out.get()
        assert np.all(got[ntok * nrows:] == np.float32(3e30)), "wrote past the output"
        got = got[:ntok * nrows].reshape(ntok, nrows)
        e = nmse(got, want)
        assert e <= 1e-10, f"call {call}: NMSE {e:.3e}"
        worst = max(nmse(got[i], want[i]) for i in range(ntok) if np.any(want[i]))
        assert worst <= 1e-9, f"worst token NMSE {worst:.3e}"
        assert np.all(got[ntok // 2] == 0)
        assert rel_l2(got, want) <= 1e-3
    dev.SetActWindow(32)
    dev.set_tuning(gemm__form=0)


def test_gemm_forms_agree_bit_for_bit(dev, devbuf):
    """The matrix cores sum the same integers in both forms and the f32 epilogue is the
    same instruction sequence, so all forms must return identical bits; a second
    weight of another shape reuses (and regrows) the expanded-weight workspace."""
    dev.SetActWindow(256)
    t = quant.Q4_K
    for ntok, nrows, k in [(200, 300, 1536), (130, 70, 512), (384, 1000, 2048)]:
        w = synth.random_weights(t, nrows, k, seed=nrows)
        x = np.stack([synth.activations(k, seed=500 + i) for i in range(ntok)])
        wd, xd = devbuf(w), devbuf(x)
        outs = []
        for form in (1, 2, 3):
            dev.set_tuning(gemm__form=form)
            out = devbuf(shape=(ntok, nrows), dtype=np.float32, fill=np.float32(-7e30))
            assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
            dev.synchronize()
            outs.append(out.get())
        for o in outs[1:]:
            assert np.array_equal(outs[0].view(np.uint32), o.view(np.uint32)), (ntok, nrows, k)
    dev.set_tuning(gemm__form=0)
    dev.SetActWindow(32)


def test_gemm_split_grid_agrees_with_single_form(dev, devbuf):
    """A grid of whole rounds plus a last round at most half full is cut: the last round's
    rows go to the 64-row tiles.  1.25 rounds of 256-token x 128-row tiles on 256 CUs
    (and a ragged last tile) against the single-form result, bit for bit; a spot check of
    one token against the oracle."""
    dev.SetActWindow(256)
    t, ntok, k = quant.Q4_K, 256, 256
    nrows = 128 * (256 + 64) + 37
    w = synth.random_weights(t, nrows, k, seed=9)
    x = np.stack([synth.activations(k, seed=900 + i) for i in range(ntok)])
    wd, xd = devbuf(w), devbuf(x)
    outs = []
    for form in (0, 1):
        dev.set_tuning(gemm__form=form)
        out = devbuf(shape=(ntok, nrows), dtype=np.float32, fill=np.float32(-7e30))
        assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
        dev.synchronize()
        outs.append(out.get())
    dev.set_tuning(gemm__form=0)
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    want = _oracle_matmul(t, w, x[5:6], nrows, k, 1, 256)
    assert nmse(outs[0][5:6], want) <= 1e-10
    dev.SetActWindow(32)


@pytest.mark.parametrize("split", [0, 2, 3, 8])
def test_gemm_k_split_vs_oracle(dev, devbuf, split):
    """Few tokens leave most of the chip idle, so K is cut across workgroups and the partial
    sums are added in a fixed order; every split count meets the same bar."""
    dev.SetActWindow(256)
    t, ntok, nrows, k = quant.Q4_K, 20, 150, 2816   # 11 super-blocks: a short last split
    w = synth.random_weights(t, nrows, k, seed=split)
    x = np.stack([synth.activations(k, seed=300 + i) for i in range(ntok)])
    want = _oracle_matmul(t, w, x, nrows, k, ntok, 256)
    wd, xd = devbuf(w), devbuf(x)
    dev.set_tuning(gemm__split=split)
    for call in range(2):
        out = devbuf(shape=(ntok * nrows + 8,), dtype=np.float32, fill=np.float32(4e30))
        assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
        dev.synchronize()
        got = out.get()
        assert np.all(got[ntok * nrows:] == np.float32(4e30))
        assert nmse(got[:ntok * nrows].reshape(ntok, nrows), want) <= 1e-10
    dev.set_tuning(gemm__split=0)
    dev.SetActWindow(32)


def test_gemm_token_equals_decode_matvec(dev, devbuf):
    ntok, nrows, k, t = 40, 256, 2048, quant.Q4_K
    dev.SetActWindow(256)
    w = synth.quantized_weights(t, nrows, k, seed=3)
    x = np.stack([synth.activations(k, seed=i) for i in range(ntok)])
    wd, xd = devbuf(w), devbuf(x)
    og = devbuf(shape=(ntok, nrows), dtype=np.float32, fill=1.0)
    om = devbuf(shape=(ntok, nrows), dtype=np.float32, fill=2.0)
    assert dev.matmul_dev(og.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    for i in range(ntok):
        assert dev.matvec_dev(om.ptr + i * nrows * 4, t, wd.ptr, xd.ptr + i * k * 4, nrows, k)
    dev.synchronize()
    assert nmse(og.get(), om.get()) <= 1e-10
    dev.SetActWindow(32)


@pytest.mark.parametrize("t,window,ntok", [(quant.Q8_0, 32, 2), (quant.Q8_0, 32, 1), (quant.Q6_K, 32, 2), (quant.Q4_K, 32, 2),
                                           (quant.Q4_K, 256, 3)])
def test_matmul_fallback_is_the_per_token_loop(dev, devbuf, t, window, ntok):
    """Types, windows and token counts the GEMM does not take still return the right values."""
    nrows, k = 100, 1024
    dev.SetActWindow(window)
    w = synth.quantized_weights(t, nrows, k, seed=1)
    x = np.stack([synth.activations(k, seed=i) for i in range(ntok)])
    want = _oracle_matmul(t, w, x, nrows, k, ntok, window)
    wd, xd = devbuf(w), devbuf(x)
    out = devbuf(shape=(ntok, nrows), dtype=np.float32, fill=5.0)
    assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    assert nmse(out.get(), want) <= 1e-10
    dev.SetActWindow(32)


@pytest.mark.parametrize("shape", [(16, 4096, 4096), (1, 48, 256), (8, 130, 512), (17, 64, 2304), (33, 200, 1024),
                                   (48, 16, 4096), (64, 1000, 2048), (5, 15, 256)],
                         ids=lambda s: "x".join(map(str, s)))
def test_gemm_few_tokens_vs_oracle(dev, devbuf, shape):
    """Up to 64 tokens: 16-row workgroups on 16x16x32 matrix instructions, K split over the
    eight wavefronts of a workgroup and summed in LDS, weights straight from memory into the
    operand registers.  The inner sums are the same exact integers as in every other form;
    only the order in which super-blocks are added differs (wavefront shares), so the bar is
    the like-for-like one, NMSE <= 1e-10 against the f64 evaluation of the same int8
    activations.  Ragged rows (not a multiple of 16), fewer super-blocks than wavefronts and
    every token-tile count are covered; nothing is written past a token's rows."""
    ntok, nrows, k = shape
    dev.SetActWindow(256)
    dev.set_tuning(gemm__form=4, gemm__min_tok=1)   # also the token counts a matvec loop would take
    w = synth.quantized_weights(quant.Q4_K, nrows, k, seed=ntok + nrows)
    x = np.stack([synth.activations(k, seed=50 + t) for t in range(ntok)])
    x[0, :min(k, 512)] = 0                    # a window of zeros
    if ntok > 2:
        x[2] *= np.float32(37.5)              # tokens of different scale
    wd, xd = devbuf(w), devbuf(x)
    out = devbuf(shape=(ntok * nrows + 5,), dtype=np.float32, fill=np.float32(3e30))
    assert dev.matmul_dev(out.ptr, quant.Q4_K, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    got = out.get()
    assert np.all(got[ntok * nrows:] == np.float32(3e30)), "wrote past the output"
    got = got[:ntok * nrows].reshape(ntok, nrows)
    want = oracle.matmul_q8act_f64(quant.Q4_K, w, x, nrows, k, ntok, 256)
    assert nmse(got, want) <= 1e-10
    for t in (0, ntok - 1):
        assert rel_l2(got[t], oracle.matvec_f64(quant.Q4_K, w, x[t], nrows, k)) <= 1e-2 or np.all(x[t] == 0)
    # the tiled form on the same operands: the same integers, another order of the f32 adds
    if ntok >= 8:
        dev.set_tuning(gemm__form=1, gemm__rows=0)
        out2 = devbuf(shape=(ntok * nrows,), dtype=np.float32, fill=0)
        assert dev.matmul_dev(out2.ptr, quant.Q4_K, wd.ptr, xd.ptr, nrows, k, ntok)
        dev.synchronize()
        assert nmse(got, out2.get().reshape(ntok, nrows)) <= 1e-12
    dev.set_tuning(gemm__form=0, gemm__min_tok=0)
    dev.SetActWindow(32)


@pytest.mark.parametrize("shape", [(128, 4096, 4096), (65, 33, 512), (100, 200, 1024), (300, 64, 768), (128, 31, 256)],
                         ids=lambda s: "x".join(map(str, s)))
def test_gemm_65_to_128_tokens_vs_oracle(dev, devbuf, shape):
    """The few-token scheme on 32x32x16 matrix instructions: 32-row x 64-token workgroups, K
    split over the wavefronts, one launch after the prep.  Chosen when the grid stays small
    (4096 rows: 65..192 tokens); forced here (gemm.form = 5), also for 300 tokens, which
    makes five token groups with a ragged last one.  Same bar as every form: NMSE <= 1e-10 against the f64 evaluation of the same int8
    activations, nothing written past the output, and agreement with the tiled form."""
    ntok, nrows, k = shape
    dev.SetActWindow(256)
    dev.set_tuning(gemm__form=5)
    w = synth.quantized_weights(quant.Q4_K, nrows, k, seed=ntok + nrows)
    x = np.stack([synth.activations(k, seed=70 + t) * np.float32(1 + t % 5) for t in range(ntok)])
    x[ntok // 3] = 0
    wd, xd = devbuf(w), devbuf(x)
    out = devbuf(shape=(ntok * nrows + 5,), dtype=np.float32, fill=np.float32(3e30))
    assert dev.matmul_dev(out.ptr, quant.Q4_K, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    got = out.get()
    assert np.all(got[ntok * nrows:] == np.float32(3e30)), "wrote past the output"
    got = got[:ntok * nrows].reshape(ntok, nrows)
    want = oracle.matmul_q8act_f64(quant.Q4_K, w, x, nrows, k, ntok, 256)
    assert nmse(got, want) <= 1e-10
    assert np.all(got[ntok // 3] == 0)
    dev.set_tuning(gemm__form=1)
    out2 = devbuf(shape=(ntok * nrows,), dtype=np.float32, fill=0)
    assert dev.matmul_dev(out2.ptr, quant.Q4_K, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    assert nmse(got, out2.get().reshape(ntok, nrows)) <= 1e-12
    dev.set_tuning(gemm__form=0)
    dev.SetActWindow(32)


@pytest.mark.parametrize("shape", [(16, 128, 256), (130, 200, 512), (8, 37, 1024), (512, 300, 1024),
                                   (129, 129, 4096), (3, 64, 2816)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("weights", ["normal", "planted"])
def test_gemm_q6k_vs_oracle(dev, devbuf, shape, weights):
    """Q6_K with the k-quant window on the matrix cores: a weight is two f16 operands (the
    int8 sub-block scale is split so that both products are f16 integers), so the sums are the
    oracle's integers.  Planted weights carry random int8 scales, -128 and odd ones included;
    token counts that leave wavefronts of a tile without a token, rows that end inside a tile
    and a grid small enough to be widened along K are among the shapes."""
    ntok, nrows, k = shape
    t = quant.Q6_K
    dev.SetActWindow(256)
    w = (synth.quantized_weights(t, nrows, k, seed=ntok) if weights == "normal"
         else synth.random_weights(t, nrows, k, seed=ntok))
    x = np.stack([synth.activations(k, seed=100 + i) * np.float32(1 + i % 7) for i in range(ntok)])
    x[ntok // 2] = 0                       # an all-zero token: scale 0, inverse 0
    want = _oracle_matmul(t, w, x, nrows, k, ntok, 256)
    wd, xd = devbuf(w), devbuf(x)
    out = devbuf(shape=(ntok * nrows + 16,), dtype=np.float32, fill=np.float32(3e30))
    n0 = dev.launch_count()
    for call in range(2):
        assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
        dev.synchronize()
        got = out.get()
        assert np.all(got[ntok * nrows:] == np.float32(3e30)), "wrote past the output"
        got = got[:ntok * nrows].reshape(ntok, nrows)
        e = nmse(got, want)
        assert e <= 1e-10, f"call {call}: NMSE {e:.3e}"
        worst = max(nmse(got[i], want[i]) for i in range(ntok) if np.any(want[i]))
        assert worst <= 1e-9, f"worst token NMSE {worst:.3e}"
        assert np.all(got[ntok // 2] == 0)
        assert rel_l2(got, want) <= 1e-3
    assert dev.launch_count() - n0 <= 6, "the matrix kernel, not a launch per token"
    dev.SetActWindow(32)


@pytest.mark.parametrize("split", [1, 2, 3, 8])
def test_gemm_q6k_k_split_and_token_loop_agree(dev, devbuf, split):
    """Every K split meets the bar, and the matrix kernel's token t is the decode matvec of
    token t (the per-token loop, tuning gemm.form = 9) to the same bar."""
    dev.SetActWindow(256)
    t, ntok, nrows, k = quant.Q6_K, 20, 150, 2816   # 11 super-blocks: a short last split
    w = synth.random_weights(t, nrows, k, seed=split)
    x = np.stack([synth.activations(k, seed=300 + i) for i in range(ntok)])
    want = _oracle_matmul(t, w, x, nrows, k, ntok, 256)
    wd, xd = devbuf(w), devbuf(x)
    dev.set_tuning(gemm__split=split)
    out = devbuf(shape=(ntok * nrows + 8,), dtype=np.float32, fill=np.float32(4e30))
    assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    got = out.get()
    assert np.all(got[ntok * nrows:] == np.float32(4e30))
    got = got[:ntok * nrows].reshape(ntok, nrows)
    assert nmse(got, want) <= 1e-10
    dev.set_tuning(gemm__split=0, gemm__form=9)
    loop = devbuf(shape=(ntok, nrows), dtype=np.float32, fill=1.0)
    assert dev.matmul_dev(loop.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    assert nmse(got, loop.get()) <= 1e-10
    dev.set_tuning(gemm__form=0)
    dev.SetActWindow(32)


@pytest.mark.parametrize("shape", [(16, 128, 128), (130, 200, 512), (8, 37, 1024), (512, 300, 1024),
                                   (129, 129, 4096), (3, 64, 2816), (40, 70, 384)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("weights", ["normal", "planted"])
@pytest.mark.parametrize("t", [quant.Q8_0, quant.Q6_K, quant.Q4_K], ids=["q8_0", "q6_k", "q4_k"])
def test_gemm_window32_vs_oracle(dev, devbuf, shape, weights, t):
    """Q8_0, Q6_K and Q4_K with the activation window of 32 on the matrix cores: the int8
    products are exact f16 integers (Q6_K: the sub-block scale split over two operands; Q4_K:
    the minimums against the prep's block sums) and the scales enter once per block of 32, so
    the sums are the oracle's.  Token counts that leave
    wavefronts of a tile without a token, rows that end inside a tile, K of one stage, K that
    is no multiple of 256 and grids widened along K are among the shapes."""
    ntok, nrows, k = shape
    if k % quant.block_elems(t):
        pytest.skip("K is not a whole number of this type's blocks")
    dev.SetActWindow(32)
    w = (synth.quantized_weights(t, nrows, k, seed=ntok) if weights == "normal"
         else synth.random_weights(t, nrows, k, seed=ntok))
    x = np.stack([synth.activations(k, seed=100 + i) * np.float32(1 + i % 7) for i in range(ntok)])
    x[ntok // 2] = 0                       # an all-zero token: scale 0, inverse 0
    x[0, 32:64] = 0                        # an all-zero window inside a token
    want = _oracle_matmul(t, w, x, nrows, k, ntok, 32)
    wd, xd = devbuf(w), devbuf(x)
    out = devbuf(shape=(ntok * nrows + 16,), dtype=np.float32, fill=np.float32(3e30))
    n0 = dev.launch_count()
    for call in range(2):
        assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
        dev.synchronize()
        got = out.get()
        assert np.all(got[ntok * nrows:] == np.float32(3e30)), "wrote past the output"
        got = got[:ntok * nrows].reshape(ntok, nrows)
        e = nmse(got, want)
        assert e <= 1e-10, f"call {call}: NMSE {e:.3e}"
        worst = max(nmse(got[i], want[i]) for i in range(ntok) if np.any(want[i]))
        assert worst <= 1e-9, f"worst token NMSE {worst:.3e}"
        assert np.all(got[ntok // 2] == 0)
        assert rel_l2(got, want) <= 1e-3
    assert dev.launch_count() - n0 <= 6, "the matrix kernel, not a launch per token"


@pytest.mark.parametrize("split", [1, 2, 3, 8])
@pytest.mark.parametrize("t", [quant.Q8_0, quant.Q6_K, quant.Q4_K], ids=["q8_0", "q6_k", "q4_k"])
def test_gemm_window32_k_split_and_token_loop_agree(dev, devbuf, split, t):
    """Every K split meets the bar, and the matrix kernel's token t is the decode matvec of
    token t (the per-token loop, tuning gemm.form = 9) to the same bar."""
    dev.SetActWindow(32)
    ntok, nrows = 20, 150
    k = 1408 if t == quant.Q8_0 else 2816   # 11 stages / 11 super-blocks: a short last split
    w = synth.random_weights(t, nrows, k, seed=split)
    x = np.stack([synth.activations(k, seed=300 + i) for i in range(ntok)])
    want = _oracle_matmul(t, w, x, nrows, k, ntok, 32)
    wd, xd = devbuf(w), devbuf(x)
    dev.set_tuning(gemm__split=split)
    out = devbuf(shape=(ntok * nrows + 8,), dtype=np.float32, fill=np.float32(4e30))
    assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    got = out.get()
    assert np.all(got[ntok * nrows:] == np.float32(4e30))
    got = got[:ntok * nrows].reshape(ntok, nrows)
    assert nmse(got, want) <= 1e-10
    dev.set_tuning(gemm__split=0, gemm__form=9)
    loop = devbuf(shape=(ntok, nrows), dtype=np.float32, fill=1.0)
    assert dev.matmul_dev(loop.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    assert nmse(got, loop.get()) <= 1e-10
    dev.set_tuning(gemm__form=0)
