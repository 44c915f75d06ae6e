"""GPU checks of the opt-in folded-scale form of the Q4_K prefill GEMM ("gemm.fold" = 1 for the
matrices jl_fold_admit_dev admits), through the C ABI.

This form is NOT exact: its f16 operands carry the scales, so its bar is the path's stated
tolerance, rel-L2 <= 1e-3 against the f64 evaluation of the same int8 activations
(oracle.matmul_q8act_f64; /root/reference/engine/nn/packedgemm_test.go:145-164 holds the
reference's GEMM to 1e-3 of its matvec loop), measured and printed at every shape of the
baseline's third configuration where the form applies.  Everything around it is exact and is
held to bits: a matrix that is not admitted, was declined (scales that can pass the f16 range)
or was withdrawn runs the exact forms and gives their bits, whatever the key says."""
import numpy as np
import pytest

import oracle
from conftest import rel_l2
from jitllm_amd import quant, synth

pytestmark = pytest.mark.gpu

POISON = np.float32(3e30)
T, WINDOW = quant.Q4_K, 256


def _run(dev, devbuf, wd, xd, nrows, k, ntok):
    out = devbuf(shape=(ntok * nrows + 16,), dtype=np.float32, fill=POISON)
    assert dev.reserve_shape(T, nrows, k, ntok)
    n0 = dev.launch_count()
    assert dev.matmul_dev(out.ptr, T, wd.ptr, xd.ptr, nrows, k, ntok)
    launches = dev.launch_count() - n0
    dev.synchronize()
    got = out.get()
    out.free()
    assert np.all(got[ntok * nrows:] == POISON), "wrote past the output"
    got = got[:ntok * nrows].reshape(ntok, nrows)
    assert np.all(np.abs(got) < 1e30), "elements left unwritten"
    return got, launches


def _sample(nrows, rng):
    picks = set(range(0, 6)) | set(range(nrows - 6, nrows)) | set(range(122, 134))
    picks |= set(int(r) for r in rng.integers(0, nrows, 48))
    return np.array(sorted(r for r in picks if 0 <= r < nrows))


# the third configuration's sweep where the 256 x 128 tile is the library's form (512 tokens x
# 4096 rows runs the whole-K tile and is checked below to keep the exact bits)
SHAPES = [(512, 14336), (2048, 4096), (2048, 14336)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"{s[0]}x4096->{s[1]}")
def test_folded_form_inside_the_tolerance_at_full_size(dev, devbuf, shape):
    ntok, nrows = shape
    k = 4096
    dev.SetActWindow(WINDOW)
    rng = np.random.default_rng(ntok + nrows)
    w = synth.quantized_weights(T, nrows, k, seed=0)          # N(0, 0.02) through the weight quantizer
    x = rng.standard_normal((ntok, k), np.float32) * (1 + np.arange(ntok, dtype=np.float32)[:, None] % 5)
    x[ntok // 3] = 0
    rows = _sample(nrows, rng)
    rb = quant.row_bytes(T, k)
    want = oracle.matmul_q8act_f64(T, np.concatenate([w[r * rb:(r + 1) * rb] for r in rows]), x, len(rows), k, ntok, WINDOW)
    wd, xd = devbuf(w), devbuf(x)
    exact, _ = _run(dev, devbuf, wd, xd, nrows, k, ntok)
    assert dev.fold_admit_dev(T, wd.ptr, nrows, k)
    try:
        for waves in (0, 4, 8):
            dev.set_tuning(gemm__fold=1, gemm__fold_waves=waves)
            got, launches = _run(dev, devbuf, wd, xd, nrows, k, ntok)
            assert launches == 2, "activation prep + one GEMM launch"
            assert np.all(np.isfinite(got))
            e_oracle = rel_l2(got[:, rows], want)
            e_exact = rel_l2(got, exact.astype(np.float64))
            worst_row = max(rel_l2(got[:, r], want[:, j]) for j, r in enumerate(rows) if np.any(want[:, j]))
            worst_tok = max(rel_l2(got[t_], exact[t_].astype(np.float64)) for t_ in range(ntok) if np.any(exact[t_]))
            print(f"\nfolded {ntok}x{k}->{nrows} waves={waves}: rel-L2 vs oracle (sampled rows) {e_oracle:.2e}, "
                  f"vs exact form (all) {e_exact:.2e}, worst sampled row {worst_row:.2e}, worst token {worst_tok:.2e}")
            assert 0 < e_exact, "the folded form was not used"
            assert e_oracle <= 1e-3 and e_exact <= 1e-3
            assert worst_row <= 2e-3 and worst_tok <= 2e-3     # no row or token far off the average
            assert np.all(got[ntok // 3] == 0), "an all-zero token stays zero"
    finally:
        dev.set_tuning(gemm__fold=0, gemm__fold_waves=0)
        dev.forget_range(wd.ptr, w.nbytes)
        for b in (wd, xd):
            b.free()
        dev.SetActWindow(32)


def test_folded_form_ragged_rows_and_tokens(dev, devbuf):
    """Rows and tokens that fill no tile, k short enough for the oracle to take every element."""
    ntok, nrows, k = 600, 2900, 1024
    dev.SetActWindow(WINDOW)
    w = synth.quantized_weights(T, nrows, k, seed=5)
    x = synth.activations(ntok * k, seed=6).reshape(ntok, k)
    want = oracle.matmul_q8act_f64(T, w, x, nrows, k, ntok, WINDOW)
    wd, xd = devbuf(w), devbuf(x)
    dev.set_tuning(gemm__form=2)
    exact, _ = _run(dev, devbuf, wd, xd, nrows, k, ntok)
    assert rel_l2(exact, want) <= 1e-5
    assert dev.fold_admit_dev(T, wd.ptr, nrows, k)
    try:
        for waves in (4, 8):
            dev.set_tuning(gemm__fold=1, gemm__fold_waves=waves)
            got, _ = _run(dev, devbuf, wd, xd, nrows, k, ntok)
            e = rel_l2(got, want)
            print(f"\nfolded ragged waves={waves}: rel-L2 vs oracle {e:.2e}")
            assert 1e-6 < e <= 1e-3
    finally:
        dev.set_tuning(gemm__fold=0, gemm__fold_waves=0, gemm__form=0)
        dev.forget_range(wd.ptr, w.nbytes)
        for b in (wd, xd):
            b.free()
        dev.SetActWindow(32)


def test_folded_form_only_for_admitted_matrices(dev, devbuf):
    """The key alone changes nothing; admission switches the form on for that matrix; planted
    scales that reach the largest f16 are declined; jl_forget withdraws an admission; shapes the
    256 x 128 tile does not serve keep the exact bits."""
    ntok, nrows, k = 2048, 4096, 4096
    dev.SetActWindow(WINDOW)
    x = np.random.default_rng(3).standard_normal((ntok, k), np.float32)
    w_ok = synth.quantized_weights(T, nrows, k, seed=0)
    w_big = synth.random_weights(T, nrows, k, seed=nrows + k)      # scales up to the largest finite f16
    xd, ok_d, big_d = devbuf(x), devbuf(w_ok), devbuf(w_big)
    try:
        exact_ok, _ = _run(dev, devbuf, ok_d, xd, nrows, k, ntok)
        exact_big, _ = _run(dev, devbuf, big_d, xd, nrows, k, ntok)
        dev.set_tuning(gemm__fold=1)
        got, _ = _run(dev, devbuf, ok_d, xd, nrows, k, ntok)
        assert np.array_equal(got.view(np.uint32), exact_ok.view(np.uint32)), "folded without admission"
        assert not dev.fold_admit_dev(T, big_d.ptr, nrows, k), "planted scales were admitted"
        got, _ = _run(dev, devbuf, big_d, xd, nrows, k, ntok)
        assert np.array_equal(got.view(np.uint32), exact_big.view(np.uint32)), "a declined matrix was folded"
        assert dev.fold_admit_dev(T, ok_d.ptr, nrows, k)
        got, _ = _run(dev, devbuf, ok_d, xd, nrows, k, ntok)
        assert not np.array_equal(got.view(np.uint32), exact_ok.view(np.uint32))
        assert rel_l2(got, exact_ok.astype(np.float64)) <= 1e-3
        # another shape over the same address is another matrix
        got, _ = _run(dev, devbuf, ok_d, xd, nrows - 128, k, ntok)
        dev.set_tuning(gemm__fold=0)
        want, _ = _run(dev, devbuf, ok_d, xd, nrows - 128, k, ntok)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        dev.set_tuning(gemm__fold=1)
        # 512 tokens x 4096 rows runs the whole-K tile: exact, admitted or not
        got, _ = _run(dev, devbuf, ok_d, xd, nrows, k, 512)
        dev.set_tuning(gemm__fold=0)
        want, _ = _run(dev, devbuf, ok_d, xd, nrows, k, 512)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        dev.set_tuning(gemm__fold=1)
        # one super-block's scale rewritten in place to a value that overflows: admitted again
        # by a new call only, and that call declines it
        w_bad = w_ok.copy()
        w_bad[(nrows // 2) * quant.row_bytes(T, k) + 144 * 3:][:2] = np.frombuffer(np.float16(60000).tobytes(), np.uint8)
        ok_d.put(w_bad)
        assert not dev.fold_admit_dev(T, ok_d.ptr, nrows, k)
        ok_d.put(w_ok)
        assert dev.fold_admit_dev(T, ok_d.ptr, nrows, k)
        dev.forget_range(ok_d.ptr, w_ok.nbytes)
        got, _ = _run(dev, devbuf, ok_d, xd, nrows, k, ntok)
        assert np.array_equal(got.view(np.uint32), exact_ok.view(np.uint32)), "folded after jl_forget"
        # other types and shapes are declined, not errors
        assert not dev.fold_admit_dev(quant.Q8_0, ok_d.ptr, nrows, k)
        assert not dev.fold_admit_dev(T, ok_d.ptr + 2, nrows, k)
    finally:
        dev.set_tuning(gemm__fold=0)
        for b in (xd, ok_d, big_d):
            b.free()
        dev.SetActWindow(32)
