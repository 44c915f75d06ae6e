"""GPU parity at the baseline's full sizes, through the C ABI, with the launch shapes the
library picks by itself at those sizes (and the forced forms beside them).

Decode matvecs are small enough for the oracle to evaluate every row.  For the prefill GEMM
the oracle evaluates a seeded sample of rows -- first, middle and last tiles and both sides of
every boundary where the grid changes kernel -- for ALL tokens, on those rows' own bytes, and
the device checks the rest of the matrix against itself: token t of the GEMM must equal the
decode matvec of token t (/root/reference/engine/nn/packedmm_test.go:15-19,
packedgemm_test.go:32-37,145-164).  Bar: NMSE <= 1e-10 against the f64 evaluation of the same
int8 activations, hence rel-L2 <= 1e-5, inside the stated 1e-3."""
import functools

import numpy as np
import pytest

import oracle
from conftest import nmse
from jitllm_amd import quant, synth
from jitllm_amd.device import Packed

pytestmark = pytest.mark.gpu

POISON = np.float32(3e30)


@functools.lru_cache(maxsize=None)
def _weights(t, nrows, k, kind):
    if kind == "normal":       # N(0, 0.02) through the weight quantizer: the baseline's weights
        return synth.quantized_weights(t, nrows, k, seed=0)
    return synth.random_weights(t, nrows, k, seed=nrows + k)   # random bytes, planted extreme scales


def _like_for_like(t, w, x, nrows, k, window):
    q, a_s, _ = oracle.quantize_act(x, window)
    return oracle.matvec_q8act_f64(t, w, q, a_s, nrows, k)


def _check_rows(got, want, what, chunk=512):
    """Whole-vector NMSE and the worst chunk of `chunk` rows: one workgroup's rows gone wrong
    must not hide in the average."""
    assert np.all(np.abs(got) < 1e30), f"{what}: rows left unwritten"
    e = nmse(got, want)
    assert e <= 1e-10, f"{what}: NMSE {e:.3e}"
    worst = max(nmse(got[i:i + chunk], want[i:i + chunk]) for i in range(0, len(want), chunk)
                if np.any(want[i:i + chunk]))
    assert worst <= 1e-9, f"{what}: worst {chunk}-row chunk NMSE {worst:.3e}"


MATVECS = [
    (quant.Q4_K, 4096, 4096, 256, "normal"),      # the headline configuration
    (quant.Q8_0, 14336, 4096, 32, "normal"),      # gate / up: more than 16 rows a CU
    (quant.Q6_K, 4096, 14336, 32, "planted"),     # down
    (quant.Q6_K, 4096, 14336, 32, "normal"),      # down with the N(0, 0.02) weights the configuration names
    (quant.Q4_K, 14336, 4096, 256, "planted"),
]


@pytest.mark.parametrize("case", MATVECS, ids=lambda c: f"{quant.NAMES[c[0]]}_{c[1]}x{c[2]}_{c[4]}")
def test_decode_matvec_full_size_rows_and_planes(dev, devbuf, case):
    """GGUF rows with the library's own launch shape (a persistent grid of 768-thread
    workgroups once a matrix has more than sixteen rows a CU) and the packed planes of the
    same bytes; every row against the oracle."""
    t, nrows, k, window, kind = case
    dev.SetActWindow(window)
    w = _weights(t, nrows, k, kind)
    x = synth.activations(k, seed=11)
    want = _like_for_like(t, w, x, nrows, k, window)
    wd, xd = devbuf(w), devbuf(x)
    out = devbuf(shape=(nrows + 8,), dtype=np.float32, fill=POISON)
    launches = dev.launch_count()
    assert dev.matvec_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k)
    dev.synchronize()
    assert dev.launch_count() == launches + 1
    got = out.get()
    assert np.all(got[nrows:] == POISON), "wrote past nrows"
    _check_rows(got[:nrows], want, "rows")
    # the same bytes as planes, packed on the device
    pl = [devbuf(shape=(max(n, 1),), dtype=np.uint32, fill=0) for n in dev.packed_words(t, nrows, k)]
    assert dev.pack_weights_dev(t, wd.ptr, nrows, k, pl[0].ptr, pl[1].ptr, pl[2].ptr)
    out2 = devbuf(shape=(nrows + 8,), dtype=np.float32, fill=POISON)
    assert dev.matvec_packed_dev(out2.ptr, t, Packed(pl[0].ptr, pl[1].ptr, pl[2].ptr, 0, nrows), xd.ptr, nrows, k)
    dev.synchronize()
    got2 = out2.get()
    assert np.all(got2[nrows:] == POISON), "planes: wrote past nrows"
    _check_rows(got2[:nrows], want, "planes")
    for b in [wd, xd, out, out2] + pl:
        b.free()
    dev.SetActWindow(32)


@pytest.mark.parametrize("t", [quant.Q4_K, quant.Q8_0, quant.Q6_K])
def test_matvec_persistent_grid_shapes(dev, devbuf, t):
    """More rows than sixteen a CU (so the default is the persistent grid) and the 768-thread
    workgroup forced beside the others (odd and even step counts, several chunks a row), on a
    matrix short enough in K to be cheap."""
    window = 32
    dev.SetActWindow(window)
    nrows, k = 16 * 256 + 200, 2176 if t == quant.Q8_0 else 4352    # 68 slots a row: two chunks, the second ragged
    w = synth.random_weights(t, nrows, k, seed=3)
    x = synth.activations(k, seed=4)
    want = _like_for_like(t, w, x, nrows, k, window)
    wd, xd = devbuf(w), devbuf(x)
    for rpw, block, grid in [(0, 0, 0), (1, 768, 0), (2, 768, 0), (1, 768, 7), (1, 768, 512), (4, 512, 0),
                             (2, 768, 7), (1, 1024, 3)]:
        dev.set_tuning(rpw=rpw, block=block, grid=grid)
        out = devbuf(shape=(nrows + 8,), dtype=np.float32, fill=POISON)
        assert dev.matvec_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k)
        dev.synchronize()
        got = out.get()
        assert np.all(got[nrows:] == POISON)
        _check_rows(got[:nrows], want, f"rpw={rpw} block={block} grid={grid}")
        out.free()
    dev.set_tuning(rpw=0, block=0, grid=0)


def _sample_rows(nrows, rng, boundaries):
    """Rows of the first, a middle and the last 128-row tile, rows either side of every kernel
    boundary, and a few anywhere: about a hundred."""
    picks = set(range(0, 8)) | set(range(nrows - 8, nrows))
    mid = (nrows // 2) // 128 * 128
    picks |= set(range(mid - 4, mid + 4)) | set(range(mid + 60, mid + 68))
    for b in boundaries:
        if 0 < b < nrows:
            picks |= set(range(b - 6, b + 6))
    picks |= set(int(r) for r in rng.integers(0, nrows, 40))
    return np.array(sorted(r for r in picks if 0 <= r < nrows))


# the baseline's sweep {16, 128, 512, 2048} tokens x {4096, 14336} rows
GEMMS = [(16, 4096), (16, 14336), (128, 4096), (128, 14336), (512, 4096), (512, 14336), (2048, 4096), (2048, 14336)]


@pytest.mark.parametrize("shape", GEMMS, ids=lambda s: f"{s[0]}x4096->{s[1]}")
def test_prefill_gemm_full_size(dev, devbuf, shape):
    """The Q4_K prefill GEMM at its real sizes (every point of the baseline's sweep): the library's
    own choice of form (the few-token forms at 16 and 128 tokens x 4096 rows, the 128 x 64 tile
    over the whole of K where the grid is half a round to one round of the chip, the 256 x 128
    tile beyond), then the 256 x 128 tile, the 128 x 64 tile and the whole-K tile forced.
    Sampled rows x all tokens against the oracle; a few tokens whole against the decode
    matvec; the forms against each other."""
    ntok, nrows = shape
    k, t, window = 4096, quant.Q4_K, 256
    dev.SetActWindow(window)
    rng = np.random.default_rng(ntok + nrows)
    w = _weights(t, nrows, k, "normal" if nrows == 4096 else "planted")
    x = rng.standard_normal((ntok, k), np.float32) * (1 + np.arange(ntok, dtype=np.float32)[:, None] % 5)
    x[ntok // 3] = 0                                  # an all-zero token
    # where the automatic form hands rows from the wide kernel to the 64-row tiles
    ntt, nrt = (ntok + 255) // 256, (nrows + 127) // 128
    full, rem = divmod(ntt * nrt, 256)
    split = full * 256 // ntt * 128 if (full >= 1 and 0 < rem <= 128) else 0
    rows = _sample_rows(nrows, rng, [split, 64, 128, nrows - 64])
    rb = quant.row_bytes(t, k)
    w_rows = np.concatenate([w[r * rb:(r + 1) * rb] for r in rows])
    want = oracle.matmul_q8act_f64(t, w_rows, x, len(rows), k, ntok, window)
    wd, xd = devbuf(w), devbuf(x)
    outs = {}
    for form in (0, 2, 1, 6):
        dev.set_tuning(gemm__form=form)
        assert dev.reserve_shape(t, nrows, k, ntok)
        out = devbuf(shape=(ntok * nrows + 16,), dtype=np.float32, fill=POISON)
        assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
        dev.synchronize()
        got = out.get()
        out.free()
        assert np.all(got[ntok * nrows:] == POISON), f"form {form}: wrote past the output"
        got = got[:ntok * nrows].reshape(ntok, nrows)
        assert np.all(np.abs(got) < 1e30), f"form {form}: elements left unwritten"
        sub = got[:, rows]
        e = nmse(sub, want)
        assert e <= 1e-10, f"form {form}: NMSE {e:.3e} on the sampled rows"
        worst = max(nmse(sub[:, j], want[:, j]) for j in range(len(rows)) if np.any(want[:, j]))
        assert worst <= 1e-9, f"form {form}: worst sampled row NMSE {worst:.3e}"
        assert np.all(got[ntok // 3] == 0)
        outs[form] = got
    dev.set_tuning(gemm__form=0)
    # every form sums the same integers and runs the same f32 epilogue, so forms that walk K in
    # one piece agree bit for bit; a form that cuts K (across workgroups, or across the
    # wavefronts of one) adds the super-blocks' terms in another association
    assert np.array_equal(outs[1].view(np.uint32), outs[2].view(np.uint32)), "128 x 64 tiles != 256 x 128 tiles"
    for form in (0, 6):
        assert nmse(outs[form], outs[1].astype(np.float64)) <= 1e-12, f"form {form} vs 128 x 64 tiles"
    k_cut = ntok <= 192 or (128 <= (ntok + 127) // 128 * ((nrows + 63) // 64) <= 256)
    if not k_cut:
        assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)), "automatic form != 128 x 64 tiles"
    # the same weights as packed planes: the tiled forms read them where they lie (no rows are
    # restored first), the same integers and the same epilogue, so the same bits
    pl = [devbuf(shape=(max(n, 1),), dtype=np.uint32, fill=0) for n in dev.packed_words(t, nrows, k)]
    assert dev.pack_weights_dev(t, wd.ptr, nrows, k, pl[0].ptr, pl[1].ptr, pl[2].ptr)
    assert dev.reserve_shape(t, nrows, k, ntok, packed=True)
    outp = devbuf(shape=(ntok * nrows + 16,), dtype=np.float32, fill=POISON)
    n0 = dev.launch_count()
    assert dev.matmul_packed_dev(outp.ptr, t, Packed(pl[0].ptr, pl[1].ptr, pl[2].ptr, 0, nrows), xd.ptr, nrows, k, ntok)
    if ntok > 192:
        assert dev.launch_count() - n0 <= 3, "a launch restored rows in front of the GEMM"
    dev.synchronize()
    gotp = outp.get()
    assert np.all(gotp[ntok * nrows:] == POISON)
    assert np.array_equal(gotp[:ntok * nrows].view(np.uint32), outs[0].reshape(-1).view(np.uint32)), "planes != rows"
    for b_ in pl + [outp]:
        b_.free()
    # token t of the GEMM == the decode matvec of token t, every row
    mv = devbuf(shape=(nrows,), dtype=np.float32, fill=POISON)
    for tok in (0, ntok // 2 + 1, ntok - 1):
        assert dev.matvec_dev(mv.ptr, t, wd.ptr, xd.ptr + tok * k * 4, nrows, k)
        dev.synchronize()
        e = nmse(outs[0][tok], mv.get().astype(np.float64))
        assert e <= 1e-10, f"token {tok}: GEMM vs decode matvec NMSE {e:.3e}"
    for b in (wd, xd, mv):
        b.free()
    dev.SetActWindow(32)


OTHER_GEMMS = [
    # (type, nrows, k, window, tokens): every other prefill GEMM the benchmark times
    (quant.Q8_0, 14336, 4096, 32, 512), (quant.Q8_0, 14336, 4096, 32, 2048),
    (quant.Q6_K, 4096, 14336, 32, 512), (quant.Q6_K, 4096, 14336, 32, 2048),
    (quant.Q6_K, 4096, 14336, 256, 512), (quant.Q6_K, 4096, 14336, 256, 2048),
]


@pytest.mark.parametrize("case", OTHER_GEMMS, ids=lambda c: f"{quant.NAMES[c[0]]}_w{c[3]}_{c[4]}x{c[2]}->{c[1]}")
def test_prefill_gemm_other_types_full_size(dev, devbuf, case):
    """The Llama-3-8B feed-forward matrices at prefill, at their real sizes: Q8_0 gate / up
    with the activation window of 32, Q6_K down with both windows; 512 and 2048 tokens.
    Sampled rows x all tokens against the oracle, and a few tokens whole against the decode
    matvec of the same token."""
    t, nrows, k, window, ntok = case
    dev.SetActWindow(window)
    rng = np.random.default_rng(ntok + nrows + window)
    w = _weights(t, nrows, k, "normal")
    x = rng.standard_normal((ntok, k), np.float32) * (1 + np.arange(ntok, dtype=np.float32)[:, None] % 5)
    x[ntok // 3] = 0
    rows = _sample_rows(nrows, rng, [64, 128, nrows - 64])
    rb = quant.row_bytes(t, k)
    w_rows = np.concatenate([w[r * rb:(r + 1) * rb] for r in rows])
    want = oracle.matmul_q8act_f64(t, w_rows, x, len(rows), k, ntok, window)
    wd, xd = devbuf(w), devbuf(x)
    assert dev.reserve_shape(t, nrows, k, ntok)
    out = devbuf(shape=(ntok * nrows + 16,), dtype=np.float32, fill=POISON)
    n0 = dev.launch_count()
    assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    assert dev.launch_count() - n0 <= 3, "the matrix kernel, not a launch per token"
    got = out.get()
    out.free()
    assert np.all(got[ntok * nrows:] == POISON), "wrote past the output"
    got = got[:ntok * nrows].reshape(ntok, nrows)
    assert np.all(np.abs(got) < 1e30), "elements left unwritten"
    sub = got[:, rows]
    e = nmse(sub, want)
    assert e <= 1e-10, f"NMSE {e:.3e} on the sampled rows"
    worst = max(nmse(sub[:, j], want[:, j]) for j in range(len(rows)) if np.any(want[:, j]))
    assert worst <= 1e-9, f"worst sampled row NMSE {worst:.3e}"
    assert np.all(got[ntok // 3] == 0)
    mv = devbuf(shape=(nrows,), dtype=np.float32, fill=POISON)
    for tok in (0, ntok // 2 + 1, ntok - 1):
        assert dev.matvec_dev(mv.ptr, t, wd.ptr, xd.ptr + tok * k * 4, nrows, k)
        dev.synchronize()
        e = nmse(got[tok], mv.get().astype(np.float64))
        assert e <= 1e-10, f"token {tok}: GEMM vs decode matvec NMSE {e:.3e}"
    for b in (wd, xd, mv):
        b.free()
    dev.SetActWindow(32)


def test_grouping_with_more_than_65535_pairs(dev, devbuf):
    """One hot expert holding more pairs than 16 bits count: the linear-time grouping keeps
    32-bit running counts from 65536 pairs up; start / perm / pos against groupPairs."""
    rows, k_used, n_expert = 70000, 1, 4
    rng = np.random.default_rng(5)
    sel = np.zeros((rows, k_used + 1), np.uint32)
    sel[:, 0] = np.where(rng.random(rows) < 0.97, 2, rng.integers(0, n_expert, rows))
    used, perm, col_e, pos = oracle.group_pairs(sel, rows, k_used, n_expert, 1)
    sd = devbuf(sel)
    start = devbuf(shape=(n_expert + 1,), dtype=np.uint32, fill=0xFFFFFFFF)
    permd = devbuf(shape=(rows * k_used,), dtype=np.uint32, fill=0xFFFFFFFF)
    posd = devbuf(shape=(rows * k_used,), dtype=np.uint32, fill=0xFFFFFFFF)
    assert dev.moe_group_dev(sd.ptr, k_used + 1, rows, k_used, n_expert, start.ptr, permd.ptr, posd.ptr)
    dev.synchronize()
    counts = np.bincount(sel[:, 0], minlength=n_expert)
    assert counts.max() > 65535
    want_start = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    assert used == rows * k_used
    assert np.array_equal(start.get(), want_start)
    assert np.array_equal(permd.get(), perm[:used])
    assert np.array_equal(posd.get(), pos)
