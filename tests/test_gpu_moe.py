"""GPU parity of the grouped expert matmul (mixture-of-experts block) against the CPU
oracle, through the C ABI.

Stages are checked on their own so each is like-for-like: grouping is integer work
(bit-exact against the oracle's groupPairs), each grouped matvec is held to NMSE
<= 1e-10 against the f64 evaluation of the same int8 activations, the combine to the
same sums in the same order; the whole block to rel-L2 <= 1e-3 against a pure-oracle
evaluation (the down projection re-quantizes act(gate)*up, so a last-bit difference in
gate/up can move an int8: the block is not a like-for-like quantity)."""
import functools

import numpy as np
import pytest

import oracle
from conftest import nmse, rel_l2
from jitllm_amd import quant, synth

pytestmark = pytest.mark.gpu


def route(rows, n_expert, k_used, seed, mode="random"):
    rng = np.random.default_rng(seed)
    sel = np.zeros((rows, k_used + 1), np.uint32)
    wt = np.zeros((rows, k_used), np.float32)
    for r in range(rows):
        logits = rng.standard_normal(n_expert).astype(np.float32)
        if mode == "one_expert":
            logits[:] = -30
            logits[5:5 + k_used] = 10 + np.arange(k_used)[::-1]
        elif mode == "mostly_empty":
            logits[k_used + 1:] -= 40
        s, w, _, _ = oracle.moe_route(logits, k_used)
        sel[r, :k_used], wt[r] = s, w
    return sel, wt


def silu(g):
    g = g.astype(np.float64)
    return g / (1 + np.exp(-g))


@pytest.mark.parametrize("form", [1, 2], ids=["every_pair_every_expert", "linear"])
@pytest.mark.parametrize("mode,rows,n_expert,k_used", [("random", 12, 16, 4), ("one_expert", 9, 16, 2),
                                                       ("mostly_empty", 7, 32, 3), ("random", 5, 8, 1),
                                                       ("random", 64, 128, 8), ("random", 300, 60, 6),
                                                       ("random", 1, 1000, 16), ("one_expert", 129, 16, 2),
                                                       ("random", 2048, 128, 8), ("random", 700, 1000, 16),
                                                       ("one_expert", 2100, 7, 2), ("random", 2600, 128, 8),
                                                       ("random", 4400, 64, 16)])
def test_grouping_is_bit_exact(dev, devbuf, mode, rows, n_expert, k_used, form):
    """Both forms of the grouping kernel against the oracle's groupPairs: integer work, exact.
    Runs of 64 pairs that end inside a row, more runs than wavefronts (300 x 6 pairs), more
    experts than pairs, every pair on a handful of experts, pair lists of many runs a wavefront
    (16,384 and 20,800 pairs) and past 65,535 pairs (70,400: 32-bit counts) are among the cases."""
    dev.set_tuning(moe__group=form)
    sel, _ = route(rows, n_expert, k_used, 3, mode)
    used, perm, col_e, pos = oracle.group_pairs(sel.reshape(-1), rows, k_used, n_expert, 1)
    assert used == rows * k_used
    want_start = np.searchsorted(col_e[:used], np.arange(n_expert + 1)).astype(np.uint32)
    sd = devbuf(sel)
    start = devbuf(shape=(n_expert + 1,), dtype=np.uint32, fill=99)
    dperm = devbuf(shape=(used,), dtype=np.uint32, fill=99)
    dpos = devbuf(shape=(used,), dtype=np.uint32, fill=99)
    assert dev.moe_group_dev(sd.ptr, k_used + 1, rows, k_used, n_expert, start.ptr, dperm.ptr, dpos.ptr)
    dev.synchronize()
    assert np.array_equal(start.get(), want_start)
    assert np.array_equal(dperm.get(), perm[:used])
    assert np.array_equal(dpos.get(), pos)
    dev.set_tuning(moe__group=0)


@functools.lru_cache(maxsize=8)
def _banks(t, n_expert, nrows, k, seed, planted):
    make = synth.random_weights if planted else synth.quantized_weights
    return np.concatenate([make(t, nrows, k, seed=seed + e) for e in range(n_expert)])


@pytest.mark.parametrize("t,nrows,k,form", [(quant.Q4_K, 96, 2048, 1), (quant.Q4_K, 200, 768, 1),
                                            (quant.Q4_K, 40, 4096, 1), (quant.Q4_K, 96, 2048, 2),
                                            (quant.Q4_K, 300, 768, 2), (quant.Q4_K, 40, 4096, 2),
                                            (quant.Q4_K, 96, 2048, 4), (quant.Q4_K, 300, 768, 4),
                                            (quant.Q4_K, 40, 4096, 4), (quant.Q4_K, 129, 256, 4),
                                            (quant.Q4_K, 96, 2048, 3), (quant.Q4_K, 300, 768, 3),
                                            (quant.Q4_K, 40, 4096, 3), (quant.Q4_K, 129, 256, 3),
                                            (quant.Q8_0, 64, 1024, 0), (quant.Q6_K, 70, 1024, 0),
                                            (quant.Q6_K, 96, 2048, 4), (quant.Q6_K, 300, 768, 4),
                                            (quant.Q6_K, 129, 256, 4), (quant.Q6_K, 96, 2048, 3),
                                            (quant.Q6_K, 300, 768, 3), (quant.Q6_K, 129, 256, 3)])
def test_grouped_matvec_vs_oracle(dev, devbuf, t, nrows, k, form):
    """form 1 = the dot-product kernel, 2 = groups of 32 columns on the matrix cores (Q4_K with
    the k-quant window), 3 = groups of 16 columns, the weights decoded in registers into the
    matrix operand, 4 = the prefill GEMM's 128-column x 64-row tile placed per expert,
    0 = what the library picks."""
    rows, n_expert, k_used, window = 13, 8, 3, 256 if t in quant.K_QUANTS else 32
    dev.SetActWindow(window)
    dev.set_tuning(moe__form=form)
    sel, _ = route(rows, n_expert, k_used, 4)
    sel[0, :k_used] = [1, 2, 3]
    sel[1:12, 0] = 6                      # one expert with 11+ columns: more than one pass of eight
    sel[1:12, 1], sel[1:12, 2] = 0, 7
    used, perm, col_e, pos = oracle.group_pairs(sel.reshape(-1), rows, k_used, n_expert, 1)
    start = np.searchsorted(col_e[:used], np.arange(n_expert + 1)).astype(np.uint32)
    bank0 = _banks(t, n_expert, nrows, k, 10, False)
    bank1 = _banks(t, n_expert, nrows, k, 50, True)
    x = np.stack([synth.activations(k, seed=200 + r) for r in range(rows)])
    sheet = nrows * quant.row_bytes(t, k)
    want0 = np.zeros((used, nrows))
    want1 = np.zeros((used, nrows))
    for c in range(used):
        e = int(col_e[c])
        q, a_s, _ = oracle.quantize_act(x[perm[c]], window)
        want0[c] = oracle.matvec_q8act_f64(t, bank0[e * sheet:(e + 1) * sheet], q, a_s, nrows, k)
        want1[c] = oracle.matvec_q8act_f64(t, bank1[e * sheet:(e + 1) * sheet], q, a_s, nrows, k)
    b0, b1, xd = devbuf(bank0), devbuf(bank1), devbuf(x)
    dstart, dperm = devbuf(start), devbuf(perm[:used].copy())
    o0 = devbuf(shape=(used, nrows), dtype=np.float32, fill=np.float32(4e30))
    o1 = devbuf(shape=(used, nrows), dtype=np.float32, fill=np.float32(4e30))
    # form 1: lanes per row -- the library's pick, then every other width; form 3: the columns
    # quantized by a prep kernel (1), by the matrix kernel itself (2), groups of 32 columns (3)
    for key, values in (("moe__group16", (1, 2, 3)),) if form == 3 else (("moe__lpr", (0, 4, 16, 32, 64)),):
        for v in values:
            dev.set_tuning(**{key: v})
            o0.put(np.full((used, nrows), 4e30, np.float32))
            o1.put(np.full((used, nrows), 4e30, np.float32))
            assert dev.moe_matvec_dev(o0.ptr, o1.ptr, t, b0.ptr, b1.ptr, xd.ptr, None, dperm.ptr, dstart.ptr,
                                      n_expert, used, nrows, k)
            dev.synchronize()
            assert nmse(o0.get(), want0) <= 1e-10 and nmse(o1.get(), want1) <= 1e-10, (key, v)
        dev.set_tuning(**{key: 0})
    # SwiGLU form: column c reads silu(x[c]) * x2[c], no gather
    g = np.stack([synth.activations(k, seed=300 + c) for c in range(used)])
    u = np.stack([synth.activations(k, seed=400 + c) for c in range(used)])
    gd, ud = devbuf(g), devbuf(u)
    assert dev.moe_matvec_dev(o0.ptr, None, t, b0.ptr, None, gd.ptr, ud.ptr, None, dstart.ptr, n_expert, used, nrows, k)
    dev.synchronize()
    got = o0.get()
    h = (silu(g) * u.astype(np.float64)).astype(np.float32)
    for c in range(used):
        e = int(col_e[c])
        q, a_s, _ = oracle.quantize_act(h[c], window)
        want = oracle.matvec_q8act_f64(t, bank0[e * sheet:(e + 1) * sheet], q, a_s, nrows, k)
        assert rel_l2(got[c], want) <= 1e-3     # exp() differs in the last bits: an int8 may move
    dev.SetActWindow(32)
    dev.set_tuning(moe__form=0)


@pytest.mark.parametrize("t", [quant.Q4_K, quant.Q6_K], ids=["q4_k", "q6_k"])
@pytest.mark.parametrize("nrows,k", [(100, 2048), (2048 + 24, 768), (48, 1280)])
def test_sixteen_column_groups_launch_shapes(dev, devbuf, nrows, k, t):
    """Form 3 under every launch shape its tuning keys reach: one to three super-blocks a step (K = 1280
    has five: a ragged last chunk), workgroups of four wavefronts, more row blocks than the library
    would take, every way of preparing the columns; ragged row counts; an expert with 19 columns."""
    window, rows, n_expert, k_used = 256, 21, 5, 2
    dev.SetActWindow(window)
    sel = np.zeros((rows, k_used + 1), np.uint32)
    sel[:, 0], sel[:, 1] = 3, 1
    sel[:2, 0], sel[19:, 1] = 0, 4
    used, perm, col_e, pos = oracle.group_pairs(sel.reshape(-1), rows, k_used, n_expert, 1)
    start = np.searchsorted(col_e[:used], np.arange(n_expert + 1)).astype(np.uint32)
    bank = _banks(t, n_expert, nrows, k, 31, True)
    x = np.stack([synth.activations(k, seed=700 + r) * np.float32(1 + r % 3) for r in range(rows)])
    sheet = nrows * quant.row_bytes(t, k)
    want = np.zeros((used, nrows))
    for c in range(used):
        e = int(col_e[c])
        q, a_s, _ = oracle.quantize_act(x[perm[c]], window)
        want[c] = oracle.matvec_q8act_f64(t, bank[e * sheet:(e + 1) * sheet], q, a_s, nrows, k)
    b, xd, dstart, dperm = devbuf(bank), devbuf(x), devbuf(start), devbuf(perm[:used].copy())
    dev.set_tuning(moe__form=3)
    for g16 in (1, 2, 3):
        for chunk, waves, shares in ((1, 0, 0), (2, 0, 0), (3, 0, 0), (0, 4, 0), (0, 0, 3), (2, 4, 5)):
            dev.set_tuning(moe__group16=g16, moe__chunk=chunk, moe__waves=waves, moe__shares=shares)
            o = devbuf(shape=(used * nrows + 8,), dtype=np.float32, fill=np.float32(4e30))
            assert dev.moe_matvec_dev(o.ptr, None, t, b.ptr, None, xd.ptr, None, dperm.ptr, dstart.ptr, n_expert,
                                      used, nrows, k)
            dev.synchronize()
            got = o.get()
            assert np.all(got[used * nrows:] == np.float32(4e30))
            assert nmse(got[:used * nrows].reshape(used, nrows), want) <= 1e-10, (g16, chunk, waves, shares)
    dev.set_tuning(moe__form=0, moe__group16=0, moe__chunk=0, moe__waves=0, moe__shares=0)
    dev.SetActWindow(32)


@pytest.mark.parametrize("t", [quant.Q4_K, quant.Q6_K], ids=["q4_k", "q6_k"])
@pytest.mark.parametrize("rows", [70, 150])
def test_grouped_matmul_more_than_one_group_of_columns(dev, devbuf, rows, t):
    """An expert chosen by 70 rows has three groups of 32 columns (the last one ragged), by 150
    rows five groups and two tiles of 128 columns; another gets one column, most get none.
    Every form against the oracle (Q6_K sheets: the dot-product kernel, the tile, the
    library's pick)."""
    nrows, k, window = 130, 512, 256
    n_expert, k_used = 6, 2
    dev.SetActWindow(window)
    sel = np.zeros((rows, k_used + 1), np.uint32)
    sel[:, 0], sel[:, 1] = 4, 1
    sel[3, 1] = 5
    used, perm, col_e, pos = oracle.group_pairs(sel.reshape(-1), rows, k_used, n_expert, 1)
    start = np.searchsorted(col_e[:used], np.arange(n_expert + 1)).astype(np.uint32)
    bank = _banks(t, n_expert, nrows, k, 77, True)
    x = np.stack([synth.activations(k, seed=600 + r) * np.float32(1 + r % 5) for r in range(rows)])
    sheet = nrows * quant.row_bytes(t, k)
    want = np.zeros((used, nrows))
    for c in range(used):
        e = int(col_e[c])
        q, a_s, _ = oracle.quantize_act(x[perm[c]], window)
        want[c] = oracle.matvec_q8act_f64(t, bank[e * sheet:(e + 1) * sheet], q, a_s, nrows, k)
    b, xd, dstart, dperm = devbuf(bank), devbuf(x), devbuf(start), devbuf(perm[:used].copy())
    # 13: form 3, fused quantization; 23: form 3, groups of 32 columns
    for form in ((1, 2, 3, 13, 23, 4) if t == quant.Q4_K else (1, 3, 13, 23, 4, 0)):
        dev.set_tuning(moe__form=form % 10, moe__group16={13: 2, 23: 3}.get(form, 1))
        o = devbuf(shape=(used * nrows + 8,), dtype=np.float32, fill=np.float32(4e30))
        assert dev.moe_matvec_dev(o.ptr, None, t, b.ptr, None, xd.ptr, None, dperm.ptr, dstart.ptr, n_expert, used,
                                  nrows, k)
        dev.synchronize()
        got = o.get()
        assert np.all(got[used * nrows:] == np.float32(4e30))
        assert nmse(got[:used * nrows].reshape(used, nrows), want) <= 1e-10, form
    dev.set_tuning(moe__form=0, moe__group16=0)
    dev.SetActWindow(32)


def test_grouped_matmul_more_experts_than_one_work_list_round(dev, devbuf):
    """The work list of groups and tiles is written 1024 experts a round: 1100 experts, columns
    on five of them across the rounds' border, one with two tiles of 128 columns."""
    t, nrows, k, window = quant.Q4_K, 64, 256, 256
    n_expert, k_used, rows = 1100, 2, 140
    dev.SetActWindow(window)
    sel = np.zeros((rows, k_used + 1), np.uint32)
    sel[:, 0], sel[:, 1] = 1023, 1024
    sel[:5, 0], sel[5:9, 1], sel[9, 0] = 3, 1099, 1025
    used, perm, col_e, pos = oracle.group_pairs(sel.reshape(-1), rows, k_used, n_expert, 1)
    start = np.searchsorted(col_e[:used], np.arange(n_expert + 1)).astype(np.uint32)
    bank = np.tile(synth.random_weights(t, nrows, k, seed=9), n_expert)
    sheet = nrows * quant.row_bytes(t, k)
    for e in (3, 1023, 1024, 1025, 1099):   # the sheets in use differ from one another
        bank[e * sheet:(e + 1) * sheet] = synth.random_weights(t, nrows, k, seed=100 + e)
    x = np.stack([synth.activations(k, seed=900 + r) for r in range(rows)])
    want = np.zeros((used, nrows))
    for c in range(used):
        e = int(col_e[c])
        q, a_s, _ = oracle.quantize_act(x[perm[c]], window)
        want[c] = oracle.matvec_q8act_f64(t, bank[e * sheet:(e + 1) * sheet], q, a_s, nrows, k)
    b, xd, dstart, dperm = devbuf(bank), devbuf(x), devbuf(start), devbuf(perm[:used].copy())
    for form in (1, 2, 3, 13, 23, 4):
        dev.set_tuning(moe__form=form % 10, moe__group16={13: 2, 23: 3}.get(form, 1))
        o = devbuf(shape=(used, nrows), dtype=np.float32, fill=np.float32(4e30))
        assert dev.moe_matvec_dev(o.ptr, None, t, b.ptr, None, xd.ptr, None, dperm.ptr, dstart.ptr, n_expert, used,
                                  nrows, k)
        dev.synchronize()
        assert nmse(o.get(), want) <= 1e-10, form
    dev.set_tuning(moe__form=0, moe__group16=0)
    dev.SetActWindow(32)


def test_combine_order_and_values(dev, devbuf):
    rows, n_expert, k_used, n_embd = 10, 16, 4, 300
    sel, wt = route(rows, n_expert, k_used, 8)
    used, perm, col_e, pos = oracle.group_pairs(sel.reshape(-1), rows, k_used, n_expert, 1)
    rng = np.random.default_rng(1)
    y = rng.standard_normal((used, n_embd)).astype(np.float32)
    resid = rng.standard_normal((rows, n_embd)).astype(np.float32)
    want = resid.copy()
    for r in range(rows):                      # ascending expert id, one f32 multiply-add at a time
        for s in np.argsort(sel[r, :k_used], kind="stable"):
            want[r] = (want[r] + (wt[r, s] * y[pos[r * k_used + s]]).astype(np.float32)).astype(np.float32)
    rd, yd, wd, sd, pd = devbuf(resid), devbuf(y), devbuf(wt), devbuf(sel), devbuf(pos)
    assert dev.moe_combine_dev(rd.ptr, yd.ptr, wd.ptr, sd.ptr, k_used + 1, pd.ptr, rows, k_used, n_embd)
    dev.synchronize()
    assert np.array_equal(rd.get().view(np.uint32), want.view(np.uint32))


def _oracle_block(t, gate, up, down, x, sel, wt, n_expert, n_ffn, n_embd, window, td=None):
    rows, k_used = wt.shape
    out = np.zeros((rows, n_embd))
    td = t if td is None else td
    gs, ds = n_ffn * quant.row_bytes(t, n_embd), n_embd * quant.row_bytes(td, n_ffn)
    for e in range(n_expert):                   # expert-major, rows ascending
        for r in range(rows):
            for s in range(k_used):
                if sel[r, s] != e:
                    continue
                q, a_s, _ = oracle.quantize_act(x[r], window)
                g = oracle.matvec_q8act_f64(t, gate[e * gs:(e + 1) * gs], q, a_s, n_ffn, n_embd)
                u = oracle.matvec_q8act_f64(t, up[e * gs:(e + 1) * gs], q, a_s, n_ffn, n_embd)
                h = (silu(g.astype(np.float32)) * u.astype(np.float32)).astype(np.float32)
                qh, ah, _ = oracle.quantize_act(h, window)
                y = oracle.matvec_q8act_f64(td, down[e * ds:(e + 1) * ds], qh, ah, n_embd, n_ffn)
                out[r] += float(wt[r, s]) * y
    return out


@functools.lru_cache(maxsize=None)
def _block_case(shape):
    """Seeded banks, routing, activations and the oracle's value of a whole block (computed once:
    the Qwen3 shape takes the oracle ten seconds)."""
    rows, n_expert, k_used, n_ffn, n_embd = shape
    t, window = quant.Q4_K, 256
    sel, wt = route(rows, n_expert, k_used, 11)
    gate = _banks(t, n_expert, n_ffn, n_embd, 1000, False)
    up = _banks(t, n_expert, n_ffn, n_embd, 2000, False)
    down = _banks(t, n_expert, n_embd, n_ffn, 3000, False)
    x = np.stack([synth.activations(n_embd, seed=500 + r) for r in range(rows)])
    want = _oracle_block(t, gate, up, down, x, sel, wt, n_expert, n_ffn, n_embd, window)
    return sel, wt, gate, up, down, x, want


@pytest.mark.parametrize("shape", [(6, 8, 2, 256, 512), (64, 128, 8, 768, 2048)],
                         ids=["tiny", "qwen3-30b-a3b"])
def test_moe_block_vs_oracle(dev, devbuf, shape):
    """The whole routed feed-forward block; the second case is the Qwen3-30B-A3B shape:
    128 experts of 768x2048 / 2048x768 in Q4_K, 64 rows routed top-8."""
    rows, n_expert, k_used, n_ffn, n_embd = shape
    t, window = quant.Q4_K, 256
    dev.SetActWindow(window)
    sel, wt, gate, up, down, x, want = _block_case(shape)
    gd, ud, dd, xd, sd, wd = devbuf(gate), devbuf(up), devbuf(down), devbuf(x), devbuf(sel), devbuf(wt)
    resid = devbuf(shape=(rows, n_embd), dtype=np.float32, fill=0)
    for call in range(2):
        resid.put(np.zeros((rows, n_embd), np.float32))
        before = dev.launch_count()
        assert dev.moe_ffn_dev(resid.ptr, t, gd.ptr, ud.ptr, dd.ptr, xd.ptr, sd.ptr, k_used + 1, wd.ptr,
                               rows, k_used, n_expert, n_ffn, n_embd)
        dev.synchronize()
        got = resid.get()
        assert rel_l2(got, want) <= 1e-3, f"call {call}: rel-L2 {rel_l2(got, want):.3e}"
        # four columns an expert on average: grouping, two matrix-core launches that quantize
        # their own columns, combine; the tiny case takes the dot-product form (two more launches)
        assert dev.launch_count() - before == (4 if rows == 64 else 6)
    dev.SetActWindow(32)


def test_moe_block_over_host_memory(dev, devbuf):
    """jl_moe_grouped: the routed block with every operand in host memory (banks resident per host
    pointer after the first call, the residual read, accumulated and written back): the oracle's
    block, and the device-pointer call's bits."""
    shape = (6, 8, 2, 256, 512)
    rows, n_expert, k_used, n_ffn, n_embd = shape
    t, window = quant.Q4_K, 256
    dev.SetActWindow(window)
    sel, wt, gate, up, down, x, want = _block_case(shape)
    r0 = synth.activations(rows * n_embd, seed=41).reshape(rows, n_embd)
    gd, ud, dd, xd, sd, wd = devbuf(gate), devbuf(up), devbuf(down), devbuf(x), devbuf(sel), devbuf(wt)
    rd = devbuf(r0)
    assert dev.moe_ffn_dev(rd.ptr, t, gd.ptr, ud.ptr, dd.ptr, xd.ptr, sd.ptr, k_used + 1, wd.ptr, rows, k_used, n_expert,
                           n_ffn, n_embd)
    dev.synchronize()
    same = rd.get()
    n_res = dev.resident_count()
    for call in range(2):
        resid = r0.copy()
        assert dev.MoEGrouped(resid, t, gate, up, down, x, sel, wt, rows, k_used, n_expert, n_ffn, n_embd) is True
        assert np.array_equal(resid.view(np.uint32), same.view(np.uint32))
        assert rel_l2(resid - r0, want) <= 1e-3
        assert dev.resident_count() == n_res + 3          # three banks, uploaded once
    for b in (gate, up, down):
        dev.Forget(b)
    assert dev.resident_count() == n_res
    assert dev.MoEGrouped(r0.copy(), quant.MXFP4, gate, up, down, x, sel, wt, rows, k_used, n_expert, n_ffn, n_embd) is False
    dev.SetActWindow(32)


def test_moe_block_prefill_1024_rows_vs_oracle_on_sampled_rows(dev, devbuf):
    """The Qwen3-30B-A3B block at a prefill batch, the size the benchmark times: 1024 rows routed
    top-8 over 128 experts (64 columns an expert on average: the matrix-core forms with groups of
    32 columns).  A row's output depends on that row alone, so the oracle evaluates a spread
    sample of rows (first, last, and evenly between) through their own eight experts."""
    rows, n_expert, k_used, n_ffn, n_embd = 1024, 128, 8, 768, 2048
    t, window = quant.Q4_K, 256
    dev.SetActWindow(window)
    sel, wt = route(rows, n_expert, k_used, 12)
    gate = _banks(t, n_expert, n_ffn, n_embd, 1000, False)
    up = _banks(t, n_expert, n_ffn, n_embd, 2000, False)
    down = _banks(t, n_expert, n_embd, n_ffn, 3000, False)
    x = np.stack([synth.activations(n_embd, seed=9000 + r) for r in range(rows)])
    sample = np.unique(np.linspace(0, rows - 1, 40).astype(int))
    want = _oracle_block(t, gate, up, down, x[sample], sel[sample], wt[sample], n_expert, n_ffn, n_embd, window)
    gd, ud, dd, xd, sd, wd = devbuf(gate), devbuf(up), devbuf(down), devbuf(x), devbuf(sel), devbuf(wt)
    resid = devbuf(shape=(rows, n_embd), dtype=np.float32, fill=0)
    for call in range(2):
        resid.put(np.zeros((rows, n_embd), np.float32))
        assert dev.moe_ffn_dev(resid.ptr, t, gd.ptr, ud.ptr, dd.ptr, xd.ptr, sd.ptr, k_used + 1, wd.ptr,
                               rows, k_used, n_expert, n_ffn, n_embd)
        dev.synchronize()
        got = resid.get()
        assert np.all(np.isfinite(got))
        assert rel_l2(got[sample], want) <= 1e-3, f"call {call}: rel-L2 {rel_l2(got[sample], want):.3e}"
        worst = max(rel_l2(got[r], want[i]) for i, r in enumerate(sample))
        assert worst <= 2e-3, f"call {call}: worst sampled row rel-L2 {worst:.3e}"
        # rows outside the sample: every one written, and of the size of its neighbours
        norms = np.sqrt(np.mean(got.astype(np.float64) ** 2, axis=1))
        assert norms.min() > 0.05 * np.median(norms) and norms.max() < 20 * np.median(norms)
    dev.SetActWindow(32)


@pytest.mark.parametrize("rows", [6, 70])
def test_moe_block_q6k_down_sheets_vs_oracle(dev, devbuf, rows):
    """Gate and up in Q4_K, down in Q6_K (the mix of a Q4_K_M file), few columns an expert (the
    dot-product kernels) and many (matrix-core tiles of both types)."""
    n_expert, k_used, n_ffn, n_embd, window = 4, 2, 256, 512, 256
    dev.SetActWindow(window)
    sel, wt = route(rows, n_expert, k_used, 21)
    gate = _banks(quant.Q4_K, n_expert, n_ffn, n_embd, 1100, False)
    up = _banks(quant.Q4_K, n_expert, n_ffn, n_embd, 2100, False)
    down = _banks(quant.Q6_K, n_expert, n_embd, n_ffn, 3100, False)
    x = np.stack([synth.activations(n_embd, seed=700 + r) for r in range(rows)])
    want = _oracle_block(quant.Q4_K, gate, up, down, x, sel, wt, n_expert, n_ffn, n_embd, window, quant.Q6_K)
    gd, ud, dd, xd, sd, wd = devbuf(gate), devbuf(up), devbuf(down), devbuf(x), devbuf(sel), devbuf(wt)
    resid = devbuf(shape=(rows, n_embd), dtype=np.float32, fill=0)
    assert dev.moe_ffn_dev(resid.ptr, quant.Q4_K, gd.ptr, ud.ptr, dd.ptr, xd.ptr, sd.ptr, k_used + 1, wd.ptr,
                           rows, k_used, n_expert, n_ffn, n_embd, down_type=quant.Q6_K)
    dev.synchronize()
    assert rel_l2(resid.get(), want) <= 1e-3
    dev.SetActWindow(32)


@pytest.mark.parametrize("case", [(64, 128, 8), (7, 16, 1), (33, 1000, 16), (5, 8, 8), (20, 130, 4), (9, 256, 8), (11, 257, 6)],
                         ids=lambda c: "x".join(map(str, c)))
def test_router_vs_oracle(dev, devbuf, case):
    """The device router against oracle.MoERouter's restatement: the selection (integer work)
    is exact, ties go to the lower index, weights are the same f32 arithmetic on the same
    scores (a score can differ in its last bit only if the f64 sum's last bit differs AND the
    narrowed value sits on a rounding boundary; the test holds exact equality of the weights
    on these seeds)."""
    rows, n_expert, k_used = case
    rng = np.random.default_rng(rows + n_expert)
    logits = rng.standard_normal((rows, n_expert)).astype(np.float32) * 3
    logits[0, :] = 0.25                       # every score equal: indices 0..k-1 in order
    if rows > 2:
        logits[1, ::2] = logits[1, 0]         # many exact ties
        logits[2, :] = -80; logits[2, n_expert - 1] = 5   # one dominant expert, the rest underflow towards zero
    want_sel = np.zeros((rows, k_used), np.uint32)
    want_wt = np.zeros((rows, k_used), np.float32)
    for r in range(rows):
        s, w, _, _ = oracle.moe_route(logits[r], k_used)
        want_sel[r], want_wt[r] = s, w
    ld = devbuf(logits)
    sel = devbuf(shape=(rows, k_used + 1), dtype=np.uint32, fill=0xFFFFFFFF)
    wt = devbuf(shape=(rows, k_used), dtype=np.float32, fill=np.float32(-1))
    assert dev.moe_route_dev(ld.ptr, rows, n_expert, k_used, sel.ptr, k_used + 1, wt.ptr)
    dev.synchronize()
    got_sel, got_wt = sel.get(), wt.get()
    assert np.array_equal(got_sel[:, :k_used], want_sel)
    assert np.all(got_sel[:, k_used] == 0xFFFFFFFF), "wrote past the selection"
    assert np.array_equal(got_wt.view(np.uint32), want_wt.view(np.uint32))
    # declines
    assert dev.moe_route_dev(ld.ptr, rows, 2000, k_used, sel.ptr, k_used + 1, wt.ptr) is False


@pytest.mark.parametrize("form", [1, 8, 0], ids=["row_a_workgroup", "eight_rows_a_workgroup", "auto"])
@pytest.mark.parametrize("case", [(64, 128, 2048, "f32"), (1, 128, 2048, "f16"), (13, 8, 4096, "f16"),
                                  (9, 16, 130, "f32"), (3, 5, 100, "f32"), (300, 130, 1000, "f16"),
                                  (515, 128, 2048, "f32")], ids=lambda c: "x".join(map(str, c)))
def test_router_logits_bit_exact_then_route(dev, devbuf, case, form):
    """The router's own matrix product on the device (kernels.RouterMatVecTok,
    /root/reference/jit/gpu/kernels/moe.go:820-917): f32 arithmetic in that kernel's
    summation order, so the logits must be the oracle's BITS (ragged k, f16 weights and a
    token count that is no multiple of the kernel's token group included); routing the device's logits on
    the device then gives the oracle's routing of the oracle's logits: the mixture block
    needs no host step from x to the selected experts."""
    ntok, n_expert, k, wdt = case
    dev.set_tuning(moe__logits=form)
    rng = np.random.default_rng(ntok * 7 + n_expert)
    w = rng.standard_normal((n_expert, k)).astype(np.float32) * np.float32(0.05)
    x = rng.standard_normal((ntok, k)).astype(np.float32)
    if wdt == "f16":
        wh = w.astype(np.float16).view(np.uint16)
        wd, wtype, want = devbuf(wh), 1, oracle.router_logits(wh, x, n_expert, k, ntok)
    else:
        wd, wtype, want = devbuf(w), 0, oracle.router_logits(w, x, n_expert, k, ntok)
    xd = devbuf(x)
    ld = devbuf(shape=(ntok * n_expert + 3,), dtype=np.float32, fill=np.float32(7e30))
    assert dev.moe_logits_dev(ld.ptr, wtype, wd.ptr, xd.ptr, n_expert, k, ntok)
    dev.synchronize()
    got = ld.get()
    assert np.all(got[ntok * n_expert:] == np.float32(7e30)), "wrote past the logits"
    got = got[:ntok * n_expert].reshape(ntok, n_expert)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    k_used = min(4, n_expert)
    sel = devbuf(shape=(ntok, k_used + 1), dtype=np.uint32, fill=0)
    wt = devbuf(shape=(ntok, k_used), dtype=np.float32, fill=0)
    assert dev.moe_route_dev(ld.ptr, ntok, n_expert, k_used, sel.ptr, k_used + 1, wt.ptr)
    dev.synchronize()
    for t in range(ntok):
        s, wgt, _, _ = oracle.moe_route(want[t], k_used)
        assert np.array_equal(sel.get()[t, :k_used], s.astype(np.uint32))
        assert np.array_equal(wt.get()[t].view(np.uint32), wgt.view(np.uint32))
    # only f32 and f16 router weights are served
    assert dev.moe_logits_dev(ld.ptr, 8, wd.ptr, xd.ptr, n_expert, k, ntok) is False
    dev.set_tuning(moe__logits=0)


def _pack_bank(dev, devbuf, t, bank, n_expert, nrows, k, layout):
    """A GGUF bank -> packed planes on the device.  layout "sheets": every expert's sheet packed
    on its own, plane sets `page` bytes apart as a container's expert pages are
    (/root/reference/format/jlm/write.go:123-180); "one": the whole bank packed as one matrix of
    n_expert * nrows rows.  Returns (jl_packed_bank, buffers to keep alive)."""
    sheet = nrows * quant.row_bytes(t, k)
    if layout == "one":
        qs, d, sc = oracle.pack_weights(t, bank, n_expert * nrows, k)
        bufs = [devbuf(qs), devbuf(d), devbuf(sc)]
        return dev.packed_bank(bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, 0, n_expert * nrows), bufs
    nq, nd, nsc = oracle.packed_words(t, nrows, k)
    o_d, o_sc = 4 * nq, 4 * (nq + nd)
    page = (4 * (nq + nd + nsc) + 4095) // 4096 * 4096 + 4096       # a page size, with slack between sheets
    host = np.full(page * n_expert, 0xA5, np.uint8)                 # poison between the sheets
    for e in range(n_expert):
        qs, d, sc = oracle.pack_weights(t, bank[e * sheet:(e + 1) * sheet], nrows, k)
        base = e * page
        host[base:base + o_d] = qs.view(np.uint8)
        host[base + o_d:base + o_sc] = d.view(np.uint8)
        host[base + o_sc:base + o_sc + 4 * nsc] = sc.view(np.uint8)
    buf = devbuf(host)
    return dev.packed_bank(buf.ptr, buf.ptr + o_d, buf.ptr + o_sc, page, nrows), [buf]


@pytest.mark.parametrize("layout", ["sheets", "one"])
@pytest.mark.parametrize("nrows,k", [(96, 2048), (200, 768), (16, 256)])
def test_grouped_matvec_over_packed_expert_sheets(dev, devbuf, layout, nrows, k):
    """jl_moe_matvec_packed_dev: the banks as packed planes, expert sheets packed on their own a
    page apart (a container's expert pages) or as row ranges of one plane set; both forms (rows
    on lanes with the columns as scalar operands; the matrix-core tile per expert) against the
    oracle over the same bytes, the tile also bit for bit against the tile over the GGUF banks."""
    t, rows, n_expert, k_used, window = quant.Q4_K, 13, 8, 3, 256
    dev.SetActWindow(window)
    sel, _ = route(rows, n_expert, k_used, 4)
    sel[1:12, 0], sel[1:12, 1], sel[1:12, 2] = 6, 0, 7
    used, perm, col_e, pos = oracle.group_pairs(sel.reshape(-1), rows, k_used, n_expert, 1)
    start = np.searchsorted(col_e[:used], np.arange(n_expert + 1)).astype(np.uint32)
    bank0 = _banks(t, n_expert, nrows, k, 10, False)
    bank1 = _banks(t, n_expert, nrows, k, 50, True)
    x = np.stack([synth.activations(k, seed=200 + r) for r in range(rows)])
    sheet = nrows * quant.row_bytes(t, k)
    want0, want1 = np.zeros((used, nrows)), np.zeros((used, nrows))
    for c in range(used):
        e = int(col_e[c])
        q, a_s, _ = oracle.quantize_act(x[perm[c]], window)
        want0[c] = oracle.matvec_q8act_f64(t, bank0[e * sheet:(e + 1) * sheet], q, a_s, nrows, k)
        want1[c] = oracle.matvec_q8act_f64(t, bank1[e * sheet:(e + 1) * sheet], q, a_s, nrows, k)
    pb0, keep0 = _pack_bank(dev, devbuf, t, bank0, n_expert, nrows, k, layout)
    pb1, keep1 = _pack_bank(dev, devbuf, t, bank1, n_expert, nrows, k, layout)
    xd, dstart, dperm = devbuf(x), devbuf(start), devbuf(perm[:used].copy())
    o0 = devbuf(shape=(used * nrows + 8,), dtype=np.float32, fill=np.float32(4e30))
    o1 = devbuf(shape=(used * nrows + 8,), dtype=np.float32, fill=np.float32(4e30))
    # the dot-product form over planes, the library's pick, groups of sixteen columns (columns from a
    # prep kernel, then quantized by the matrix kernel itself), then the tile
    for form in (1, 0, 3, 13, 23, 4):
        dev.set_tuning(moe__form=form % 10, moe__group16={3: 1, 13: 2, 23: 3}.get(form, 0))
        o0.put(np.full(used * nrows + 8, 4e30, np.float32))
        o1.put(np.full(used * nrows + 8, 4e30, np.float32))
        assert dev.moe_matvec_packed_dev(o0.ptr, o1.ptr, t, pb0, pb1, xd.ptr, None, dperm.ptr, dstart.ptr, n_expert,
                                         used, nrows, k)
        dev.synchronize()
        g0, g1 = o0.get(), o1.get()
        assert np.all(g0[used * nrows:] == np.float32(4e30)) and np.all(g1[used * nrows:] == np.float32(4e30))
        assert nmse(g0[:used * nrows].reshape(used, nrows), want0) <= 1e-10, form
        assert nmse(g1[:used * nrows].reshape(used, nrows), want1) <= 1e-10, form
    dev.set_tuning(moe__form=0, moe__group16=0)
    # the tile form over the same weights as GGUF banks: the same integers, the same epilogue
    b0, b1 = devbuf(bank0), devbuf(bank1)
    r0 = devbuf(shape=(used * nrows,), dtype=np.float32, fill=0)
    r1 = devbuf(shape=(used * nrows,), dtype=np.float32, fill=0)
    dev.set_tuning(moe__form=4)
    assert dev.moe_matvec_dev(r0.ptr, r1.ptr, t, b0.ptr, b1.ptr, xd.ptr, None, dperm.ptr, dstart.ptr, n_expert, used,
                              nrows, k)
    dev.synchronize()
    dev.set_tuning(moe__form=0)
    assert np.array_equal(g0[:used * nrows].view(np.uint32), r0.get().view(np.uint32))
    assert np.array_equal(g1[:used * nrows].view(np.uint32), r1.get().view(np.uint32))
    # what the plane form does not serve is declined, never approximated
    dev.SetActWindow(32)
    assert not dev.moe_matvec_packed_dev(o0.ptr, None, t, pb0, None, xd.ptr, None, dperm.ptr, dstart.ptr, n_expert,
                                         used, nrows, k)
    assert not dev.moe_matvec_packed_dev(o0.ptr, None, quant.Q6_K, pb0, None, xd.ptr, None, dperm.ptr, dstart.ptr,
                                         n_expert, used, nrows, k)


def test_grouped_matvec_over_the_expert_pages_of_the_reference_written_container(dev, devbuf):
    """The four exp_gate_bank sheets of each block of v29.jlm.gz, uploaded as the file holds them
    (one device copy of the container's bytes, the bank addressed by the entry's plane offsets
    and the header's expert page size, /root/reference/format/jlm/read.go:447-469) and fed to
    the mixture's grouped matvec; the expectation comes from the regenerated GGUF source
    bytes, which are independent of the packing."""
    import os
    from conftest import GOLDEN
    from v29_source import source_tensors
    from jitllm_amd import jlm
    f = jlm.File.open(os.path.join(GOLDEN, "v29.jlm.gz"))
    src = {(n, b): p for n, b, kind, p in source_tensors() if kind == "q4k"}
    t, window = quant.Q4_K, 256
    dev.SetActWindow(window)
    data = np.frombuffer(f.data, np.uint8)
    file_d = devbuf(np.concatenate([data, np.zeros((-len(data)) % 16, np.uint8)]))
    seen = 0
    for e in f.entries:
        if e.name != "exp_gate_bank":
            continue
        n_expert, nrows, k = e.sheets, e.rows, e.k
        assert (n_expert, nrows, k) == (4, 16, 256)
        pb = dev.packed_bank(file_d.ptr + e.qs_off, file_d.ptr + e.d_off, file_d.ptr + e.sc_off, f.exp_page_size, nrows)
        rows, k_used = 9, 2
        sel = np.zeros((rows, k_used + 1), np.uint32)
        sel[:, 0] = np.arange(rows) % n_expert
        sel[:, 1] = (np.arange(rows) + 1 + e.block) % n_expert
        used, perm, col_e, pos = oracle.group_pairs(sel.reshape(-1), rows, k_used, n_expert, 1)
        start = np.searchsorted(col_e[:used], np.arange(n_expert + 1)).astype(np.uint32)
        x = np.stack([synth.activations(k, seed=40 + r) for r in range(rows)])
        bank = src[(e.name, e.block)]
        sheet = nrows * quant.row_bytes(t, k)
        want = np.zeros((used, nrows))
        for c in range(used):
            q, a_s, _ = oracle.quantize_act(x[perm[c]], window)
            ex = int(col_e[c])
            want[c] = oracle.matvec_q8act_f64(t, bank[ex * sheet:(ex + 1) * sheet], q, a_s, nrows, k)
        xd, dstart, dperm = devbuf(x), devbuf(start), devbuf(perm[:used].copy())
        o = devbuf(shape=(used, nrows), dtype=np.float32, fill=np.float32(4e30))
        assert dev.moe_matvec_packed_dev(o.ptr, None, t, pb, None, xd.ptr, None, dperm.ptr, dstart.ptr, n_expert, used,
                                         nrows, k)
        dev.synchronize()
        assert nmse(o.get(), want) <= 1e-10, (e.name, e.block)
        seen += 1
    assert seen == 2
    dev.SetActWindow(32)


@pytest.mark.parametrize("layout", ["sheets", "one"])
@pytest.mark.parametrize("shape", [(6, 8, 2, 256, 512), (64, 128, 8, 768, 2048)], ids=["tiny", "qwen3-30b-a3b"])
def test_moe_block_over_packed_banks_vs_oracle(dev, devbuf, shape, layout):
    """The whole routed feed-forward block with the three banks as packed planes."""
    rows, n_expert, k_used, n_ffn, n_embd = shape
    t, window = quant.Q4_K, 256
    dev.SetActWindow(window)
    sel, wt, gate, up, down, x, want = _block_case(shape)
    pg, k0 = _pack_bank(dev, devbuf, t, gate, n_expert, n_ffn, n_embd, layout)
    pu, k1 = _pack_bank(dev, devbuf, t, up, n_expert, n_ffn, n_embd, layout)
    pd, k2 = _pack_bank(dev, devbuf, t, down, n_expert, n_embd, n_ffn, layout)
    xd, sd, wd = devbuf(x), devbuf(sel), devbuf(wt)
    resid = devbuf(shape=(rows, n_embd), dtype=np.float32, fill=0)
    for call in range(2):
        resid.put(np.zeros((rows, n_embd), np.float32))
        assert dev.moe_ffn_packed_dev(resid.ptr, t, pg, pu, pd, xd.ptr, sd.ptr, k_used + 1, wd.ptr, rows, k_used,
                                      n_expert, n_ffn, n_embd)
        dev.synchronize()
        got = resid.get()
        assert rel_l2(got, want) <= 1e-3, f"call {call}: rel-L2 {rel_l2(got, want):.3e}"
    dev.SetActWindow(32)


@pytest.mark.parametrize("layout", ["rows", "planes"])
@pytest.mark.parametrize("rows", [64, 5])
def test_block_in_one_call_is_router_then_ffn_bit_for_bit(dev, devbuf, layout, rows):
    """jl_moe_block_dev: the logits, router and feed-forward calls in one, bit for bit."""
    t, n_expert, k_used, n_ffn, n_embd = quant.Q4_K, 32, 4, 512, 1024
    dev.SetActWindow(256)
    gate, up = _banks(t, n_expert, n_ffn, n_embd, 1000, False), _banks(t, n_expert, n_ffn, n_embd, 2000, False)
    down = _banks(t, n_expert, n_embd, n_ffn, 3000, False)
    rng = np.random.default_rng(rows)
    router = (rng.standard_normal((n_expert, n_embd)) / np.sqrt(n_embd)).astype(np.float32)
    x = rng.standard_normal((rows, n_embd)).astype(np.float32)
    resid0 = rng.standard_normal((rows, n_embd)).astype(np.float32)
    xd, rd = devbuf(x), devbuf(router)
    if layout == "planes":
        keep = [_pack_bank(dev, devbuf, t, b, n_expert, r, k, "one")
                for b, r, k in ((gate, n_ffn, n_embd), (up, n_ffn, n_embd), (down, n_embd, n_ffn))]
        banks = [kb[0] for kb in keep]
    else:
        keep = [devbuf(gate), devbuf(up), devbuf(down)]
        banks = [b.ptr for b in keep]
    ld = devbuf(shape=(rows, n_expert), dtype=np.float32, fill=0)
    sel = devbuf(shape=(rows, k_used + 1), dtype=np.uint32, fill=0)
    wt = devbuf(shape=(rows, k_used), dtype=np.float32, fill=0)
    want = devbuf(resid0)
    try:
        separate = dev.launch_count()
        assert dev.moe_logits_dev(ld.ptr, 0, rd.ptr, xd.ptr, n_expert, n_embd, rows)
        assert dev.moe_route_dev(ld.ptr, rows, n_expert, k_used, sel.ptr, k_used + 1, wt.ptr)
        if layout == "planes":
            assert dev.moe_ffn_packed_dev(want.ptr, t, banks[0], banks[1], banks[2], xd.ptr, sel.ptr, k_used + 1, wt.ptr,
                                          rows, k_used, n_expert, n_ffn, n_embd)
        else:
            assert dev.moe_ffn_dev(want.ptr, t, banks[0], banks[1], banks[2], xd.ptr, sel.ptr, k_used + 1, wt.ptr, rows,
                                   k_used, n_expert, n_ffn, n_embd)
        separate = dev.launch_count() - separate
        dev.synchronize()
        for i in range(2):
            got = devbuf(resid0)
            sel2 = devbuf(shape=(rows, k_used + 1), dtype=np.uint32, fill=0)
            wt2 = devbuf(shape=(rows, k_used), dtype=np.float32, fill=0)
            before = dev.launch_count()
            assert dev.moe_block_dev(got.ptr, t, banks[0], banks[1], banks[2], rd.ptr, xd.ptr, rows, k_used, n_expert,
                                     n_ffn, n_embd, sel=sel2.ptr, wt=wt2.ptr)
            assert dev.launch_count() == before + separate
            dev.synchronize()
            assert np.array_equal(sel2.get()[:, :k_used], sel.get()[:, :k_used])
            assert np.array_equal(wt2.get().view(np.uint32), wt.get().view(np.uint32))
            assert np.array_equal(got.get().view(np.uint32), want.get().view(np.uint32))
        # the routing kept in the context's own workspace
        got = devbuf(resid0)
        assert dev.moe_block_dev(got.ptr, t, banks[0], banks[1], banks[2], rd.ptr, xd.ptr, rows, k_used, n_expert,
                                 n_ffn, n_embd)
        dev.synchronize()
        assert np.array_equal(got.get().view(np.uint32), want.get().view(np.uint32))
    finally:
        dev.SetActWindow(32)
