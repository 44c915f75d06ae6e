"""CPU tests: the oracle against the golden vectors the reference's own tests hold,
against independent numpy restatements, and against what the mathematics fixes."""
import json
import os

import numpy as np
import pytest

import oracle
from conftest import GOLDEN, nmse
from jitllm_amd import quant, synth

Q8_0, Q4_K, Q6_K, MXFP4 = quant.Q8_0, quant.Q4_K, quant.Q6_K, quant.MXFP4
ALL = [Q8_0, Q4_K, Q6_K, MXFP4]


# ------------------------------------------------------------------ half codec
def test_half_decode_all_patterns():
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([oracle.half_to_f32(int(h)) for h in allh], np.float32)
    fin = ~np.isnan(want)
    assert np.array_equal(got[fin].view(np.uint32), want[fin].view(np.uint32))
    assert np.all(np.isnan(got[~fin]))


def test_half_encode_round_trips_and_rounds_to_nearest_even():
    allh = np.arange(65536, dtype=np.uint16)
    vals = allh.view(np.float16).astype(np.float32)
    for h, v in zip(allh[::7], vals[::7]):
        if np.isnan(v):
            continue
        assert oracle.f32_to_half(v) == h
    rng = np.random.default_rng(0)
    f = np.concatenate([rng.standard_normal(3000).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 5, 3000),
                        np.array([65504, 65519.99, 65520, 1e-8, 6e-8, 2.98e-8, 0, -0.0], np.float32)])
    want = f.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_half(v) for v in f], np.uint16)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- golden dequant
@pytest.mark.parametrize("name,t", [("q4_k_tiny", Q4_K), ("q6_k_tiny", Q6_K), ("q8_0_gemma", Q8_0),
                                    ("q8_0_minilm", Q8_0), ("q8_0_stories", Q8_0)])
def test_dequant_matches_libggml_golden(name, t):
    """testdata/golden/dequant of the reference: libggml output, compared as uint32
    (/root/reference/convert/gguf/gguf_test.go:251-315)."""
    src = np.fromfile(os.path.join(GOLDEN, name + ".in"), np.uint8)
    want = np.fromfile(os.path.join(GOLDEN, name + ".f32"), np.uint32)
    got = oracle.dequant(t, src, want.size).view(np.uint32)
    assert np.array_equal(got, want)
    assert np.unique(want).size > 16, "degenerate window"


def test_dequant_mxfp4_matches_gguf_py_golden():
    """format/quant/testdata/mxfp4.json of the reference (/root/reference/format/quant/mxfp4_test.go:18-66)."""
    j = json.load(open(os.path.join(GOLDEN, "mxfp4.json")))
    blocks = np.frombuffer(bytes.fromhex(j["blocks"]), np.uint8)
    bits = np.array(j["bits"], np.uint32)
    assert blocks.size == 336 * 17 and bits.size == 336 * 32
    assert np.array_equal(oracle.dequant(MXFP4, blocks, bits.size).view(np.uint32), bits)


def test_block_geometry():
    assert [(oracle.block_elems(t), oracle.block_bytes(t)) for t in ALL] == [(32, 34), (256, 144), (256, 210), (32, 17)]
    for t in ALL:
        assert (oracle.block_elems(t), oracle.block_bytes(t)) == quant.BLOCK[t]


# ------------------------------------------------------------------ packed layout
def test_pack_q4k_matches_planes_written_by_the_reference_writer():
    """v29.jlm.gz was written by the reference's container writer from regenerable source
    bytes; every Q4_K tensor and expert sheet must re-pack to the same bytes."""
    from v29_source import source_tensors
    from jitllm_amd import jlm
    f = jlm.File.open(os.path.join(GOLDEN, "v29.jlm.gz"))
    src = {(n, b): (kind, p) for n, b, kind, p in source_tensors()}
    checked = 0
    for e in f.entries:
        kind, payload = src[(e.name, e.block)]
        if kind == "f32":  # the generator restatement checks itself on the verbatim norms
            got = np.frombuffer(f.data, np.float32, e.k, e.qs_off)
            assert np.array_equal(got.view(np.uint32), payload.view(np.uint32))
        elif kind == "q4k":
            rb = e.rows * quant.row_bytes(Q4_K, e.k)
            for x in range(e.sheets):
                t, qs, d, sc = f.planes(e, x)
                assert t == Q4_K
                mq, md, msc = oracle.pack_weights(Q4_K, payload[x * rb:(x + 1) * rb], e.rows, e.k)
                assert np.array_equal(mq, qs) and np.array_equal(md, d) and np.array_equal(msc, sc)
                checked += 1
    assert checked == 11  # token_embd, 2 attn_k, 2 banks x 4 sheets


Q5_K = 13   # not a type of the matmul path: the one format whose secondary plane the reference wrote into a fixture


def test_dequant_q5k_matches_libggml_golden():
    """testdata/golden/dequant/q5_k_tiny of the reference (libggml on real weights): the oracle's
    Q5_K decoder is only the yardstick for the packed reader below."""
    src = np.fromfile(os.path.join(GOLDEN, "q5_k_tiny.in"), np.uint8)
    want = np.fromfile(os.path.join(GOLDEN, "q5_k_tiny.f32"), np.uint32)
    assert src.size == 32 * 176 and want.size == 8192
    assert np.array_equal(oracle.dequant(Q5_K, src, want.size).view(np.uint32), want)


def test_pack_q5k_secondary_plane_matches_planes_written_by_the_reference_writer():
    """The secondary (high-bit) plane half of packSub
    (/root/reference/jit/gpu/kernels/pack.go:229-235), which Q6_K shares with two bits a
    weight, against bytes the reference's own writer produced: both attn_q tensors and the
    eight exp_down_bank sheets of v29.jlm.gz are Q5_K (4-bit primary + 1-bit secondary plane,
    D word, 96-bit SC stream) and must re-pack to the same bytes."""
    from v29_source import source_tensors
    from jitllm_amd import jlm
    f = jlm.File.open(os.path.join(GOLDEN, "v29.jlm.gz"))
    src = {(n, b): (kind, p) for n, b, kind, p in source_tensors()}
    checked = 0
    for e in f.entries:
        kind, payload = src[(e.name, e.block)]
        if kind != "q5k":
            continue
        assert e.type == 7                      # Q5S, /root/reference/format/jlm/schema.go:25-58
        nq, nd, nsc = oracle.packed_words(Q5_K, e.rows, e.k)
        assert (nq, nd, nsc) == (e.rows * 8 * 5, e.rows, e.rows * 3)
        rb = e.rows * oracle.row_bytes(Q5_K, e.k)
        for x in range(e.sheets):
            x0 = x * f.exp_page_size if e.sheets > 1 else 0
            qs = np.frombuffer(f.data, np.uint32, nq, e.qs_off + x0)
            d = np.frombuffer(f.data, np.uint32, nd, e.d_off + x0)
            sc = np.frombuffer(f.data, np.uint32, nsc, e.sc_off + x0)
            mq, md, msc = oracle.pack_weights(Q5_K, payload[x * rb:(x + 1) * rb], e.rows, e.k)
            assert np.array_equal(md, d) and np.array_equal(msc, sc)
            # primary words 0..3 and the secondary word 4 of every sub-block, separately
            mq5, qs5 = mq.reshape(-1, 5, e.rows), qs.reshape(-1, 5, e.rows)
            assert np.array_equal(mq5[:, :4], qs5[:, :4]), "primary plane"
            assert np.array_equal(mq5[:, 4], qs5[:, 4]), "secondary plane"
            assert np.any(qs5[:, 4] != 0)
            # and the reader of the secondary plane: the reference-written planes read back
            # to what Dequant32 gives for the source blocks
            for r in (0, e.rows - 1):
                got = oracle.row_packed(Q5_K, qs, d, sc, r, e.rows, e.k)
                want = oracle.dequant(Q5_K, payload[x * rb:(x + 1) * rb], e.rows * e.k)[r * e.k:(r + 1) * e.k]
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
            checked += 1
    assert checked == 10  # 2 attn_q, 2 banks x 4 sheets


def test_row_packed_q5k_reads_the_golden_values_back():
    """pack -> RowPacked over the libggml golden blocks (k = 512: two super-blocks a row, so the
    cross-super strides the k = 256 fixture cannot show are exercised) gives the golden bits:
    writer and reader of the secondary plane agree with each other AND with libggml."""
    src = np.fromfile(os.path.join(GOLDEN, "q5_k_tiny.in"), np.uint8)
    want = np.fromfile(os.path.join(GOLDEN, "q5_k_tiny.f32"), np.uint32)
    for k in (256, 512, 2048):
        nrows = 8192 // k
        qs, d, sc = oracle.pack_weights(Q5_K, src, nrows, k)
        for r in range(nrows):
            got = oracle.row_packed(Q5_K, qs, d, sc, r, nrows, k)
            assert np.array_equal(got.view(np.uint32), want[r * k:(r + 1) * k]), (k, r)


def test_packed_words_closed_form():
    """Bytes per 256 weights: Q4_K 144 (= GGUF), Q6_K 212, Q8_0 8*34, MXFP4 8*17
    (/root/reference/internal/oracle/packed_test.go:177-213)."""
    for t, per256 in [(Q4_K, 144), (Q6_K, 212), (Q8_0, 272), (MXFP4, 136)]:
        for nrows, k in [(8, 256), (300, 512), (16, 2048)]:
            nq, nd, nsc = oracle.packed_words(t, nrows, k)
            assert (nq + nd + nsc) * 4 == nrows * k // 256 * per256
            assert (nq, nd, nsc) == quant.packed_words(t, nrows, k)
    # a ragged row count rounds the shared d words up
    assert oracle.packed_words(Q8_0, 9, 512)[1] == 16 * 5
    assert oracle.packed_words(MXFP4, 9, 512)[1] == 16 * 3


def _numpy_row_reader(t, qs, d, sc, r, nrows, k):
    """An independent, vectorised reader of one row of the planes, written from the layout
    description rather than from the oracle's loops.  Its indexing is also what the reference's
    own independent gate restates (/root/reference/jit/gpu/kernels/realpack_test.go:67-195,
    checkPack: "restated, not called"): the Q8_0 D word at sup*((nrows+1)/2) + r/2 with the odd
    row in the high half (:109-116), the MXFP4 D byte r%4 of word sup*((nrows+3)/4) + r/4 shifted
    left 23 (:101-107), the Q6_K scale byte (si%4) of word si/4 plus the offset -128 (:138-146),
    the secondary plane's bit position (:181-187).  So the packer's text (pack.go) and a second
    statement inside the reference both agree with what is checked here."""
    P = quant.PACKED[t]
    sub, words = P["sub"], P["words"]
    nsub = k // sub
    w = qs.reshape(nsub, words, nrows)[:, :, r]                     # [nsub][words]
    by = (w[:, :, None] >> (8 * np.arange(4))[None, None, :]) & 0xFF  # bytes [nsub][words][4]
    if t == Q8_0:
        q = by.reshape(nsub, 32).astype(np.int8).astype(np.float64)
        dw = d.reshape(nsub, (nrows + 1) // 2)[:, r // 2]
        scale = ((dw >> (16 * (r % 2))) & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float64)
        return (q * scale[:, None]).reshape(-1)
    if t == MXFP4:
        b = by.reshape(nsub, 16)
        codes = np.concatenate([b & 0xF, b >> 4], axis=1)
        table = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.float64)
        dw = d.reshape(nsub, (nrows + 3) // 4)[:, r // 4]
        e = (dw >> (8 * (r % 4))) & 0xFF
        scale = (e.astype(np.uint32) << 23).view(np.float32).astype(np.float64)
        return (table[codes] * scale[:, None]).reshape(-1)
    if t == Q4_K:
        b = by.reshape(nsub, 16)
        q = np.concatenate([b & 0xF, b >> 4], axis=1).astype(np.float64)
        nsup = nsub // 8
        dw = d.reshape(nsup, nrows)[:, r]
        dd = (dw & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32)
        dm = (dw >> 16).astype(np.uint16).view(np.float16).astype(np.float32)
        st = sc.reshape(nsup, 3, nrows)[:, :, r]
        # the sixteen 6-bit fields are one 96-bit little-endian integer per super-block
        stream = [int(a0) | (int(a1) << 32) | (int(a2) << 64) for a0, a1, a2 in st]
        out = np.empty((nsub, 32))
        for s in range(8):
            scv = np.array([(v >> (12 * s)) & 63 for v in stream], np.float32)
            mv = np.array([(v >> (12 * s + 6)) & 63 for v in stream], np.float32)
            sl = slice(s, nsub, 8)
            out[sl] = (dd * scv).astype(np.float32)[:, None] * q[sl] - (dm * mv).astype(np.float32)[:, None]
        return out.reshape(-1)
    if t == Q6_K:
        lo = by[:, 0:2, :].reshape(nsub, 8)
        prim = np.concatenate([lo & 0xF, lo >> 4], axis=1)            # elems 0..15
        hb = by[:, 2, :]                                               # [nsub][4]
        l = np.arange(16)
        hi2 = (hb[:, l % 4] >> (2 * (l // 4))) & 3
        q = (prim | (hi2 << 4)).astype(np.float64) - 32
        nsup = nsub // 16
        dd = (d.reshape(nsup, nrows)[:, r] & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32)
        sw = sc.reshape((nsub + 3) // 4, nrows)[:, r]
        si = np.arange(nsub)
        scb = ((sw[si // 4] >> (8 * (si % 4))) & 0xFF).astype(np.int32) - 128
        scale = (np.repeat(dd, 16) * scb.astype(np.float32)).astype(np.float32)
        return (scale[:, None].astype(np.float64) * q).reshape(-1)
    raise AssertionError


@pytest.mark.parametrize("t", ALL)
@pytest.mark.parametrize("shape", [(9, 512), (300, 512), (5, 2048)])
def test_pack_round_trip_and_independent_reader(t, shape):
    """RowPacked(pack(src)) == Dequant32(src) (/root/reference/internal/oracle/packed_test.go:54-114),
    and a second reader written from the layout description agrees on every row checked."""
    nrows, k = shape
    src = synth.random_weights(t, nrows, k, seed=nrows)
    want = oracle.dequant(t, src, nrows * k).reshape(nrows, k)
    qs, d, sc = oracle.pack_weights(t, src, nrows, k)
    for r in sorted({0, 1, nrows // 2, nrows - 1}):
        got = oracle.row_packed(t, qs, d, sc, r, nrows, k)
        assert np.array_equal(got, want[r]), f"row {r}"     # value equality (Q6_K's -0.0 reads back +0.0)
        ind = _numpy_row_reader(t, qs, d, sc, r, nrows, k)
        assert nmse(ind, want[r]) < 1e-12, f"independent reader, row {r}"


def test_pack_round_trip_on_golden_blocks():
    for name, t in [("q4_k_tiny", Q4_K), ("q6_k_tiny", Q6_K)]:
        src = np.fromfile(os.path.join(GOLDEN, name + ".in"), np.uint8)
        want = np.fromfile(os.path.join(GOLDEN, name + ".f32"), np.float32)
        for nrows, k in [(32, 256), (4, 2048), (1, 8192)]:
            qs, d, sc = oracle.pack_weights(t, src, nrows, k)
            got = np.stack([oracle.row_packed(t, qs, d, sc, r, nrows, k) for r in range(nrows)]).reshape(-1)
            assert np.array_equal(got, want)


def test_mxfp4_pack_refuses_exponents_an_f32_scale_cannot_hold():
    """/root/reference/jit/gpu/kernels/pack.go:407-420, /root/reference/internal/oracle/packed_test.go:220-247."""
    blk = np.zeros(17 * 32, np.uint8)            # 1 row, k = 1024
    blk[0::17] = 127
    oracle.pack_weights(MXFP4, blk, 1, 1024)     # fine
    for e in (0, 1, 255):
        bad = blk.copy()
        bad[17 * 3] = e
        oracle.pack_weights(MXFP4, bad, 1, 1024)  # all-zero codes pass at any exponent
        bad[17 * 3 + 5] = 0x08                    # -0 codes are still zero
        oracle.pack_weights(MXFP4, bad, 1, 1024)
        bad[17 * 3 + 5] = 0x21
        with pytest.raises(ValueError):
            oracle.pack_weights(MXFP4, bad, 1, 1024)


# ------------------------------------------------------------ activation quantizer
def _numpy_quantize(x, window):
    """Independent vectorised statement: f32 divisions by numpy, halves away from zero."""
    k = x.size
    per = max(1, window // 32) * 32
    q = np.empty(k, np.int8)
    a_s = np.empty(k // 32, np.float32)
    for w0 in range(0, k, per):
        seg = x[w0:min(w0 + per, k)]
        amax = np.abs(seg).max() if seg.size else np.float32(0)
        d = np.float32(amax) / np.float32(127)
        inv = np.float32(1) / d if d != 0 else np.float32(0)
        p = (seg * inv).astype(np.float32).astype(np.float64)
        q[w0:w0 + seg.size] = (np.sign(p) * np.floor(np.abs(p) + 0.5)).astype(np.int8)
        a_s[w0 // 32:(w0 + seg.size) // 32] = d
    s16 = q.reshape(-1, 16).astype(np.int32).sum(axis=1).astype(np.float32)
    return q, a_s, s16


@pytest.mark.parametrize("window", [32, 256])
def test_quantizer_against_numpy_on_random_and_boundary_inputs(window):
    from test_gpu_matvec import boundary_activations
    rng = np.random.default_rng(window)
    for k in (32, 288, 4096):
        for x in (rng.standard_normal(k).astype(np.float32), boundary_activations(rng, k, window),
                  np.zeros(k, np.float32), (rng.standard_normal(k) * 1e-30).astype(np.float32)):
            q, a_s, s16 = oracle.quantize_act(x, window)
            wq, wa, ws = _numpy_quantize(x, window)
            assert np.array_equal(q, wq)
            assert np.array_equal(a_s.view(np.uint32), wa.view(np.uint32))
            assert np.array_equal(s16, ws)
            assert np.abs(q.astype(np.int32)).max() <= 127


def test_quantizer_host_form_is_the_device_form_rescaled():
    """pairs[2b+1] = -sum*biasC/8 and half[h] = -sum16*biasC/4
    (/root/reference/internal/oracle/quantize.go:53-61,116-117)."""
    x = synth.activations(1024, seed=5)
    q, a_s, s16 = oracle.quantize_act(x, 32)
    for t, bc in [(Q4_K, 1), (Q8_0, 128), (Q6_K, 32), (MXFP4, 12)]:
        assert oracle.bias_c(t) == bc
        q2, pairs, half = oracle.quantize_q8_window(x, bc, 32, halves=True)
        assert np.array_equal(q, q2) and np.array_equal(pairs[0::2], a_s)
        s32 = s16[0::2] + s16[1::2]
        assert np.array_equal(pairs[1::2], (-s32.astype(np.float64) * bc / 8).astype(np.float32))
        assert np.array_equal(half, (-s16.astype(np.float64) * bc / 4).astype(np.float32))


def test_round_half_away_trick_is_exact():
    """trunc(p + copysign(0.5 - 2^-25, p)) == round-half-away(p): every f32 in [1/4, 4) and a
    sweep of larger magnitudes, the form the GPU and CPU-baseline quantizers use."""
    c = np.uint32(0x3EFFFFFF).view(np.float32)
    for e in (-2, -1, 0, 1, 6):
        bits = (np.uint32((e + 127) << 23) + np.arange(0, 1 << 23, 1 if e < 2 else 64, dtype=np.uint32)).astype(np.uint32)
        p = bits.view(np.float32)
        got = np.trunc((p + c).astype(np.float32)).astype(np.int64)
        assert np.array_equal(got, np.floor(p.astype(np.float64) + 0.5).astype(np.int64))


# ------------------------------------------------------------------ matvec forms
@pytest.mark.parametrize("t", ALL)
def test_matvec_forms_agree(t):
    """Three routes to W x over f32 activations: Dequant32 + Neumaier f32, Dequant32 + f64,
    and the packed-plane reader (/root/reference/internal/oracle/packed_test.go:119-173)."""
    nrows, k = 9, 512
    w = synth.quantized_weights(t, nrows, k, seed=2)
    x = synth.activations(k, seed=3)
    ref = oracle.matvec_f64(t, w, x, nrows, k)
    assert nmse(oracle.matvec(t, w, x, nrows, k), ref) < 1e-12
    qs, d, sc = oracle.pack_weights(t, w, nrows, k)
    assert nmse(oracle.matvec_packed_rows(t, qs, d, sc, x, nrows, k), ref) < 1e-10
    part = oracle.matvec_packed_rows(t, qs, d, sc, x, nrows, k, lo=3, hi=5)
    assert np.all(part[:3] == 0) and np.all(part[5:] == 0) and nmse(part[3:5], ref[3:5]) < 1e-10
    # brute force on the dequantised row, no oracle arithmetic involved
    wd = oracle.dequant(t, w, nrows * k).reshape(nrows, k).astype(np.float64)
    assert nmse(ref, wd @ x.astype(np.float64)) < 1e-28


@pytest.mark.parametrize("t", ALL)
@pytest.mark.parametrize("window", [32, 256])
def test_int8_activation_evaluators(t, window):
    """The like-for-like form equals dequant(W) . (q * d_a) as a real-number identity, so a
    dropped bias term, a wrong sub-block scale or a misplaced activation scale fails here."""
    nrows, k = 7, 1024
    for w in (synth.quantized_weights(t, nrows, k, seed=4), synth.random_weights(t, nrows, k, seed=5)):
        x = synth.activations(k, seed=6)
        q, a_s, s16 = oracle.quantize_act(x, window)
        xhat = q.astype(np.float64) * np.repeat(a_s.astype(np.float64), 32)
        wd = oracle.dequant(t, w, nrows * k).reshape(nrows, k).astype(np.float64)
        # dequant rounds d*sc*q - dmin*m to f32; the like-for-like form keeps the exact products
        want = wd @ xhat
        got = oracle.matvec_q8act_f64(t, w, q, a_s, nrows, k)
        assert nmse(got, want) < 1e-12
        assert nmse(oracle.matvec_q8act_f32(t, w, q, a_s, s16, nrows, k), got) < 1e-10


@pytest.mark.parametrize("t,window", [(Q4_K, 256), (Q4_K, 32), (Q8_0, 32), (Q6_K, 32)])
def test_cpu_baseline_restatement(t, window):
    nrows, k = 264, 1024
    w = synth.random_weights(t, nrows, k, seed=3)
    x = synth.activations(k, seed=4)
    qs, d, sc = oracle.pack_weights(t, w, nrows, k)
    q, a_s, _ = oracle.quantize_act(x, window)
    want = oracle.matvec_q8act_f64(t, w, q, a_s, nrows, k)
    for threads in (1, 3):
        cp = oracle.CpuPath(threads)
        got = cp.matvec_packed(t, qs, d, sc, x, nrows, k, window)
        cp.close()
        assert nmse(got, want) < 1e-10


@pytest.mark.parametrize("ntok,window", [(1, 256), (5, 256), (70, 256), (9, 32)])
def test_cpu_baseline_gemm_restatement(ntok, window):
    """The weight-stationary prefill GEMM of the CPU baseline (the port of
    /root/reference/jit/cpu/packedgemm.go:37-75): token t of the GEMM is the fused matvec of
    token t bit for bit (the reference's own gate, nn.TestMatMulPackedMatchesTheRowLoopExactly),
    and every token meets the oracle's like-for-like bar.  Ragged token blocks (70 = 64 + 6), a
    row count that is not a multiple of 16, an expert's sheet inside a bank's planes."""
    t, nrows, k = Q4_K, 264, 1024
    w = synth.random_weights(t, nrows, k, seed=3)
    x = np.stack([synth.activations(k, seed=40 + i) * np.float32(1 + i % 3) for i in range(ntok)])
    qs, d, sc = oracle.pack_weights(t, w, nrows, k)
    want = oracle.matmul_q8act_f64(t, w, x, nrows, k, ntok, window)
    for threads in (1, 3):
        cp = oracle.CpuPath(threads)
        got = cp.matmul_packed(t, qs, d, sc, x, nrows, k, ntok, window)
        assert nmse(got, want) < 1e-10
        for tok in (0, ntok - 1):
            mv = cp.matvec_packed(t, qs, d, sc, x[tok], nrows, k, window)
            assert np.array_equal(got[tok].view(np.uint32), mv.view(np.uint32)), "GEMM token != fused matvec"
        # rows 64..199 of the same planes as a matrix of their own (an expert's sheet)
        sub = cp.matmul_packed(t, qs, d, sc, x, 136, k, ntok, window, row0=64, stride=nrows)
        assert np.array_equal(sub.view(np.uint32), got[:, 64:200].view(np.uint32))
        cp.close()


def test_cpu_baseline_mixture_block_restatement():
    """The CPU baseline's routed feed-forward block (the port of moeBatchExpert,
    /root/reference/engine/model/moe.go:697-761) against the block built from the oracle's
    own pieces: per (row, expert) the like-for-like matvecs, silu(g) * u, the weighted sum."""
    rows, n_expert, k_used, n_ffn, n_embd, window = 9, 6, 2, 256, 512, 256
    rng = np.random.default_rng(3)
    sel = np.zeros((rows, k_used + 1), np.uint32)
    wt = np.zeros((rows, k_used), np.float32)
    for r in range(rows):
        s, wv, _, _ = oracle.moe_route(rng.standard_normal(n_expert).astype(np.float32), k_used)
        sel[r, :k_used], wt[r] = s, wv
    mk = lambda nr, kk, seed: np.concatenate([synth.quantized_weights(Q4_K, nr, kk, seed=seed + e) for e in range(n_expert)])
    gate, up, down = mk(n_ffn, n_embd, 100), mk(n_ffn, n_embd, 200), mk(n_embd, n_ffn, 300)
    x = np.stack([synth.activations(n_embd, seed=50 + r) for r in range(rows)])
    gs, ds = n_ffn * quant.row_bytes(Q4_K, n_embd), n_embd * quant.row_bytes(Q4_K, n_ffn)
    want = np.zeros((rows, n_embd))
    for r in range(rows):
        q, a_s, _ = oracle.quantize_act(x[r], window)
        for s_ in range(k_used):
            e = int(sel[r, s_])
            g = oracle.matvec_q8act_f64(Q4_K, gate[e * gs:(e + 1) * gs], q, a_s, n_ffn, n_embd).astype(np.float32)
            u = oracle.matvec_q8act_f64(Q4_K, up[e * gs:(e + 1) * gs], q, a_s, n_ffn, n_embd).astype(np.float32)
            h = (g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u).astype(np.float32)
            qh, ah, _ = oracle.quantize_act(h, window)
            want[r] += float(wt[r, s_]) * oracle.matvec_q8act_f64(Q4_K, down[e * ds:(e + 1) * ds], qh, ah, n_embd, n_ffn)
    planes = lambda bank, nr, kk: oracle.pack_weights(Q4_K, bank, n_expert * nr, kk)
    cp = oracle.CpuPath(3)
    got = cp.moe_block(planes(gate, n_ffn, n_embd), planes(up, n_ffn, n_embd), planes(down, n_embd, n_ffn), x, sel, wt,
                       n_expert, n_ffn, n_embd, window)
    cp.close()
    err = float(np.sqrt(np.sum((got - want) ** 2) / np.sum(want ** 2)))
    assert err <= 1e-4, f"rel-L2 {err:.3e}"


# ------------------------------------------------------------------------- MoE
def test_rmsnorm32_known_answers_and_invariants():
    """RMSNorm32 (/root/reference/internal/oracle/oracle.go:230-240) pinned without retyping
    it: a hand-computed case, exact rational arithmetic on a small vector, unit mean square
    of the output for w = 1 and eps = 0, bit-identical output when x is scaled by a power of
    two (eps = 0), and the large-eps limit x * w / sqrt(eps)."""
    from fractions import Fraction
    import math
    y = oracle.rmsnorm32(np.array([3, 4], np.float32), np.array([1, 1], np.float32), 0.0)
    assert np.array_equal(y, np.array([3 / math.sqrt(12.5), 4 / math.sqrt(12.5)], np.float64).astype(np.float32))
    rng = np.random.default_rng(5)
    x = rng.standard_normal(37).astype(np.float32)
    w = rng.standard_normal(37).astype(np.float32)
    eps = 1e-6
    mean = sum(Fraction(float(v)) ** 2 for v in x) / 37 + Fraction(eps)     # exact
    want = np.array([float(Fraction(float(v)) * Fraction(float(u))) / math.sqrt(float(mean)) for v, u in zip(x, w)])
    got = oracle.rmsnorm32(x, w, eps)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-30)) <= 2.0 ** -23   # one f32 rounding
    x = rng.standard_normal(4096).astype(np.float32)
    ones = np.ones(4096, np.float32)
    y = oracle.rmsnorm32(x, ones, 0.0)
    assert abs(np.sum(y.astype(np.float64) ** 2) / 4096 - 1) <= 1e-6
    assert np.array_equal(oracle.rmsnorm32(x * np.float32(1024), ones, 0.0), y)
    big = oracle.rmsnorm32(x, w := rng.standard_normal(4096).astype(np.float32), 1e12)
    assert np.allclose(big, x.astype(np.float64) * w / 1e6, rtol=1e-5, atol=0)


def test_router_logits_order_pinned_by_cancellation_cases():
    """The router's logits (/root/reference/jit/gpu/kernels/moe.go:843-917) are an f32 sum in
    a stated order: 128 strided partial sums, then a binary tree that pairs thread j with
    j + 64, j + 32, ...  The order only shows in roundings, so it is pinned by cases built
    to round differently under other orders: 2^24 absorbs a lone +1 but not a +2.
    Answers are worked out by hand from the stated order, not computed by the same code."""
    big = np.float32(2.0 ** 24)
    def one(places, k=256):
        w = np.zeros((1, k), np.float32)
        w[0, 0] = big
        for i in places:
            w[0, i] = 1
        return float(oracle.router_logits(w, np.ones(k, np.float32), 1, k)[0, 0])
    assert one([128]) == 2.0 ** 24            # same thread as the big term: added one by one, lost
    assert one([128, 129]) == 2.0 ** 24       # threads 0 and 1; thread 1's lone 1 meets 2^24 at the last step
    assert one([64, 192]) == 2.0 ** 24 + 2    # both in thread 64: 1 + 1 = 2 survives meeting 2^24 at s = 64
    assert one([32, 96]) == 2.0 ** 24 + 2     # threads 32 and 96 meet each other (s = 64) before the big term (s = 32)
    assert one([32, 64]) == 2.0 ** 24         # thread 64 meets the big term alone (s = 64), thread 32 alone (s = 32)
    assert one([1, 2, 3]) == 2.0 ** 24 + 2    # s = 2: threads 1 and 3 make 2, thread 2's lone 1 is lost to 2^24; s = 1: 2^24 + 2
    # a sequential sum would give 2^24 for every one of these, an f64 sum 2^24 + 2 or + 4
    # values: against f64 on random data, ragged k (tail trips add +0), f16 weights exact
    rng = np.random.default_rng(3)
    for rows, k, ntok in [(5, 2048, 3), (3, 130, 2), (2, 100, 1), (4, 4097, 2)]:
        w = rng.standard_normal((rows, k)).astype(np.float32)
        x = rng.standard_normal((ntok, k)).astype(np.float32)
        got = oracle.router_logits(w, x, rows, k, ntok)
        want = x.astype(np.float64) @ w.astype(np.float64).T
        assert np.max(np.abs(got - want)) <= 1e-5 * np.sqrt(k)
        wh = w.astype(np.float16)
        got16 = oracle.router_logits(wh.view(np.uint16), x, rows, k, ntok)
        assert np.array_equal(got16, oracle.router_logits(wh.astype(np.float32), x, rows, k, ntok))
    # small integers are exact in any order: the plain dot product
    w = rng.integers(-8, 9, (6, 300)).astype(np.float32)
    x = rng.integers(-8, 9, (2, 300)).astype(np.float32)
    assert np.array_equal(oracle.router_logits(w, x, 6, 300, 2), (x.astype(np.int64) @ w.astype(np.int64).T).astype(np.float32))


def test_moe_route_against_brute_force():
    rng = np.random.default_rng(0)
    for n, k in [(128, 8), (16, 2), (8, 1), (4, 4)]:
        for trial in range(20):
            logits = rng.standard_normal(n).astype(np.float32)
            if trial % 4 == 0:
                logits[rng.integers(n, size=n // 2)] = logits[0]   # ties: lowest index wins
            sel, wt, ordr, owt = oracle.moe_route(logits, k)
            p = np.exp(logits.astype(np.float64) - float(logits.max()))
            p32 = p.astype(np.float32)
            scores = (p32.astype(np.float64) / p.sum()).astype(np.float32)
            want = sorted(range(n), key=lambda e: (-scores[e], e))[:k]
            assert list(sel) == want
            s = np.float32(0)
            for e in want:
                s = np.float32(s + scores[e])
            s = np.float32(s + np.float32(1e-20))
            assert np.array_equal(wt, (scores[want] / s).astype(np.float32))
            assert list(ordr) == sorted(want)
            assert all(owt[i] == wt[list(sel).index(e)] for i, e in enumerate(ordr))
            assert abs(float(wt.sum()) - 1) < 1e-6


def test_moe_route_never_selects_nan():
    logits = np.array([0.5, np.nan, 0.25, 0.1], np.float32)
    # a NaN logit poisons the softmax; the selection rule itself is what is under test
    sel, _, _, _ = oracle.moe_route(np.array([0.5, -1e30, 0.25, 0.1], np.float32), 2)
    assert list(sel) == [0, 2]
    sel, _, _, _ = oracle.moe_route(logits, 2)
    assert len(sel) == 0  # every score is NaN: nothing is eligible


def _brute_group(sel, rows, k, n_exp, unit):
    pairs = sorted((int(sel[r * (k + 1) + s]), r, s) for r in range(rows) for s in range(k))
    perm, col_e, pos = [], [], {}
    for e in range(n_exp):
        mine = [(r, s) for ee, r, s in pairs if ee == e]
        for r, s in mine:
            pos[(r, s)] = len(perm)
            perm.append(r)
            col_e.append(e)
        while len(perm) % unit:
            perm.append(rows)
            col_e.append(e)
    return perm, col_e, pos


@pytest.mark.parametrize("case", ["random", "one_expert", "mostly_empty", "k1", "unit1"])
def test_group_pairs_against_brute_force(case):
    """/root/reference/jit/gpu/tier/grouppairs_test.go:84-137."""
    rng = np.random.default_rng(1)
    rows, k, n_exp, unit = 12, 4, 16, 8
    if case == "k1":
        k = 1
    if case == "unit1":
        unit = 1
    sel = np.zeros((rows, k + 1), np.uint32)
    for r in range(rows):
        if case == "one_expert":
            sel[r, :k] = 5
        elif case == "mostly_empty":
            sel[r, :k] = rng.choice([2, 9, 10, 15], size=k, replace=False) if k <= 4 else 2
        else:
            sel[r, :k] = rng.choice(n_exp, size=k, replace=False)
    used, perm, col_e, pos = oracle.group_pairs(sel.reshape(-1), rows, k, n_exp, unit)
    bperm, bcol, bpos = _brute_group(sel.reshape(-1), rows, k, n_exp, unit)
    assert used == len(bperm) and used % unit == 0
    assert list(perm[:used]) == bperm
    assert [int(col_e[j]) for j in range(used) if perm[j] != rows] == [e for e, p in zip(bcol, bperm) if p != rows]
    for r in range(rows):
        for s in range(k):
            assert pos[r * k + s] == bpos[(r, s)]
            assert perm[pos[r * k + s]] == r and col_e[pos[r * k + s]] == sel[r, s]


# -------------------------------------------------------------- synthetic weights
@pytest.mark.parametrize("t,tol", [(Q8_0, 0.01), (Q6_K, 0.03), (Q4_K, 0.12), (MXFP4, 0.2)])
def test_synthetic_quantizers_round_trip(t, tol):
    w = synth.normal_weights(16, 1024, seed=3)
    b = synth.QUANTIZERS[t](w)
    assert b.size == 16 * quant.row_bytes(t, 1024)
    dq = oracle.dequant(t, b, 16 * 1024).reshape(16, 1024)
    assert np.linalg.norm(dq - w) / np.linalg.norm(w) < tol
    assert np.array_equal(synth.quantized_weights(t, 16, 1024, seed=3, chunk=5)[:b.size], b)


def test_planted_scales_are_finite_and_reach_the_extremes():
    for t in ALL:
        b = synth.random_weights(t, 8, 4096, seed=1)
        assert np.all(np.isfinite(oracle.dequant(t, b, 8 * 4096)))
    b = synth.random_weights(Q4_K, 8, 4096, seed=0).reshape(-1, 144)
    d = b[:, 0].astype(np.uint16) | (b[:, 1].astype(np.uint16) << 8)
    assert {0x0001, 0x03FF, 0x0400, 0x7BFF} <= set(d.tolist()) | set((b[:, 2].astype(np.uint16) | (b[:, 3].astype(np.uint16) << 8)).tolist())
