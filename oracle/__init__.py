"""ctypes binding of the CPU oracle (libjl_oracle.so).

TEST INFRASTRUCTURE ONLY.  Importable from tests/, from the smoke check and
from bench.py's cpu_baseline leg; the product package never imports it.  All
arrays are numpy; sizes are checked here so a test cannot hand the C code a
short buffer.
"""
import ctypes as C
import os
import subprocess

import numpy as np

Q8_0, Q4_K, Q6_K, MXFP4 = 8, 12, 14, 39
TYPES = (Q8_0, Q4_K, Q6_K, MXFP4)

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libjl_oracle.so")


def build(force=False):
    """Compile the oracle with the Makefile beside this file."""
    args = ["make", "-C", _HERE, "-s"]
    if force:
        args.append("-B")
    subprocess.run(args, check=True)


def _load():
    if not os.path.exists(_LIB):
        build()
    return C.CDLL(_LIB)


_l = _load()
_u8p, _i8p = C.POINTER(C.c_uint8), C.POINTER(C.c_int8)
_f32p, _f64p = C.POINTER(C.c_float), C.POINTER(C.c_double)
_u32p, _i32p = C.POINTER(C.c_uint32), C.POINTER(C.c_int32)
_szp = C.POINTER(C.c_size_t)


def _p(a, t):
    return a.ctypes.data_as(t)


def _chk(a, dtype, n=None):
    a = np.ascontiguousarray(a, dtype=dtype)
    if n is not None and a.size < n:
        raise ValueError(f"buffer of {a.size} {dtype} is shorter than {n}")
    return a


_l.jlo_block_elems.restype = C.c_int
_l.jlo_block_bytes.restype = C.c_int
_l.jlo_half_to_f32.restype = C.c_float
_l.jlo_half_to_f32.argtypes = [C.c_uint16]
_l.jlo_f32_to_half.restype = C.c_uint16
_l.jlo_f32_to_half.argtypes = [C.c_float]
_l.jlo_dequant.argtypes = [C.c_int, _u8p, _f32p, C.c_size_t]
_l.jlo_packed_words.argtypes = [C.c_int, C.c_int, C.c_int, _szp, _szp, _szp]
_l.jlo_pack_weights.argtypes = [C.c_int, _u8p, C.c_int, C.c_int, _u32p, _u32p, _u32p]
_l.jlo_row_packed.argtypes = [_f32p, C.c_int, _u32p, _u32p, _u32p, C.c_int, C.c_int, C.c_int]
_l.jlo_matvec_packed_rows.argtypes = [_f32p, C.c_int, _u32p, _u32p, _u32p, _f32p,
                                      C.c_int, C.c_int, C.c_int, C.c_int]
_l.jlo_matvec.argtypes = [_f32p, C.c_int, _u8p, _f32p, C.c_int, C.c_int]
_l.jlo_matvec_f64.argtypes = [_f64p, C.c_int, _u8p, _f32p, C.c_int, C.c_int]
_l.jlo_quantize_act.argtypes = [_i8p, _f32p, _f32p, _f32p, C.c_int, C.c_int]
_l.jlo_quantize_q8_window.argtypes = [_i8p, _f32p, _f32p, _f32p, C.c_int, C.c_double, C.c_int]
_l.jlo_bias_c.restype = C.c_double
_l.jlo_bias_c.argtypes = [C.c_int]
_l.jlo_matvec_q8act_f64.argtypes = [_f64p, C.c_int, _u8p, _i8p, _f32p, C.c_int, C.c_int]
_l.jlo_matvec_q8act_f32.argtypes = [_f32p, C.c_int, _u8p, _i8p, _f32p, _f32p, C.c_int, C.c_int]
_l.jlo_rmsnorm32.restype = None
_l.jlo_rmsnorm32.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_double]
_l.jlo_router_logits.restype = None
_l.jlo_router_logits.argtypes = [_f32p, C.c_void_p, C.c_int, _f32p, C.c_int, C.c_int, C.c_int]
_l.jlo_moe_route.argtypes = [_f32p, C.c_int, C.c_int, _i32p, _f32p, _i32p, _f32p]
_l.jlo_group_pairs.argtypes = [_u32p, C.c_int, C.c_int, C.c_int, C.c_int, _u32p, _u32p, _u32p,
                               C.c_int]


def block_elems(t):
    return _l.jlo_block_elems(t)


def block_bytes(t):
    return _l.jlo_block_bytes(t)


def row_bytes(t, k):
    return k // block_elems(t) * block_bytes(t)


def half_to_f32(h):
    return _l.jlo_half_to_f32(int(h))


def f32_to_half(f):
    return _l.jlo_f32_to_half(float(np.float32(f)))


def dequant(t, src, n):
    """Dequant32 of n elements of GGUF blocks of type t."""
    be = block_elems(t)
    if be == 0 or n % be:
        raise ValueError("not a whole number of blocks")
    src = _chk(src, np.uint8, n // be * block_bytes(t))
    dst = np.empty(n, np.float32)
    if _l.jlo_dequant(t, _p(src, _u8p), _p(dst, _f32p), n) != 0:
        raise ValueError("dequant refused")
    return dst


def packed_words(t, nrows, k):
    nq, nd, nsc = C.c_size_t(), C.c_size_t(), C.c_size_t()
    if _l.jlo_packed_words(t, nrows, k, C.byref(nq), C.byref(nd), C.byref(nsc)) != 0:
        raise ValueError("packed_words refused")
    return nq.value, nd.value, nsc.value


def pack_weights(t, src, nrows, k):
    """PackWeights: GGUF row-major bytes -> (qs, d, sc) u32 planes."""
    src = _chk(src, np.uint8, nrows * row_bytes(t, k))
    nq, nd, nsc = packed_words(t, nrows, k)
    qs = np.zeros(nq, np.uint32)
    d = np.zeros(nd, np.uint32)
    sc = np.zeros(max(nsc, 1), np.uint32)
    rc = _l.jlo_pack_weights(t, _p(src, _u8p), nrows, k, _p(qs, _u32p), _p(d, _u32p), _p(sc, _u32p))
    if rc != 0:
        raise ValueError(f"pack refused ({rc})")
    return qs, d, sc[:nsc]


def _planes(t, qs, d, sc, nrows, k):
    nq, nd, nsc = packed_words(t, nrows, k)
    qs, d = _chk(qs, np.uint32, nq), _chk(d, np.uint32, nd)
    sc = _chk(sc if nsc else np.zeros(1, np.uint32), np.uint32, max(nsc, 1))
    return qs, d, sc


def row_packed(t, qs, d, sc, r, nrows, k):
    qs, d, sc = _planes(t, qs, d, sc, nrows, k)
    dst = np.empty(k, np.float32)
    if _l.jlo_row_packed(_p(dst, _f32p), t, _p(qs, _u32p), _p(d, _u32p), _p(sc, _u32p), r, nrows, k):
        raise ValueError("row_packed refused")
    return dst


def matvec_packed_rows(t, qs, d, sc, x, nrows, k, lo=0, hi=None):
    hi = nrows if hi is None else hi
    qs, d, sc = _planes(t, qs, d, sc, nrows, k)
    x = _chk(x, np.float32, k)
    out = np.zeros(nrows, np.float32)
    if _l.jlo_matvec_packed_rows(_p(out, _f32p), t, _p(qs, _u32p), _p(d, _u32p), _p(sc, _u32p),
                                 _p(x, _f32p), nrows, k, lo, hi):
        raise ValueError("matvec_packed_rows refused")
    return out


def matvec(t, w, x, nrows, k):
    """oracle.MatVec: Dequant32 + Neumaier f32 dot with f32 activations."""
    w = _chk(w, np.uint8, nrows * row_bytes(t, k))
    x = _chk(x, np.float32, k)
    out = np.empty(nrows, np.float32)
    if _l.jlo_matvec(_p(out, _f32p), t, _p(w, _u8p), _p(x, _f32p), nrows, k):
        raise ValueError("matvec refused")
    return out


def matvec_f64(t, w, x, nrows, k):
    w = _chk(w, np.uint8, nrows * row_bytes(t, k))
    x = _chk(x, np.float32, k)
    out = np.empty(nrows, np.float64)
    if _l.jlo_matvec_f64(_p(out, _f64p), t, _p(w, _u8p), _p(x, _f32p), nrows, k):
        raise ValueError("matvec_f64 refused")
    return out


def quantize_act(x, window=32):
    """Device-form activation quantizer: (q int8[k], as f32[k/32], sum16 f32[k/16])."""
    x = _chk(x, np.float32)
    k = x.size
    q = np.empty(k, np.int8)
    a_s = np.empty(k // 32, np.float32)
    s16 = np.empty(k // 16, np.float32)
    if _l.jlo_quantize_act(_p(q, _i8p), _p(a_s, _f32p), _p(s16, _f32p), _p(x, _f32p), k, window):
        raise ValueError("quantize_act refused")
    return q, a_s, s16


def quantize_q8_window(x, bias_c, window=32, halves=False):
    """Host-form activation quantizer: (q, pairs f32[2*k/32], half f32[k/16] or None)."""
    x = _chk(x, np.float32)
    k = x.size
    q = np.empty(k, np.int8)
    pairs = np.empty(2 * (k // 32), np.float32)
    half = np.empty(k // 16, np.float32) if halves else None
    hp = _p(half, _f32p) if halves else C.cast(None, _f32p)
    if _l.jlo_quantize_q8_window(_p(q, _i8p), _p(pairs, _f32p), hp, _p(x, _f32p), k,
                                 float(bias_c), window):
        raise ValueError("quantize_q8_window refused")
    return q, pairs, half


def bias_c(t):
    return _l.jlo_bias_c(t)


def matvec_q8act_f64(t, w, q, a_s, nrows, k):
    w = _chk(w, np.uint8, nrows * row_bytes(t, k))
    q, a_s = _chk(q, np.int8, k), _chk(a_s, np.float32, k // 32)
    out = np.empty(nrows, np.float64)
    if _l.jlo_matvec_q8act_f64(_p(out, _f64p), t, _p(w, _u8p), _p(q, _i8p), _p(a_s, _f32p), nrows, k):
        raise ValueError("matvec_q8act_f64 refused")
    return out


def matvec_q8act_f32(t, w, q, a_s, s16, nrows, k):
    w = _chk(w, np.uint8, nrows * row_bytes(t, k))
    q, a_s = _chk(q, np.int8, k), _chk(a_s, np.float32, k // 32)
    s16 = _chk(s16, np.float32, k // 16)
    out = np.empty(nrows, np.float32)
    if _l.jlo_matvec_q8act_f32(_p(out, _f32p), t, _p(w, _u8p), _p(q, _i8p), _p(a_s, _f32p),
                               _p(s16, _f32p), nrows, k):
        raise ValueError("matvec_q8act_f32 refused")
    return out


def matmul_q8act_f64(t, w, x, nrows, k, ntok, window):
    """out[ntok][nrows]: each token quantized on its own, then the f64 like-for-like form."""
    x = _chk(x, np.float32, ntok * k).reshape(ntok, k)
    out = np.empty((ntok, nrows), np.float64)
    for i in range(ntok):
        q, a_s, _ = quantize_act(x[i], window)
        out[i] = matvec_q8act_f64(t, w, q, a_s, nrows, k)
    return out


def rmsnorm32(x, w, eps):
    """RMSNorm over an f32 vector with f64 accumulation (oracle.RMSNorm32)."""
    x, w = _chk(x, np.float32), _chk(w, np.float32, np.asarray(x).size)
    y = np.empty(x.size, np.float32)
    _l.jlo_rmsnorm32(_p(y, _f32p), _p(x, _f32p), _p(w, _f32p), x.size, float(eps))
    return y


def router_logits(w, x, rows, k, ntok=1):
    """Router logits [ntok][rows] in the reference device kernel's summation order
    (kernels.RouterMatVecTok); w is f32 [rows][k], or f16 bits (uint16) of the same shape."""
    w = np.ascontiguousarray(w)
    f16 = w.dtype == np.uint16
    if not f16:
        w = _chk(w, np.float32, rows * k)
    elif w.size != rows * k:
        raise ValueError("router_logits: weight size")
    x = _chk(x, np.float32, ntok * k)
    out = np.empty((ntok, rows), np.float32)
    _l.jlo_router_logits(_p(out, _f32p), w.ctypes.data_as(C.c_void_p), int(f16), _p(x, _f32p), rows, k, ntok)
    return out


def moe_route(logits, k):
    """Softmax over all experts, lexicographic top-k, renormalised weights.

    Returns (sel, wt) in selection order and (ord, owt) in ascending expert id."""
    logits = _chk(logits, np.float32)
    n = logits.size
    sel, ordr = np.zeros(k, np.int32), np.zeros(k, np.int32)
    wt, owt = np.zeros(k, np.float32), np.zeros(k, np.float32)
    got = _l.jlo_moe_route(_p(logits, _f32p), n, k, _p(sel, _i32p), _p(wt, _f32p),
                           _p(ordr, _i32p), _p(owt, _f32p))
    if got < 0:
        raise ValueError("moe_route refused")
    return sel[:got], wt[:got], ordr[:got], owt[:got]


def group_pairs(sel, rows, k, n_exp, unit):
    """groupPairs: sel is [rows][k+1] u32.  Returns (used, perm, col_e, pos)."""
    sel = _chk(sel, np.uint32, rows * (k + 1))
    ncols = rows * k + n_exp * unit
    perm, col_e = np.zeros(ncols, np.uint32), np.zeros(ncols, np.uint32)
    pos = np.zeros(rows * k, np.uint32)
    used = _l.jlo_group_pairs(_p(sel, _u32p), rows, k, n_exp, unit, _p(perm, _u32p),
                              _p(col_e, _u32p), _p(pos, _u32p), ncols)
    if used < 0:
        raise ValueError("group_pairs refused")
    return used, perm, col_e, pos


# --------------------------------------------------------------- CPU baseline
class CpuPath:
    """The intrinsic restatement of the reference's host kernels (jl_cpu_path.c):
    activation quantizer + fused packed matvec on a spinning worker pool."""

    def __init__(self, threads):
        lib = os.path.join(_HERE, "libjl_cpu_path.so")
        if not os.path.exists(lib):
            build()
        self._l = C.CDLL(lib)
        self._l.jlc_pool_create.restype = C.c_void_p
        self._l.jlc_pool_create.argtypes = [C.c_int]
        self._l.jlc_pool_destroy.argtypes = [C.c_void_p]
        self._l.jlc_has_vnni.argtypes = [C.c_void_p]
        self._l.jlc_matvec_packed.argtypes = [C.c_void_p, _f32p, C.c_int, _u32p, _u32p, _u32p, _f32p,
                                              C.c_int, C.c_int, C.c_int]
        pp = C.POINTER(_u32p)
        self._l.jlc_time_matvec.restype = C.c_double
        self._l.jlc_time_matvec.argtypes = [C.c_void_p, _f32p, C.c_int, pp, pp, pp, C.c_int, _f32p,
                                            C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        self._l.jlc_membw.restype = C.c_double
        self._l.jlc_membw.argtypes = [C.c_int, C.c_size_t, C.c_int]
        self._l.jlc_matmul_packed.argtypes = [C.c_void_p, _f32p, C.c_int, _u32p, _u32p, _u32p, C.c_int, C.c_int,
                                              _f32p, C.c_int, C.c_int, C.c_int, C.c_int]
        self._l.jlc_time_matmul.restype = C.c_double
        self._l.jlc_time_matmul.argtypes = [C.c_void_p, _f32p, C.c_int, _u32p, _u32p, _u32p, _f32p, C.c_int, C.c_int,
                                            C.c_int, C.c_int, C.c_int]
        moe = [C.c_void_p, _f32p, pp, pp, pp, _f32p, _u32p, C.c_int, _f32p] + [C.c_int] * 6
        self._l.jlc_moe_block.argtypes = moe
        self._l.jlc_time_moe_block.restype = C.c_double
        self._l.jlc_time_moe_block.argtypes = moe + [C.c_int]
        self.threads = threads
        self._p = self._l.jlc_pool_create(threads)

    def close(self):
        if self._p:
            self._l.jlc_pool_destroy(self._p)
            self._p = None

    @property
    def vnni(self):
        return bool(self._l.jlc_has_vnni(self._p))

    def matvec_packed(self, t, qs, d, sc, x, nrows, k, window):
        qs, d, sc = _planes(t, qs, d, sc, nrows, k)
        x = _chk(x, np.float32, k)
        out = np.zeros(nrows, np.float32)
        if self._l.jlc_matvec_packed(self._p, _p(out, _f32p), t, _p(qs, _u32p), _p(d, _u32p),
                                     _p(sc, _u32p), _p(x, _f32p), nrows, k, window):
            raise ValueError("cpu matvec refused")
        return out

    def time_matvec(self, t, copies, x, nrows, k, window, reps=9, sweeps=1):
        """copies: list of (qs, d, sc) distinct plane sets.  Seconds per call: the median of `reps`
        timed passes of `sweeps` sweeps over all the copies."""
        n = len(copies)
        arr = lambda i: (_u32p * n)(*[_p(c[i], _u32p) for c in copies])
        x = _chk(x, np.float32, k)
        out = np.zeros(nrows, np.float32)
        s = self._l.jlc_time_matvec(self._p, _p(out, _f32p), t, arr(0), arr(1), arr(2), n,
                                    _p(x, _f32p), nrows, k, window, reps, sweeps)
        if s < 0:
            raise ValueError("cpu timing refused")
        return s

    def matmul_packed(self, t, qs, d, sc, x, nrows, k, ntok, window, row0=0, stride=None):
        """The weight-stationary prefill GEMM over Q4_K planes (rows row0.. of planes `stride`
        rows long): out [ntok][nrows]."""
        stride = nrows if stride is None else stride
        qs, d, sc = _planes(t, qs, d, sc, stride, k)
        x = _chk(x, np.float32, ntok * k)
        out = np.zeros((ntok, nrows), np.float32)
        if self._l.jlc_matmul_packed(self._p, _p(out, _f32p), t, _p(qs, _u32p), _p(d, _u32p), _p(sc, _u32p),
                                     row0, stride, _p(x, _f32p), nrows, k, ntok, window):
            raise ValueError("cpu matmul refused")
        return out

    def time_matmul(self, t, qs, d, sc, x, nrows, k, ntok, window, reps=9):
        """Seconds per call: 3 warm calls, then the median of `reps` timed calls."""
        qs, d, sc = _planes(t, qs, d, sc, nrows, k)
        x = _chk(x, np.float32, ntok * k)
        out = np.zeros((ntok, nrows), np.float32)
        s = self._l.jlc_time_matmul(self._p, _p(out, _f32p), t, _p(qs, _u32p), _p(d, _u32p), _p(sc, _u32p),
                                    _p(x, _f32p), nrows, k, ntok, window, reps)
        if s < 0:
            raise ValueError("cpu timing refused")
        return s

    def _moe_args(self, gate, up, down, x, sel, wt, n_expert, n_ffn, n_embd):
        rows, k_used = wt.shape
        banks = []
        for planes, r, kk in ((gate, n_ffn, n_embd), (up, n_ffn, n_embd), (down, n_embd, n_ffn)):
            pl = _planes(Q4_K, planes[0], planes[1], planes[2], n_expert * r, kk)
            banks.append((pl, (_u32p * 3)(*[_p(a, _u32p) for a in pl])))
        x = _chk(x, np.float32, rows * n_embd)
        sel = np.ascontiguousarray(sel, np.uint32)
        wt = np.ascontiguousarray(wt, np.float32)
        return banks, x, sel, wt, rows, k_used

    def moe_block(self, gate, up, down, x, sel, wt, n_expert, n_ffn, n_embd, window):
        """The routed feed-forward block over banks of Q4_K planes (each a (qs, d, sc) plane set of
        n_expert * rows rows): resid [rows][n_embd], starting from zero."""
        banks, x, sel, wt, rows, k_used = self._moe_args(gate, up, down, x, sel, wt, n_expert, n_ffn, n_embd)
        resid = np.zeros((rows, n_embd), np.float32)
        if self._l.jlc_moe_block(self._p, _p(resid, _f32p), banks[0][1], banks[1][1], banks[2][1], _p(x, _f32p),
                                 _p(sel, _u32p), sel.shape[1], _p(wt, _f32p), rows, k_used, n_expert, n_ffn, n_embd,
                                 window):
            raise ValueError("cpu mixture block refused")
        return resid

    def time_moe_block(self, gate, up, down, x, sel, wt, n_expert, n_ffn, n_embd, window, reps=9):
        banks, x, sel, wt, rows, k_used = self._moe_args(gate, up, down, x, sel, wt, n_expert, n_ffn, n_embd)
        resid = np.zeros((rows, n_embd), np.float32)
        s = self._l.jlc_time_moe_block(self._p, _p(resid, _f32p), banks[0][1], banks[1][1], banks[2][1], _p(x, _f32p),
                                       _p(sel, _u32p), sel.shape[1], _p(wt, _f32p), rows, k_used, n_expert, n_ffn,
                                       n_embd, window, reps)
        if s < 0:
            raise ValueError("cpu timing refused")
        return s

    def membw(self, nbytes=1 << 30, reps=3):
        return self._l.jlc_membw(self.threads, nbytes, reps)
