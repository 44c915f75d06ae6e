"""Host-side mirror of the reference's accelerator seam over the C ABI.

`Device` is the shape of nn.Device (/root/reference/engine/nn/device.go:23-31):
MatVec(out, t, w, x, nrows, k) -> bool, False meaning "declined, run your own
path".  The *_dev methods take device pointers (ints, e.g. tensor.data_ptr())
and enqueue on a stream without waiting: that is the boundary a resident engine
and the benchmarks use.  Failures (as opposed to declines) raise DeviceError,
where the reference's entry points panic.
"""
import ctypes as C

import numpy as np

from . import _lib, quant


class DeviceError(RuntimeError):
    pass


def _ptr(a):
    """Address of a numpy array or a raw int address."""
    if isinstance(a, np.ndarray):
        return a.ctypes.data
    return int(a)


def _opt(a):
    return None if a is None else _ptr(a)


class Packed:
    """nn.Packed (/root/reference/engine/nn/device.go:70-80): the three planes of a weight,
    and which rows of them a matrix is.  Planes are numpy uint32 arrays or device addresses."""

    def __init__(self, qs, d, sc, row=0, stride=0):
        self.qs, self.d, self.sc, self.row, self.stride = qs, d, sc, row, stride


class MVGroup:
    """nn.MVGroup (/root/reference/engine/nn/packedgroup.go:18-37): up to MAX_GROUP packed matvecs
    that read one activation X[:K]; Out[i] gets Rows[i] rows of P[i] (type T[i])."""

    def __init__(self, Out, T, P, Rows, X, K, ActUp=None, Act=0, Resid=None, Alpha=0.0):
        self.N = len(P)
        self.Out, self.T, self.P, self.Rows, self.X, self.K = list(Out), list(T), list(P), list(Rows), X, K
        self.ActUp, self.Act, self.Resid, self.Alpha = ActUp, Act, Resid, Alpha


class Device:
    def __init__(self, device=0, act_window=32, code_object=None):
        self._l = _lib.load()
        self._ctx = C.c_void_p()
        opts = _lib.Options(device, act_window,
                            (code_object or _lib.CODE_OBJECT_PATH).encode())
        rc = self._l.jl_ctx_create(C.byref(self._ctx), C.byref(opts))
        if rc != _lib.OK:
            msg = self._l.jl_last_error(None).decode()
            self._ctx = None
            raise DeviceError(f"jl_ctx_create failed ({rc}): {msg}")

    def launch_count(self):
        """Kernels launched so far by this device."""
        return int(self._l.jl_launch_count(self._ctx))

    def close(self):
        if getattr(self, "_ctx", None):
            self._l.jl_ctx_destroy(self._ctx)
            self._ctx = None

    def __del__(self):
        self.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _served(self, rc, what):
        if rc == _lib.OK:
            return True
        if rc == _lib.DECLINED:
            return False
        raise DeviceError(f"{what} failed ({rc}): {self._l.jl_last_error(self._ctx).decode()}")

    # -- configuration -------------------------------------------------------
    def SetActWindow(self, n):
        """nn.ActWindower.SetActWindow (/root/reference/engine/nn/device.go:1566-1568)."""
        self._served(self._l.jl_set_act_window(self._ctx, n), "jl_set_act_window")

    def Reserve(self, max_tok, max_k):
        """nn.LayerDevice.Reserve: size the prefill workspace ahead of time."""
        self._served(self._l.jl_reserve(self._ctx, max_tok, max_k), "jl_reserve")

    def PrepLayer(self, li, kind, t, n_embd, n_ffn, gate, up, down, down_type=None, norm_w=None, norm_eps=0.0,
                  n_expert=0, k_used=0, router=None):
        """nn.LayerDevice.PrepLayer for a block's feed-forward weights
        (/root/reference/engine/nn/device.go:1096-1131): uploaded once from host memory and kept until
        ReleaseLayers.  gate / up / down are numpy arrays of GGUF bytes, or (qs, d, sc) tuples of
        packed planes (sc None for Q8_0); router f32 [n_expert][n_embd] for a mixture.  False when
        the block is declined (no kernel for it, or it does not fit): it then stays on the host."""
        keep = []

        def host(a):
            if a is None:
                return None
            a = np.ascontiguousarray(a)
            keep.append(a)
            return a.ctypes.data

        packed = isinstance(gate, tuple)
        if packed:
            def planes(m):
                hp = _lib.HostPlanes(host(m[0]), host(m[1]), host(m[2]))
                keep.append(hp)
                return C.cast(C.pointer(hp), C.c_void_p).value
            g, u, d = planes(gate), planes(up), planes(down)
        else:
            g, u, d = host(gate), host(up), host(down)
        plan = _lib.LayerPlan(int(kind), int(t), int(t if down_type is None else down_type), int(n_embd), int(n_ffn),
                              int(packed), g, u, d, host(norm_w), float(norm_eps), int(n_expert), int(k_used),
                              host(router))
        return self._served(self._l.jl_prep_layer(self._ctx, int(li), C.byref(plan)), "jl_prep_layer")

    def layer_ffn_dev(self, li, h, resid, n, stream=None):
        """Run prepared block li's feed-forward for n rows: resid [n][n_embd] += ffn(h [n][n_embd])."""
        return self._served(self._l.jl_layer_ffn_dev(self._ctx, int(li), _ptr(h), _ptr(resid), int(n), stream),
                            "jl_layer_ffn_dev")

    def ReleaseLayers(self, lo, hi):
        """nn.LayerDevice.ReleaseLayers (/root/reference/engine/nn/device.go:1160-1176)."""
        self._served(self._l.jl_release_layers(self._ctx, int(lo), int(hi)), "jl_release_layers")

    def Layers(self):
        """nn.LayerDevice.Layers: how many blocks are resident."""
        return int(self._l.jl_layer_count(self._ctx))

    def reserve_shape(self, t, nrows, k, ntok, packed=False):
        """Grow every workspace a matmul of this shape would grow, launching nothing."""
        return self._served(self._l.jl_reserve_shape(self._ctx, t, nrows, k, ntok, int(packed)), "jl_reserve_shape")

    def probe_dev(self, kind, src, nbytes, grid=0, block=0, stream=None):
        """An empty kernel (kind 0) or a kernel that only reads nbytes at src (kind 1)."""
        return self._served(self._l.jl_probe_dev(self._ctx, kind, src, nbytes, grid, block, stream), "jl_probe_dev")

    def lock(self):
        """The lock host-pointer calls hold while they run (jl_ctx_lock)."""
        self._served(self._l.jl_ctx_lock(self._ctx), "jl_ctx_lock")

    def unlock(self):
        self._served(self._l.jl_ctx_unlock(self._ctx), "jl_ctx_unlock")

    def resident_count(self):
        return int(self._l.jl_resident_count(self._ctx))

    def forget_range(self, address, nbytes):
        self._served(self._l.jl_forget(self._ctx, int(address), int(nbytes)), "jl_forget")

    def set_tuning(self, **kw):
        for k, v in kw.items():
            key = (k.replace("__", ".") if "__" in k else "matvec." + k).encode()
            self._served(self._l.jl_set_tuning(self._ctx, key, int(v)), "jl_set_tuning")

    @property
    def stream(self):
        return self._l.jl_stream(self._ctx)

    def synchronize(self):
        self._served(self._l.jl_synchronize(self._ctx), "jl_synchronize")

    # -- host-pointer seam ---------------------------------------------------
    def MatVec(self, out, t, w, x, nrows, k):
        """nn.Device.MatVec: out[0:nrows] = W x over raw GGUF bytes; False = declined."""
        if t not in quant.BLOCK:
            return False
        assert out.dtype == np.float32 and x.dtype == np.float32 and w.dtype == np.uint8
        assert out.size >= nrows and x.size >= k
        return self._served(self._l.jl_matvec(self._ctx, _ptr(out), t, _ptr(w), w.nbytes, _ptr(x),
                                              nrows, k), "jl_matvec")

    def MatMul(self, out, t, w, x, nrows, k, ntok):
        """JIT.MatMul (/root/reference/engine/nn/matmul.go:27): x [ntok][k] -> out [ntok][nrows]."""
        if t not in quant.BLOCK:
            return False
        assert out.dtype == np.float32 and x.dtype == np.float32 and w.dtype == np.uint8
        assert out.size >= ntok * nrows and x.size >= ntok * k
        return self._served(self._l.jl_matmul(self._ctx, _ptr(out), t, _ptr(w), w.nbytes, _ptr(x),
                                              nrows, k, ntok), "jl_matmul")

    def Forget(self, w):
        """nn.CopyForgetter.Forget: drop the device copy keyed on this host buffer."""
        self._served(self._l.jl_forget(self._ctx, _ptr(w), w.nbytes), "jl_forget")

    # -- packed planes, host pointers -----------------------------------------
    def packed_words(self, t, nrows, k):
        """kernels.PackedWords: (QS, D, SC) plane sizes in u32 words, or None if undefined."""
        nq, nd, nsc = C.c_size_t(), C.c_size_t(), C.c_size_t()
        rc = self._l.jl_packed_words(t, nrows, k, C.byref(nq), C.byref(nd), C.byref(nsc))
        return (nq.value, nd.value, nsc.value) if rc == _lib.OK else None

    def MatVecPacked(self, out, t, p, x, nrows, k):
        """JIT.MatVecPacked (/root/reference/engine/nn/packed.go:24); p = Packed(qs, d, sc, row, stride)."""
        assert out.dtype == np.float32 and x.dtype == np.float32
        return self._served(self._l.jl_matvec_packed(self._ctx, _ptr(out), t, _ptr(p.qs), _ptr(p.d),
                                                     _opt(p.sc), p.row, p.stride, _ptr(x), nrows, k),
                            "jl_matvec_packed")

    def MatMulPacked(self, out, t, p, x, nrows, k, ntok):
        """JIT.MatMulPacked (/root/reference/engine/nn/packedmm.go:23)."""
        assert out.dtype == np.float32 and x.dtype == np.float32
        return self._served(self._l.jl_matmul_packed(self._ctx, _ptr(out), t, _ptr(p.qs), _ptr(p.d),
                                                     _opt(p.sc), p.row, p.stride, _ptr(x), nrows, k, ntok),
                            "jl_matmul_packed")

    def _packed_multi(self, outs, t, ps, x, xstride, up, act, nrows, k, what):
        m = len(ps)
        assert len(outs) == m and x.dtype == np.float32 and all(o.dtype == np.float32 for o in outs)
        po = (C.c_void_p * m)(*[_ptr(o) for o in outs])
        pq = (C.c_void_p * m)(*[_ptr(p.qs) for p in ps])
        pd = (C.c_void_p * m)(*[_ptr(p.d) for p in ps])
        psc = (C.c_void_p * m)(*[_opt(p.sc) for p in ps])
        pr = (C.c_int * m)(*[p.row for p in ps])
        stride = ps[0].stride if m else 0
        assert all(p.stride == stride for p in ps)
        return self._served(self._l.jl_matvec_packed_multi(self._ctx, po, t, pq, pd, psc, pr, stride, _ptr(x), xstride,
                                                           _opt(up), act, nrows, k, m), what)

    def MatVecPackedMulti(self, outs, t, ps, x, nrows, k):
        """JIT.MatVecPackedMulti (/root/reference/engine/nn/packedmulti.go:24): several packed matvecs
        that share one activation; outs and ps are lists (numpy arrays, Packed)."""
        return self._packed_multi(outs, t, ps, x, 0, None, 0, nrows, k, "jl_matvec_packed_multi")

    def MatVecPackedGather(self, outs, t, ps, x, xstride, nrows, k):
        """JIT.MatVecPackedGather (/root/reference/engine/nn/packedmulti.go:84): matrix j reads
        x[j*xstride : j*xstride+k]."""
        return self._packed_multi(outs, t, ps, x, xstride, None, 0, nrows, k, "jl_matvec_packed_multi")

    def MatVecPackedGatherAct(self, outs, t, ps, x, up, act, xstride, nrows, k):
        """JIT.MatVecPackedGatherAct (/root/reference/engine/nn/packedmulti.go:93): matrix j reads
        act(x_j) * up_j; x is left as it was."""
        assert up.dtype == np.float32
        return self._packed_multi(outs, t, ps, x, xstride, up, act, nrows, k, "jl_matvec_packed_multi")

    def MatVecPackedGroup(self, g):
        """JIT.MatVecPackedGroup (/root/reference/engine/nn/packedgroup.go:51); g = MVGroup."""
        n = g.N
        po = (C.c_void_p * n)(*[_ptr(o) for o in g.Out[:n]])
        pt = (C.c_int * n)(*g.T[:n])
        pq = (C.c_void_p * n)(*[_ptr(p.qs) for p in g.P[:n]])
        pd = (C.c_void_p * n)(*[_ptr(p.d) for p in g.P[:n]])
        psc = (C.c_void_p * n)(*[_opt(p.sc) for p in g.P[:n]])
        pr = (C.c_int * n)(*[p.row for p in g.P[:n]])
        pst = (C.c_int * n)(*[p.stride for p in g.P[:n]])
        prw = (C.c_int * n)(*g.Rows[:n])
        return self._served(self._l.jl_matvec_packed_group(self._ctx, n, po, pt, pq, pd, psc, pr, pst, prw, _ptr(g.X), g.K,
                                                           _opt(g.ActUp), g.Act, _opt(g.Resid), float(g.Alpha)),
                            "jl_matvec_packed_group")

    def MoEGrouped(self, resid, t, gate_bank, up_bank, down_bank, x, sel, wt, rows, k_used, n_expert, n_ffn, n_embd):
        """One routed feed-forward block over host memory (moeBatchFrom,
        /root/reference/engine/model/moe.go:510-761): resid [rows][n_embd] accumulated in place."""
        assert resid.dtype == np.float32 and x.dtype == np.float32 and wt.dtype == np.float32 and sel.dtype == np.uint32
        return self._served(self._l.jl_moe_grouped(self._ctx, _ptr(resid), t, _ptr(gate_bank), _ptr(up_bank), _ptr(down_bank),
                                                   _ptr(x), _ptr(sel), sel.shape[1], _ptr(wt), rows, k_used, n_expert,
                                                   n_ffn, n_embd), "jl_moe_grouped")

    def ForgetPacked(self, p):
        self._served(self._l.jl_forget(self._ctx, _ptr(p.qs), 4), "jl_forget")

    # -- device-pointer entry points ------------------------------------------
    def pack_weights_dev(self, t, src, nrows, k, qs, d, sc, stream=None):
        """kernels.PackWeightsInto on the device: GGUF rows -> planes."""
        return self._served(self._l.jl_pack_weights_dev(self._ctx, t, _ptr(src), nrows, k, _ptr(qs), _ptr(d),
                                                        _opt(sc), stream), "jl_pack_weights_dev")

    def fold_admit_dev(self, t, w, nrows, k, stream=None):
        """Admits a Q4_K matrix to the folded-scale GEMM form ("gemm.fold" = 1); False when its
        scales can pass the f16 range."""
        return self._served(self._l.jl_fold_admit_dev(self._ctx, t, _ptr(w), nrows, k, stream), "jl_fold_admit_dev")

    def unpack_weights_dev(self, t, p, nrows, k, dst, stream=None):
        return self._served(self._l.jl_unpack_weights_dev(self._ctx, t, _ptr(p.qs), _ptr(p.d), _opt(p.sc),
                                                          p.row, p.stride, nrows, k, _ptr(dst), stream),
                            "jl_unpack_weights_dev")

    def matvec_packed_dev(self, out, t, p, x, nrows, k, stream=None):
        return self._served(self._l.jl_matvec_packed_dev(self._ctx, _ptr(out), t, _ptr(p.qs), _ptr(p.d),
                                                         _opt(p.sc), p.row, p.stride, _ptr(x), nrows, k,
                                                         stream), "jl_matvec_packed_dev")

    def matvec_packed_q8_dev(self, out, t, p, q, a_s, sum16, nrows, k, stream=None):
        return self._served(self._l.jl_matvec_packed_q8_dev(self._ctx, _ptr(out), t, _ptr(p.qs), _ptr(p.d),
                                                            _opt(p.sc), p.row, p.stride, _ptr(q), _ptr(a_s),
                                                            _ptr(sum16), nrows, k, stream),
                            "jl_matvec_packed_q8_dev")

    def matmul_packed_dev(self, out, t, p, x, nrows, k, ntok, stream=None):
        return self._served(self._l.jl_matmul_packed_dev(self._ctx, _ptr(out), t, _ptr(p.qs), _ptr(p.d),
                                                         _opt(p.sc), p.row, p.stride, _ptr(x), nrows, k,
                                                         ntok, stream), "jl_matmul_packed_dev")

    def quantize_act_dev(self, x, ntok, k, q, a_s, sum16, stream=None):
        return self._served(self._l.jl_quantize_act_dev(self._ctx, _ptr(x), ntok, k, _ptr(q),
                                                        _ptr(a_s), _ptr(sum16), stream),
                            "jl_quantize_act_dev")

    def dequant_dev(self, t, src, dst, n, stream=None):
        return self._served(self._l.jl_dequant_dev(self._ctx, t, _ptr(src), _ptr(dst), n, stream),
                            "jl_dequant_dev")

    def matvec_dev(self, out, t, w, x, nrows, k, stream=None):
        return self._served(self._l.jl_matvec_dev(self._ctx, _ptr(out), t, _ptr(w), _ptr(x),
                                                  nrows, k, stream), "jl_matvec_dev")

    def matvec_q8_dev(self, out, t, w, q, a_s, sum16, nrows, k, stream=None):
        return self._served(self._l.jl_matvec_q8_dev(self._ctx, _ptr(out), t, _ptr(w), _ptr(q),
                                                     _ptr(a_s), _ptr(sum16), nrows, k, stream),
                            "jl_matvec_q8_dev")

    def matvec_group_dev(self, outs, types, ws, rows, x, k, act_up=None, resid=None, alpha=0.0, stream=None,
                         norm_w=None, norm_eps=0.0, norm_out=None, resid_gate=None):
        """JIT.MatVecPackedGroup: up to four matvecs reading one activation, optional
        RMSNorm(x) * norm_w first, optional silu(x) * act_up and resid += alpha * out[0]
        (alpha * sigmoid(*resid_gate) when a device logit gates the add), in one launch."""
        g = _lib.MVGroup()
        g.n = len(outs)
        for i in range(g.n):
            g.out[i], g.type[i], g.w[i], g.rows[i] = _ptr(outs[i]), types[i], _ptr(ws[i]), rows[i]
        g.x, g.k, g.act_up, g.resid, g.alpha = _ptr(x), k, _opt(act_up), _opt(resid), alpha
        g.norm_w, g.norm_eps, g.norm_out, g.resid_gate = _opt(norm_w), norm_eps, _opt(norm_out), _opt(resid_gate)
        return self._served(self._l.jl_matvec_group_dev(self._ctx, C.byref(g), stream), "jl_matvec_group_dev")

    def matvec_gather_dev(self, outs, t, ws, x, xstride, up, nrows, k, stream=None):
        """JIT.MatVecPackedGather[Act] (xstride > 0) / MatVecPackedMulti (xstride 0, up None)."""
        m = len(outs)
        po = (C.c_void_p * m)(*[_ptr(o) for o in outs])
        pw = (C.c_void_p * m)(*[_ptr(w) for w in ws])
        return self._served(self._l.jl_matvec_gather_dev(self._ctx, po, t, pw, _ptr(x), xstride, _opt(up),
                                                         nrows, k, m, stream), "jl_matvec_gather_dev")

    def matvec_packed_multi_dev(self, outs, t, planes, row0, stride, x, xstride, up, nrows, k, stream=None,
                                resid=None, alpha=0.0, norm_w=None, norm_eps=0.0, norm_out=None, resid_gate=None):
        """MatVecPackedMulti / Gather / GatherAct over packed planes: planes is a list of
        (qs, d, sc) device pointers, row0 the first row of each matrix in its buffer;
        resid += alpha * out[0] rides on the launch when given, and norm_w puts an RMSNorm
        in front of the quantizer (not together with up)."""
        return self.packed_multi_call(self.packed_multi_args(outs, t, planes, row0, stride, x, xstride, up,
                                                             nrows, k, resid, alpha, norm_w, norm_eps, norm_out,
                                                             resid_gate), stream)

    def packed_multi_args(self, outs, t, planes, row0, stride, x, xstride, up, nrows, k, resid=None, alpha=0.0,
                          norm_w=None, norm_eps=0.0, norm_out=None, resid_gate=None):
        """The argument block of a packed multi call, built once by a caller that repeats it."""
        m = len(outs)
        po = (C.c_void_p * m)(*[_ptr(o) for o in outs])
        pq = (C.c_void_p * m)(*[_ptr(p[0]) for p in planes])
        pd = (C.c_void_p * m)(*[_ptr(p[1]) for p in planes])
        ps = (C.c_void_p * m)(*[_opt(p[2]) for p in planes])
        pr = (C.c_int * m)(*row0)
        return (po, t, pq, pd, ps, pr, stride, _ptr(x), xstride, _opt(up), _opt(resid), alpha, _opt(resid_gate), _opt(norm_w), norm_eps,
                _opt(norm_out), nrows, k, m)

    def packed_multi_call(self, args, stream=None):
        return self._served(self._l.jl_matvec_packed_multi_dev(self._ctx, *args, stream),
                            "jl_matvec_packed_multi_dev")

    def matmul_dev(self, out, t, w, x, nrows, k, ntok, stream=None):
        """x [ntok][k] -> out [ntok][nrows] on device operands (JIT.MatMulPacked semantics)."""
        return self._served(self._l.jl_matmul_dev(self._ctx, _ptr(out), t, _ptr(w), _ptr(x),
                                                  nrows, k, ntok, stream), "jl_matmul_dev")

    def matmul_static_dev(self, out, t, w, x, nrows, k, ntok, stream=None):
        """jl_matmul_dev on the library's static device workspace: allocates nothing."""
        return self._served(self._l.jl_matmul_static_dev(self._ctx, _ptr(out), t, _ptr(w), _ptr(x),
                                                         nrows, k, ntok, stream), "jl_matmul_static_dev")

    # -- mixture of experts -----------------------------------------------------
    def moe_logits_dev(self, logits, wtype, w, x, n_expert, k, ntok, stream=None):
        """Router logits [ntok][n_expert] = x [ntok][k] . W^T, W f32 (wtype 0) or f16 (1), in the
        reference device kernel's summation order (kernels.RouterMatVecTok)."""
        return self._served(self._l.jl_moe_logits_dev(self._ctx, _ptr(logits), wtype, _ptr(w), _ptr(x),
                                                      n_expert, k, ntok, stream), "jl_moe_logits_dev")

    def moe_route_dev(self, logits, rows, n_expert, k_used, sel, sel_stride, wt, stream=None):
        """oracle.MoERouter on the device: softmax, lexicographic top-k, renormalised weights."""
        return self._served(self._l.jl_moe_route_dev(self._ctx, _ptr(logits), rows, n_expert, k_used,
                                                     _ptr(sel), sel_stride, _ptr(wt), stream),
                            "jl_moe_route_dev")

    def moe_group_dev(self, sel, sel_stride, rows, k_used, n_expert, start, perm, pos, stream=None):
        return self._served(self._l.jl_moe_group_dev(self._ctx, _ptr(sel), sel_stride, rows, k_used,
                                                     n_expert, _ptr(start), _ptr(perm), _ptr(pos), stream),
                            "jl_moe_group_dev")

    def moe_matvec_dev(self, out0, out1, t, bank0, bank1, x, x2, src, start, n_expert, ncols, nrows, k,
                       stream=None):
        opt = lambda a: None if a is None else _ptr(a)
        return self._served(self._l.jl_moe_matvec_dev(self._ctx, _ptr(out0), opt(out1), t, _ptr(bank0),
                                                      opt(bank1), _ptr(x), opt(x2), opt(src), _ptr(start),
                                                      n_expert, ncols, nrows, k, stream), "jl_moe_matvec_dev")

    @staticmethod
    def packed_bank(qs, d, sc, sheet_bytes, stride):
        """jl_packed_bank: expert 0's planes (device addresses); sheet_bytes between experts' sheets
        (0: one plane set of `stride` rows holding every expert)."""
        return _lib.PackedBank(_ptr(qs), _ptr(d), _ptr(sc), int(sheet_bytes), int(stride))

    def moe_matvec_packed_dev(self, out0, out1, t, bank0, bank1, x, x2, src, start, n_expert, ncols, nrows, k,
                              stream=None):
        """jl_moe_matvec_dev over banks of packed planes (packed_bank(...))."""
        opt = lambda a: None if a is None else _ptr(a)
        return self._served(self._l.jl_moe_matvec_packed_dev(
            self._ctx, _ptr(out0), opt(out1), t, C.byref(bank0), None if bank1 is None else C.byref(bank1), _ptr(x),
            opt(x2), opt(src), _ptr(start), n_expert, ncols, nrows, k, stream), "jl_moe_matvec_packed_dev")

    def moe_ffn_packed_dev(self, resid, t, gate, up, down, x, sel, sel_stride, wt, rows, k_used, n_expert, n_ffn,
                           n_embd, stream=None):
        """One routed feed-forward block over banks of packed planes."""
        return self._served(self._l.jl_moe_ffn_packed_dev(
            self._ctx, _ptr(resid), t, C.byref(gate), C.byref(up), C.byref(down), _ptr(x), _ptr(sel), sel_stride,
            _ptr(wt), rows, k_used, n_expert, n_ffn, n_embd, stream), "jl_moe_ffn_packed_dev")

    def moe_combine_dev(self, resid, y, wt, sel, sel_stride, pos, rows, k_used, n_embd, stream=None):
        return self._served(self._l.jl_moe_combine_dev(self._ctx, _ptr(resid), _ptr(y), _ptr(wt), _ptr(sel),
                                                       sel_stride, _ptr(pos), rows, k_used, n_embd, stream),
                            "jl_moe_combine_dev")

    def moe_ffn_dev(self, resid, t, gate, up, down, x, sel, sel_stride, wt, rows, k_used, n_expert,
                    n_ffn, n_embd, stream=None, down_type=None):
        """One routed feed-forward block (moeBatchFrom): resid [rows][n_embd] += mixture output.
        down_type: the down bank's type where it differs from gate and up."""
        return self._served(self._l.jl_moe_ffn_types_dev(self._ctx, _ptr(resid), t, t if down_type is None else down_type,
                                                         _ptr(gate), _ptr(up), _ptr(down), _ptr(x), _ptr(sel),
                                                         sel_stride, _ptr(wt), rows, k_used, n_expert, n_ffn, n_embd,
                                                         stream),
                            "jl_moe_ffn_types_dev")

    def moe_block_dev(self, resid, t, gate, up, down, router, x, rows, k_used, n_expert, n_ffn, n_embd, sel=None,
                      wt=None, stream=None, down_type=None, router_type=0):
        """The whole mixture block, router included: resid [rows][n_embd] += mixture output.  gate / up /
        down: banks of GGUF sheets (device addresses), or three packed_bank(...) structures."""
        if isinstance(gate, _lib.PackedBank):
            return self._served(self._l.jl_moe_block_packed_dev(
                self._ctx, _ptr(resid), t, C.byref(gate), C.byref(up), C.byref(down), router_type, _ptr(router), _ptr(x),
                rows, k_used, n_expert, n_ffn, n_embd, _opt(sel), _opt(wt), stream), "jl_moe_block_packed_dev")
        return self._served(self._l.jl_moe_block_dev(
            self._ctx, _ptr(resid), t, t if down_type is None else down_type, _ptr(gate), _ptr(up), _ptr(down),
            router_type, _ptr(router), _ptr(x), rows, k_used, n_expert, n_ffn, n_embd, _opt(sel), _opt(wt), stream),
            "jl_moe_block_dev")

    def matmul_mxfp4_bf16_dev(self, out, w, x, nrows, k, ntok, stream=None):
        """MXFP4 weights x bf16 activations (bits as uint16) -> f32 out [ntok][nrows]."""
        return self._served(self._l.jl_matmul_mxfp4_bf16_dev(self._ctx, _ptr(out), _ptr(w), _ptr(x),
                                                             nrows, k, ntok, stream),
                            "jl_matmul_mxfp4_bf16_dev")

    def matmul_mxfp4_packed_bf16_dev(self, out, p, x, nrows, k, ntok, stream=None):
        """The same over packed MXFP4 planes; p = Packed(qs, d, None, row, stride)."""
        return self._served(self._l.jl_matmul_mxfp4_packed_bf16_dev(self._ctx, _ptr(out), _ptr(p.qs), _ptr(p.d),
                                                                    p.row, p.stride, _ptr(x), nrows, k, ntok,
                                                                    stream), "jl_matmul_mxfp4_packed_bf16_dev")
