#!/usr/bin/env python3
"""Headline benchmark: Q4_K decode matvec, batch 1, 4096x4096, on one MI355X.

One step = one pass of the hot path over one activation vector: quantize x to
int8 and compute out = W x, both inside one fused kernel launch
(jl_matvec_dev), which is what the reference's own protocol times (NewInput +
MatVecPacked per call, /root/reference/engine/nn/perbyte_test.go:131-144).
Weights rotate through enough distinct device copies to exceed twice the
256 MB Infinity Cache, so no launch is served from cache (same file,
:184-189, :246-253).  Inputs are resident in HBM before the timed region.

Timing protocol (the reference's: warm calls, then the median of nine timed
runs, perbyte_test.go:131-144): at least 200 untimed launches, then NINE timed
windows of exactly --steps launches each, each window bracketed by HIP events
on the launch stream; the reported step time is the median window's.  Every
window is enqueued behind a wait kernel (one wavefront watching the clock, no
memory traffic), so its launches are already queued when the first one starts
and a short window measures the device, not the host's launch rate.  Every section checks the output it timed
against dequantize (on the device) + an f64 product on rows spread over the grid.

Prints ONE JSON line.  `value` is algorithmic bytes per second (weight bytes +
x + out per launch), `roofline` prices the same figure against the 8 TB/s HBM
peak; `cpu_baseline` is the intrinsic restatement of the reference's host
kernels timed on this box's cores (a reported baseline, not a target).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
CACHE_BYTES = 256 << 20  # Infinity Cache; rotate through more than twice this

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# script (profiles/), scaled by the same counters over a plain copy of known
# size (profiles/matvec_q4k_4096_hbm_traffic.md: fetch 4723.0 x 1.9950 KiB + write 16 KiB).
MEASURED_TRAFFIC = {"c1": 9638349}


def matvec_bytes(t, nrows, k):
    from jitllm_amd import quant
    return nrows * quant.row_bytes(t, k) + 4 * k + 4 * nrows


def spread_rows(nrows, n):
    """About n row indices: the first and last eight and the rest evenly over the matrix."""
    picks = set(range(min(8, nrows))) | set(range(max(0, nrows - 8), nrows))
    picks |= set(int(v) for v in np.linspace(0, nrows - 1, n))
    return np.array(sorted(picks))


def dequant_rows(dev, t, w_host, rows, k):
    """Rows of a GGUF weight dequantized ON THE DEVICE (jl_dequant_dev) -> f64 [len(rows)][k]."""
    from jitllm_amd import quant
    from jitllm_amd.hipmem import DeviceArray
    rb = quant.row_bytes(t, k)
    rows = np.asarray(rows)
    if len(rows) > 1 and np.all(np.diff(rows) == 1):      # a contiguous range (an expert's sheet)
        src = DeviceArray(w_host[int(rows[0]) * rb:(int(rows[-1]) + 1) * rb])
    else:
        src = DeviceArray(np.concatenate([w_host[r * rb:(r + 1) * rb] for r in rows]))
    dst = DeviceArray(shape=(len(rows) * k,), dtype=np.float32, fill=0)
    if not dev.dequant_dev(t, src.ptr, dst.ptr, len(rows) * k):
        raise RuntimeError("the device declined to dequantize")
    dev.synchronize()
    out = dst.get().reshape(len(rows), k).astype(np.float64)
    src.free()
    dst.free()
    return out


def rel_err(got, want, what, bar=2e-2):
    got = np.asarray(got, np.float64)
    if not np.all(np.isfinite(got)):
        raise RuntimeError(f"{what}: non-finite output")
    err = float(np.sqrt(np.mean((got - want) ** 2)) / max(np.sqrt(np.mean(want ** 2)), 1e-30))
    if not err <= bar:
        raise RuntimeError(f"{what}: output differs from dequantize + f64 product by {err:.3e}")
    return err


def measure(dev, run, steps, gate, warm=3, windows=9):
    """warm untimed calls of run(i), then the median over nine windows of `steps` calls, each
    window enqueued behind the gate."""
    from jitllm_amd.hipmem import timed_windows
    for i in range(warm):
        run(i)
    dev.synchronize()
    ms, _ = timed_windows(run, steps, dev.stream, windows, gate)
    return ms


class Workload:
    """A weight matrix replicated into rotating device copies plus x and out."""

    def __init__(self, dev, t, nrows, k, window, seed=0, packed=False):
        """packed=False: GGUF row-major bytes (jl_matvec_dev); packed=True: the reference's
        QS/D/SC planes, packed on the device from the same bytes (jl_matvec_packed_dev)."""
        from jitllm_amd import quant, synth
        from jitllm_amd.device import Packed
        from jitllm_amd.hipmem import DeviceArray, check, hip
        self.dev, self.t, self.nrows, self.k, self.window = dev, t, nrows, k, window
        self.packed = packed
        self.name = f"{quant.NAMES[t]} matvec {nrows}x{k} batch 1"
        self.w_host = synth.quantized_weights(t, nrows, k, seed=seed)
        self.x_host = synth.activations(k, seed=seed + 1)
        one = DeviceArray(self.w_host)
        if packed:
            nq, nd, nsc = dev.packed_words(t, nrows, k)
            up = lambda v: (v + 255) & ~255
            o_d = up(nq * 4)
            o_sc = o_d + up(nd * 4)
            self.wbytes = o_sc + up(nsc * 4)
            self.alg_bytes = (nq + nd + nsc) * 4 + 4 * k + 4 * nrows
        else:
            self.wbytes = self.w_host.nbytes
            self.alg_bytes = matvec_bytes(t, nrows, k)
        self.ncopies = max(2, min(128, (2 * CACHE_BYTES + 64 * (1 << 20)) // self.wbytes + 1))
        self.pool = DeviceArray(shape=(self.ncopies * self.wbytes,), dtype=np.uint8)
        self.planes = []
        for i in range(self.ncopies):
            base = self.pool.ptr + i * self.wbytes
            if packed:
                pl = Packed(base, base + o_d, base + o_sc if nsc else None, 0, nrows)
                if not dev.pack_weights_dev(t, one.ptr, nrows, k, pl.qs, pl.d, pl.sc):
                    raise RuntimeError(f"{self.name}: the device declined to pack")
                self.planes.append(pl)
            else:
                check(hip().hipMemcpy(base, one.ptr, self.wbytes, 3), "copy")
        dev.synchronize()
        one.free()
        self.x = DeviceArray(self.x_host)
        self.out = DeviceArray(shape=(nrows,), dtype=np.float32, fill=0)

    def step(self, i):
        if self.packed:
            ok = self.dev.matvec_packed_dev(self.out.ptr, self.t, self.planes[i % self.ncopies], self.x.ptr,
                                            self.nrows, self.k)
        else:
            ok = self.dev.matvec_dev(self.out.ptr, self.t, self.pool.ptr + (i % self.ncopies) * self.wbytes,
                                     self.x.ptr, self.nrows, self.k)
        if not ok:
            raise RuntimeError(f"{self.name}: the device declined")

    def timed(self, steps, warmup, gate=None):
        """(ms per step of the median of nine windows of `steps` launches, by HIP events on the
        launch stream; every window's ms per step; host microseconds to enqueue one launch)."""
        from jitllm_amd.hipmem import synchronize, timed_windows
        self.dev.SetActWindow(self.window)
        for i in range(max(warmup, 200)):
            self.step(i)
        self.dev.synchronize()
        synchronize()
        t0 = time.perf_counter()
        for i in range(64):
            self.step(i)
        host_us = (time.perf_counter() - t0) * 1e6 / 64
        self.dev.synchronize()
        ms, per = timed_windows(self.step, steps, self.dev.stream, 9, gate, host_us)
        synchronize()
        return ms, per, host_us

    def timed_hot(self, steps, gate=None):
        """ms per step over copy 0 alone (weights cache resident)."""
        from jitllm_amd.hipmem import timed_windows
        self.dev.SetActWindow(self.window)
        for _ in range(50):
            self.step(0)
        self.dev.synchronize()
        ms, _ = timed_windows(lambda i: self.step(0), steps, self.dev.stream, 9, gate)
        return ms

    def check(self):
        """The last step's output: every row finite, and 96 rows spread over the whole grid
        (first, last, and evenly between) within 2 % (of the rows' RMS) of dequantize (on the
        device) + f64 dot with the f32 activation; the int8 activation accounts for a few parts
        in a thousand.  A sanity gate on what was timed, not the parity test."""
        got = self.out.get()
        if not np.all(np.isfinite(got)):
            raise RuntimeError(f"{self.name}: non-finite output")
        rows = spread_rows(self.nrows, 96)
        want = dequant_rows(self.dev, self.t, self.w_host, rows, self.k) @ self.x_host.astype(np.float64)
        return rel_err(got[rows], want, self.name)

    def free(self):
        self.pool.free()
        self.x.free()
        self.out.free()


def cpu_baseline(t, nrows, k, window, seed=0):
    """The reference's host path (restated with intrinsics, oracle/jl_cpu_path.c) on this
    box's cores: packed planes, rotating copies >= 192 MiB, 3 warm calls, then the median of nine
    timed passes (the reference's protocol), each pass long enough that the leg is about 20
    core-seconds of work."""
    import oracle
    from jitllm_amd import synth
    cores = min(16, len(os.sched_getaffinity(0)))
    w = synth.quantized_weights(t, nrows, k, seed=seed)
    x = synth.activations(k, seed=seed + 1)
    qs, d, sc = oracle.pack_weights(t, w, nrows, k)
    one = qs.nbytes + d.nbytes + sc.nbytes
    n = max(1, (192 << 20) // one)
    copies = [(qs.copy(), d.copy(), sc.copy()) for _ in range(n)]
    cp = oracle.CpuPath(cores)
    probe = cp.time_matvec(t, copies, x, nrows, k, window, reps=1)
    sweeps = max(1, int(0.14 / max(probe * n, 1e-6)))       # ~0.14 s a pass, nine passes
    sec = cp.time_matvec(t, copies, x, nrows, k, window, reps=9, sweeps=sweeps)
    wall = cp.membw(1 << 30, 3)
    vnni = cp.vnni
    cp.close()
    return {
        "value": round(one / sec / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
        "sample": f"{n} distinct packed copies ({n * one >> 20} MiB), 3 warm calls, median of 9 passes of "
                  f"{sweeps} sweeps over the copies ({9 * sweeps * n} calls); "
                  f"activation quantizer included per call; "
                  f"{'AVX-VNNI VPDPBUSD' if vnni else 'AVX2 VPMADDUBSW'} 256-bit; "
                  f"host read wall {wall / 1e9:.1f} GB/s",
        "us_per_call": round(sec * 1e6, 1),
    }


MFMA_F16_PEAK_TFLOPS = 2500.0


def cpu_baseline_gemm(nrows, k, ntok, window=256, seed=0):
    """The reference's weight-stationary prefill GEMM on this box's cores (restated with
    intrinsics, oracle/jl_cpu_path.c; Q4_K planes, the activation quantizer inside every call):
    3 warm calls, then the median of nine timed calls of the whole matmul."""
    import oracle
    from jitllm_amd import quant, synth
    cores = min(16, len(os.sched_getaffinity(0)))
    w = synth.quantized_weights(quant.Q4_K, nrows, k, seed=seed)
    x = np.random.default_rng(2).standard_normal((ntok, k), np.float32)
    qs, d, sc = oracle.pack_weights(quant.Q4_K, w, nrows, k)
    cp = oracle.CpuPath(cores)
    sec = cp.time_matmul(quant.Q4_K, qs, d, sc, x, nrows, k, ntok, window, reps=9)
    vnni = cp.vnni
    cp.close()
    return {"value": round(2.0 * nrows * k * ntok / sec / 1e12, 3), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{ntok} tokens x {k} -> {nrows}, Q4_K planes, window {window}: 3 warm calls, median of 9 calls "
                      f"(12 calls, {12 * sec:.2f} s); work items of 16 rows x 64 tokens handed to {cores} spinning workers; "
                      f"{'AVX-VNNI VPDPBUSD' if vnni else 'AVX2 VPMADDUBSW'} 256-bit",
            "ms_per_call": round(sec * 1e3, 2)}


def cpu_baseline_moe(hosts, x_host, sel, wt, n_expert, n_ffn, n_embd, window=256):
    """The reference's routed feed-forward block on this box's cores (oracle/jl_cpu_path.c: expert
    by expert, gather, gate and up through the GEMM, silu(g) * u, down, the residual add), over
    the same banks (as planes), rows, selection and weights the device block was given."""
    import oracle
    from jitllm_amd import quant
    cores = min(16, len(os.sched_getaffinity(0)))
    shapes = [(n_ffn, n_embd), (n_ffn, n_embd), (n_embd, n_ffn)]
    planes = [oracle.pack_weights(quant.Q4_K, h, n_expert * r, k) for h, (r, k) in zip(hosts, shapes)]
    cp = oracle.CpuPath(cores)
    sec = cp.time_moe_block(planes[0], planes[1], planes[2], x_host, sel, wt, n_expert, n_ffn, n_embd, window, reps=9)
    cp.close()
    return {"us_per_step": round(sec * 1e6, 1), "cores": cores, "kind": "port",
            "sample": f"one warm block, median of 9 blocks; selection and weights given (the router is not in the CPU "
                      f"figure); {cores} spinning workers"}


def gemm_section(dev, gate, shapes=None, t=None, k=4096, window=256, packed=False):
    """Prefill GEMM (x [ntok][k] f32 -> out [ntok][nrows]), activation quantizer and layout
    kernel included in every step; flops = 2*nrows*k*ntok, priced against the dense f16 MFMA
    peak (the kernel runs exact integer operands on the f16 matrix cores).
    shapes: {nrows: [ntok, ...]}; default = the baseline's prefill configurations.
    t = Q6_K / Q8_0: the same model's other tensors.  packed: the weights as packed planes
    (jl_matmul_packed_dev).  Output check: 96 rows spread over the matrix x every token.
    Q4_K rows also run the opt-in folded-scale form ("gemm.fold" = 1) where it applies, reported
    beside the exact form with its measured rel-L2 against the exact result."""
    from jitllm_amd import quant, synth
    from jitllm_amd.device import Packed
    from jitllm_amd.hipmem import DeviceArray
    t = quant.Q4_K if t is None else t
    dev.SetActWindow(window)
    out = {}
    shapes = shapes or {4096: (16, 128, 512, 2048), 14336: (16, 128, 512, 2048)}
    for nrows, toks in shapes.items():
        w_host = synth.quantized_weights(t, nrows, k, seed=0)
        w = DeviceArray(w_host)
        rows = spread_rows(nrows, 96)
        wrows = dequant_rows(dev, t, w_host, rows, k)
        pl = None
        folded = t == quant.Q4_K and not packed and dev.fold_admit_dev(t, w.ptr, nrows, k)
        if packed:
            bufs = [DeviceArray(shape=(max(n, 1),), dtype=np.uint32, fill=0) for n in dev.packed_words(t, nrows, k)]
            if not dev.pack_weights_dev(t, w.ptr, nrows, k, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr):
                raise RuntimeError("the device declined to pack")
            dev.synchronize()
            pl = Packed(bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, 0, nrows)
        for ntok in toks:
            x_host = np.random.default_rng(2).standard_normal((ntok, k), np.float32)
            x = DeviceArray(x_host)
            o = DeviceArray(shape=(ntok, nrows), dtype=np.float32, fill=np.float32(np.nan))
            if not dev.reserve_shape(t, nrows, k, ntok, packed):
                raise RuntimeError("the device declined the prefill GEMM's shape")

            def run(_):
                ok = (dev.matmul_packed_dev(o.ptr, t, pl, x.ptr, nrows, k, ntok) if packed
                      else dev.matmul_dev(o.ptr, t, w.ptr, x.ptr, nrows, k, ntok))
                if not ok:
                    raise RuntimeError("the device declined the prefill GEMM")
            ms = measure(dev, run, 20, gate)
            got = o.get()
            if not np.all(np.isfinite(got)):
                raise RuntimeError(f"prefill GEMM {ntok}x{k}->{nrows}: non-finite or unwritten output")
            err = rel_err(got[:, rows], x_host.astype(np.float64) @ wrows.T, f"prefill GEMM {ntok}x{k}->{nrows}")
            tf = 2.0 * nrows * k * ntok / (ms * 1e-3) / 1e12
            out[f"{ntok}x{k}->{nrows}"] = {"us_per_step": round(ms * 1e3, 1), "TFLOP/s": round(tf, 1),
                                          "frac_of_f16_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                                          "checked_rel_err": float(f"{err:.2e}")}
            if folded:
                # the opt-in folded-scale form beside the exact one: never the line above, and
                # its time only together with its measured distance from the exact result
                dev.set_tuning(gemm__fold=1)
                try:
                    ms_f = measure(dev, run, 20, gate)
                    got_f = o.get()
                finally:
                    dev.set_tuning(gemm__fold=0)
                if not np.array_equal(got_f.view(np.uint32), got.view(np.uint32)):   # else: a shape the form does not serve
                    if not np.all(np.isfinite(got_f)):
                        raise RuntimeError(f"folded prefill GEMM {ntok}x{k}->{nrows}: non-finite output")
                    e = got.astype(np.float64)
                    rel = float(np.sqrt(np.sum((got_f - e) ** 2) / np.sum(e * e)))
                    if rel > 1e-3:
                        raise RuntimeError(f"folded prefill GEMM {ntok}x{k}->{nrows}: rel-L2 {rel:.2e} against the exact form")
                    tf_f = 2.0 * nrows * k * ntok / (ms_f * 1e-3) / 1e12
                    out[f"{ntok}x{k}->{nrows}"]["folded_opt_in"] = {
                        "us_per_step": round(ms_f * 1e3, 1), "TFLOP/s": round(tf_f, 1),
                        "frac_of_f16_mfma_peak": round(tf_f / MFMA_F16_PEAK_TFLOPS, 4),
                        "rel_l2_vs_exact_form": float(f"{rel:.2e}")}
            x.free()
            o.free()
        if folded:
            dev.forget_range(w.ptr, w_host.nbytes)
        w.free()
        if packed:
            for b in bufs:
                b.free()
    return out


def _silu(v):
    return v / (1.0 + np.exp(-v))


def _ffn_check(dev, quant, wg, wd, x_host, gate, up, y, resid, n_embd, n_ffn, what):
    """gate / up rows against dequantize + f64 dot of the normed x (norm weight 1), and y rows
    against dequantize + f64 dot of silu(gate) * up taken from the device's own gate and up."""
    g, u, yy, r = gate.get(), up.get(), y.get(), resid.get()
    xn = x_host.astype(np.float64)
    xn = xn / np.sqrt(np.mean(xn * xn) + 1e-5)
    rows = spread_rows(n_ffn, 64)
    want = dequant_rows(dev, quant.Q8_0, wg, rows, n_embd) @ xn
    e1 = rel_err(g[rows], want, what + " gate")
    rel_err(u[rows], want, what + " up")
    rows = spread_rows(n_embd, 64)
    h = _silu(g.astype(np.float64)) * u.astype(np.float64)
    e2 = rel_err(yy[rows], dequant_rows(dev, quant.Q6_K, wd, rows, n_ffn) @ h, what + " down")
    rel_err(r[rows], yy[rows].astype(np.float64), what + " residual add", 1e-5)
    return max(e1, e2)


def ffn_section(dev, gate_):
    """A gated feed-forward block at decode, the baseline's second configuration: RMSNorm folded
    into the quantizer of gate and up (Q8_0 14336x4096), one grouped launch; then down (Q6_K
    4096x14336) over silu(gate) * up formed inside its quantizer with the residual add riding
    on the launch: two launches per block.  Four rotating sets of the three matrices
    (692 MiB) keep every step out of cache."""
    from jitllm_amd import quant, synth
    from jitllm_amd.hipmem import DeviceArray
    n_embd, n_ffn = 4096, 14336
    dev.SetActWindow(32)
    wg = synth.quantized_weights(quant.Q8_0, n_ffn, n_embd, seed=0)
    wd = synth.quantized_weights(quant.Q6_K, n_embd, n_ffn, seed=1)
    sets = []
    for i in range(4):
        g, u, d = DeviceArray(wg), DeviceArray(wg), DeviceArray(wd)
        sets.append((g, u, d))
    x_host = synth.activations(n_embd, seed=2)
    x = DeviceArray(x_host)
    norm_w = DeviceArray(np.ones(n_embd, np.float32))
    gate = DeviceArray(shape=(n_ffn,), dtype=np.float32, fill=0)
    up = DeviceArray(shape=(n_ffn,), dtype=np.float32, fill=0)
    y = DeviceArray(shape=(n_embd,), dtype=np.float32, fill=0)
    resid = DeviceArray(shape=(n_embd,), dtype=np.float32, fill=0)

    def run(i):
        g, u, d = sets[i % len(sets)]
        ok = dev.matvec_group_dev([gate.ptr, up.ptr], [quant.Q8_0, quant.Q8_0], [g.ptr, u.ptr], [n_ffn, n_ffn],
                                  x.ptr, n_embd, norm_w=norm_w.ptr, norm_eps=1e-5)
        ok = ok and dev.matvec_group_dev([y.ptr], [quant.Q6_K], [d.ptr], [n_embd], gate.ptr, n_ffn, act_up=up.ptr,
                                         resid=resid.ptr, alpha=1.0)
        if not ok:
            raise RuntimeError("the device declined the feed-forward block")
    ms = measure(dev, run, 20, gate_, warm=8)
    resid.zero()
    run(0)
    dev.synchronize()
    err = _ffn_check(dev, quant, wg, wd, x_host, gate, up, y, resid, n_embd, n_ffn, "feed-forward block")
    nbytes = 2 * wg.nbytes + wd.nbytes + 4 * (n_embd + 2 * n_ffn) + 4 * (2 * n_ffn + 2 * n_embd)
    for g, u, d in sets:
        g.free(); u.free(); d.free()
    for b in (x, norm_w, gate, up, y, resid):
        b.free()
    return {"us_per_step": round(ms * 1e3, 2), "launches_per_step": 2, "bytes_per_step": nbytes,
            "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "checked_rel_err": float(f"{err:.2e}")}


def ffn_packed_section(dev, gate_):
    """The same gated feed-forward block over packed planes, the layout a .jlm file holds:
    gate and up (Q8_0 14336x4096) one launch of two packed matvecs sharing x, down (Q6_K
    4096x14336) one launch over silu(gate) * up with the residual add riding on it; the
    RMSNorm in front of gate and up is folded into their quantizer.  Four rotating sets of
    planes keep every step out of cache."""
    from jitllm_amd import quant, synth
    from jitllm_amd.hipmem import DeviceArray
    n_embd, n_ffn = 4096, 14336
    dev.SetActWindow(32)
    wg = synth.quantized_weights(quant.Q8_0, n_ffn, n_embd, seed=0)
    wd = synth.quantized_weights(quant.Q6_K, n_embd, n_ffn, seed=1)

    def planes_of(t, w_host, nrows, k):
        src = DeviceArray(w_host)
        pl = [DeviceArray(shape=(max(n, 1),), dtype=np.uint32, fill=0) for n in dev.packed_words(t, nrows, k)]
        if not dev.pack_weights_dev(t, src.ptr, nrows, k, pl[0].ptr, pl[1].ptr, pl[2].ptr):
            raise RuntimeError("the device declined to pack a matrix")
        dev.synchronize()
        src.free()
        return pl
    sets = [(planes_of(quant.Q8_0, wg, n_ffn, n_embd), planes_of(quant.Q8_0, wg, n_ffn, n_embd),
             planes_of(quant.Q6_K, wd, n_embd, n_ffn)) for _ in range(4)]
    x_host = synth.activations(n_embd, seed=2)
    x = DeviceArray(x_host)
    gate = DeviceArray(shape=(n_ffn,), dtype=np.float32, fill=0)
    up = DeviceArray(shape=(n_ffn,), dtype=np.float32, fill=0)
    y = DeviceArray(shape=(n_embd,), dtype=np.float32, fill=0)
    resid = DeviceArray(shape=(n_embd,), dtype=np.float32, fill=0)
    norm_w = DeviceArray(np.ones(n_embd, np.float32))
    tri = lambda pl: (pl[0].ptr, pl[1].ptr, pl[2].ptr)
    calls = [(dev.packed_multi_args([gate.ptr, up.ptr], quant.Q8_0, [tri(g), tri(u)], [0, 0], n_ffn, x.ptr, 0, None,
                                    n_ffn, n_embd, norm_w=norm_w.ptr, norm_eps=1e-5),
              dev.packed_multi_args([y.ptr], quant.Q6_K, [tri(d)], [0], n_embd, gate.ptr, 0, up.ptr, n_embd, n_ffn,
                                    resid=resid.ptr, alpha=1.0)) for g, u, d in sets]

    def run(i):
        a, b = calls[i % len(calls)]
        if not (dev.packed_multi_call(a) and dev.packed_multi_call(b)):
            raise RuntimeError("the device declined the packed feed-forward block")
    ms = measure(dev, run, 20, gate_, warm=8)
    resid.zero()
    run(0)
    dev.synchronize()
    err = _ffn_check(dev, quant, wg, wd, x_host, gate, up, y, resid, n_embd, n_ffn, "packed feed-forward block")
    nbytes = 2 * n_ffn * quant.row_bytes(quant.Q8_0, n_embd) + n_embd * quant.row_bytes(quant.Q6_K, n_ffn) \
        + 4 * (n_embd + 2 * n_ffn) + 4 * (2 * n_ffn + 2 * n_embd)
    for st in sets:
        for pl in st:
            for b in pl:
                b.free()
    for b in (x, gate, up, y, resid, norm_w):
        b.free()
    return {"us_per_step": round(ms * 1e3, 2), "launches_per_step": 2, "bytes_per_step": nbytes,
            "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "checked_rel_err": float(f"{err:.2e}")}


def moe_section(dev, gate_, rows=64, packed=False, cpu=False):
    """Qwen3-30B-A3B routed feed-forward block: 128 experts (gate/up 768x2048, down 2048x768,
    Q4_K), 64 rows routed top-8; one step = router logits (f32 router matrix, rows ~ N(0, 1/k)
    so the logits are ~ N(0,1)) + softmax/top-8 + group + gate/up + down + combine, all on the
    device.  Bytes = the touched experts' three sheets + router matrix + x in + resid out.
    Output check: three rows of the block recomputed in f64 from sheets dequantized on the
    device, with the device's own selection and weights.
    packed: the three banks are packed planes on the device (one plane set per bank, as a .jlm
    file holds them), read where they lie."""
    from jitllm_amd import quant, synth
    from jitllm_amd.hipmem import DeviceArray
    t, n_expert, k_used, n_ffn, n_embd = quant.Q4_K, 128, 8, 768, 2048
    dev.SetActWindow(256)
    rng = np.random.default_rng(0)
    x_host = rng.standard_normal((rows, n_embd)).astype(np.float32)
    x = DeviceArray(x_host)
    router = DeviceArray((rng.standard_normal((n_expert, n_embd)) / np.sqrt(n_embd)).astype(np.float32))
    ld = DeviceArray(shape=(rows, n_expert), dtype=np.float32, fill=0)
    sd = DeviceArray(shape=(rows, k_used + 1), dtype=np.uint32, fill=0)
    wd = DeviceArray(shape=(rows, k_used), dtype=np.float32, fill=0)
    if not (dev.moe_logits_dev(ld.ptr, 0, router.ptr, x.ptr, n_expert, n_embd, rows) and
            dev.moe_route_dev(ld.ptr, rows, n_expert, k_used, sd.ptr, k_used + 1, wd.ptr)):
        raise RuntimeError("the device declined the router")
    dev.synchronize()
    touched = len(np.unique(sd.get()[:, :k_used]))
    gs = n_ffn * quant.row_bytes(t, n_embd)
    ds = n_embd * quant.row_bytes(t, n_ffn)
    banks, hosts = [], []
    for i, (r, k) in enumerate([(n_ffn, n_embd), (n_ffn, n_embd), (n_embd, n_ffn)]):
        hosts.append(synth.quantized_weights(t, r * n_expert, k, seed=10 + i))
        banks.append(DeviceArray(hosts[-1]))
    resid = DeviceArray(shape=(rows, n_embd), dtype=np.float32, fill=0)
    pbanks = []
    if packed:
        for i, (r, k) in enumerate([(n_ffn, n_embd), (n_ffn, n_embd), (n_embd, n_ffn)]):
            nq, nd, nsc = dev.packed_words(t, r * n_expert, k)
            pl = [DeviceArray(shape=(n,), dtype=np.uint32, fill=0) for n in (nq, nd, nsc)]
            if not dev.pack_weights_dev(t, banks[i].ptr, r * n_expert, k, pl[0].ptr, pl[1].ptr, pl[2].ptr):
                raise RuntimeError("the device declined to pack a bank")
            dev.synchronize()
            banks[i].free()
            banks[i] = pl[0]
            banks += pl[1:]
            pbanks.append(dev.packed_bank(pl[0].ptr, pl[1].ptr, pl[2].ptr, 0, r * n_expert))

    def run(_):
        # one call: router logits, softmax + top-8, grouping, gate + up, down, combine
        b = pbanks if packed else [bk.ptr for bk in banks[:3]]
        if not dev.moe_block_dev(resid.ptr, t, b[0], b[1], b[2], router.ptr, x.ptr, rows, k_used, n_expert, n_ffn,
                                 n_embd, sel=sd.ptr, wt=wd.ptr):
            raise RuntimeError("the device declined the mixture block")
    ms = measure(dev, run, 20, gate_)
    resid.zero()
    run(0)
    dev.synchronize()
    got, sel, wt = resid.get(), sd.get(), wd.get()
    if not np.all(np.isfinite(got)):
        raise RuntimeError("mixture block: non-finite output")
    err = 0.0
    for r in (0, rows // 2, rows - 1):
        want = np.zeros(n_embd)
        xr = x_host[r].astype(np.float64)
        for s_ in range(k_used):
            e = int(sel[r, s_])
            g = dequant_rows(dev, t, hosts[0], np.arange(e * n_ffn, (e + 1) * n_ffn), n_embd) @ xr
            u = dequant_rows(dev, t, hosts[1], np.arange(e * n_ffn, (e + 1) * n_ffn), n_embd) @ xr
            want += float(wt[r, s_]) * (dequant_rows(dev, t, hosts[2], np.arange(e * n_embd, (e + 1) * n_embd), n_ffn)
                                        @ (_silu(g) * u))
        err = max(err, rel_err(got[r], want, f"mixture block row {r}", 3e-2))
    nbytes = touched * (2 * gs + ds) + 2 * rows * n_embd * 4 + n_expert * n_embd * 4
    for b in banks + [x, sd, wd, resid, ld, router]:
        b.free()
    out = {"us_per_step": round(ms * 1e3, 1), "experts_touched": touched, "bytes_per_step": nbytes,
           "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
           "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
           "TFLOP/s": round(rows * k_used * 3 * 2.0 * n_ffn * n_embd / (ms * 1e-3) / 1e12, 2),
           "checked_rel_err": float(f"{err:.2e}")}
    if cpu:
        base = cpu_baseline_moe(hosts, x_host, sel, wt, n_expert, n_ffn, n_embd)
        base["GB/s"] = round(nbytes / (base["us_per_step"] * 1e-6) / 1e9, 1)
        out["cpu_baseline"] = base
    return out


def moe_decode_section(dev, gate_):
    """The same mixture at decode: one token, its eight experts.  The three banks are packed
    planes on the device (one set per bank, as a .jlm file holds them); gate and up of the eight
    experts are ONE launch of sixteen packed matvecs sharing x, the eight down projections one
    launch over silu(gate) * up.  Every step takes another eight experts, so the sheets come
    from memory.  Bytes = 24 sheets + activations.  Output check: the last step's first and
    last expert recomputed in f64 from their sheets dequantized on the device."""
    from jitllm_amd import quant, synth
    from jitllm_amd.hipmem import DeviceArray
    t, n_expert, k_used, n_ffn, n_embd = quant.Q4_K, 128, 8, 768, 2048
    dev.SetActWindow(256)
    planes, hosts = [], []
    for i, (r, k) in enumerate([(n_ffn, n_embd), (n_ffn, n_embd), (n_embd, n_ffn)]):
        hosts.append(synth.quantized_weights(t, r * n_expert, k, seed=10 + i))
        src = DeviceArray(hosts[-1])
        nq, nd, nsc = dev.packed_words(t, r * n_expert, k)
        pl = [DeviceArray(shape=(n,), dtype=np.uint32, fill=0) for n in (nq, nd, nsc)]
        if not dev.pack_weights_dev(t, src.ptr, r * n_expert, k, pl[0].ptr, pl[1].ptr, pl[2].ptr):
            raise RuntimeError("the device declined to pack a bank")
        dev.synchronize()
        src.free()
        planes.append(pl)
    x_host = synth.activations(n_embd, seed=4)
    x = DeviceArray(x_host)
    g = DeviceArray(shape=(k_used, n_ffn), dtype=np.float32, fill=0)
    u = DeviceArray(shape=(k_used, n_ffn), dtype=np.float32, fill=0)
    ys = [DeviceArray(shape=(n_embd,), dtype=np.float32, fill=0) for _ in range(k_used)]
    rng = np.random.default_rng(1)
    picks = [sorted(rng.choice(n_expert, k_used, replace=False).tolist()) for _ in range(32)]
    gp = [(planes[0][0].ptr, planes[0][1].ptr, planes[0][2].ptr)] * k_used + \
         [(planes[1][0].ptr, planes[1][1].ptr, planes[1][2].ptr)] * k_used
    dp = [(planes[2][0].ptr, planes[2][1].ptr, planes[2][2].ptr)] * k_used
    gouts = [g.ptr + j * n_ffn * 4 for j in range(k_used)] + [u.ptr + j * n_ffn * 4 for j in range(k_used)]

    # argument blocks are built once per expert set: the timed loop is two library calls a step
    calls = [(dev.packed_multi_args(gouts, t, gp, [e * n_ffn for e in ex] * 2, n_expert * n_ffn, x.ptr, 0, None,
                                    n_ffn, n_embd),
              dev.packed_multi_args([y.ptr for y in ys], t, dp, [e * n_embd for e in ex], n_expert * n_embd,
                                    g.ptr, n_ffn, u.ptr, n_embd, n_ffn)) for ex in picks]

    def run(i):
        a, b = calls[i % len(calls)]
        if not (dev.packed_multi_call(a) and dev.packed_multi_call(b)):
            raise RuntimeError("the device declined the decode mixture")
    ms = measure(dev, run, 32, gate_, warm=4)
    run(5)
    dev.synchronize()
    err, xr = 0.0, x_host.astype(np.float64)
    for j in (0, k_used - 1):
        e = picks[5][j]
        gg = dequant_rows(dev, t, hosts[0], np.arange(e * n_ffn, (e + 1) * n_ffn), n_embd) @ xr
        uu = dequant_rows(dev, t, hosts[1], np.arange(e * n_ffn, (e + 1) * n_ffn), n_embd) @ xr
        err = max(err, rel_err(g.get()[j], gg, "decode mixture gate"), rel_err(u.get()[j], uu, "decode mixture up"))
        want = dequant_rows(dev, t, hosts[2], np.arange(e * n_embd, (e + 1) * n_embd), n_ffn) @ (_silu(gg) * uu)
        err = max(err, rel_err(ys[j].get(), want, "decode mixture down", 3e-2))
    sheet = n_ffn * quant.row_bytes(t, n_embd)
    nbytes = 3 * k_used * sheet + 4 * n_embd + 4 * (4 * k_used * n_ffn) + 4 * k_used * n_embd
    for pl in planes:
        for b in pl:
            b.free()
    for b in [x, g, u] + ys:
        b.free()
    return {"us_per_step": round(ms * 1e3, 2), "launches_per_step": 2, "bytes_per_step": nbytes,
            "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "checked_rel_err": float(f"{err:.2e}")}


def mxfp4_section(dev, gate_):
    """gpt-oss-20B expert shape: MXFP4 2880x2880, bf16 activations, tokens 1 / 64 / 1024.  The
    1- and 64-token cases are bound by the weight stream, so they rotate through enough
    distinct weight copies to exceed twice the Infinity Cache, like the headline; 1024 tokens
    is bound by the matrix cores and reads one copy.  Output check: rows spread over the matrix
    against dequantize (on the device) + f64 dot with the bf16 activations (exact inputs, so
    the bar is 1e-5)."""
    from jitllm_amd import quant, synth
    from jitllm_amd.hipmem import DeviceArray, check, hip
    nrows = k = 2880
    w_host = synth.quantized_weights(quant.MXFP4, nrows, k, seed=0)
    wbytes = (w_host.nbytes + 255) & ~255
    ncopies = (2 * CACHE_BYTES + (64 << 20)) // wbytes + 1
    one = DeviceArray(w_host)
    pool = DeviceArray(shape=(ncopies * wbytes,), dtype=np.uint8)
    for i in range(ncopies):
        check(hip().hipMemcpy(pool.ptr + i * wbytes, one.ptr, w_host.nbytes, 3), "copy")
    rows = spread_rows(nrows, 96)
    wrows = dequant_rows(dev, quant.MXFP4, w_host, rows, k)
    out = {}
    for ntok in (1, 64, 1024):
        xf = np.random.default_rng(3).standard_normal((ntok, k)).astype(np.float32)
        xb = (xf.view(np.uint32) >> 16).astype(np.uint16)
        x = DeviceArray(xb)
        o = DeviceArray(shape=(ntok, nrows), dtype=np.float32, fill=np.float32(np.nan))
        rotate = ntok <= 64
        if not dev.reserve_shape(quant.MXFP4, nrows, k, ntok):
            raise RuntimeError("the device declined the MXFP4 shape")

        def run(i):
            wp = pool.ptr + (i % ncopies) * wbytes if rotate else one.ptr
            if not dev.matmul_mxfp4_bf16_dev(o.ptr, wp, x.ptr, nrows, k, ntok):
                raise RuntimeError("the device declined the MXFP4 matmul")
        ms = measure(dev, run, 40, gate_, warm=20)
        got = o.get()
        if not np.all(np.isfinite(got)):
            raise RuntimeError(f"MXFP4 {ntok} tokens: non-finite or unwritten output")
        xe = (xb.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        err = rel_err(got[:, rows], xe @ wrows.T, f"MXFP4 {ntok} tokens", 1e-5)
        nbytes = nrows * (k // 32) * 17 + ntok * k * 2 + ntok * nrows * 4
        tf = 2.0 * nrows * k * ntok / (ms * 1e-3) / 1e12
        out[f"{ntok} tokens"] = {"us_per_step": round(ms * 1e3, 1), "TFLOP/s": round(tf, 2),
                                 "frac_of_bf16_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                                 "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
                                 "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                 "weights": f"{ncopies} rotating copies" if rotate else "single copy (cache resident)",
                                 "checked_rel_err": float(f"{err:.2e}")}
        x.free()
        o.free()
    # the same matrix as packed planes (the device packer's), one token: a lane a row
    from jitllm_amd.device import Packed
    nq, nd, _ = dev.packed_words(quant.MXFP4, nrows, k)
    pbytes = ((nq + nd) * 4 + 255) & ~255
    pcopies = min(ncopies, pool.nbytes // pbytes)
    if not dev.pack_weights_dev(quant.MXFP4, one.ptr, nrows, k, pool.ptr, pool.ptr + nq * 4, None):
        raise RuntimeError("the device declined to pack the MXFP4 matrix")
    dev.synchronize()
    for i in range(1, pcopies):
        check(hip().hipMemcpy(pool.ptr + i * pbytes, pool.ptr, (nq + nd) * 4, 3), "copy")
    xf = np.random.default_rng(3).standard_normal((1, k)).astype(np.float32)
    xb = (xf.view(np.uint32) >> 16).astype(np.uint16)
    x = DeviceArray(xb)
    o = DeviceArray(shape=(1, nrows), dtype=np.float32, fill=np.float32(np.nan))

    def run_planes(i):
        base = pool.ptr + (i % pcopies) * pbytes
        if not dev.matmul_mxfp4_packed_bf16_dev(o.ptr, Packed(base, base + nq * 4, None, 0, nrows), x.ptr, nrows, k, 1):
            raise RuntimeError("the device declined the packed MXFP4 matmul")
    ms = measure(dev, run_planes, 40, gate_, warm=20)
    got = o.get()
    if not np.all(np.isfinite(got)):
        raise RuntimeError("MXFP4 planes: non-finite or unwritten output")
    xe = (xb.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    err = rel_err(got[:, rows], xe @ wrows.T, "MXFP4 planes 1 token", 1e-5)
    nbytes = (nq + nd) * 4 + k * 2 + nrows * 4
    out["1 token, packed planes"] = {"us_per_step": round(ms * 1e3, 1), "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
                                     "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                     "weights": f"{pcopies} rotating copies", "checked_rel_err": float(f"{err:.2e}")}
    x.free()
    o.free()
    # more tokens over the planes: the exact bf16 form (the planes feed the matrix instruction
    # where they lie), and the opt-in block-scaled form (fp8 activations x the planes' fp4 codes on
    # the scaled matrix instruction): never the default; its loss against the bf16 activations is
    # the rel-L2 beside its time (the bar there is 5e-2)
    for ntok in (64, 1024):
        xf = np.random.default_rng(3).standard_normal((ntok, k)).astype(np.float32)
        xb = (xf.view(np.uint32) >> 16).astype(np.uint16)
        x = DeviceArray(xb)
        xe = (xb.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        rotate = ntok <= 64
        for scaled in (0, 1):
            o = DeviceArray(shape=(ntok, nrows), dtype=np.float32, fill=np.float32(np.nan))
            dev.set_tuning(mxfp4__scaled=scaled)
            try:
                def run_packed(i):
                    base = pool.ptr + (i % pcopies) * pbytes if rotate else pool.ptr
                    if not dev.matmul_mxfp4_packed_bf16_dev(o.ptr, Packed(base, base + nq * 4, None, 0, nrows), x.ptr,
                                                            nrows, k, ntok):
                        raise RuntimeError("the device declined the packed MXFP4 matmul")
                run_packed(0)    # grows the workspace outside the timed windows
                ms = measure(dev, run_packed, 40, gate_, warm=20)
            finally:
                dev.set_tuning(mxfp4__scaled=0)
            got = o.get()
            what = "block-scaled fp8 x fp4 (opt-in, lossy)" if scaled else "bf16"
            err = rel_err(got[:, rows], xe @ wrows.T, f"MXFP4 planes {what} {ntok} tokens", 5e-2 if scaled else 1e-5)
            tf = 2.0 * nrows * k * ntok / (ms * 1e-3) / 1e12
            line = {"us_per_step": round(ms * 1e3, 1), "TFLOP/s": round(tf, 2),
                    "weights": f"{pcopies} rotating copies" if rotate else "single copy (cache resident)"}
            if scaled:
                line["frac_of_fp8_mfma_peak"] = round(tf / 5000.0, 4)
                line["rel_l2_vs_bf16_activations"] = float(f"{err:.2e}")
            else:
                line["frac_of_bf16_mfma_peak"] = round(tf / MFMA_F16_PEAK_TFLOPS, 4)
                line["checked_rel_err"] = float(f"{err:.2e}")
            out[f"{ntok} tokens, packed planes, {what}"] = line
            o.free()
        x.free()
    one.free()
    pool.free()
    return out


def ceiling_section(dev, gate_, vendor_gemm=False):
    """What a single launch costs on this machine before any arithmetic, beside the kernels it
    bounds: back-to-back empty kernels, and a kernel that only READS n bytes (every thread
    keeps eight 128-bit loads in flight; nothing is stored), over rotating buffers that exceed
    twice the Infinity Cache, at the sizes of the decode matvecs.  Median of nine windows.
    vendor_gemm (--section ceiling only: it imports torch): the vendor library's plain f16 GEMM
    at the prefill shapes."""
    from jitllm_amd.hipmem import DeviceArray
    out = {}
    ms = measure(dev, lambda i: dev.probe_dev(0, None, 0, 512, 1024), 200, gate_, warm=50)
    out["empty_kernel"] = {"us_per_launch": round(ms * 1e3, 3), "grid": 512, "block": 1024}
    # the floor as a function of the grid: workgroups x threads
    out["empty_kernel_by_grid_us"] = {
        f"{grid}x{block}": round(measure(dev, lambda i: dev.probe_dev(0, None, 0, grid, block), 200, gate_, warm=20) * 1e3, 3)
        for grid in (64, 256, 1024, 2048) for block in (64, 256, 1024)}
    # the matrix cores with nothing to wait for: 8 wavefronts a CU, 2000 rounds of four
    # 32x32x16 f16 matrix instructions each; then the same with five vector instructions
    # after each matrix instruction, the prefill GEMM loop's share
    rounds, ncu = 2000, 256   # one 512-thread workgroup for each of the MI355X's 256 CUs
    for key, kind in [("matrix_cores_f16", 3), ("matrix_cores_f16_with_5_vector_instructions_each", 4)]:
        ms = measure(dev, lambda i: dev.probe_dev(kind, None, rounds, ncu, 512), 5, gate_, warm=2)
        tf = ncu * 8 * rounds * 4 * 32768.0 / (ms * 1e-3) / 1e12
        out[key] = {"TFLOP/s": round(tf, 1), "frac_of_f16_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                    "us_per_launch": round(ms * 1e3, 1)}
    pool = DeviceArray(np.random.default_rng(0).integers(0, 1 << 32, (640 << 20) // 4, dtype=np.uint32))
    for name, nbytes in [("9.4 MB (Q4_K 4096x4096)", 9437184), ("33 MB (Q4_K 14336x4096)", 33030144),
                         ("48 MB (Q6_K 4096x14336)", 48168960), ("62 MB (Q8_0 14336x4096)", 62390272)]:
        stride = (nbytes + 4095) & ~4095
        ncopies = pool.nbytes // stride
        best, by_shape = None, {}
        for grid, block in [(256, 1024), (512, 1024), (1024, 512), (2048, 256), (512, 768)]:
            ms = measure(dev, lambda i: dev.probe_dev(1, pool.ptr + (i % ncopies) * stride, nbytes, grid, block),
                         100, gate_, warm=20)
            by_shape[f"{grid}x{block}"] = round(ms * 1e3, 3)
            if best is None or ms < best[0]:
                best = (ms, grid, block)
        ms, grid, block = best
        out[name] = {"us_per_launch": round(ms * 1e3, 3), "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
                     "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "grid": grid, "block": block, "copies": ncopies, "us_by_grid_x_block": by_shape}
    if vendor_gemm:
        # (--section ceiling only) how many CUs a read needs: the mixture block's bytes, 320 MB, through
        # 64 to 512 workgroups -- half the CUs read nearly as fast as all of them, a quarter does not
        nbytes = 320 << 20
        out["pure_read_320MB_us_by_grid_x_block"] = {
            f"{grid}x{block}": round(measure(dev, lambda i: dev.probe_dev(1, pool.ptr + (i % 2) * nbytes, nbytes, grid, block),
                                             20, gate_, warm=4) * 1e3, 1)
            for grid, block in [(512, 1024), (256, 1024), (256, 512), (128, 1024), (128, 512), (126, 1024), (64, 1024)]}
    pool.free()
    if vendor_gemm:
        out["vendor_f16_gemm"] = vendor_gemm_section()
    return out


def vendor_gemm_section():
    """A yardstick, not a part of the path: the vendor library's plain f16 GEMM (torch.matmul, which
    runs hipBLASLt) at the prefill GEMM's shapes and the MXFP4 section's, its weights ALREADY f16 / bf16 in memory -- no activation
    quantizer, no dequantization, none of the exact integer arithmetic.  What a tuned kernel reaches
    on this machine at these shapes when it has none of that to do."""
    import torch
    out = {}
    # the Q4_K prefill shapes in f16, then the MXFP4 section's 2880 x 2880 in bf16
    for ntok, k, nrows, dt in ((512, 4096, 4096, torch.float16), (2048, 4096, 4096, torch.float16),
                               (512, 4096, 14336, torch.float16), (2048, 4096, 14336, torch.float16),
                               (64, 2880, 2880, torch.bfloat16), (1024, 2880, 2880, torch.bfloat16)):
        a = torch.randn(ntok, k, device="cuda", dtype=dt)
        b = torch.randn(nrows, k, device="cuda", dtype=dt)
        for _ in range(5):
            c = a @ b.t()
        torch.cuda.synchronize()
        windows = []
        for _ in range(9):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(20):
                c = a @ b.t()
            e1.record()
            e1.synchronize()
            windows.append(e0.elapsed_time(e1) / 20)
        ms = sorted(windows)[len(windows) // 2]
        tf = 2.0 * nrows * k * ntok / (ms * 1e-3) / 1e12
        out[f"{ntok}x{k}->{nrows} {str(dt).split('.')[-1]}"] = {
            "us_per_step": round(ms * 1e3, 1), "TFLOP/s": round(tf, 1),
            "frac_of_f16_mfma_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
        del a, b, c
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="headline workload only")
    ap.add_argument("--gemm", metavar="NTOK,NROWS", help="only the prefill GEMM of this shape (k = 4096), "
                    "for profiling one kernel; prints its section alone")
    ap.add_argument("--matvec", metavar="TYPE,NROWS,K[,packed][,w32]", help="only this decode matvec (TYPE q4_k, q6_k or "
                    "q8_0; packed = packed planes; w32 = activation window 32), for profiling one kernel; "
                    "prints its section alone")
    ap.add_argument("--section", choices=["mxfp4", "moe", "moe_packed", "moe_prefill", "moe_decode", "ffn", "ffn_packed", "ceiling", "gemm_packed"],
                    help="only this section of the default run, for profiling its kernels; prints the section alone")
    ap.add_argument("--tune", metavar="KEY=VALUE", action="append", default=[],
                    help="a tuning key of the library (include/jlmi.h, jl_set_tuning), e.g. gemm.form=6; repeatable")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU (no sharding, no collectives); use --gpus 1")

    from jitllm_amd import quant
    from jitllm_amd.device import Device
    from jitllm_amd.hipmem import Gate

    dev = Device(device=0, act_window=256)
    gate = Gate(dev)
    for kv in args.tune:
        key, value = kv.split("=")
        dev.set_tuning(**{key.replace(".", "__"): int(value)})
    if args.gemm:
        ntok, nrows = (int(v) for v in args.gemm.split(","))
        print(json.dumps({"prefill_gemm": gemm_section(dev, gate, {nrows: (ntok,)})}), flush=True)
        dev.close()
        return
    if args.matvec:
        f = args.matvec.split(",")
        t = {"q4_k": quant.Q4_K, "q6_k": quant.Q6_K, "q8_0": quant.Q8_0}[f[0]]
        wl = Workload(dev, t, int(f[1]), int(f[2]), 32 if t == quant.Q8_0 or "w32" in f else 256,
                      packed="packed" in f)
        ms, per, host_us = wl.timed(args.steps, args.warmup, gate)
        wl.check()
        g = wl.alg_bytes / (ms * 1e-3) / 1e9
        print(json.dumps({"matvec": wl.name, "packed": wl.packed, "us_per_step": round(ms * 1e3, 3),
                          "GB/s": round(g, 1), "frac_of_hbm_peak": round(g / HBM_PEAK_GBS, 4),
                          "bytes_per_step": wl.alg_bytes}), flush=True)
        dev.close()
        return
    if args.section:
        fn = {"mxfp4": mxfp4_section, "moe": moe_section, "moe_packed": lambda d, g: moe_section(d, g, packed=True),
              "moe_prefill": lambda d, g: moe_section(d, g, 1024),
              "moe_decode": moe_decode_section, "ffn": ffn_section,
              "ffn_packed": ffn_packed_section, "ceiling": lambda d, g: ceiling_section(d, g, vendor_gemm=True),
              "gemm_packed": lambda d, g: gemm_section(d, g, {4096: (512,), 14336: (512,)}, packed=True)}[args.section]
        print(json.dumps({args.section: fn(dev, gate)}), flush=True)
        dev.close()
        return
    head = Workload(dev, quant.Q4_K, 4096, 4096, window=256)
    ms, per, host_us = head.timed(args.steps, args.warmup, gate)
    head.check()
    gbs = head.alg_bytes / (ms * 1e-3) / 1e9
    line = {
        "metric": "Q4_K matvec GB/s (% of HBM peak)",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "i8 dot, f32 accumulate", "data": "synthetic",
        "config": {"workload": head.name + ", weights N(0,0.02) seed 0 quantized to Q4_K, x N(0,1); "
                               f"activation quantizer (window 256) fused into the launch; "
                               f"{head.ncopies} rotating weight copies ({head.ncopies * head.wbytes >> 20} MiB)",
                   "bytes_per_step": head.alg_bytes},
        "timing": {"protocol": f">= 200 untimed launches, then 9 timed windows of {args.steps} launches each, HIP events "
                               "on the launch stream, each window enqueued behind a wait kernel (one wavefront, no memory "
                               "traffic) that lasts 1.5 x the host's enqueue time of the window, so the launches "
                               "run back to back; ms_per_step is the median window",
                   "windows_us_per_step": [round(v * 1e3, 3) for v in per],
                   "host_enqueue_us_per_launch": round(host_us, 2)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC.get("c1"),
                     "kernel": "jl_matvec_q4k_r1", "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2)},
    }
    # the same launch over ONE copy of the weights (cache resident): what the memory side costs
    head_hot = head.timed_hot(max(200, args.steps // 4), gate)
    line["headline_single_copy"] = {"us_per_step": round(head_hot * 1e3, 2),
                                    "GB/s": round(head.alg_bytes / (head_hot * 1e-3) / 1e9, 1),
                                    "weights": "single copy (cache resident); not the metric"}
    head.free()

    if not args.no_extra:
        # the other decode matvecs, over GGUF rows and over the reference's packed planes
        extra = {}
        for key, t, nrows, k, window in [("q4_k_4096x4096", quant.Q4_K, 4096, 4096, 256),
                                         ("q8_0_14336x4096", quant.Q8_0, 14336, 4096, 32),
                                         ("q6_k_4096x14336", quant.Q6_K, 4096, 14336, 32),
                                         ("q4_k_14336x4096", quant.Q4_K, 14336, 4096, 256)]:
            for layout, packed in (("gguf_rows", False), ("packed_planes", True)):
                if key == "q4_k_4096x4096" and not packed:
                    continue  # the headline above
                wl = Workload(dev, t, nrows, k, window, packed=packed)
                ems, _, _ = wl.timed(max(50, min(args.steps, 200)), args.warmup, gate)
                err = wl.check()
                g = wl.alg_bytes / (ems * 1e-3) / 1e9
                extra.setdefault(key, {})[layout] = {
                    "us_per_step": round(ems * 1e3, 2), "GB/s": round(g, 1),
                    "frac_of_hbm_peak": round(g / HBM_PEAK_GBS, 4), "bytes_per_step": wl.alg_bytes,
                    "checked_rel_err": float(f"{err:.2e}")}
                wl.free()
        line["other_configs"] = extra
        line["launch_ceiling"] = ceiling_section(dev, gate)
        line["ffn_block_decode"] = ffn_section(dev, gate)
        line["ffn_block_decode_packed"] = ffn_packed_section(dev, gate)
        line["prefill_gemm"] = gemm_section(dev, gate)
        g512 = line["prefill_gemm"]["512x4096->4096"]
        line["roofline_prefill_gemm"] = {"bound": "mfma", "achieved": g512["TFLOP/s"], "peak": MFMA_F16_PEAK_TFLOPS,
                                         "unit": "TFLOP/s", "frac": g512["frac_of_f16_mfma_peak"], "traffic": None,
                                         "workload": "Q4_K prefill GEMM 512 tokens x 4096 -> 4096, prep + GEMM per step"}
        if not args.no_cpu:
            line["roofline_prefill_gemm"]["cpu_baseline"] = cpu_baseline_gemm(4096, 4096, 512)
        line["prefill_gemm_packed_planes"] = gemm_section(dev, gate, {4096: (512,), 14336: (512,)}, packed=True)
        line["prefill_gemm_q6k"] = gemm_section(dev, gate, {4096: (512, 2048)}, quant.Q6_K, 14336)
        # the second configuration's matrices at prefill: the activation window is 32 there
        line["prefill_gemm_window32"] = {
            "q8_0": gemm_section(dev, gate, {14336: (512, 2048)}, quant.Q8_0, 4096, 32),
            "q6_k": gemm_section(dev, gate, {4096: (512, 2048)}, quant.Q6_K, 14336, 32)}
        line["moe_block"] = moe_section(dev, gate, cpu=not args.no_cpu)
        line["moe_block_packed_planes"] = moe_section(dev, gate, packed=True)
        line["moe_block_prefill_1024_rows"] = moe_section(dev, gate, 1024)   # groups of 32 columns per expert
        line["moe_decode"] = moe_decode_section(dev, gate)
        line["mxfp4_gemm"] = mxfp4_section(dev, gate)

    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(quant.Q4_K, 4096, 4096, 256)
    gate.free()
    dev.close()
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
