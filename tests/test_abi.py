"""CPU tests of the host side: the C ABI library loads and exports every symbol the
header declares, the container reader parses the reference-written fixture, and the
product never reaches into the oracle."""
import os
import re

import numpy as np
import pytest

from conftest import GOLDEN, ROOT
from jitllm_amd import _lib, jlm, quant


def _declared():
    text = open(os.path.join(ROOT, "include", "jlmi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(jl_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"libjlmi.so lacks {n}"
    assert sorted(_lib.SIGNATURES) == names, "the ctypes table and the header disagree"


def test_code_object_is_built():
    assert os.path.getsize(_lib.CODE_OBJECT_PATH) > 1000


def test_context_creation_fails_loudly_without_a_gpu():
    import ctypes as C
    lib = _lib.load()
    ctx = C.c_void_p()
    opts = _lib.Options(0, 32, b"/nonexistent/code_object.hsaco")
    rc = lib.jl_ctx_create(C.byref(ctx), C.byref(opts))
    assert rc < 0 and not ctx.value           # no device here, or no such code object on a GPU box
    assert lib.jl_last_error(None)


def test_product_never_imports_the_oracle():
    """The oracle is test infrastructure: nothing under jitllm_amd/ may import, load or
    link it (the reference enforces the same for its own, internal/oracle/oracle.go:4-5)."""
    pkg = os.path.join(ROOT, "jitllm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".h", ".hip", "Makefile")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(import|from)\s+oracle\b", text, re.M), f
                assert "jl_oracle" not in text and "libjl_cpu_path" not in text, f


def test_act_window_rule():
    assert quant.act_window([quant.Q4_K, quant.Q6_K]) == 256
    assert quant.act_window([quant.Q4_K, quant.Q8_0]) == 32
    assert quant.act_window([]) == 32


def test_jlm_reader_on_the_reference_written_container():
    f = jlm.File.open(os.path.join(GOLDEN, "v29.jlm.gz"))
    assert (f.version, f.n_blocks, f.n_tensors, f.n_exp_pages) == (29, 2, 12, 8)
    assert (f.page_size, f.exp_page_size, f.exp_data_off, f.dense_off) == (24576, 24576, 77824, 4096)
    assert len(f.entries) == 12
    bank = [e for e in f.entries if e.name == "exp_gate_bank" and e.block == 1][0]
    assert (bank.k, bank.rows, bank.sheets) == (256, 16, 4)
    t, qs, d, sc = f.planes(bank, 3)
    assert t == quant.Q4_K and (qs.size, d.size, sc.size) == quant.packed_words(quant.Q4_K, 16, 256)
    with pytest.raises(ValueError):
        f.planes(bank, 4)
    q5 = [e for e in f.entries if e.name == "attn_q"][0]
    with pytest.raises(ValueError):
        f.planes(q5)                       # Q5_K is not a type of this path
    with pytest.raises(ValueError):
        jlm.File(b"not a container" * 20)


def test_bench_refuses_more_than_one_gpu():
    """The bench runs on one GPU: asking for more ends with a message, before anything
    touches a device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr
    assert r.stdout.strip() == ""


def test_forget_returns_while_another_thread_holds_the_context_lock():
    """nn.CopyForgetter.Forget "must not block on the device's own work" and may be called
    from inside a page-in the device started (/root/reference/engine/nn/device.go:1570-1581).
    The host-pointer entry points hold the context lock for their whole synchronous run; a
    context bound to no device lets this be shown without a GPU: while another thread sits on
    that lock, jl_forget returns at once, and the lock holder itself may call it too."""
    import ctypes as C
    import threading
    import time
    lib = _lib.load()
    ctx = C.c_void_p()
    opts = _lib.Options(-1, 32, None)
    assert lib.jl_ctx_create(C.byref(ctx), C.byref(opts)) == _lib.OK and ctx.value
    held, release, done = threading.Event(), threading.Event(), threading.Event()

    def holder():
        assert lib.jl_ctx_lock(ctx) == _lib.OK
        buf = np.zeros(64, np.uint8)
        assert lib.jl_forget(ctx, buf.ctypes.data, buf.nbytes) == _lib.OK   # same thread, lock held
        held.set()
        release.wait(30)
        assert lib.jl_ctx_unlock(ctx) == _lib.OK
        done.set()

    th = threading.Thread(target=holder)
    th.start()
    assert held.wait(30)
    buf = np.zeros(4096, np.uint8)
    t0 = time.perf_counter()
    for _ in range(1000):
        assert lib.jl_forget(ctx, buf.ctypes.data, buf.nbytes) == _lib.OK
    dt = time.perf_counter() - t0
    assert not done.is_set(), "the holder released before the forgets returned"
    assert dt < 1.0, f"1000 forgets took {dt:.3f} s with the context lock held elsewhere"
    release.set()
    th.join(30)
    assert done.is_set()
    assert lib.jl_resident_count(ctx) == 0        # takes the lock itself: free again, queue applied
    # a context without a device fails every compute entry point loudly
    out = np.zeros(4, np.float32)
    w = np.zeros(144, np.uint8)
    x = np.zeros(256, np.float32)
    rc = lib.jl_matvec(ctx, out.ctypes.data, quant.Q4_K, w.ctypes.data, w.nbytes, x.ctypes.data, 1, 256)
    assert rc < 0 and lib.jl_last_error(ctx)
    lib.jl_ctx_destroy(ctx)


def test_block_seam_argument_checks_without_a_gpu():
    """jl_prep_layer / jl_layer_ffn_dev / jl_release_layers / jl_layer_count on a context bound
    to no device: broken plans are errors, a type without a kernel is a decline (the reference's
    PrepLayer returns false and the block stays on the CPU, /root/reference/engine/nn/device.go:
    1096-1131), a good plan fails loudly at the device, and nothing is left prepared."""
    import ctypes as C
    lib = _lib.load()
    ctx = C.c_void_p()
    opts = _lib.Options(-1, 32, None)
    assert lib.jl_ctx_create(C.byref(ctx), C.byref(opts)) == _lib.OK and ctx.value
    E, F = 256, 512
    gate = np.zeros(F * (E // 32) * 34, np.uint8)
    down = np.zeros(E * (F // 32) * 34, np.uint8)

    def plan(**kw):
        p = _lib.LayerPlan(_lib.LAYER_DENSE, quant.Q8_0, quant.Q8_0, E, F, 0, gate.ctypes.data, gate.ctypes.data,
                           down.ctypes.data, None, 0.0, 0, 0, None)
        for k, v in kw.items():
            setattr(p, k, v)
        return p

    assert lib.jl_layer_count(ctx) == 0
    assert lib.jl_prep_layer(ctx, 0, None) < 0
    assert lib.jl_prep_layer(ctx, -1, C.byref(plan())) < 0
    assert lib.jl_prep_layer(ctx, 0, C.byref(plan(gate=None))) < 0
    assert lib.jl_prep_layer(ctx, 0, C.byref(plan(kind=7))) < 0
    assert lib.jl_prep_layer(ctx, 0, C.byref(plan(kind=_lib.LAYER_MOE, n_expert=4, k_used=2))) < 0      # no router
    assert lib.jl_prep_layer(ctx, 0, C.byref(plan(type=99))) == _lib.DECLINED                            # no kernel
    assert lib.jl_prep_layer(ctx, 0, C.byref(plan(type=quant.Q4_K, n_embd=96))) == _lib.DECLINED         # k % 256
    rc = lib.jl_prep_layer(ctx, 0, C.byref(plan()))
    assert rc < 0 and lib.jl_last_error(ctx)            # a good plan: no device to put it on
    assert lib.jl_layer_count(ctx) == 0
    x = np.zeros(E, np.float32)
    assert lib.jl_layer_ffn_dev(ctx, 0, x.ctypes.data, x.ctypes.data, 1, None) < 0
    assert b"not prepared" in lib.jl_last_error(ctx)
    assert lib.jl_release_layers(ctx, 0, 100) == _lib.OK
    lib.jl_ctx_destroy(ctx)


def test_fold_admission_argument_checks_without_a_gpu():
    """jl_fold_admit_dev on a context bound to no device: what the folded-scale GEMM form does
    not serve is a decline, a null matrix an error, and a good request fails at the device."""
    import ctypes as C
    lib = _lib.load()
    ctx = C.c_void_p()
    opts = _lib.Options(-1, 32, None)
    assert lib.jl_ctx_create(C.byref(ctx), C.byref(opts)) == _lib.OK and ctx.value
    w = np.zeros(4 * 144, np.uint8)
    assert lib.jl_fold_admit_dev(ctx, quant.Q8_0, w.ctypes.data, 4, 256, None) == _lib.DECLINED
    assert lib.jl_fold_admit_dev(ctx, quant.Q4_K, w.ctypes.data, 4, 96, None) == _lib.DECLINED
    assert lib.jl_fold_admit_dev(ctx, quant.Q4_K, w.ctypes.data + 1, 4, 256, None) == _lib.DECLINED
    assert lib.jl_fold_admit_dev(ctx, quant.Q4_K, None, 4, 256, None) < 0
    assert lib.jl_fold_admit_dev(ctx, quant.Q4_K, w.ctypes.data, 4, 256, None) < 0
    assert lib.jl_set_tuning(ctx, b"gemm.fold", 1) == _lib.OK and lib.jl_set_tuning(ctx, b"gemm.fold_waves", 8) == _lib.OK
    lib.jl_ctx_destroy(ctx)


def test_grouped_host_forms_argument_checks_without_a_gpu():
    """jl_matvec_packed_multi / jl_matvec_packed_group on a context bound to no device: the
    reference's declines are declines (one matrix is not a batch, an activation the kernels do not
    bake in, more matrices than a group holds), null operands are errors, and a good call fails
    at the device."""
    import ctypes as C
    lib = _lib.load()
    ctx = C.c_void_p()
    opts = _lib.Options(-1, 32, None)
    assert lib.jl_ctx_create(C.byref(ctx), C.byref(opts)) == _lib.OK and ctx.value
    nrows, k, m = 32, 256, 2
    qs, d = np.zeros(nrows * k // 4, np.uint32), np.zeros(nrows * k // 32, np.uint32)
    x = np.zeros(2 * k, np.float32)
    outs = [np.zeros(nrows, np.float32) for _ in range(m)]
    po = (C.c_void_p * m)(*[o.ctypes.data for o in outs])
    pq = (C.c_void_p * m)(*[qs.ctypes.data] * m)
    pd = (C.c_void_p * m)(*[d.ctypes.data] * m)
    psc = (C.c_void_p * m)(None, None)
    pr = (C.c_int * m)(0, 0)
    call = lambda **kw: lib.jl_matvec_packed_multi(ctx, kw.get("outs", po), quant.Q8_0, pq, pd, psc, pr, nrows, x.ctypes.data,
                                                   kw.get("xstride", 0), kw.get("up"), kw.get("act", 0), nrows, k, kw.get("m", m))
    assert call(m=1) == _lib.DECLINED
    assert call(xstride=k - 1) == _lib.DECLINED
    assert call(xstride=k, up=x.ctypes.data, act=3) == _lib.DECLINED
    assert call(outs=None) < 0
    assert call(up=x.ctypes.data) < 0                      # a gated activation with one shared x
    assert call() < 0 and b"no device" in lib.jl_last_error(ctx)
    pt = (C.c_int * m)(quant.Q8_0, quant.Q8_0)
    pst = (C.c_int * m)(0, 0)
    prw = (C.c_int * m)(nrows, nrows)
    grp = lambda n, **kw: lib.jl_matvec_packed_group(ctx, n, po, pt, pq, pd, psc, pr, pst, prw, kw.get("x", x.ctypes.data), k,
                                                     kw.get("up"), kw.get("act", 0), None, C.c_float(0))
    assert grp(0) == _lib.DECLINED and grp(_lib.MAX_GROUP + 1) == _lib.DECLINED
    assert grp(2, up=x.ctypes.data, act=2) == _lib.DECLINED
    assert grp(2, x=None) < 0
    assert grp(2) < 0 and b"no device" in lib.jl_last_error(ctx)
    lib.jl_ctx_destroy(ctx)
