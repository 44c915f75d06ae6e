"""The entry point that allocates nothing, jl_matmul_static_dev, against jl_matmul_dev:
same operands, same launches, workspaces carved from the library's static device array.

Bar: the outputs are the same bits (the kernels and their order are the same; only the
address of the workspace differs).  Two calls in a row, the second with a smaller input, so
the second call runs over the first call's leftovers in the shared array; then a shape whose
workspace does not fit must be refused with a clear error and launch nothing."""
import numpy as np
import pytest

from jitllm_amd import quant, synth
from jitllm_amd.device import DeviceError
from jitllm_amd.hipmem import mem_info

pytestmark = pytest.mark.gpu

POISON = np.float32(-5e30)


def _both(dev, devbuf, t, window, ntok, nrows, k, seed):
    dev.SetActWindow(window)
    w = synth.random_weights(t, nrows, k, seed=seed)
    x = np.stack([synth.activations(k, seed=seed * 100 + i) for i in range(ntok)])
    wd, xd = devbuf(w), devbuf(x)
    want = devbuf(shape=(ntok * nrows + 16,), dtype=np.float32, fill=POISON)
    got = devbuf(shape=(ntok * nrows + 16,), dtype=np.float32, fill=POISON)
    assert dev.matmul_dev(want.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)      # grows its workspaces here
    dev.synchronize()
    free_before, _ = mem_info()
    launches = dev.launch_count()
    assert dev.matmul_static_dev(got.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    n_static = dev.launch_count() - launches
    dev.synchronize()
    free_after, _ = mem_info()
    assert free_after == free_before, "the call changed the amount of free device memory"
    launches = dev.launch_count()
    assert dev.matmul_dev(want.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    assert n_static == dev.launch_count() - launches, "not the same launches as jl_matmul_dev"
    a, b = got.get(), want.get()
    assert np.all(a[ntok * nrows:] == POISON), "wrote past the output"
    assert np.all(np.abs(b[:ntok * nrows]) < 1e30)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), \
        f"{quant.NAMES[t]} {ntok}x{k}->{nrows}: {np.sum(a != b)} elements differ from jl_matmul_dev"
    for buf in (wd, xd, want, got):
        buf.free()


def test_static_matmul_equals_matmul_two_calls_in_a_row(dev, devbuf):
    """A large call, then a smaller one over its leftovers; K-split shapes (few tokens, two
    workspaces), the wide tiles, the few-token form, and the window-32 forms of the other
    types."""
    cases = [
        (quant.Q4_K, 256, 512, 4096, 2048),     # 64 wide tiles cut four ways along K: fragments + 32 MiB of partial sums
        (quant.Q4_K, 256, 130, 300, 1024),      # smaller, ragged, over the leftovers
        (quant.Q4_K, 256, 512, 9000, 1024),     # 256 x 128 tiles
        (quant.Q4_K, 256, 16, 700, 512),        # few-token form
        (quant.Q6_K, 256, 140, 520, 1024),
        (quant.Q8_0, 32, 200, 333, 1024),       # window 32: its own prep layout
        (quant.Q8_0, 32, 5, 1000, 512),         # a handful of tokens: the grouped dot-product kernel
        (quant.Q6_K, 32, 2, 100, 512),          # token by token: no workspace at all
        (quant.Q4_K, 256, 40, 200, 256),        # tiny, last
    ]
    for i, (t, window, ntok, nrows, k) in enumerate(cases):
        _both(dev, devbuf, t, window, ntok, nrows, k, seed=7 + i)
    dev.SetActWindow(32)


def test_static_matmul_on_a_stream_of_the_callers(dev, devbuf):
    """The callers this entry point is for bring their own stream (a serving loop's, one under
    graph capture): the same bits as jl_matmul_dev, with the work enqueued on that stream (the
    context's stream is kept busy behind a wait kernel meanwhile, so an answer can only come
    from the caller's)."""
    from jitllm_amd.hipmem import Gate, Stream
    t, window, ntok, nrows, k = quant.Q4_K, 256, 300, 520, 1024
    dev.SetActWindow(window)
    w = synth.random_weights(t, nrows, k, seed=3)
    x = np.stack([synth.activations(k, seed=300 + i) for i in range(ntok)])
    wd, xd = devbuf(w), devbuf(x)
    want = devbuf(shape=(ntok * nrows,), dtype=np.float32, fill=POISON)
    got = devbuf(shape=(ntok * nrows,), dtype=np.float32, fill=POISON)
    assert dev.matmul_dev(want.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    st = Stream()
    free_before, _ = mem_info()
    Gate(dev).hold(dev.stream, 20000)                      # 20 ms of nothing on the context's stream
    assert dev.matmul_static_dev(got.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok, stream=st.handle)
    st.synchronize()
    a = got.get()                                          # (a blocking copy: the caller's stream has finished)
    dev.synchronize()
    free_after, _ = mem_info()
    assert free_after == free_before
    assert np.array_equal(a.view(np.uint32), want.get().view(np.uint32))
    st.destroy()
    for buf in (wd, xd, want, got):
        buf.free()
    dev.SetActWindow(32)


def test_static_matmul_refuses_what_does_not_fit(dev, devbuf):
    """A shape whose activation fragments alone exceed the array: a clear error, and the
    output untouched."""
    t, ntok, nrows, k = quant.Q4_K, 8192, 64, 4096      # fragments: 16 x 2 x 256 x 9 KiB = 72 MiB > 64 MiB
    dev.SetActWindow(256)
    assert dev._l.jl_static_scratch_bytes() == 64 << 20
    w = synth.random_weights(t, nrows, k, seed=1)
    wd = devbuf(w)
    xd = devbuf(shape=(ntok, k), dtype=np.float32, fill=1.0)
    out = devbuf(shape=(ntok * nrows,), dtype=np.float32, fill=POISON)
    launches = dev.launch_count()
    with pytest.raises(DeviceError, match="static scratch"):
        dev.matmul_static_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    assert dev.launch_count() == launches, "launched although the shape was refused"
    dev.synchronize()
    assert np.all(out.get() == POISON)
    # the same context still serves what fits, and the ordinary entry point serves the large shape
    assert dev.matmul_dev(out.ptr, t, wd.ptr, xd.ptr, nrows, k, ntok)
    dev.synchronize()
    assert np.all(np.abs(out.get()) < 1e30)
    dev.SetActWindow(32)
