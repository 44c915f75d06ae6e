"""MI355X-native quantized-weight matmul path behind jitllm's operator interface.

The compute lives in hand-written HIP kernels (csrc/) behind a C ABI
(include/jlmi.h); this package is the thin host-side mirror of the reference's
`engine/nn` device seam on top of it.
"""
from . import quant  # noqa: F401
