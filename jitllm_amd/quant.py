"""Quantization type numbers and block geometry.

The numbers are the ggml_type values a GGUF file carries, the same ones the
reference's quant.Type uses (/root/reference/format/quant/types.go:14-85).
"""

Q8_0 = 8
Q4_K = 12
Q6_K = 14
MXFP4 = 39

# type -> (elements per block, bytes per block)
BLOCK = {Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210), MXFP4: (32, 17)}
NAMES = {Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K", MXFP4: "MXFP4"}
K_QUANTS = (Q4_K, Q6_K)

# Packed-plane geometry per format: elements per sub-block scale, payload words
# per sub-block (primary + secondary plane), sub-blocks per super-scale, rows
# sharing one d word (/root/reference/jit/gpu/kernels/matvec.go:137-166,
# pack.go:543-556).
PACKED = {
    Q8_0: dict(sub=32, words=8, per_super=1, dslots=2, sc="none"),
    Q4_K: dict(sub=32, words=4, per_super=8, dslots=1, sc="stream"),
    Q6_K: dict(sub=16, words=3, per_super=16, dslots=1, sc="bytes"),
    MXFP4: dict(sub=32, words=4, per_super=1, dslots=4, sc="none"),
}


def block_elems(t):
    return BLOCK[t][0]


def block_bytes(t):
    return BLOCK[t][1]


def row_bytes(t, k):
    """Bytes of one GGUF row of k elements."""
    be, bb = BLOCK[t]
    if k <= 0 or k % be:
        raise ValueError(f"k={k} is not a multiple of {NAMES[t]}'s {be} elements per block")
    return k // be * bb


def packed_words(t, nrows, k):
    """Lengths in u32 words of the QS, D and SC planes of a packed tensor
    (/root/reference/jit/gpu/kernels/pack.go:580-621)."""
    p = PACKED[t]
    unit = p["sub"] * p["per_super"]
    if k <= 0 or nrows <= 0 or k % unit:
        raise ValueError(f"k={k} is not a multiple of {unit}")
    nsub = k // p["sub"]
    nsuper = nsub // p["per_super"]
    qs = nrows * nsub * p["words"]
    n = p["dslots"]
    d = nsuper * ((nrows + n - 1) // n)
    if p["sc"] == "stream":
        sc = nrows * nsuper * 3
    elif p["sc"] == "bytes":
        sc = nrows * ((nsub + 3) // 4)
    else:
        sc = 0
    return qs, d, sc


def act_window(types):
    """Activation amax window for a model whose matvec types are `types`: 256
    when every one is a k-quant, else 32
    (/root/reference/jit/cpu/matvec.go:46-62)."""
    types = list(types)
    if types and all(t in K_QUANTS for t in types):
        return 256
    return 32
