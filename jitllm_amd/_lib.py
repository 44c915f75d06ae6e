"""Loads the C ABI (libjlmi.so, built in-tree by csrc/Makefile) with ctypes.

There is no fallback: when the library or its gfx950 code object is missing,
loading raises, and so does every operator built on it.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libjlmi.so")
CODE_OBJECT_PATH = os.path.join(_HERE, "jlmi_gfx950.hsaco")

OK, DECLINED = 0, 1


class Options(C.Structure):
    _fields_ = [("device", C.c_int), ("act_window", C.c_int), ("code_object", C.c_char_p)]


_vp, _sz, _int = C.c_void_p, C.c_size_t, C.c_int
ACT_SILU = 0   # kernels.ActSiLU
MAX_GROUP = 4

MAX_GROUP = 4


class MVGroup(C.Structure):
    """jl_mv_group: the reference's nn.MVGroup over device pointers."""
    _fields_ = [("n", C.c_int), ("out", C.c_void_p * MAX_GROUP), ("type", C.c_int * MAX_GROUP),
                ("w", C.c_void_p * MAX_GROUP), ("rows", C.c_int * MAX_GROUP), ("x", C.c_void_p),
                ("k", C.c_int), ("act_up", C.c_void_p), ("resid", C.c_void_p), ("alpha", C.c_float),
                ("resid_gate", C.c_void_p), ("norm_w", C.c_void_p), ("norm_eps", C.c_float), ("norm_out", C.c_void_p)]


class PackedBank(C.Structure):
    """jl_packed_bank: a mixture's bank as packed planes (device addresses)."""
    _fields_ = [("qs", C.c_void_p), ("d", C.c_void_p), ("sc", C.c_void_p), ("sheet_bytes", C.c_size_t),
                ("stride", C.c_int)]


class HostPlanes(C.Structure):
    """jl_host_planes: a matrix's (a bank's) three packed planes in host memory."""
    _fields_ = [("qs", C.c_void_p), ("d", C.c_void_p), ("sc", C.c_void_p)]


class LayerPlan(C.Structure):
    """jl_layer_plan: a block's feed-forward weights as jl_prep_layer takes them (host memory)."""
    _fields_ = [("kind", C.c_int), ("type", C.c_int), ("down_type", C.c_int), ("n_embd", C.c_int),
                ("n_ffn", C.c_int), ("packed", C.c_int), ("gate", C.c_void_p), ("up", C.c_void_p),
                ("down", C.c_void_p), ("norm_w", C.c_void_p), ("norm_eps", C.c_float), ("n_expert", C.c_int),
                ("k_used", C.c_int), ("router", C.c_void_p)]


LAYER_DENSE, LAYER_MOE = 0, 1

# name -> (restype, argtypes); every symbol include/jlmi.h declares
SIGNATURES = {
    "jl_hip_runtime": (C.c_char_p, []),
    "jl_ctx_create": (_int, [C.POINTER(_vp), C.POINTER(Options)]),
    "jl_launch_count": (C.c_ulonglong, [_vp]),
    "jl_ctx_destroy": (None, [_vp]),
    "jl_last_error": (C.c_char_p, [_vp]),
    "jl_set_act_window": (_int, [_vp, _int]),
    "jl_stream": (_vp, [_vp]),
    "jl_synchronize": (_int, [_vp]),
    "jl_set_tuning": (_int, [_vp, C.c_char_p, _int]),
    "jl_matvec": (_int, [_vp, _vp, _int, _vp, _sz, _vp, _int, _int]),
    "jl_forget": (_int, [_vp, _vp, _sz]),
    "jl_probe_dev": (_int, [_vp, _int, _vp, _sz, _int, _int, _vp]),
    "jl_ctx_lock": (_int, [_vp]),
    "jl_ctx_unlock": (_int, [_vp]),
    "jl_resident_count": (_sz, [_vp]),
    "jl_reserve_shape": (_int, [_vp, _int, _int, _int, _int, _int]),
    "jl_matmul": (_int, [_vp, _vp, _int, _vp, _sz, _vp, _int, _int, _int]),
    "jl_quantize_act_dev": (_int, [_vp, _vp, _int, _int, _vp, _vp, _vp, _vp]),
    "jl_dequant_dev": (_int, [_vp, _int, _vp, _vp, _sz, _vp]),
    "jl_matvec_dev": (_int, [_vp, _vp, _int, _vp, _vp, _int, _int, _vp]),
    "jl_matvec_q8_dev": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _vp, _int, _int, _vp]),
    "jl_matvec_group_dev": (_int, [_vp, C.POINTER(MVGroup), _vp]),
    "jl_matvec_multi_dev": (_int, [_vp, C.POINTER(_vp), _int, C.POINTER(_vp), _vp, _int, _int, _int, _vp]),
    "jl_matvec_gather_dev": (_int, [_vp, C.POINTER(_vp), _int, C.POINTER(_vp), _vp, _sz, _vp, _int, _int, _int,
                                    _vp]),
    "jl_moe_grouped": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _vp, _vp, _int, _vp, _int, _int, _int, _int, _int]),
    "jl_matvec_packed_multi": (_int, [_vp, C.POINTER(_vp), _int, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp),
                                      C.POINTER(C.c_int), _int, _vp, _sz, _vp, _int, _int, _int, _int]),
    "jl_matvec_packed_group": (_int, [_vp, _int, C.POINTER(_vp), C.POINTER(C.c_int), C.POINTER(_vp), C.POINTER(_vp),
                                      C.POINTER(_vp), C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int), _vp,
                                      _int, _vp, _int, _vp, C.c_float]),
    "jl_matvec_packed_multi_dev": (_int, [_vp, _vp, _int, _vp, _vp, _vp, C.POINTER(C.c_int), _int, _vp, C.c_size_t,
                                          _vp, _vp, C.c_float, _vp, _vp, C.c_float, _vp, _int, _int, _int, _vp]),
    "jl_matmul_dev": (_int, [_vp, _vp, _int, _vp, _vp, _int, _int, _int, _vp]),
    "jl_matmul_static_dev": (_int, [_vp, _vp, _int, _vp, _vp, _int, _int, _int, _vp]),
    "jl_static_scratch_bytes": (_sz, []),
    "jl_reserve": (_int, [_vp, _int, _int]),
    "jl_prep_layer": (_int, [_vp, _int, C.POINTER(LayerPlan)]),
    "jl_layer_ffn_dev": (_int, [_vp, _int, _vp, _vp, _int, _vp]),
    "jl_release_layers": (_int, [_vp, _int, _int]),
    "jl_layer_count": (_int, [_vp]),
    "jl_packed_words": (_int, [_int, _int, _int, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz)]),
    "jl_matvec_packed": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _int, _int, _vp, _int, _int]),
    "jl_matmul_packed": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _int, _int, _vp, _int, _int, _int]),
    "jl_pack_weights_dev": (_int, [_vp, _int, _vp, _int, _int, _vp, _vp, _vp, _vp]),
    "jl_fold_admit_dev": (_int, [_vp, _int, _vp, _int, _int, _vp]),
    "jl_unpack_weights_dev": (_int, [_vp, _int, _vp, _vp, _vp, _int, _int, _int, _int, _vp, _vp]),
    "jl_matvec_packed_dev": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _int, _int, _vp, _int, _int, _vp]),
    "jl_matvec_packed_q8_dev": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _int, _int, _vp, _vp, _vp, _int,
                                       _int, _vp]),
    "jl_matmul_packed_dev": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _int, _int, _vp, _int, _int, _int,
                                    _vp]),
    "jl_matmul_mxfp4_bf16_dev": (_int, [_vp, _vp, _vp, _vp, _int, _int, _int, _vp]),
    "jl_matmul_mxfp4_packed_bf16_dev": (_int, [_vp, _vp, _vp, _vp, _int, _int, _vp, _int, _int, _int, _vp]),
    "jl_moe_logits_dev": (_int, [_vp, _vp, _int, _vp, _vp, _int, _int, _int, _vp]),
    "jl_moe_route_dev": (_int, [_vp, _vp, _int, _int, _int, _vp, _int, _vp, _vp]),
    "jl_moe_group_dev": (_int, [_vp, _vp, _int, _int, _int, _int, _vp, _vp, _vp, _vp]),
    "jl_moe_matvec_dev": (_int, [_vp, _vp, _vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp]),
    "jl_moe_matvec_packed_dev": (_int, [_vp, _vp, _vp, _int, C.POINTER(PackedBank), C.POINTER(PackedBank), _vp, _vp, _vp,
                                        _vp, _int, _int, _int, _int, _vp]),
    "jl_moe_ffn_packed_dev": (_int, [_vp, _vp, _int, C.POINTER(PackedBank), C.POINTER(PackedBank), C.POINTER(PackedBank),
                                     _vp, _vp, _int, _vp, _int, _int, _int, _int, _int, _vp]),
    "jl_moe_combine_dev": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _vp, _int, _int, _int, _vp]),
    "jl_moe_ffn_dev": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _vp, _vp, _int, _vp, _int, _int, _int, _int,
                              _int, _vp]),
    "jl_moe_ffn_types_dev": (_int, [_vp, _vp, _int, _int, _vp, _vp, _vp, _vp, _vp, _int, _vp, _int, _int, _int,
                                    _int, _int, _vp]),
    "jl_moe_block_dev": (_int, [_vp, _vp, _int, _int, _vp, _vp, _vp, _int, _vp, _vp, _int, _int, _int, _int, _int,
                                _vp, _vp, _vp]),
    "jl_moe_block_packed_dev": (_int, [_vp, _vp, _int, C.POINTER(PackedBank), C.POINTER(PackedBank),
                                       C.POINTER(PackedBank), _int, _vp, _vp, _int, _int, _int, _int, _int, _vp, _vp,
                                       _vp]),
}

_lib = None


def load():
    """The loaded library with argtypes set.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C jitllm_amd/csrc` "
                "(or __graft_entry__.build()); there is no fallback path")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib
