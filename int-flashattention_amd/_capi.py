"""ctypes binding of libintfa.so (the C ABI declared in include/intfa.h).

The library is built in-tree by ``build.py`` (hipcc, gfx950).  There is no fallback: when the shared
object is absent or does not load, every entry point raises.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libintfa.so")

ABI_VERSION = 8          # INTFA_VERSION of include/intfa.h this mirror was written against
INTFA_F16, INTFA_BF16, INTFA_F32 = 0, 1, 2
PROUND_REFERENCE, PROUND_RNE = 0, 1
STATIC_SCRATCH_BYTES = 32 << 20      # INTFA_STATIC_SCRATCH_BYTES


class FwdParams(ctypes.Structure):
    """Mirror of ``intfa_fwd_params`` (include/intfa.h); field order and types must match exactly."""
    _fields_ = (
        [(n, ctypes.c_void_p) for n in ("q", "k", "v", "out", "q_scale", "k_scale", "v_scale", "lse")]
        + [(n, ctypes.c_int64) for n in (
            "q_stride_b", "q_stride_h", "q_stride_n",
            "k_stride_b", "k_stride_h", "k_stride_n",
            "v_stride_b", "v_stride_h", "v_stride_n",
            "o_stride_b", "o_stride_h", "o_stride_n",
            "qs_stride_b", "qs_stride_h", "qs_stride_n",
            "ks_stride_b", "ks_stride_h", "ks_stride_n",
            "vs_stride_b", "vs_stride_h")]
        + [(n, ctypes.c_int32) for n in ("batch", "heads", "seqlen", "head_dim", "scale_dtype", "io_dtype", "causal")]
        + [("sm_scale", ctypes.c_float), ("p_round", ctypes.c_int32), ("num_splits", ctypes.c_int32),
           ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
           ("heads_kv", ctypes.c_int32), ("seqlen_k", ctypes.c_int32),
           ("v_scale_block", ctypes.c_int32), ("reserved0", ctypes.c_int32), ("vs_stride_blk", ctypes.c_int64),
           ("seqlens_k", ctypes.c_void_p), ("causal_rows", ctypes.c_int32), ("reserved1", ctypes.c_int32)]
    )


class AppendParams(ctypes.Structure):
    """Mirror of ``intfa_append_params`` (include/intfa.h)."""
    _fields_ = (
        [("k_new", ctypes.c_void_p), ("v_new", ctypes.c_void_p)]
        + [(n, ctypes.c_int64) for n in ("kn_stride_b", "kn_stride_h", "kn_stride_n", "vn_stride_b", "vn_stride_h", "vn_stride_n")]
        + [("k_cache", ctypes.c_void_p), ("v_cache", ctypes.c_void_p)]
        + [(n, ctypes.c_int64) for n in ("kc_stride_b", "kc_stride_h", "kc_stride_n", "vc_stride_b", "vc_stride_h", "vc_stride_n")]
        + [("k_scale_cache", ctypes.c_void_p)]
        + [(n, ctypes.c_int64) for n in ("ksc_stride_b", "ksc_stride_h", "ksc_stride_n")]
        + [("v_scale", ctypes.c_void_p), ("vs_stride_b", ctypes.c_int64), ("vs_stride_h", ctypes.c_int64),
           ("seqlens_k", ctypes.c_void_p)]
        + [(n, ctypes.c_int32) for n in ("seqlen_filled", "batch", "heads_kv", "seqlen_new", "seqlen_cache", "head_dim", "dtype")]
    )


VARIANT_FULL_INT8, VARIANT_HALF_INT8, VARIANT_FP16 = 0, 1, 2

EXPORTS = ("intfa_version", "intfa_error_string", "intfa_fwd_block_n", "intfa_fwd_workspace_bytes", "intfa_fwd_suggest_splits",
           "intfa_fwd_full_int8", "intfa_fwd_half_int8", "intfa_fwd_fp16", "intfa_fwd_full_int8_static", "intfa_debug_qk_int32",
           "intfa_quant_pertoken", "intfa_quant_pertensor_workspace_bytes", "intfa_quant_pertensor",
           "intfa_quant_perblock_channel", "intfa_kvcache_append_int8")

_lib = None


def load():
    """Loads libintfa.so once and declares the prototypes.  Raises if the library is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} not found: the HIP extension is not built. Run `python -m int_flashattention_amd.build` "
            "(needs hipcc). There is no CPU or PyTorch fallback for the attention kernels.")
    lib = ctypes.CDLL(LIB_PATH)
    pp = ctypes.POINTER(FwdParams)
    lib.intfa_version.restype = ctypes.c_int
    lib.intfa_version.argtypes = []
    lib.intfa_fwd_block_n.restype = ctypes.c_int
    lib.intfa_fwd_block_n.argtypes = [ctypes.c_int, ctypes.c_int]
    lib.intfa_error_string.restype = ctypes.c_char_p
    lib.intfa_error_string.argtypes = [ctypes.c_int]
    lib.intfa_fwd_suggest_splits.restype = ctypes.c_int
    lib.intfa_fwd_suggest_splits.argtypes = [pp, ctypes.c_int, ctypes.c_int]
    lib.intfa_fwd_workspace_bytes.restype = ctypes.c_size_t
    lib.intfa_fwd_workspace_bytes.argtypes = [pp]
    for name in ("intfa_fwd_full_int8", "intfa_fwd_half_int8", "intfa_fwd_fp16", "intfa_fwd_full_int8_static"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [pp, ctypes.c_void_p]
    lib.intfa_debug_qk_int32.restype = ctypes.c_int
    lib.intfa_debug_qk_int32.argtypes = [pp, ctypes.c_void_p, ctypes.c_void_p]
    i64, i32, vp = ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p
    lib.intfa_quant_pertoken.restype = ctypes.c_int
    lib.intfa_quant_pertoken.argtypes = [vp, i64, i64, i64, vp, vp, i32, i32, i32, i32, i32, vp]
    lib.intfa_quant_pertensor_workspace_bytes.restype = ctypes.c_size_t
    lib.intfa_quant_pertensor_workspace_bytes.argtypes = [i32, i32]
    lib.intfa_quant_pertensor.restype = ctypes.c_int
    lib.intfa_quant_pertensor.argtypes = [vp, i64, i64, i64, vp, vp, i32, i32, i32, i32, i32, vp, ctypes.c_size_t, vp]
    lib.intfa_quant_perblock_channel.restype = ctypes.c_int
    lib.intfa_quant_perblock_channel.argtypes = [vp, i64, i64, i64, vp, vp, i32, i32, i32, i32, i32, i32, vp]
    lib.intfa_kvcache_append_int8.restype = ctypes.c_int
    lib.intfa_kvcache_append_int8.argtypes = [ctypes.POINTER(AppendParams), vp]
    if lib.intfa_version() != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH} has ABI version {lib.intfa_version()}, this package expects {ABI_VERSION}: rebuild it")
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().intfa_error_string(rc).decode()
        raise RuntimeError(f"{what} failed with code {rc}: {msg}")
