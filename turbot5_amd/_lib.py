"""ctypes binding of libt5attn.so (the C ABI declared in include/t5attn.h).

There is no fallback: if the library is missing or a call fails, an exception
is raised.  Build the library with ``python -m turbot5_amd.build``.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libt5attn.so")

T5A_BF16, T5A_F32, T5A_F16 = 0, 1, 2
ABI_VERSION = 116   # T5A_ABI_VERSION of include/t5attn.h
PATTERN_LOCAL, PATTERN_BLOCK, PATTERN_TGLOBAL = 1, 2, 3
SCORES_DEFAULT, SCORES_EXACT, SCORES_PRESCALED = 0, 1, 2   # the exact_scores field
STATIC_SCRATCH_BYTES = 8 * 1024 * 1024   # T5A_STATIC_SCRATCH_BYTES

EXPORTS = (
    "t5a_version", "t5a_last_error", "t5a_bucket_lut", "t5a_fwd_dense", "t5a_bwd_dense", "t5a_bwd_workspace_bytes", "t5a_bwd_varlen", "t5a_bwd_varlen_workspace_bytes", "t5a_fwd_varlen",
    "t5a_varlen_workspace_bytes", "t5a_bias_lut_bytes", "t5a_bias_lut_bytes_windowed",
    "t5a_fwd_sparse", "t5a_sparse_launch_plan", "t5a_sparse_workspace_bytes", "t5a_sparse_key_bits_words", "t5a_splitk_workspace_bytes", "t5a_fwd_splitk", "t5a_fwd_splitk_static",
    "t5a_rmsnorm",
)


class T5ABias(C.Structure):
    _fields_ = [("table", C.c_void_p), ("table_dtype", C.c_int32), ("num_buckets", C.c_int32),
                ("max_distance", C.c_int32), ("lut_ready", C.c_int32),
                ("stride_bucket", C.c_int64), ("stride_head", C.c_int64),
                ("lut", C.c_void_p), ("lut_bytes", C.c_int64),
                ("lut_window", C.c_int32), ("reserved", C.c_int32)]


class T5ADenseArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p), ("lse", C.c_void_p),
                ("q_strides", C.c_int64 * 3), ("k_strides", C.c_int64 * 3), ("v_strides", C.c_int64 * 3),
                ("o_strides", C.c_int64 * 3),
                ("dtype", C.c_int32), ("B", C.c_int32), ("H", C.c_int32), ("M", C.c_int32), ("N", C.c_int32),
                ("D", C.c_int32), ("causal", C.c_int32), ("sm_scale", C.c_float),
                ("exact_scores", C.c_int32), ("reserved", C.c_int32),
                ("bias", T5ABias)]


class T5ADenseBwdArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p), ("dout", C.c_void_p),
                ("lse", C.c_void_p), ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p), ("dtable", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64),
                ("q_strides", C.c_int64 * 3), ("k_strides", C.c_int64 * 3), ("v_strides", C.c_int64 * 3),
                ("o_strides", C.c_int64 * 3), ("dout_strides", C.c_int64 * 3),
                ("dq_strides", C.c_int64 * 3), ("dk_strides", C.c_int64 * 3), ("dv_strides", C.c_int64 * 3),
                ("dtype", C.c_int32), ("B", C.c_int32), ("H", C.c_int32), ("M", C.c_int32), ("N", C.c_int32),
                ("D", C.c_int32), ("causal", C.c_int32), ("sm_scale", C.c_float),
                ("exact_scores", C.c_int32), ("fp32_math", C.c_int32),
                ("bias", T5ABias)]


class T5AVarlenArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p), ("lse", C.c_void_p),
                ("q_strides", C.c_int64 * 2), ("k_strides", C.c_int64 * 2), ("v_strides", C.c_int64 * 2),
                ("o_strides", C.c_int64 * 2),
                ("cu_seqlens_q", C.c_void_p), ("cu_seqlens_k", C.c_void_p),
                ("seq_lens_q", C.c_void_p), ("seq_lens_k", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64),
                ("dtype", C.c_int32), ("B", C.c_int32), ("H", C.c_int32), ("D", C.c_int32),
                ("total_q", C.c_int32), ("total_k", C.c_int32), ("max_seqlen_q", C.c_int32),
                ("max_seqlen_k", C.c_int32), ("causal", C.c_int32), ("sm_scale", C.c_float),
                ("workspace_ready", C.c_int32), ("exact_scores", C.c_int32),
                ("bias", T5ABias)]


class T5AVarlenBwdArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p), ("dout", C.c_void_p),
                ("lse", C.c_void_p), ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p), ("dtable", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64),
                ("q_strides", C.c_int64 * 2), ("k_strides", C.c_int64 * 2), ("v_strides", C.c_int64 * 2),
                ("o_strides", C.c_int64 * 2), ("dout_strides", C.c_int64 * 2),
                ("dq_strides", C.c_int64 * 2), ("dk_strides", C.c_int64 * 2), ("dv_strides", C.c_int64 * 2),
                ("cu_seqlens_q", C.c_void_p), ("cu_seqlens_k", C.c_void_p),
                ("seq_lens_q", C.c_void_p), ("seq_lens_k", C.c_void_p),
                ("dtype", C.c_int32), ("B", C.c_int32), ("H", C.c_int32), ("D", C.c_int32),
                ("total_q", C.c_int32), ("total_k", C.c_int32), ("max_seqlen_q", C.c_int32), ("max_seqlen_k", C.c_int32),
                ("causal", C.c_int32), ("sm_scale", C.c_float),
                ("exact_scores", C.c_int32), ("fp32_math", C.c_int32),
                ("bias", T5ABias)]


class T5ASparseArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
                ("side_k", C.c_void_p), ("side_v", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64),
                ("q_strides", C.c_int64 * 3), ("k_strides", C.c_int64 * 3), ("v_strides", C.c_int64 * 3),
                ("o_strides", C.c_int64 * 3), ("side_k_strides", C.c_int64 * 3), ("side_v_strides", C.c_int64 * 3),
                ("dtype", C.c_int32), ("B", C.c_int32), ("H", C.c_int32), ("L", C.c_int32), ("D", C.c_int32),
                ("pattern", C.c_int32), ("block_len", C.c_int32), ("aux", C.c_int32), ("n_side", C.c_int32),
                ("sm_scale", C.c_float), ("exact_scores", C.c_int32),
                ("bias", T5ABias), ("seq_lens", C.c_void_p), ("seq_starts", C.c_void_p),
                ("key_bits", C.c_void_p), ("key_bits_stride", C.c_int64), ("side_counts", C.c_void_p),
                ("run_len", C.c_int32), ("reserved", C.c_int32)]


class T5ASplitKArgs(C.Structure):
    _fields_ = [("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
                ("attn_bias", C.c_void_p), ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64),
                ("q_strides", C.c_int64 * 3), ("k_strides", C.c_int64 * 3), ("v_strides", C.c_int64 * 3),
                ("o_strides", C.c_int64 * 3), ("bias_strides", C.c_int64 * 4),
                ("dtype", C.c_int32), ("B", C.c_int32), ("H", C.c_int32), ("M", C.c_int32), ("N", C.c_int32),
                ("D", C.c_int32), ("num_splits", C.c_int32), ("sm_scale", C.c_float),
                ("key_lens", C.c_void_p), ("key_starts", C.c_void_p)]


class T5ARmsNormArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("weight", C.c_void_p), ("y", C.c_void_p),
                ("x_strides", C.c_int64 * 2),
                ("batches", C.c_int64), ("rows_per_batch", C.c_int32), ("dim", C.c_int32), ("group", C.c_int32),
                ("x_dtype", C.c_int32), ("weight_dtype", C.c_int32), ("eps", C.c_float),
                ("reserved", C.c_int32),
                ("residual", C.c_void_p), ("sum_out", C.c_void_p), ("residual_row_stride", C.c_int64),
                ("seq_lens", C.c_void_p), ("seq_starts", C.c_void_p),
                ("key_bits", C.c_void_p), ("key_bits_stride", C.c_int64), ("group_counts", C.c_void_p)]


_lib = None
_lock = threading.Lock()


class T5AError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"libt5attn error {code}: {message}")
        self.code = code


def load() -> C.CDLL:
    """Load (once) and return the shared library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: the HIP extension is not built (run `python -m turbot5_amd.build`); "
                "there is no fallback path")
        lib = C.CDLL(LIB_PATH)
        lib.t5a_version.restype = C.c_int
        if lib.t5a_version() != ABI_VERSION:   # the structs below would not match what the library reads
            raise ImportError(f"{LIB_PATH} has ABI version {lib.t5a_version()}, this binding expects {ABI_VERSION}: "
                              "rebuild it (`python -m turbot5_amd.build`)")
        lib.t5a_last_error.restype = C.c_char_p
        lib.t5a_bucket_lut.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int32)]
        lib.t5a_bucket_lut.restype = C.c_int
        for name, typ in (("t5a_fwd_dense", T5ADenseArgs), ("t5a_bwd_dense", T5ADenseBwdArgs), ("t5a_fwd_varlen", T5AVarlenArgs),
                          ("t5a_bwd_varlen", T5AVarlenBwdArgs),
                          ("t5a_fwd_sparse", T5ASparseArgs), ("t5a_fwd_splitk", T5ASplitKArgs),
                          ("t5a_fwd_splitk_static", T5ASplitKArgs)):
            fn = getattr(lib, name)
            fn.argtypes = [C.POINTER(typ), C.c_void_p]
            fn.restype = C.c_int
        lib.t5a_bwd_workspace_bytes.argtypes = [C.c_int32] * 3
        lib.t5a_bwd_workspace_bytes.restype = C.c_int64
        lib.t5a_bwd_varlen_workspace_bytes.argtypes = [C.c_int32] * 2
        lib.t5a_bwd_varlen_workspace_bytes.restype = C.c_int64
        lib.t5a_splitk_workspace_bytes.argtypes = [C.c_int32] * 5
        lib.t5a_splitk_workspace_bytes.restype = C.c_int64
        lib.t5a_rmsnorm.argtypes = [C.POINTER(T5ARmsNormArgs), C.c_void_p]
        lib.t5a_rmsnorm.restype = C.c_int
        lib.t5a_bias_lut_bytes.argtypes = [C.c_int32] * 4
        lib.t5a_bias_lut_bytes.restype = C.c_int64
        lib.t5a_bias_lut_bytes_windowed.argtypes = [C.c_int32] * 4
        lib.t5a_bias_lut_bytes_windowed.restype = C.c_int64
        lib.t5a_varlen_workspace_bytes.argtypes = [C.c_int32] * 3
        lib.t5a_varlen_workspace_bytes.restype = C.c_int64
        lib.t5a_sparse_workspace_bytes.argtypes = [C.c_int32] * 7
        lib.t5a_sparse_workspace_bytes.restype = C.c_int64
        lib.t5a_sparse_launch_plan.argtypes = [C.c_int32] * 11 + [C.POINTER(C.c_int32)]
        lib.t5a_sparse_launch_plan.restype = C.c_int
        lib.t5a_sparse_key_bits_words.argtypes = [C.c_int32] * 3
        lib.t5a_sparse_key_bits_words.restype = C.c_int64
        _lib = lib
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise T5AError(rc, load().t5a_last_error().decode("utf-8", "replace"))


def bucket_lut(bidirectional: bool, num_buckets: int, max_distance: int):
    """Host-side integer bucket table for rel in [-max_distance, max_distance] as a python list."""
    out = (C.c_int32 * (2 * max_distance + 1))()
    check(load().t5a_bucket_lut(int(bool(bidirectional)), num_buckets, max_distance, out))
    return list(out)
