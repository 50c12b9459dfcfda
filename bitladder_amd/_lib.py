"""ctypes binding of libbitdecode.so (the C ABI declared in include/bitdecode.h).

There is no fallback: if the library is missing the import of the first entry point raises.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libbitdecode.so")

ABI_VERSION = 5
FP16, BF16 = 0, 1
K_CHANNEL, K_TENSOR = 0, 1

_i32, _i64, _vp, _f32 = ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p, ctypes.c_float


class QpackArgs(ctypes.Structure):
    _fields_ = [
        ("k", _vp), ("v", _vp),
        ("k_stride_b", _i64), ("k_stride_t", _i64), ("k_stride_h", _i64),
        ("v_stride_b", _i64), ("v_stride_t", _i64), ("v_stride_h", _i64),
        ("k_pack", _vp), ("k_params", _vp), ("v_pack", _vp), ("v_params", _vp),
        ("b", _i32), ("n_tokens", _i32), ("h_k", _i32), ("d", _i32),
        ("cache_tokens", _i32), ("dst_offset", _i32),
        ("dst_offsets", _vp),
        ("bits", _i32), ("group_size", _i32), ("dtype", _i32),
        ("block_table", _vp), ("block_table_stride", _i64),
        ("max_pages_per_seq", _i32), ("num_pages", _i32),
        ("quant_mode", _i32),
    ]


class FwdArgs(ctypes.Structure):
    _fields_ = [
        ("q", _vp), ("q_stride_b", _i64), ("q_stride_h", _i64),
        ("k_pack", _vp), ("k_params", _vp), ("v_pack", _vp), ("v_params", _vp),
        ("cache_tokens", _i32), ("seqlen_k", _i32),
        ("seqlens_k", _vp),
        ("k_res", _vp), ("v_res", _vp),
        ("kres_stride_b", _i64), ("kres_stride_t", _i64), ("kres_stride_h", _i64),
        ("vres_stride_b", _i64), ("vres_stride_t", _i64), ("vres_stride_h", _i64),
        ("res_len", _i32),
        ("res_lens", _vp),
        ("max_seqlen_k", _i32), ("max_res_len", _i32),
        ("out", _vp), ("out_stride_b", _i64), ("out_stride_h", _i64),
        ("softmax_lse", _vp),
        ("workspace", _vp), ("workspace_bytes", ctypes.c_size_t),
        ("b", _i32), ("h", _i32), ("h_k", _i32), ("d", _i32),
        ("bits", _i32), ("group_size", _i32), ("dtype", _i32),
        ("softmax_scale", _f32),
        ("num_splits", _i32),
        ("block_table", _vp), ("block_table_stride", _i64),
        ("max_pages_per_seq", _i32), ("num_pages", _i32),
        ("quant_mode", _i32),
    ]


class FwdAppendArgs(ctypes.Structure):
    _fields_ = [
        ("fwd", FwdArgs),
        ("lengths", _vp),
        ("k_new", _vp), ("v_new", _vp),
        ("knew_stride_b", _i64), ("knew_stride_h", _i64),
        ("vnew_stride_b", _i64), ("vnew_stride_h", _i64),
        ("max_len", _i32),
    ]


EXPORTS = ("bitdecode_abi_version", "bitdecode_last_error", "bitdecode_num_splits",
           "bitdecode_fwd_workspace_bytes", "bitdecode_num_splits_for", "bitdecode_qpack", "bitdecode_fwd",
           "bitdecode_fwd_append", "bitdecode_fwd_append_workspace_bytes", "bitdecode_fwd_static")

_lib = None


class BitDecodeError(RuntimeError):
    """Raised when a C-ABI call returns a non-zero status (the reference raises RuntimeError
    through TORCH_CHECK, csrc/bit_decode/decode_api.cpp:18-20)."""

    def __init__(self, code: int, message: str):
        super().__init__(f"bitdecode error {code}: {message}")
        self.code = code


def lib():
    """Load libbitdecode.so once.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m bitladder_amd.build` "
                "(there is no CPU or PyTorch fallback for the HIP kernels)")
        L = ctypes.CDLL(LIB_PATH)
        L.bitdecode_abi_version.restype = ctypes.c_int
        L.bitdecode_last_error.restype = ctypes.c_char_p
        L.bitdecode_num_splits.restype = ctypes.c_int
        L.bitdecode_num_splits.argtypes = [_i32] * 7
        L.bitdecode_num_splits_for.restype = ctypes.c_int
        L.bitdecode_num_splits_for.argtypes = [_i32] * 8
        L.bitdecode_fwd_workspace_bytes.restype = ctypes.c_size_t
        L.bitdecode_fwd_workspace_bytes.argtypes = [_i32] * 3
        L.bitdecode_qpack.restype = ctypes.c_int
        L.bitdecode_qpack.argtypes = [ctypes.POINTER(QpackArgs), _vp]
        L.bitdecode_fwd.restype = ctypes.c_int
        L.bitdecode_fwd.argtypes = [ctypes.POINTER(FwdArgs), _vp]
        L.bitdecode_fwd_static.restype = ctypes.c_int
        L.bitdecode_fwd_static.argtypes = [ctypes.POINTER(FwdArgs), _vp]
        L.bitdecode_fwd_append.restype = ctypes.c_int
        L.bitdecode_fwd_append.argtypes = [ctypes.POINTER(FwdAppendArgs), _vp]
        L.bitdecode_fwd_append_workspace_bytes.restype = ctypes.c_size_t
        L.bitdecode_fwd_append_workspace_bytes.argtypes = [_i32] * 3
        if L.bitdecode_abi_version() != ABI_VERSION:
            raise ImportError("libbitdecode.so ABI version mismatch; rebuild it")
        _lib = L
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise BitDecodeError(rc, lib().bitdecode_last_error().decode())
