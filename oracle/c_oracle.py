"""ctypes binding of oracle/bitdecode_oracle.c (test infrastructure only)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

from .bitdecode_oracle import QuantKV

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle_c.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle_c.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_round_fp16.restype = ctypes.c_float
        _lib.oracle_round_fp16.argtypes = [ctypes.c_float]
        _lib.oracle_round_bf16.restype = ctypes.c_float
        _lib.oracle_round_bf16.argtypes = [ctypes.c_float]
    return _lib


def _p(a, t):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(t))


def quantize_kv_c(k: np.ndarray, v: np.ndarray, bits: int, gs: int, dtype: str = "fp16") -> QuantKV:
    k = np.ascontiguousarray(k, dtype=np.float32)
    v = np.ascontiguousarray(v, dtype=np.float32)
    b, S, h, d = k.shape
    kc = np.empty((b, S, h, d), np.uint8)
    vc = np.empty((b, S, h, d), np.uint8)
    ks = np.empty((b, S // gs, h, d), np.float32)
    kz = np.empty_like(ks)
    vs = np.empty((b, S, h, d // gs), np.float32)
    vz = np.empty_like(vs)
    f, u8 = ctypes.c_float, ctypes.c_uint8
    lib().oracle_quantize_kv(_p(k, f), _p(v, f), b, S, h, d, bits, gs, int(dtype == "bf16"),
                             _p(kc, u8), _p(ks, f), _p(kz, f), _p(vc, u8), _p(vs, f), _p(vz, f))
    return QuantKV(bits, gs, dtype, kc, ks, kz, vc, vs, vz)


def attend_c(q: np.ndarray, qkv: QuantKV | None, softmax_scale: float, k_res=None, v_res=None,
             seqlens_k=None, res_lens=None):
    q = np.ascontiguousarray(q, dtype=np.float32)
    b, _, h, d = q.shape
    f, u8, i32 = ctypes.c_float, ctypes.c_uint8, ctypes.c_int
    if qkv is not None:
        S, hk, gs = qkv.k_codes.shape[1], qkv.k_codes.shape[2], qkv.group_size
        arrs = [np.ascontiguousarray(a) for a in
                (qkv.k_codes, qkv.k_scale, qkv.k_zero, qkv.v_codes, qkv.v_scale, qkv.v_zero)]
    else:
        S, hk, gs = 0, k_res.shape[2], 128
        arrs = [None] * 6
    R = 0 if k_res is None else k_res.shape[1]
    kr = None if k_res is None else np.ascontiguousarray(k_res, dtype=np.float32)
    vr = None if v_res is None else np.ascontiguousarray(v_res, dtype=np.float32)
    sl = None if seqlens_k is None else np.ascontiguousarray(seqlens_k, dtype=np.int32)
    rl = None if res_lens is None else np.ascontiguousarray(res_lens, dtype=np.int32)
    out = np.empty((b, 1, h, d), np.float32)
    lse = np.empty((b, h), np.float32)
    lib().oracle_attend(_p(q, f), _p(arrs[0], u8), _p(arrs[1], f), _p(arrs[2], f),
                        _p(arrs[3], u8), _p(arrs[4], f), _p(arrs[5], f),
                        _p(kr, f), _p(vr, f), _p(sl, i32), _p(rl, i32),
                        b, h, hk, d, S, R, gs, ctypes.c_float(softmax_scale),
                        _p(out, f), _p(lse, f))
    return out, lse
