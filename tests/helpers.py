"""Shared test plumbing: numpy oracle <-> torch device tensors."""
from __future__ import annotations

import numpy as np
import torch

from oracle import bitdecode_oracle as O


def torch_dtype(dtype: str):
    return torch.float16 if dtype == "fp16" else torch.bfloat16


def to_dev(x: np.ndarray, dtype: str, device) -> torch.Tensor:
    """fp32 numpy holding storage-representable values -> device tensor of that dtype."""
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch_dtype(dtype)).to(device)


def bits16(x: np.ndarray, dtype: str) -> np.ndarray:
    """fp32 values representable in dtype -> their 16-bit patterns."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if dtype == "fp16":
        return x.astype(np.float16).view(np.uint16)
    return (x.view(np.uint32) >> 16).astype(np.uint16)


def alloc_cache(b, S, h_k, bits, gs, device, fill=None, k_tensor=False):
    """Caller-side allocation with the reference's shapes (evaluation/test.py:74-83); in "k-tensor" mode
    k_params has v_params' shape."""
    pn = 16 // bits
    d = 128
    mk = torch.zeros if fill is None else (lambda *a, **k: torch.full(*a, fill_value=fill, **k))
    k_pack = mk((b, S // pn, h_k, d), dtype=torch.uint16, device=device)
    k_params = torch.zeros((b, d // gs, h_k, S) if k_tensor else (b, S // gs, h_k, d), dtype=torch.float32, device=device)
    v_pack = mk((b, S, h_k, d // pn), dtype=torch.uint16, device=device)
    v_params = torch.zeros((b, d // gs, h_k, S), dtype=torch.float32, device=device)
    return k_pack, k_params, v_pack, v_params


def cache_to_numpy(k_pack, k_params, v_pack, v_params):
    return (k_pack.cpu().view(torch.int16).numpy().view(np.uint16),
            k_params.cpu().numpy(),
            v_pack.cpu().view(torch.int16).numpy().view(np.uint16),
            v_params.cpu().numpy())


def cache_from_numpy(arrs, device):
    kp, kpar, vp, vpar = arrs
    return (torch.from_numpy(kp.view(np.int16).copy()).view(torch.uint16).to(device),
            torch.from_numpy(kpar.copy()).to(device),
            torch.from_numpy(vp.view(np.int16).copy()).view(torch.uint16).to(device),
            torch.from_numpy(vpar.copy()).to(device))


def oracle_physical(qkv: O.QuantKV):
    """Quantizer-oracle output laid out in the physical format (host-side packing)."""
    from bitladder_amd import layout as L
    dt = qkv.dtype
    return L.pack_physical(qkv.k_codes, bits16(qkv.k_scale, dt), bits16(qkv.k_zero, dt),
                           qkv.v_codes, bits16(qkv.v_scale, dt), bits16(qkv.v_zero, dt),
                           qkv.bits, qkv.group_size, dt, qkv.quant_mode)


def assert_cache_equals_oracle(cache_np, qkv: O.QuantKV):
    """Bit-exact comparison of a packed cache with the quantizer oracle.  Codes are compared as
    codes; scale and zero are compared as the fp16 bit patterns the cache stores (for a bf16 cache:
    the oracle's bf16 value converted to fp16 with round-to-nearest-even, which is the identity
    inside the fp16 normal range)."""
    from bitladder_amd import layout as L
    dt = qkv.dtype
    kc, ks, kz, vc, vs, vz = L.unpack_physical(*cache_np, qkv.bits, qkv.group_size, "fp16", qkv.quant_mode)
    np.testing.assert_array_equal(kc, qkv.k_codes, err_msg="K codes")
    np.testing.assert_array_equal(vc, qkv.v_codes, err_msg="V codes")

    def stored(x):
        b = bits16(x, dt)
        return L._bf16_bits_to_fp16_bits(b) if dt == "bf16" else b

    np.testing.assert_array_equal(ks, stored(qkv.k_scale), err_msg="K scale")
    np.testing.assert_array_equal(kz, stored(qkv.k_zero), err_msg="K zero")
    np.testing.assert_array_equal(vs, stored(qkv.v_scale), err_msg="V scale")
    np.testing.assert_array_equal(vz, stored(qkv.v_zero), err_msg="V zero")


def out_tolerance(want: np.ndarray, dtype: str, atol: float = 2e-3) -> np.ndarray:
    """Element-wise bound on |output - oracle|: 2e-3 for the arithmetic, plus, for a bf16 output, half a
    bf16 unit in the last place of the expected value (what rounding the result to 8 significant bits adds)."""
    want = np.asarray(want, dtype=np.float32)
    if dtype == "fp16":
        return np.full(want.shape, atol, np.float32)
    mag = np.maximum(np.abs(want), np.float32(2.0 ** -126))
    ulp = np.exp2(np.floor(np.log2(mag)) - 7).astype(np.float32)
    return (atol + 0.5 * ulp).astype(np.float32)
