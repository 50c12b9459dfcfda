"""Multi-threaded torch (CPU) form of the oracle.  TEST INFRASTRUCTURE ONLY: used as the timed
"reference semantics on host cores" leg of the benchmark and checked against the numpy oracle
in tests/test_oracle.py.  Follows the same reference lines as oracle/bitdecode_oracle.py
(qpack.h:224-296, dequantize.h:291,372, flash_fwd_kernel.h:406-534, softmax.h:250-310).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass
class TorchQuantKV:
    bits: int
    group_size: int
    k_codes: torch.Tensor   # uint8 [b,S,h,d]
    k_scale: torch.Tensor   # storage dtype [b,S/gs,h,d]
    k_zero: torch.Tensor
    v_codes: torch.Tensor   # uint8 [b,S,h,d]
    v_scale: torch.Tensor   # storage dtype [b,S,h,d/gs]
    v_zero: torch.Tensor


def _roundf(t: torch.Tensor) -> torch.Tensor:
    a = t.abs()
    f = a.floor()
    return torch.copysign(f + ((a - f) >= 0.5).to(t.dtype), t)


def _quant(x: torch.Tensor, dim: int, bits: int, dtype: torch.dtype):
    M = float((1 << bits) - 1)
    mx = x.amax(dim=dim, keepdim=True)
    mn = x.amin(dim=dim, keepdim=True)
    # a zero minimum takes the sign of -0 if the group holds one (IEEE 754-2019 minimum)
    neg0 = ((x == 0) & torch.signbit(x)).any(dim=dim, keepdim=True)
    mn = torch.where((mn == 0) & neg0, torch.full_like(mn, -0.0), mn)
    rng = mx - mn
    pos = rng > 0
    # tensor / tensor: torch evaluates `python_scalar / tensor` as reciprocal-then-multiply (two
    # roundings), which is not the IEEE division of qpack.h:246,250
    one = torch.ones_like(rng)
    scale_inv = torch.where(pos, (one * M) / torch.where(pos, rng, one), torch.zeros_like(rng))
    nz = scale_inv != 0
    scale = torch.where(nz, one / torch.where(nz, scale_inv, one), torch.zeros_like(rng))
    t = (x - mn) * scale_inv
    codes = _roundf(t).clamp_(0, M).to(torch.uint8)
    return codes, scale.to(dtype), mn.to(dtype)


def quantize_kv(k: torch.Tensor, v: torch.Tensor, bits: int, gs: int, dtype: torch.dtype) -> TorchQuantKV:
    """k, v: fp32 [b,S,h,d] holding values representable in `dtype`."""
    b, S, h, d = k.shape
    kc, ks, kz = _quant(k.reshape(b, S // gs, gs, h, d), 2, bits, dtype)
    vc, vs, vz = _quant(v.reshape(b, S, h, d // gs, gs), 4, bits, dtype)
    return TorchQuantKV(bits, gs, kc.reshape(b, S, h, d), ks.squeeze(2), kz.squeeze(2),
                        vc.reshape(b, S, h, d), vs.squeeze(4), vz.squeeze(4))


def dequant_attend(q: torch.Tensor, qkv: TorchQuantKV, softmax_scale: float,
                   k_res: torch.Tensor | None = None, v_res: torch.Tensor | None = None) -> torch.Tensor:
    """Dequantize the whole cache to fp32, then fp32 softmax attention over [packed || residual].
    q fp32 [b,1,h,d]; returns fp32 [b,1,h,d]."""
    gs = qkv.group_size
    b, S, h_k, d = qkv.k_codes.shape
    h = q.shape[2]
    g = h // h_k
    k_hat = (qkv.k_codes.float().reshape(b, S // gs, gs, h_k, d) * qkv.k_scale.float().unsqueeze(2)
             + qkv.k_zero.float().unsqueeze(2)).reshape(b, S, h_k, d)
    v_hat = (qkv.v_codes.float().reshape(b, S, h_k, d // gs, gs) * qkv.v_scale.float().unsqueeze(4)
             + qkv.v_zero.float().unsqueeze(4)).reshape(b, S, h_k, d)
    if k_res is not None and k_res.shape[1]:
        k_hat = torch.cat([k_hat, k_res.float()], dim=1)
        v_hat = torch.cat([v_hat, v_res.float()], dim=1)
    qq = q.float().reshape(b, h_k, g, d)                       # head hq -> kv head hq // g
    s = torch.einsum("bkgd,bskd->bkgs", qq, k_hat) * softmax_scale
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("bkgs,bskd->bkgd", p, v_hat)
    return o.reshape(b, 1, h, d)
