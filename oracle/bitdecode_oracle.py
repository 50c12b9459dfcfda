"""CPU oracle for the low-bit KV-cache decode path.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy fp32, the arithmetic of the reference's quantize-pack
and decode-attention kernels.  It is the checker for the HIP kernels; nothing in the
product package imports it.  Only tests, the smoke entry and the CPU-baseline leg of
the benchmark may use it.

Every function cites the reference code it follows (paths relative to the reference
tree).  The reference cannot be compiled here (CUDA/PTX only, CUTLASS submodule
absent), so each function is pinned by closed forms, invariants, brute force and a
second, independently written C restatement (oracle/bitdecode_oracle.c); the tests
that do so live in tests/test_oracle.py.

Pin status
----------
quantize_group / quantize_kv_ref : pinned (closed forms, invariants, brute-force
    rounding cases, C cross-check).  The reference binary is built with
    --use_fast_math (setup.py:149); the contract here is the IEEE-754 fp32 reading
    of csrc/bit_decode/src/include/qpack.h:224-252, so the exact bits of the CUDA
    binary's `scale` on rare groups are "parity unpinned".  So is the sign of a
    stored zero-point that is a zero of a group holding both -0 and +0: the reference
    reduces with `x < y ? x : y`, order-dependent; here -0 orders below +0.
dequantize_ref  : pinned (exactness on an exact grid, error bound scale/2 against the input, one-hot
    probes of the K and V grouping axes; tests/test_oracle.py).
attend_ref      : pinned (reduces to softmax(QK^T)V; block-order invariance).
lse_combine_ref : pinned (closed form, split-count invariance).
num_splits_heuristic_ref : pinned (known answers from the reference's own comment).
"k-tensor" mode : quantize_kv_ref / dequantize_ref with K grouped like V; pinned by the same closed
    forms and one-hot axis probes (tests/test_oracle.py); no C witness for this mode.
bf16 variants   : the reference has no bf16 kernel; "parity unpinned" by any
    reference artefact, pinned only by the same invariants as fp16.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np

F32 = np.float32


# --------------------------------------------------------------------------------------
# storage-type helpers (fp16 is numpy-native; bf16 is carried as fp32 values that are
# exactly representable in bf16)
# --------------------------------------------------------------------------------------
def round_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round fp32 -> bf16 (nearest even), returned as fp32 holding the bf16 value."""
    x = np.ascontiguousarray(x, dtype=F32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16) << 16
    out = (r & 0xFFFFFFFF).astype(np.uint32).view(F32).reshape(x.shape).copy()
    nan = np.isnan(x)
    out[nan] = np.nan
    return out


def round_to_storage(x: np.ndarray, dtype: str) -> np.ndarray:
    """Round fp32 values to the storage type ('fp16' or 'bf16'); result is fp32."""
    if dtype == "fp16":
        with np.errstate(over="ignore"):
            return np.asarray(x, dtype=F32).astype(np.float16).astype(F32)
    if dtype == "bf16":
        return round_to_bf16(x)
    raise ValueError(dtype)


def roundf(t: np.ndarray) -> np.ndarray:
    """C `roundf`: nearest integer, halves away from zero (qpack.h:282-285 uses roundf)."""
    t = np.asarray(t, dtype=F32)
    a = np.abs(t)
    f = np.floor(a)
    # a - f is exact in fp32, so the comparison with .5 is exact
    r = f + ((a - f) >= F32(0.5)).astype(F32)
    return np.copysign(r, t).astype(F32)


# --------------------------------------------------------------------------------------
# quantizer  (csrc/bit_decode/src/include/qpack.h:224-296 for 4-bit, :115-209 for 2-bit;
#             the arithmetic is identical, only the packing differs)
# --------------------------------------------------------------------------------------
def quantize_group(x: np.ndarray, bits: int, axis: int, dtype: str = "fp16"):
    """Quantize along `axis` as ONE group.

    x: values exactly representable in the storage dtype, any shape.
    Returns (codes uint8 same shape, scale fp32-holding-storage-value, zero likewise),
    scale/zero with `axis` reduced (keepdims).

    Follows qpack.h:238-252: range = max - min; scale_inv = range > 0 ? M/range : 0;
    stored scale = scale_inv == 0 ? 0 : 1/scale_inv (rounded to the storage type when
    written as half2, flash_fwd_kernel.h:939-964); stored zero = min;
    qpack.h:272-285: code = clamp(roundf((x - min) * scale_inv), 0, M).
    """
    x = np.asarray(x, dtype=F32)
    M = F32((1 << bits) - 1)
    mx = np.max(x, axis=axis, keepdims=True)
    mn = np.min(x, axis=axis, keepdims=True)
    # signed zeros: the minimum orders -0 below +0 (IEEE 754-2019 minimum).  The reference reduces with
    # `x < y ? x : y` (qpack.h:11-105), which leaves the sign of a zero minimum to the reduction order;
    # the value, the scale and every code are the same either way.
    has_neg_zero = np.any((x == 0) & np.signbit(x), axis=axis, keepdims=True)
    mn = np.where((mn == 0) & has_neg_zero, F32(-0.0), mn).astype(F32)
    rng = (mx - mn).astype(F32)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        scale_inv = np.where(rng > 0, M / np.where(rng > 0, rng, F32(1)), F32(0)).astype(F32)
        scale_f = np.where(scale_inv == 0, F32(0),
                           F32(1) / np.where(scale_inv == 0, F32(1), scale_inv)).astype(F32)
        t = ((x - mn).astype(F32) * scale_inv).astype(F32)
    r = roundf(t)
    codes = np.fmin(np.fmax(r, F32(0)), M).astype(np.uint8)
    scale = round_to_storage(scale_f, dtype)
    zero = round_to_storage(mn, dtype)  # exact: mn is one of the inputs
    return codes, scale, zero


@dataclass
class QuantKV:
    """Canonical logical form of a quantized cache (layout-free)."""
    bits: int
    group_size: int
    dtype: str
    k_codes: np.ndarray   # uint8 [b, S, h_k, d]
    k_scale: np.ndarray   # fp32  [b, S/gs, h_k, d]   (values representable in dtype)
    k_zero: np.ndarray    # fp32  [b, S/gs, h_k, d]
    v_codes: np.ndarray   # uint8 [b, S, h_k, d]
    v_scale: np.ndarray   # fp32  [b, S, h_k, d/gs]
    v_zero: np.ndarray    # fp32  [b, S, h_k, d/gs]
    quant_mode: str = "k-channel"   # "k-tensor": k_scale / k_zero are [b, S, h_k, d/gs] like V's


def quantize_kv_ref(k: np.ndarray, v: np.ndarray, bits: int, group_size: int,
                    dtype: str = "fp16", quant_mode: str = "k-channel") -> QuantKV:
    """K per-channel (groups of `group_size` consecutive tokens of one channel),
    V per-token (groups of `group_size` consecutive channels of one token).

    quant_mode "k-tensor" (qpack.h:378-470, quant_Ktensor; its dispatch is commented out in the
    reference, decode_api.cpp:195-203, 217-225): K is quantized like V, per token over groups of
    `group_size` consecutive channels -- the reduction runs over the fragment's channel index and the
    four lanes of a quad (qpack.h:313-375: thread_reduce_g over size<1>/num_params columns, then
    quad_allreduce_g), i.e. over channels of one token; same arithmetic (qpack.h:398-411, 424-449).
    The reference has it for 4 bits only (qpack.h:385).

    Grouping axes: the K operand is reduced over the token index of the MMA fragment and
    the V operand over its channel index (qpack.h:11-84 applied at
    flash_fwd_kernel.h:919-937 to sK[token, channel] and the transposed view of sV);
    tensor shapes k_params (b, S/gs, h_k, d) / v_params (b, d/gs, h_k, S) in
    evaluation/test.py:76-83 say the same.
    """
    k = np.asarray(k, dtype=F32)
    v = np.asarray(v, dtype=F32)
    b, S, h, d = k.shape
    gs = group_size
    if S % gs or d % gs:
        raise ValueError("S and d must be multiples of group_size")
    if quant_mode not in ("k-channel", "k-tensor"):
        raise ValueError(quant_mode)
    vg = v.reshape(b, S, h, d // gs, gs)
    vc, vs, vz = quantize_group(vg, bits, axis=4, dtype=dtype)
    if quant_mode == "k-tensor":
        kc, ks, kz = quantize_group(k.reshape(b, S, h, d // gs, gs), bits, axis=4, dtype=dtype)
        ks, kz = ks[..., 0], kz[..., 0]
    else:
        kc, ks, kz = quantize_group(k.reshape(b, S // gs, gs, h, d), bits, axis=2, dtype=dtype)
        ks, kz = ks[:, :, 0], kz[:, :, 0]
    return QuantKV(bits, gs, dtype, kc.reshape(b, S, h, d), ks, kz,
                   vc.reshape(b, S, h, d), vs[..., 0], vz[..., 0], quant_mode)


def dequantize_ref(qkv: QuantKV):
    """x_hat = code * scale + zero in fp32 (dequantize.h:291,372 computes the same
    expression with an fp16 fma; the fp32 form is the accuracy oracle).
    Returns (k_hat, v_hat) fp32 [b, S, h_k, d]."""
    gs = qkv.group_size
    b, S, h, d = qkv.k_codes.shape
    k_axis = 3 if qkv.quant_mode == "k-tensor" else 1      # dequantize.h:403-475 / :291
    ks = np.repeat(qkv.k_scale, gs, axis=k_axis)
    kz = np.repeat(qkv.k_zero, gs, axis=k_axis)
    k_hat = qkv.k_codes.astype(F32) * ks + kz
    vs = np.repeat(qkv.v_scale, gs, axis=3)
    vz = np.repeat(qkv.v_zero, gs, axis=3)
    v_hat = qkv.v_codes.astype(F32) * vs + vz
    return k_hat.astype(F32), v_hat.astype(F32)


# --------------------------------------------------------------------------------------
# attention (flash_fwd_kernel.h:406-534 hot loop, softmax.h:188-214,250-310, mask.h:128-165;
#            GQA mapping decode_api.cpp:362-368: q head hq uses kv head hq // g)
# --------------------------------------------------------------------------------------
def attend_ref(q: np.ndarray, k_hat: np.ndarray, v_hat: np.ndarray, softmax_scale: float,
               k_res: np.ndarray | None = None, v_res: np.ndarray | None = None,
               seqlens_k: np.ndarray | None = None, res_lens: np.ndarray | None = None):
    """fp32 softmax attention of one query token over [packed prefix || fp16 residual].

    q [b,1,h,d]; k_hat/v_hat [b,S,h_k,d] fp32 (dequantized) or None; k_res/v_res
    [b,R,h_k,d]; seqlens_k[b] = valid packed tokens (default S); res_lens[b] = valid
    residual tokens (default R).  Tokens past the valid length are masked to -inf
    (mask.h:160-162).  Returns (out fp32 [b,1,h,d], lse fp32 [b,h]) with
    lse = ln sum exp(softmax_scale * q.k)  (softmax.h:303).
    A row with no valid token gives out = 0, lse = -inf (flash_fwd_kernel.h:116-155
    with the combine guard :1223-1231 turning it into +inf only for the final LSE;
    this function reports -inf and leaves that convention to lse_combine_ref).
    """
    q = np.asarray(q, dtype=F32)
    b, one, h, d = q.shape
    assert one == 1
    if k_hat is not None:
        h_k = k_hat.shape[2]
        S = k_hat.shape[1]
    else:
        h_k = k_res.shape[2]
        S = 0
    R = 0 if k_res is None else k_res.shape[1]
    g = h // h_k
    out = np.zeros((b, 1, h, d), dtype=F32)
    lse = np.full((b, h), -np.inf, dtype=F32)
    sc = F32(softmax_scale)
    for bi in range(b):
        sp = S if seqlens_k is None else int(seqlens_k[bi])
        rl = R if res_lens is None else int(res_lens[bi])
        for hk in range(h_k):
            parts_k, parts_v = [], []
            if sp:
                parts_k.append(np.asarray(k_hat[bi, :sp, hk], dtype=F32))
                parts_v.append(np.asarray(v_hat[bi, :sp, hk], dtype=F32))
            if rl:
                parts_k.append(np.asarray(k_res[bi, :rl, hk], dtype=F32))
                parts_v.append(np.asarray(v_res[bi, :rl, hk], dtype=F32))
            if not parts_k:
                continue
            kk = np.concatenate(parts_k, axis=0)
            vv = np.concatenate(parts_v, axis=0)
            qq = q[bi, 0, hk * g:(hk + 1) * g]                 # [g, d]
            s = (qq @ kk.T).astype(F32) * sc                   # [g, n]
            m = s.max(axis=1, keepdims=True)
            p = np.exp((s - m).astype(F32)).astype(F32)
            l = p.sum(axis=1, keepdims=True, dtype=F32)
            out[bi, 0, hk * g:(hk + 1) * g] = ((p @ vv).astype(F32) / l).astype(F32)
            lse[bi, hk * g:(hk + 1) * g] = (m + np.log(l))[:, 0]
    return out, lse


def lse_combine_ref(o_parts: np.ndarray, lse_parts: np.ndarray):
    """Cross-split combine (flash_fwd_kernel.h:1217-1248, 1280-1298).

    o_parts [n, ..., d] fp32 normalised partial outputs, lse_parts [n, ...] natural-log
    LSE (-inf for an empty split).  M = max lse (0 if all -inf);
    L = ln sum exp(lse - M) + M (+inf if the sum is 0 or NaN);
    O = sum exp(lse_s - L) * O_s.  Returns (O fp32, L fp32).
    """
    o_parts = np.asarray(o_parts, dtype=F32)
    lse_parts = np.asarray(lse_parts, dtype=F32)
    M = lse_parts.max(axis=0)
    M = np.where(np.isneginf(M), F32(0), M).astype(F32)
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        ssum = np.exp((lse_parts - M).astype(F32)).sum(axis=0, dtype=F32)
        L = np.where((ssum == 0) | np.isnan(ssum), F32(np.inf), np.log(ssum) + M).astype(F32)
        w = np.exp((lse_parts - L).astype(F32)).astype(F32)
    O = (w[..., None] * o_parts).sum(axis=0, dtype=F32)
    return O.astype(F32), L


def num_splits_heuristic_ref(batch_nheads_mblocks: int, num_sms: int, num_n_blocks: int,
                             max_splits: int) -> int:
    """Restatement of decode_api.cpp:234-268 (kept for its known-answer test; the
    MI355X build tunes its own split choice)."""
    if batch_nheads_mblocks >= 0.8 * num_sms:
        return 1
    max_splits = min(max_splits, num_sms, num_n_blocks)
    cd = lambda a, b: (a + b - 1) // b
    elig = lambda n: n == 1 or cd(num_n_blocks, n) != cd(num_n_blocks, n - 1)
    eff = []
    best = 0.0
    for n in range(1, max_splits + 1):
        if not elig(n):
            eff.append(0.0)
            continue
        waves = np.float32(batch_nheads_mblocks * n) / np.float32(num_sms)
        e = float(waves / np.ceil(waves))
        best = max(best, e)
        eff.append(e)
    for n in range(1, max_splits + 1):
        if elig(n) and eff[n - 1] >= 0.85 * best:
            return n
    return 1


# --------------------------------------------------------------------------------------
# synthetic inputs (the benchmark/test distribution: seeded N(0,1), 2 % of K channels x10)
# --------------------------------------------------------------------------------------
def make_inputs(b: int, h: int, h_k: int, S: int, R: int, seed: int = 0, dtype: str = "fp16",
                d: int = 128):
    """Returns q [b,1,h,d], k [b,S+R,h_k,d], v [b,S+R,h_k,d] as fp32 arrays holding values
    exactly representable in `dtype`.  round(0.02*d) = 3 outlier channels per kv-head,
    drawn with the same generator, have K multiplied by 10."""
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((b, 1, h, d), dtype=F32)
    k = rng.standard_normal((b, S + R, h_k, d), dtype=F32)
    v = rng.standard_normal((b, S + R, h_k, d), dtype=F32)
    n_out = int(round(0.02 * d))
    for hk in range(h_k):
        ch = rng.choice(d, size=n_out, replace=False)
        k[:, :, hk, ch] *= F32(10)
    return (round_to_storage(q, dtype), round_to_storage(k, dtype), round_to_storage(v, dtype))


def algorithmic_bytes(b: int, h: int, h_k: int, S_total_packed: int, R_total: int, bits: int,
                      gs: int, d: int = 128) -> int:
    """Bytes one decode step must move: packed codes + scale/zero, fp16 residual, Q in,
    O out.  S_total_packed / R_total are summed over the batch."""
    packed = h_k * S_total_packed * d * 2 * (bits / 8 + 4 / gs)
    resid = h_k * R_total * d * 2 * 2
    qo = 2 * b * h * d * 2
    return int(packed + resid + qo)
