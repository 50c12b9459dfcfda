"""Cache management around the two kernels: a packed low-bit prefix plus an fp16 residual window per
sequence, kept in step with the tokens a decode loop appends.

This is the bookkeeping the reference's figures describe (imgs/overview.png, imgs/scheme.png: the most
recent `L mod N_r` tokens stay fp16 and are attended in fp16; when the window reaches `N_r` tokens it is
quantize-packed and appended to the cache) and that its kernel traits still name
(csrc/bit_decode/src/include/kernel_traits.h:76,85: residual_block_size).  The reference's main branch
ships no code for it; here it is host logic over `kvcache_pack_int(dst_offsets=...)` and
`fwd_kvcache_int(seqlens_k=..., residual_len=...)`, or one launch per token with
`fwd_kvcache_int_append` (`step`).  Lengths are tracked on the host (they are a pure function of the
calls made) and mirrored in a device counter that `step` advances, so nothing is read back from the
device.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import torch

from .interface import fwd_kvcache_int, fwd_kvcache_int_append, kvcache_pack_int, plan_fwd_kvcache_int_append

BLOCK = 128          # tokens per packed block = residual window size N_r


class BitKVCache:
    """One attention layer's KV cache: `k_pack/k_params/v_pack/v_params` with the reference's tensor
    contract (evaluation/test.py:74-83) and `k_res/v_res [b, 128, h_k, 128]` for the window.

    Sequences may have different lengths.  `packed_len[i]` is always a multiple of 128 and
    `res_len[i] < 128` after every call.
    """

    def __init__(self, batch: int, kv_heads: int, max_tokens: int, *, num_bits: int = 4, group_size: int = 128,
                 dtype: torch.dtype = torch.float16, device="cuda", head_dim: int = 128,
                 quant_mode: str = "k-channel"):
        if head_dim != 128:
            raise NotImplementedError("head_dim must be 128")
        if quant_mode not in ("k-channel", "k-tensor"):
            raise ValueError(f"quant_mode must be 'k-channel' or 'k-tensor', got {quant_mode!r}")
        if quant_mode == "k-tensor" and num_bits != 4:
            raise NotImplementedError("quant_mode 'k-tensor' is implemented for num_bits=4 only")
        self.b, self.h_k, self.bits, self.gs, self.dtype = batch, kv_heads, num_bits, group_size, dtype
        self.quant_mode = quant_mode
        self.device = torch.device(device)
        self.capacity = (max_tokens + BLOCK - 1) // BLOCK * BLOCK
        pn, S, d = 16 // num_bits, self.capacity, head_dim
        dev = self.device
        self.k_pack = torch.zeros((batch, S // pn, kv_heads, d), dtype=torch.uint16, device=dev)
        # "k-tensor": one (scale, zero) per token and channel group for K as well, shaped like V's
        k_params_shape = (batch, d // group_size, kv_heads, S) if quant_mode == "k-tensor" \
            else (batch, S // group_size, kv_heads, d)
        self.k_params = torch.zeros(k_params_shape, dtype=torch.float32, device=dev)
        self.v_pack = torch.zeros((batch, S, kv_heads, d // pn), dtype=torch.uint16, device=dev)
        self.v_params = torch.zeros((batch, d // group_size, kv_heads, S), dtype=torch.float32, device=dev)
        self.k_res = torch.zeros((batch, BLOCK, kv_heads, d), dtype=dtype, device=dev)
        self.v_res = torch.zeros_like(self.k_res)
        self.packed_len = [0] * batch
        self.res_len = [0] * batch
        self.total = torch.zeros(batch, dtype=torch.int32, device=dev)     # tokens held, as `step` needs them
        self._rows = torch.arange(batch, device=dev)

    # ------------------------------------------------------------------ lengths
    @property
    def lengths(self) -> list[int]:
        return [p + r for p, r in zip(self.packed_len, self.res_len)]

    def _i32(self, values: Sequence[int]) -> torch.Tensor:
        return torch.tensor(list(values), dtype=torch.int32, device=self.device)

    # ------------------------------------------------------------------ writes
    def prefill(self, k: torch.Tensor, v: torch.Tensor, lengths: Optional[Sequence[int]] = None) -> None:
        """Start the cache from prompt K/V `[b, L, h_k, 128]` (`lengths[i] <= L` valid tokens per sequence,
        default L): whole 128-token blocks are quantize-packed in one launch, each sequence's last
        `length mod 128` tokens go to its fp16 window."""
        b, L = k.shape[0], k.shape[1]
        lengths = [L] * b if lengths is None else [int(x) for x in lengths]
        if b != self.b or len(lengths) != b or max(lengths) > L or min(lengths) < 0:
            raise ValueError("prefill: batch or lengths do not match")
        if max(lengths) > self.capacity:
            raise ValueError(f"prefill: {max(lengths)} tokens exceed the capacity of {self.capacity}")
        self.packed_len = [x // BLOCK * BLOCK for x in lengths]
        self.res_len = [x - p for x, p in zip(lengths, self.packed_len)]
        n_pack = max(self.packed_len)
        if n_pack:
            # sequences shorter than n_pack get blocks of padding packed behind their prefix; decode never
            # reads them (seqlens_k) and later appends overwrite them
            kvcache_pack_int(k[:, :n_pack], self.k_pack, self.k_params, v[:, :n_pack], self.v_pack, self.v_params,
                             None, None, n_pack, self.quant_mode, self.gs, self.bits)
        for i, (p, r) in enumerate(zip(self.packed_len, self.res_len)):
            if r:
                self.k_res[i, :r].copy_(k[i, p:p + r])
                self.v_res[i, :r].copy_(v[i, p:p + r])
        self.total.copy_(self._i32(lengths))

    def append(self, k_new: torch.Tensor, v_new: torch.Tensor) -> None:
        """Append one token per sequence, `[b, 1, h_k, 128]` (or `[b, h_k, 128]`).  A window that reaches 128
        tokens is quantize-packed behind its sequence's prefix in the same call (one launch for all
        sequences that filled up; the others are skipped through a negative offset)."""
        if k_new.dim() == 4:
            k_new, v_new = k_new[:, 0], v_new[:, 0]
        if any(p + r + 1 > self.capacity for p, r in zip(self.packed_len, self.res_len)):
            raise ValueError("append: cache capacity exceeded")
        pos = self._i32(self.res_len).long()
        self.k_res[self._rows, pos] = k_new.to(self.dtype)
        self.v_res[self._rows, pos] = v_new.to(self.dtype)
        self.res_len = [r + 1 for r in self.res_len]
        if BLOCK in self.res_len:
            full = [r == BLOCK for r in self.res_len]
            offsets = self._i32([p if f else -1 for p, f in zip(self.packed_len, full)])
            kvcache_pack_int(self.k_res, self.k_pack, self.k_params, self.v_res, self.v_pack, self.v_params,
                             None, None, BLOCK, self.quant_mode, self.gs, self.bits, dst_offsets=offsets)
            self.packed_len = [p + BLOCK if f else p for p, f in zip(self.packed_len, full)]
            self.res_len = [0 if f else r for r, f in zip(self.res_len, full)]
        self.total += 1

    # ------------------------------------------------------------------ read
    def decode(self, q: torch.Tensor, softmax_scale: Optional[float] = None, **kw) -> torch.Tensor:
        """Attention of one query token per sequence, `q [b, 1, h, 128]`, over everything appended so far."""
        if softmax_scale is None:
            softmax_scale = 1.0 / math.sqrt(q.shape[-1])
        max_p, max_r = max(self.packed_len), max(self.res_len)
        return fwd_kvcache_int(q, self.k_pack, self.k_params, self.v_pack, self.v_params, None, softmax_scale,
                               self.quant_mode, self.gs, self.bits,
                               seqlens_k=self._i32(self.packed_len), max_seqlen_k=max_p,
                               k_residual=self.k_res, v_residual=self.v_res,
                               residual_len=self._i32(self.res_len), max_residual_len=max_r, **kw)

    # ------------------------------------------------------------------ one launch per token
    def plan_step(self, q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
                  softmax_scale: Optional[float] = None, **kw):
        """A `DecodePlan` whose `run()` is one decode step in one launch: attend `q` over everything held
        plus the new token, append the token, pack the window if it became full.  The plan reads
        `q / k_new / v_new` in place and sizes its grid for the cache's capacity, so it can be run (or
        captured in a HIP graph and replayed) once per token.  Lengths advance on the device; the host
        copies do not follow a plan that is run directly: call `sync_lengths()` before mixing it with the
        other methods."""
        if softmax_scale is None:
            softmax_scale = 1.0 / math.sqrt(q.shape[-1])
        return plan_fwd_kvcache_int_append(q, k_new, v_new, self.k_pack, self.k_params, self.v_pack, self.v_params,
                                           self.k_res, self.v_res, self.total, self.capacity + BLOCK - 1, None,
                                           softmax_scale, self.quant_mode, self.gs, self.bits, **kw)

    def step(self, q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
             softmax_scale: Optional[float] = None, **kw) -> torch.Tensor:
        """`append` and `decode` in one launch, except that a window filled by this token is attended in
        fp16 once more before its packed form takes over.  A sequence that has no room left is attended
        but not extended."""
        if k_new.dim() == 3:
            k_new, v_new = k_new[:, None], v_new[:, None]
        if any(p + r + 1 > self.capacity for p, r in zip(self.packed_len, self.res_len)):
            raise ValueError("step: cache capacity exceeded")
        if softmax_scale is None:
            softmax_scale = 1.0 / math.sqrt(q.shape[-1])
        # (the plain entry point: its workspace comes from the per-stream cache and its argument block is
        # found again when the same buffers are passed step after step)
        out = fwd_kvcache_int_append(q, k_new.to(self.dtype), v_new.to(self.dtype), self.k_pack, self.k_params,
                                     self.v_pack, self.v_params, self.k_res, self.v_res, self.total,
                                     self.capacity + BLOCK - 1, None, softmax_scale, self.quant_mode, self.gs, self.bits,
                                     **kw)
        for i, (p, r) in enumerate(zip(self.packed_len, self.res_len)):
            if r + 1 < BLOCK:
                self.res_len[i] = r + 1
            elif p + BLOCK <= self.capacity:
                self.packed_len[i], self.res_len[i] = p + BLOCK, 0
        return out

    def sync_lengths(self) -> None:
        """Reads the device counter back (synchronises) and rebuilds the host copies from it."""
        totals = self.total.tolist()
        self.packed_len = [t // BLOCK * BLOCK for t in totals]
        self.res_len = [t - p for t, p in zip(totals, self.packed_len)]
