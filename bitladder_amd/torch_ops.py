"""`torch.library` registration of the entry points, so that they can sit inside `torch.compile`d or
exported graphs: `torch.ops.bitladder_amd.kvcache_pack_int`, `.fwd_kvcache_int`, `.fwd_kvcache_int_append`.

The operators forward to `bitladder_amd.interface` (same argument meaning, `quant_mode` last; optional tensors
may be None) and
declare what they write: the pack call mutates the four cache tensors, the step call mutates the cache, the
window and the lengths.  Their fake implementations only describe the output, so tracing runs no kernel.
The reference registers its functions through pybind only (csrc/bit_decode/decode_api.cpp:605-611).
"""
from __future__ import annotations

from typing import Optional

import torch

from . import interface as I

_CACHE = ("k_pack", "k_params", "v_pack", "v_params")


@torch.library.custom_op("bitladder_amd::kvcache_pack_int", mutates_args=_CACHE, device_types="cuda")
def kvcache_pack_int(k_cache: torch.Tensor, k_pack: torch.Tensor, k_params: torch.Tensor,
                     v_cache: torch.Tensor, v_pack: torch.Tensor, v_params: torch.Tensor,
                     block_table: Optional[torch.Tensor] = None, group_size: int = 128, num_bits: int = 4,
                     dst_offset: int = 0, dst_offsets: Optional[torch.Tensor] = None,
                     quant_mode: str = "k-channel") -> None:
    I.kvcache_pack_int(k_cache, k_pack, k_params, v_cache, v_pack, v_params, block_table, None, 0, quant_mode,
                       group_size, num_bits, dst_offset=dst_offset, dst_offsets=dst_offsets)


@kvcache_pack_int.register_fake
def _(k_cache, k_pack, k_params, v_cache, v_pack, v_params, block_table=None, group_size=128, num_bits=4,
      dst_offset=0, dst_offsets=None, quant_mode="k-channel") -> None:
    return None


@torch.library.custom_op("bitladder_amd::fwd_kvcache_int", mutates_args=(), device_types="cuda")
def fwd_kvcache_int(q: torch.Tensor, k_pack: torch.Tensor, k_params: torch.Tensor,
                    v_pack: torch.Tensor, v_params: torch.Tensor,
                    block_table: Optional[torch.Tensor] = None, softmax_scale: float = 1.0,
                    group_size: int = 128, num_bits: int = 4,
                    seqlens_k: Optional[torch.Tensor] = None, max_seqlen_k: Optional[int] = None,
                    k_residual: Optional[torch.Tensor] = None, v_residual: Optional[torch.Tensor] = None,
                    residual_len: Optional[torch.Tensor] = None, num_splits: int = 0,
                    quant_mode: str = "k-channel") -> torch.Tensor:
    return I.fwd_kvcache_int(q, k_pack, k_params, v_pack, v_params, block_table, softmax_scale, quant_mode,
                             group_size, num_bits, seqlens_k=seqlens_k, max_seqlen_k=max_seqlen_k,
                             k_residual=k_residual, v_residual=v_residual, residual_len=residual_len,
                             num_splits=num_splits)


@fwd_kvcache_int.register_fake
def _(q, k_pack, k_params, v_pack, v_params, block_table=None, softmax_scale=1.0, group_size=128, num_bits=4,
      seqlens_k=None, max_seqlen_k=None, k_residual=None, v_residual=None, residual_len=None, num_splits=0,
      quant_mode="k-channel"):
    return torch.empty_like(q)


@torch.library.custom_op("bitladder_amd::fwd_kvcache_int_append",
                         mutates_args=_CACHE + ("k_residual", "v_residual", "lengths"), device_types="cuda")
def fwd_kvcache_int_append(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
                           k_pack: torch.Tensor, k_params: torch.Tensor,
                           v_pack: torch.Tensor, v_params: torch.Tensor,
                           k_residual: torch.Tensor, v_residual: torch.Tensor,
                           lengths: torch.Tensor, max_len: int,
                           block_table: Optional[torch.Tensor] = None, softmax_scale: float = 1.0,
                           group_size: int = 128, num_bits: int = 4, num_splits: int = 0,
                           quant_mode: str = "k-channel") -> torch.Tensor:
    return I.fwd_kvcache_int_append(q, k_new, v_new, k_pack, k_params, v_pack, v_params, k_residual, v_residual,
                                    lengths, max_len, block_table, softmax_scale, quant_mode, group_size, num_bits,
                                    num_splits=num_splits)


@fwd_kvcache_int_append.register_fake
def _(q, k_new, v_new, k_pack, k_params, v_pack, v_params, k_residual, v_residual, lengths, max_len,
      block_table=None, softmax_scale=1.0, group_size=128, num_bits=4, num_splits=0, quant_mode="k-channel"):
    return torch.empty_like(q)
