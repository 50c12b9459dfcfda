"""quant_mode "k-tensor" (K quantized per token over channel groups, like V; 4 bits): pack kernel bit-exact
against the oracle, decode within 2e-3 of dequantize-then-attend, through the same entry points."""
import math

import numpy as np
import pytest
import torch

from oracle import bitdecode_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

ATOL = 2e-3
SCALE = 1.0 / math.sqrt(128)


def _pack_gpu(k, v, gs, dtype, device, S):
    from bitladder_amd import kvcache_pack_int
    b, _, h_k, _ = k.shape
    cache = H.alloc_cache(b, S, h_k, 4, gs, device, k_tensor=True)
    kvcache_pack_int(H.to_dev(k[:, :S], dtype, device), cache[0], cache[1], H.to_dev(v[:, :S], dtype, device),
                     cache[2], cache[3], None, None, S, "k-tensor", gs, 4)
    return cache


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("gs", [32, 64, 128])
def test_qpack_ktensor_bit_exact(device, gs, dtype):
    b, h_k, S = 2, 3, 384
    _, k, v = O.make_inputs(b, h_k, h_k, S, 0, seed=300 + gs, dtype=dtype)
    k[0, 7, 1, :gs] = -2.25                                   # constant K group of one token
    k[1, 3, 2, :] = 0.0
    k[0, 0, 2, 17], k[0, 0, 2, 18] = 65504.0, -65504.0        # full fp16 range inside one token's group
    k, v = O.round_to_storage(k, dtype), O.round_to_storage(v, dtype)
    want = O.quantize_kv_ref(k, v, 4, gs, dtype, "k-tensor")
    cache = _pack_gpu(k, v, gs, dtype, device, S)
    torch.cuda.synchronize()
    assert cache[1].shape == cache[3].shape
    H.assert_cache_equals_oracle(H.cache_to_numpy(*cache), want)


@pytest.mark.parametrize("gs", [128, 64, 32])
@pytest.mark.parametrize("h,h_k", [(4, 4), (8, 2), (8, 1)])
def test_decode_ktensor_from_host_packed_cache(device, gs, h, h_k):
    """Decode kernel alone: the cache is laid out on the host from the quantizer oracle."""
    from bitladder_amd import fwd_kvcache_int
    b, S = 2, 1024
    q, k, v = O.make_inputs(b, h, h_k, S, 0, seed=17)
    qkv = O.quantize_kv_ref(k, v, 4, gs, "fp16", "k-tensor")
    cache = H.cache_from_numpy(H.oracle_physical(qkv), device)
    k_hat, v_hat = O.dequantize_ref(qkv)
    want, want_lse = O.attend_ref(q, k_hat, v_hat, SCALE)
    for ns in (0, 1, 3):
        out, lse = fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-tensor", gs, 4,
                                   num_splits=ns, return_lse=True)
        err = np.abs(out.float().cpu().numpy() - want).max()
        assert err < ATOL, (gs, h, h_k, ns, err)
        np.testing.assert_allclose(lse.cpu().numpy(), want_lse, atol=3e-3, rtol=1e-4)


@pytest.mark.parametrize("dtype,gs", [("fp16", 128), ("bf16", 64), ("fp16", 32)])
def test_pack_then_decode_ktensor_ragged_with_window(device, dtype, gs):
    """Both kernels together on a ragged batch with an fp16 window, many units per wave and several splits."""
    from bitladder_amd import fwd_kvcache_int
    b, h, h_k, S, R = 3, 8, 2, 4096, 128
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=400 + gs, dtype=dtype)
    cache = _pack_gpu(k, v, gs, dtype, device, S)
    qkv = O.quantize_kv_ref(k[:, :S], v[:, :S], 4, gs, dtype, "k-tensor")
    k_hat, v_hat = O.dequantize_ref(qkv)
    seqlens = np.array([S, 1280, 128], np.int32)
    reslens = np.array([128, 5, 77], np.int32)
    want, _ = O.attend_ref(q, k_hat, v_hat, -SCALE, k[:, S:], v[:, S:], seqlens_k=seqlens, res_lens=reslens)
    for ns in (0, 5):
        out = fwd_kvcache_int(H.to_dev(q, dtype, device), *cache, None, -SCALE, "k-tensor", gs, 4,
                              seqlens_k=torch.from_numpy(seqlens).to(device), max_seqlen_k=S,
                              k_residual=H.to_dev(k[:, S:], dtype, device), v_residual=H.to_dev(v[:, S:], dtype, device),
                              residual_len=torch.from_numpy(reslens).to(device), max_residual_len=R, num_splits=ns)
        diff = np.abs(out.float().cpu().numpy() - want)
        assert (diff < H.out_tolerance(want, dtype, ATOL)).all(), (dtype, gs, ns, diff.max())


def test_ktensor_is_rejected_at_two_bits(device):
    from bitladder_amd import fwd_kvcache_int_append, kvcache_pack_int
    t = torch.zeros(1, 128, 2, 128, dtype=torch.float16, device=device)
    cache = H.alloc_cache(1, 128, 2, 2, 128, device, k_tensor=True)
    with pytest.raises(NotImplementedError):
        kvcache_pack_int(t, cache[0], cache[1], t, cache[2], cache[3], None, None, 128, "k-tensor", 128, 2)
    with pytest.raises(NotImplementedError):
        fwd_kvcache_int_append(t[:, :1], t[:, :1], t[:, :1], *cache, t, t, torch.zeros(1, dtype=torch.int32, device=device),
                               0, None, 1.0, "k-tensor", 128, 2)
