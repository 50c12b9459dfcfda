"""Golden vectors (tests/golden/kv_golden.npz, written by tests/golden/make_golden.py).
CPU: the oracle still reproduces them bit for bit.  GPU: the HIP kernels reproduce them."""
import os

import numpy as np
import pytest

from oracle import bitdecode_oracle as O
from tests import helpers as H

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kv_golden.npz")
CASES = [(4, 128), (4, 64), (4, 32), (2, 128), (2, 64), (2, 32)]


def _f32(bits16):
    return bits16.view(np.float16).astype(np.float32)


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD)


@pytest.mark.parametrize("bits,gs", CASES)
def test_oracle_reproduces_golden_vectors(gold, bits, gs):
    S = int(gold["packed_tokens"])
    q, k, v = _f32(gold["q"]), _f32(gold["k"]), _f32(gold["v"])
    qkv = O.quantize_kv_ref(k[:, :S], v[:, :S], bits, gs)
    tag = f"b{bits}g{gs}"
    np.testing.assert_array_equal(qkv.k_codes, gold[f"{tag}_k_codes"])
    np.testing.assert_array_equal(qkv.v_codes, gold[f"{tag}_v_codes"])
    np.testing.assert_array_equal(H.bits16(qkv.k_scale, "fp16"), gold[f"{tag}_k_scale"])
    np.testing.assert_array_equal(H.bits16(qkv.v_zero, "fp16"), gold[f"{tag}_v_zero"])
    for name, arr in zip(("k_pack", "k_params", "v_pack", "v_params"), H.oracle_physical(qkv)):
        np.testing.assert_array_equal(arr.view(np.uint8), gold[f"{tag}_{name}"].view(np.uint8), err_msg=name)
    k_hat, v_hat = O.dequantize_ref(qkv)
    out, lse = O.attend_ref(q, k_hat, v_hat, float(gold["softmax_scale"]), k[:, S:], v[:, S:])
    np.testing.assert_allclose(out, gold[f"{tag}_out"], atol=1e-6)
    np.testing.assert_allclose(lse, gold[f"{tag}_lse"], atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("bits,gs", CASES)
def test_kernels_reproduce_golden_vectors(gold, device, bits, gs):
    import torch
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    S = int(gold["packed_tokens"])
    to_t = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(torch.float16).to(device)
    q, k, v = to_t(gold["q"]), to_t(gold["k"]), to_t(gold["v"])
    b, _, h_k, _ = k.shape
    cache = H.alloc_cache(b, S, h_k, bits, gs, device)
    kvcache_pack_int(k[:, :S], cache[0], cache[1], v[:, :S], cache[2], cache[3], None, None, S, "k-channel", gs, bits)
    tag = f"b{bits}g{gs}"
    got = H.cache_to_numpy(*cache)
    for name, arr in zip(("k_pack", "k_params", "v_pack", "v_params"), got):
        np.testing.assert_array_equal(arr.view(np.uint8), gold[f"{tag}_{name}"].view(np.uint8), err_msg=name)
    out, lse = fwd_kvcache_int(q, *cache, None, float(gold["softmax_scale"]), "k-channel", gs, bits,
                               k_residual=k[:, S:], v_residual=v[:, S:], return_lse=True)
    assert np.abs(out.float().cpu().numpy() - gold[f"{tag}_out"]).max() < 2e-3
    np.testing.assert_allclose(lse.cpu().numpy(), gold[f"{tag}_lse"], atol=2e-3)
