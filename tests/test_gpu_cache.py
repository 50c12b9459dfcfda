"""BitKVCache: ragged prefill, token-by-token append with pack-on-full, decode -- against the oracle on the
full token history of every sequence."""
import math

import numpy as np
import pytest
import torch

from oracle import bitdecode_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

SCALE = 1.0 / math.sqrt(128)


def _expected(q, hist_k, hist_v, bits, gs):
    """Per sequence: the first floor(L/128)*128 tokens quantized (blocks are group-aligned, so packing
    block by block equals packing the prefix at once), the rest fp16; fp32 attention over both."""
    outs = []
    for i, (k, v) in enumerate(zip(hist_k, hist_v)):
        L = k.shape[0]
        P = L // 128 * 128
        k_hat = v_hat = None
        if P:
            qkv = O.quantize_kv_ref(k[None, :P], v[None, :P], bits, gs)
            k_hat, v_hat = O.dequantize_ref(qkv)
        kr = k[None, P:] if L > P else None
        vr = v[None, P:] if L > P else None
        o, _ = O.attend_ref(q[i:i + 1], k_hat, v_hat, SCALE, kr, vr)
        outs.append(o)
    return np.concatenate(outs, 0)


@pytest.mark.parametrize("bits,gs", [(4, 128), (2, 64)])
def test_cache_prefill_append_decode(device, bits, gs):
    from bitladder_amd import BitKVCache
    b, h, h_k, steps = 3, 8, 2, 150
    lengths = [200, 128, 37]
    Lmax = 256
    q_all, k_all, v_all = O.make_inputs(b, h, h_k, Lmax + steps, 0, seed=91)
    rng = np.random.default_rng(5)
    cache = BitKVCache(b, h_k, Lmax + steps, num_bits=bits, group_size=gs, device=device)
    kd, vd = H.to_dev(k_all, "fp16", device), H.to_dev(v_all, "fp16", device)
    # positions past each sequence's length hold NaN: they must never reach a result
    kp, vp = kd[:, :Lmax].clone(), vd[:, :Lmax].clone()
    for i, L in enumerate(lengths):
        kp[i, L:] = float("nan")
        vp[i, L:] = float("nan")
    cache.prefill(kp, vp, lengths)
    hist_k = [k_all[i, :L].copy() for i, L in enumerate(lengths)]
    hist_v = [v_all[i, :L].copy() for i, L in enumerate(lengths)]
    assert cache.lengths == lengths and cache.packed_len == [128, 128, 0] and cache.res_len == [72, 0, 37]
    checks = {0, 27, 55, 56, 90, 91, 92, steps}
    for step in range(steps + 1):
        if step in checks:
            q = O.round_to_storage(rng.standard_normal((b, 1, h, 128)).astype(np.float32), "fp16")
            out = cache.decode(H.to_dev(q, "fp16", device), SCALE)
            want = _expected(q, hist_k, hist_v, bits, gs)
            err = np.abs(out.float().cpu().numpy() - want).max()
            assert err < 2e-3, (step, err, cache.packed_len, cache.res_len)
        if step < steps:
            t = Lmax + step
            cache.append(kd[:, t:t + 1], vd[:, t:t + 1])
            for i in range(b):
                hist_k[i] = np.concatenate([hist_k[i], k_all[i, t:t + 1]], 0)
                hist_v[i] = np.concatenate([hist_v[i], v_all[i, t:t + 1]], 0)
    assert cache.lengths == [L + steps for L in lengths]
    assert all(p % 128 == 0 for p in cache.packed_len) and all(r < 128 for r in cache.res_len)


def test_cache_capacity_is_enforced(device):
    from bitladder_amd import BitKVCache
    cache = BitKVCache(1, 1, 128, device=device)
    k = torch.zeros((1, 128, 1, 128), dtype=torch.float16, device=device)
    cache.prefill(k, k)
    with pytest.raises(ValueError):
        cache.append(k[:, :1], k[:, :1])
    with pytest.raises(ValueError):
        cache.prefill(torch.zeros((1, 256, 1, 128), dtype=torch.float16, device=device),
                      torch.zeros((1, 256, 1, 128), dtype=torch.float16, device=device))
