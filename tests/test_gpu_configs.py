"""GPU parity at the benchmark configurations' real shapes (full size where the CPU oracle
finishes in seconds, otherwise on a slice of the batch plus size-independent properties)."""
import math

import numpy as np
import pytest
import torch

from oracle import bitdecode_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu
ATOL = 2e-3
SCALE = 1.0 / math.sqrt(128)


def _run_config(device, b, h, h_k, S, R, bits, gs, dtype, seed=0, check_batches=None, check_kv_heads=None,
                num_splits=0):
    """Pack + decode the whole configuration on the GPU; compare the batches / kv-heads named in
    check_* (default: all) with the oracle: cache bytes bit-exact, output within tolerance."""
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=seed, dtype=dtype)
    cache = H.alloc_cache(b, S, h_k, bits, gs, device)
    kd, vd = H.to_dev(k, dtype, device), H.to_dev(v, dtype, device)
    kvcache_pack_int(kd[:, :S], cache[0], cache[1], vd[:, :S], cache[2], cache[3], None, None, S,
                     "k-channel", gs, bits)
    out = fwd_kvcache_int(H.to_dev(q, dtype, device), *cache, None, SCALE, "k-channel", gs, bits,
                          k_residual=kd[:, S:], v_residual=vd[:, S:], num_splits=num_splits)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    cache_np = H.cache_to_numpy(*cache)
    worst = 0.0
    g = h // h_k
    for bi in (range(b) if check_batches is None else check_batches):
        # kv heads compared for this batch row: all, a fixed set, or a choice per row
        hks = (list(range(h_k)) if check_kv_heads is None else
               list(check_kv_heads(bi)) if callable(check_kv_heads) else list(check_kv_heads))
        hqs = [hk * g + j for hk in hks for j in range(g)]
        sl = slice(bi, bi + 1)
        qkv = O.quantize_kv_ref(k[sl, :S][:, :, hks], v[sl, :S][:, :, hks], bits, gs, dtype)
        # k_pack (b, S/pn, h_k, d), k_params (b, S/gs, h_k, d), v_pack (b, S, h_k, d/pn), v_params (b, d/gs, h_k, S)
        # are containers of per-(batch, kv-head) regions: slice the regions through the byte view
        sub = tuple(a.reshape(b, h_k, -1)[sl][:, hks].reshape((1, a.shape[1], len(hks), a.shape[3]))
                    for a in cache_np)
        H.assert_cache_equals_oracle(sub, qkv)
        k_hat, v_hat = O.dequantize_ref(qkv)
        want, _ = O.attend_ref(q[sl][:, :, hqs], k_hat, v_hat, SCALE, k[sl, S:][:, :, hks], v[sl, S:][:, :, hks])
        diff = np.abs(got[sl][:, :, hqs] - want)
        err = float(diff.max())
        worst = max(worst, err)
        # 2e-3, plus half a bf16 ulp of the expected value for a bf16 output
        assert (diff < H.out_tolerance(want, dtype, ATOL)).all(), (bi, err)
    return worst


def test_c1_llama2_7b_mha_4k(device):
    _run_config(device, 1, 32, 32, 4096, 128, 4, 128, "fp16")


def test_c2_llama3_8b_gqa_32k(device):
    _run_config(device, 1, 32, 8, 32768, 128, 4, 128, "fp16")


def test_c2_statistical_crosscheck_vs_unquantized(device):
    """Same comparison as the reference's own smoke test (evaluation/test.py:110-113): mean-abs
    error against attention on the UNquantized cache; the reference notebook records 0.002773
    for 4-bit g128 at S=4096 (benchmark/bench_single_decode.ipynb:92).  Same order expected."""
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    b, h, h_k, S = 1, 32, 32, 4096
    rng = np.random.default_rng(0)
    q = O.round_to_storage(rng.standard_normal((b, 1, h, 128), dtype=np.float32), "fp16")
    k = O.round_to_storage(rng.standard_normal((b, S, h_k, 128), dtype=np.float32), "fp16")
    v = O.round_to_storage(rng.standard_normal((b, S, h_k, 128), dtype=np.float32), "fp16")
    cache = H.alloc_cache(b, S, h_k, 4, 128, device)
    kvcache_pack_int(H.to_dev(k, "fp16", device), cache[0], cache[1], H.to_dev(v, "fp16", device), cache[2],
                     cache[3], None, None, S, "k-channel", 128, 4)
    out = fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-channel", 128, 4)
    want, _ = O.attend_ref(q, k, v, SCALE)
    mae = float(np.abs(out.float().cpu().numpy() - want).mean())
    assert 1e-3 < mae < 6e-3, mae


def test_c3_llama3_8b_gqa_128k_2bit_g64(device):
    """Long split-KV partitioning and the cross-split combine; oracle on all eight kv heads."""
    _run_config(device, 1, 32, 8, 131072, 128, 2, 64, "fp16")


def test_c5_llama3_70b_layer_bf16_2bit(device):
    """b8, 64 q / 8 kv heads (group of 8), S=65536, 2-bit g128, bf16; oracle on one kv head of every batch row
    (a different one per row, so every kv head index is compared once)."""
    _run_config(device, 8, 64, 8, 65536, 128, 2, 128, "bf16", check_kv_heads=lambda bi: ((3 * bi + 1) % 8,))


def test_longest_sequence_of_the_reference_sweep_524288_tokens(device):
    """The far end of the reference's sweep (benchmark/bench_single_decode.ipynb:207: one sequence, MHA 32 x 128,
    S = 524288, 4-bit g128).  Inputs are generated on the GPU (4 GiB per tensor); one kv head travels to the host
    and is compared with the oracle (cache bytes bit-exact, output within tolerance), and the result must not
    depend on the split count."""
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    b, h, h_k, S, R, bits, gs, hk = 1, 32, 32, 524288, 128, 4, 128, 21
    g = torch.Generator(device=device).manual_seed(524288)
    q = torch.randn((b, 1, h, 128), generator=g, device=device).half()
    k = torch.randn((b, S + R, h_k, 128), generator=g, device=device, dtype=torch.float16)
    v = torch.randn((b, S + R, h_k, 128), generator=g, device=device, dtype=torch.float16)
    k[:, :, :, 5::43] *= 10.0                              # a few outlier channels, as in the other inputs
    cache = H.alloc_cache(b, S, h_k, bits, gs, device)
    kvcache_pack_int(k[:, :S], cache[0], cache[1], v[:, :S], cache[2], cache[3], None, None, S, "k-channel", gs, bits)
    kw = dict(k_residual=k[:, S:], v_residual=v[:, S:])
    outs = {ns: fwd_kvcache_int(q, *cache, None, SCALE, "k-channel", gs, bits, num_splits=ns, **kw) for ns in (0, 1, 5, 64)}
    torch.cuda.synchronize()
    k1 = k[:, :, hk:hk + 1].float().cpu().numpy()
    v1 = v[:, :, hk:hk + 1].float().cpu().numpy()
    qkv = O.quantize_kv_ref(k1[:, :S], v1[:, :S], bits, gs, "fp16")
    # the cache tensors are containers of per-(batch, kv-head) regions: the head's region through the flat view
    cache_np = H.cache_to_numpy(*(t.reshape(b, h_k, -1)[:, hk:hk + 1].reshape(1, t.shape[1], 1, t.shape[3]).contiguous()
                                  for t in cache))
    H.assert_cache_equals_oracle(cache_np, qkv)
    k_hat, v_hat = O.dequantize_ref(qkv)
    want, _ = O.attend_ref(q[:, :, hk:hk + 1].float().cpu().numpy(), k_hat, v_hat, SCALE, k1[:, S:], v1[:, S:])
    errs = {ns: float(np.abs(o[:, :, hk:hk + 1].float().cpu().numpy() - want).max()) for ns, o in outs.items()}
    spread = {ns: (o.float() - outs[0].float()).abs().max().item() for ns, o in outs.items()}
    print("max-abs error against the oracle by split count:", errs, "; against the chosen split count:", spread)
    assert max(errs.values()) < ATOL, errs
    assert max(spread.values()) < 1e-3, spread


def test_c4_ragged_batch_decode_and_append(device):
    """Batch 16, per-sequence KV length uniform in [1024, 8192] (seeded).  The packed part of
    each sequence is its length rounded down to a multiple of 128; the remainder plus 128 new
    tokens live in the fp16 window.  Then the step's append: the oldest 128 window tokens of
    every sequence are quantize-packed at its own offset and decode runs on the new state."""
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    b, h, h_k, bits, gs, cap, rcap = 16, 32, 8, 4, 128, 8192 + 128, 256
    rng = np.random.default_rng(4)
    lens = rng.integers(1024, 8193, size=b)
    packed = (lens // 128) * 128
    res = lens - packed + 128                          # 128 .. 255 tokens in the window
    q, k, v = O.make_inputs(b, h, h_k, cap, rcap, seed=44)
    kd, vd = H.to_dev(k, "fp16", device), H.to_dev(v, "fp16", device)
    cache = H.alloc_cache(b, cap, h_k, bits, gs, device, fill=0x5a5a)   # junk beyond the valid prefix
    kvcache_pack_int(kd[:, :cap], cache[0], cache[1], vd[:, :cap], cache[2], cache[3], None, None, cap,
                     "k-channel", gs, bits)
    # window of sequence i = tokens packed_i .. packed_i + res_i of its stream
    kres = torch.zeros(b, rcap, h_k, 128, dtype=torch.float16, device=device)
    vres = torch.zeros_like(kres)
    for i in range(b):
        kres[i, :res[i]] = kd[i, packed[i]:packed[i] + res[i]]
        vres[i, :res[i]] = vd[i, packed[i]:packed[i] + res[i]]
    seqlens = torch.tensor(packed, dtype=torch.int32, device=device)
    reslens = torch.tensor(res, dtype=torch.int32, device=device)
    qd = H.to_dev(q, "fp16", device)
    out = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, seqlens_k=seqlens,
                          max_seqlen_k=int(packed.max()), k_residual=kres, v_residual=vres,
                          residual_len=reslens, max_residual_len=int(res.max()))
    got = out.float().cpu().numpy()
    qkv = O.quantize_kv_ref(k[:, :cap], v[:, :cap], bits, gs)
    k_hat, v_hat = O.dequantize_ref(qkv)
    kres_np = np.stack([np.pad(k[i, packed[i]:packed[i] + res[i]], ((0, rcap - res[i]), (0, 0), (0, 0))) for i in range(b)])
    vres_np = np.stack([np.pad(v[i, packed[i]:packed[i] + res[i]], ((0, rcap - res[i]), (0, 0), (0, 0))) for i in range(b)])
    want, _ = O.attend_ref(q, k_hat, v_hat, SCALE, kres_np, vres_np, packed.astype(np.int32), res.astype(np.int32))
    assert np.abs(got - want).max() < ATOL

    # ---- append: pack the oldest 128 window tokens of every sequence at its own offset
    before = [t.clone() for t in cache]
    cache2 = H.alloc_cache(b, cap, h_k, bits, gs, device, fill=0x3c3c)
    # start from a cache that holds only the valid prefixes (rest junk), as a serving loop would
    for dst, src in zip(cache2, before):
        dst.copy_(src)
    kvcache_pack_int(kres[:, :128], cache2[0], cache2[1], vres[:, :128], cache2[2], cache2[3], None, None, 128,
                     "k-channel", gs, bits, dst_offsets=seqlens)
    torch.cuda.synchronize()
    # the appended chunk equals what the full pack wrote there; everything else is untouched
    for a, c in zip(before, cache2):
        assert torch.equal(a, c)
    seqlens2 = seqlens + 128
    out2 = fwd_kvcache_int(qd, *cache2, None, SCALE, "k-channel", gs, bits, seqlens_k=seqlens2,
                           max_seqlen_k=int(packed.max()) + 128, k_residual=kres[:, 128:].contiguous(),
                           v_residual=vres[:, 128:].contiguous(), residual_len=reslens - 128,
                           max_residual_len=int(res.max()) - 128)
    want2, _ = O.attend_ref(q, k_hat, v_hat, SCALE, kres_np[:, 128:], vres_np[:, 128:],
                            (packed + 128).astype(np.int32), (res - 128).astype(np.int32))
    assert np.abs(out2.float().cpu().numpy() - want2).max() < ATOL


# ------------------------------------------------------------------ size-independent properties
def _c2_state(device, seed=9):
    from bitladder_amd import kvcache_pack_int
    b, h, h_k, S, R, bits, gs = 1, 32, 8, 32768, 128, 4, 128
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=seed)
    kd, vd, qd = H.to_dev(k, "fp16", device), H.to_dev(v, "fp16", device), H.to_dev(q, "fp16", device)
    cache = H.alloc_cache(b, S, h_k, bits, gs, device)
    kvcache_pack_int(kd[:, :S], cache[0], cache[1], vd[:, :S], cache[2], cache[3], None, None, S, "k-channel", gs, bits)
    return qd, kd, vd, cache, S


def test_full_size_split_count_invariance_and_determinism(device):
    from bitladder_amd import fwd_kvcache_int
    qd, kd, vd, cache, S = _c2_state(device)
    kw = dict(k_residual=kd[:, S:], v_residual=vd[:, S:])
    base = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", 128, 4, **kw)
    again = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", 128, 4, **kw)
    assert torch.equal(base, again)                        # deterministic: fixed merge order
    for ns in (1, 2, 7, 32, 64, 256):
        o = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", 128, 4, num_splits=ns, **kw)
        assert (o.float() - base.float()).abs().max().item() < 5e-4, ns


def test_full_size_token_permutation_inside_chunks(device):
    """Permuting the tokens of every 128-token chunk (K and V rows together) leaves each K group's
    min/max and each V token's group untouched, so the attention output may only move by summation order."""
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    qd, kd, vd, cache, S = _c2_state(device, seed=10)
    base = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", 128, 4)
    perm = torch.stack([torch.randperm(128, device=device) + 128 * c for c in range(S // 128)]).reshape(-1)
    cache2 = H.alloc_cache(1, S, 8, 4, 128, device)
    kvcache_pack_int(kd[:, :S][:, perm].contiguous(), cache2[0], cache2[1], vd[:, :S][:, perm].contiguous(),
                     cache2[2], cache2[3], None, None, S, "k-channel", 128, 4)
    o = fwd_kvcache_int(qd, *cache2, None, SCALE, "k-channel", 128, 4)
    assert (o.float() - base.float()).abs().max().item() < 5e-4


def test_full_size_value_scaling_is_linear(device):
    """V -> 2V is exact in fp16: scale and zero double, codes stay, so the output doubles."""
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    qd, kd, vd, cache, S = _c2_state(device, seed=11)
    base = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", 128, 4)
    cache2 = H.alloc_cache(1, S, 8, 4, 128, device)
    kvcache_pack_int(kd[:, :S], cache2[0], cache2[1], (vd[:, :S] * 2).contiguous(), cache2[2], cache2[3], None, None,
                     S, "k-channel", 128, 4)
    assert torch.equal(cache[2], cache2[2])                # V codes unchanged
    o = fwd_kvcache_int(qd, *cache2, None, SCALE, "k-channel", 128, 4)
    assert (o.float() - 2 * base.float()).abs().max().item() < 1e-3


def test_full_size_pack_is_idempotent_and_error_bounded(device):
    from bitladder_amd import kvcache_pack_int, layout as L
    qd, kd, vd, cache, S = _c2_state(device, seed=12)
    cache2 = H.alloc_cache(1, S, 8, 4, 128, device, fill=0x7777)
    kvcache_pack_int(kd[:, :S], cache2[0], cache2[1], vd[:, :S], cache2[2], cache2[3], None, None, S, "k-channel", 128, 4)
    for a, c in zip(cache, cache2):
        assert torch.equal(a, c)
    kc, ks, kz, vc, vs, vz = L.unpack_physical(*H.cache_to_numpy(*cache), 4, 128)
    f = lambda a: a.view(np.float16).astype(np.float32)
    k_hat = kc.astype(np.float32) * np.repeat(f(ks), 128, axis=1) + np.repeat(f(kz), 128, axis=1)
    k = kd[:, :S].float().cpu().numpy()
    bound = np.repeat(f(ks), 128, axis=1) * (0.5 + 15 * 2.0 ** -11) + 1e-6
    assert (np.abs(k_hat - k) <= bound).all()
    assert kc.max() == 15 and kc.min() == 0
