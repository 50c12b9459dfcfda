"""GPU parity tests: HIP kernels (through the C ABI) against the CPU oracle.

Bars: packed codes and scale/zero bit-exact; attention output within 2e-3 max-abs of
dequantize-then-attend computed in fp32.
"""
import math

import numpy as np
import pytest
import torch

from oracle import bitdecode_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

ATOL = 2e-3
SCALE = 1.0 / math.sqrt(128)


def _pack_gpu(k, v, bits, gs, dtype, device, S):
    from bitladder_amd import kvcache_pack_int
    b, _, h_k, _ = k.shape
    cache = H.alloc_cache(b, S, h_k, bits, gs, device)
    kd, vd = H.to_dev(k[:, :S], dtype, device), H.to_dev(v[:, :S], dtype, device)
    cu = torch.arange(0, (b + 1) * S, S, dtype=torch.int32, device=device)
    kvcache_pack_int(kd, cache[0], cache[1], vd, cache[2], cache[3], None, cu, S, "k-channel", gs, bits)
    return cache


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("bits", [2, 4])
def test_qpack_bit_exact(device, bits, gs, dtype):
    b, h_k, S = 2, 3, 384
    q, k, v = O.make_inputs(b, h_k, h_k, S, 0, seed=bits * 100 + gs, dtype=dtype)
    # edge groups: constant K group, constant V group, max-range values, exact .5 ties
    k[0, :gs, 0, 5] = 1.5
    v[0, 7, 1, :gs] = -2.25
    k[1, gs:2 * gs, 1, 9] = np.linspace(-3, 3, gs, dtype=np.float32)
    v[1, 3, 2, :] = 0.0
    k[0, 0, 2, 17], k[0, 1, 2, 17] = 65504.0, -65504.0
    k, v = O.round_to_storage(k, dtype), O.round_to_storage(v, dtype)
    want = O.quantize_kv_ref(k, v, bits, gs, dtype)
    cache = _pack_gpu(k, v, bits, gs, dtype, device, S)
    torch.cuda.synchronize()
    H.assert_cache_equals_oracle(H.cache_to_numpy(*cache), want)


@pytest.mark.parametrize("bits,gs", [(4, 128), (4, 32), (2, 128), (2, 64), (4, 64), (2, 32)])
@pytest.mark.parametrize("h,h_k", [(4, 4), (8, 2), (8, 1)])
def test_decode_from_host_packed_cache(device, bits, gs, h, h_k):
    """Decode kernel alone: the cache is laid out on the host from the quantizer oracle."""
    from bitladder_amd import fwd_kvcache_int
    b, S = 2, 1024
    q, k, v = O.make_inputs(b, h, h_k, S, 0, seed=7)
    qkv = O.quantize_kv_ref(k, v, bits, gs)
    cache = H.cache_from_numpy(H.oracle_physical(qkv), device)
    k_hat, v_hat = O.dequantize_ref(qkv)
    want, want_lse = O.attend_ref(q, k_hat, v_hat, SCALE)
    for ns in (0, 1, 3):
        out, lse = fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-channel", gs, bits,
                                   num_splits=ns, return_lse=True)
        err = np.abs(out.float().cpu().numpy() - want).max()
        assert err < ATOL, (ns, err)
        np.testing.assert_allclose(lse.cpu().numpy(), want_lse, atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("res_len", [0, 1, 31, 32, 33, 100, 128])
@pytest.mark.parametrize("bits,gs", [(4, 128), (2, 64)])
def test_decode_with_residual_window(device, bits, gs, res_len):
    from bitladder_amd import fwd_kvcache_int
    b, h, h_k, S, R = 2, 8, 2, 512, 128
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=11)
    qkv = O.quantize_kv_ref(k[:, :S], v[:, :S], bits, gs)
    cache = _pack_gpu(k, v, bits, gs, "fp16", device, S)
    k_hat, v_hat = O.dequantize_ref(qkv)
    rl = np.full(b, res_len, np.int32)
    want, _ = O.attend_ref(q, k_hat, v_hat, SCALE, k[:, S:], v[:, S:], res_lens=rl)
    kres, vres = H.to_dev(k[:, S:], "fp16", device), H.to_dev(v[:, S:], "fp16", device)
    # poison the invalid tail: it must not be read into the result
    kres[:, res_len:] = float("nan")
    vres[:, res_len:] = float("nan")
    out = fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-channel", gs, bits,
                          k_residual=kres, v_residual=vres, residual_len=res_len)
    err = np.abs(out.float().cpu().numpy() - want).max()
    assert err < ATOL, err


def test_decode_residual_only(device):
    """No packed prefix at all: the fp16 path alone (also the fp16-KV baseline kernel)."""
    from bitladder_amd import fwd_kvcache_int
    b, h, h_k, R = 2, 8, 2, 1000
    q, k, v = O.make_inputs(b, h, h_k, 0, R, seed=5)
    want, _ = O.attend_ref(q, None, None, SCALE, k, v)
    cache = H.alloc_cache(b, 128, h_k, 4, 128, device)
    for ns in (0, 1, 5):
        out = fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-channel", 128, 4,
                              seqlen_k=0, k_residual=H.to_dev(k, "fp16", device),
                              v_residual=H.to_dev(v, "fp16", device), num_splits=ns)
        err = np.abs(out.float().cpu().numpy() - want).max()
        assert err < ATOL, (ns, err)


@pytest.mark.parametrize("bits,gs", [(4, 128), (4, 64), (4, 32), (2, 128), (2, 64), (2, 32)])
def test_decode_many_chunks_per_wave(device, bits, gs):
    """Few splits over a long prefix: every wave loops over several chunks (running max carried
    across chunks, loads of the next chunk issued while the current one is consumed)."""
    from bitladder_amd import fwd_kvcache_int
    b, h, h_k, S = 1, 8, 2, 4096 + 128 * 3          # 35 chunks: uneven tail across the 8 waves
    q, k, v = O.make_inputs(b, h, h_k, S, 0, seed=21)
    qkv = O.quantize_kv_ref(k, v, bits, gs)
    cache = _pack_gpu(k, v, bits, gs, "fp16", device, S)
    k_hat, v_hat = O.dequantize_ref(qkv)
    want, _ = O.attend_ref(q, k_hat, v_hat, SCALE)
    for ns in (1, 2):
        out = fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-channel", gs, bits, num_splits=ns)
        err = np.abs(out.float().cpu().numpy() - want).max()
        assert err < ATOL, (ns, err)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("gs", [128, 64, 32])
def test_decode_both_wave_count_variants_of_the_4bit_kernels(device, gs, dtype):
    """The 4-bit kernels exist with 16 (12 at group 32) and with 8 waves per workgroup; the library takes the
    8-wave one when a workgroup has at most 16 packed units.  32 units here: one split runs the large variant,
    two splits the small one with two units per wave (its deeper row pipeline runs on into the second unit),
    four splits the small one with one unit per wave.  Same bar for all."""
    from bitladder_amd import fwd_kvcache_int
    b, h, h_k, S, R, bits = 2, 8, 2, 2048, 40, 4
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=91, dtype=dtype)
    qkv = O.quantize_kv_ref(k[:, :S], v[:, :S], bits, gs, dtype=dtype)
    cache = _pack_gpu(k, v, bits, gs, dtype, device, S)
    k_hat, v_hat = O.dequantize_ref(qkv)
    want, want_lse = O.attend_ref(q, k_hat, v_hat, SCALE, k[:, S:], v[:, S:])
    kres, vres = H.to_dev(k[:, S:], dtype, device), H.to_dev(v[:, S:], dtype, device)
    tol = H.out_tolerance(want, dtype)
    for ns in (1, 2, 4):
        out, lse = fwd_kvcache_int(H.to_dev(q, dtype, device), *cache, None, SCALE, "k-channel", gs, bits,
                                   k_residual=kres, v_residual=vres, num_splits=ns, return_lse=True)
        err = np.abs(out.float().cpu().numpy() - want)
        assert (err <= tol).all(), (ns, err.max())
        np.testing.assert_allclose(lse.cpu().numpy(), want_lse, atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("bits,gs", [(4, 128), (4, 32), (2, 128), (2, 32)])
def test_decode_many_splits(device, bits, gs):
    """More splits than one batch of the final merge handles at once (33, 70), and more splits than
    packed units (100 over 40 or 80 units: most splits are empty and must contribute nothing).  The
    result and the LSE must not depend on the split count."""
    from bitladder_amd import fwd_kvcache_int
    b, h, h_k, S, R = 2, 8, 2, 128 * 40, 48
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=33)
    qkv = O.quantize_kv_ref(k[:, :S], v[:, :S], bits, gs)
    cache = _pack_gpu(k, v, bits, gs, "fp16", device, S)
    k_hat, v_hat = O.dequantize_ref(qkv)
    want, want_lse = O.attend_ref(q, k_hat, v_hat, SCALE, k[:, S:], v[:, S:])
    kres, vres = H.to_dev(k[:, S:], "fp16", device), H.to_dev(v[:, S:], "fp16", device)
    for ns in (33, 70, 100, 512):
        out, lse = fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-channel", gs, bits,
                                   k_residual=kres, v_residual=vres, num_splits=ns, return_lse=True)
        err = np.abs(out.float().cpu().numpy() - want).max()
        assert err < ATOL, (ns, err)
        np.testing.assert_allclose(lse.cpu().numpy(), want_lse, atol=2e-3, rtol=1e-4)


def test_plan_and_pack_replay_in_hip_graph(device):
    """A decode plan (split workspace included) and an append-pack call are captured in one HIP graph
    and replayed several times with eager work and synchronisations in between; every replay must
    reproduce the eager result bit for bit, also after the inputs behind the captured pointers change."""
    from bitladder_amd import kvcache_pack_int, plan_fwd_kvcache_int
    b, h, h_k, S, R, bits, gs = 2, 8, 2, 128 * 12, 128, 4, 128
    q, k, v = O.make_inputs(b, h, h_k, S + 128, R, seed=44)
    kd, vd = H.to_dev(k, "fp16", device), H.to_dev(v, "fp16", device)
    qd = H.to_dev(q, "fp16", device)
    cache = H.alloc_cache(b, S + 128, h_k, bits, gs, device)
    kvcache_pack_int(kd[:, :S], cache[0], cache[1], vd[:, :S], cache[2], cache[3], None, None, S, "k-channel", gs, bits)
    new_k, new_v = kd[:, S:S + 128].clone(), vd[:, S:S + 128].clone()      # block appended inside the graph
    kres, vres = kd[:, S + 128:].contiguous(), vd[:, S + 128:].contiguous()
    plan = plan_fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, seqlen_k=S + 128,
                                k_residual=kres, v_residual=vres, num_splits=5)

    def step():
        kvcache_pack_int(new_k, cache[0], cache[1], new_v, cache[2], cache[3], None, None, 128, "k-channel", gs,
                         bits, dst_offset=S)
        return plan.run()

    eager = step().clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream(device).wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step()
    for rep in range(4):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
        # eager work between replays, then new contents behind the captured pointers
        _ = (kd.float().sum() + vd.float().sum()).item()
        if rep == 1:
            qd.mul_(-0.5)
            new_k.copy_(kd[:, 128:256])
            new_v.copy_(vd[:, 128:256])
            eager = step().clone()
            torch.cuda.synchronize()
    want_cache = H.alloc_cache(b, S + 128, h_k, bits, gs, device)
    kvcache_pack_int(torch.cat([kd[:, :S], new_k], 1), want_cache[0], want_cache[1], torch.cat([vd[:, :S], new_v], 1),
                     want_cache[2], want_cache[3], None, None, S + 128, "k-channel", gs, bits)
    for a, c in zip(cache, want_cache):
        assert torch.equal(a, c)


@pytest.mark.parametrize("seed", range(12))
def test_decode_random_shapes(device, seed):
    """Seeded sweep over the argument space: batch, GQA ratio, bits, group size, element type, packed
    length per sequence (ragged, including empty), window length per sequence, split count and the
    sign of the softmax scale, each against dequantize-then-attend on the same inputs."""
    from bitladder_amd import fwd_kvcache_int
    rng = np.random.default_rng(1000 + seed)
    bits = int(rng.choice([2, 4]))
    gs = int(rng.choice([32, 64, 128]))
    dtype = "bf16" if seed % 3 == 2 else "fp16"
    h_k = int(rng.choice([1, 2, 3]))
    g = int(rng.choice([1, 2, 4, 5, 8]))
    b = int(rng.integers(1, 4))
    S = 128 * int(rng.integers(1, 20))
    R = int(rng.choice([0, 16, 77, 128]))
    ns = int(rng.choice([0, 1, 2, 3, 7, 19]))
    scale = SCALE * (-1.0 if seed % 4 == 3 else 1.0)
    h = h_k * g
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=2000 + seed, dtype=dtype)
    qkv = O.quantize_kv_ref(k[:, :S], v[:, :S], bits, gs, dtype)
    cache = _pack_gpu(k, v, bits, gs, dtype, device, S)
    k_hat, v_hat = O.dequantize_ref(qkv)
    seqlens = (128 * rng.integers(0, S // 128 + 1, b)).astype(np.int32)
    seqlens[rng.integers(0, b)] = S                       # at least one full-length sequence
    reslens = rng.integers(0, R + 1, b).astype(np.int32) if R else np.zeros(b, np.int32)
    if R and seqlens.min() == 0:
        reslens[seqlens == 0] = np.maximum(reslens[seqlens == 0], 1)     # keep every row non-empty here
    kres = vres = None
    kw = dict(seqlens_k=torch.from_numpy(seqlens).to(device), max_seqlen_k=S, num_splits=ns, return_lse=True)
    if R:
        kw.update(k_residual=H.to_dev(k[:, S:], dtype, device), v_residual=H.to_dev(v[:, S:], dtype, device),
                  residual_len=torch.from_numpy(reslens).to(device), max_residual_len=R)
        kres, vres = k[:, S:], v[:, S:]
    elif seqlens.min() == 0:
        seqlens[seqlens == 0] = 128
        kw["seqlens_k"] = torch.from_numpy(seqlens).to(device)
    want, want_lse = O.attend_ref(q, k_hat, v_hat, scale, kres, vres, seqlens_k=seqlens,
                                  res_lens=reslens if R else None)
    out, lse = fwd_kvcache_int(H.to_dev(q, dtype, device), *cache, None, scale, "k-channel", gs, bits, **kw)
    diff = np.abs(out.float().cpu().numpy() - want)      # 2e-3, plus half a bf16 ulp for a bf16 output
    assert (diff < H.out_tolerance(want, dtype, ATOL)).all(), (bits, gs, dtype, b, h, h_k, S, R, ns, diff.max())
    np.testing.assert_allclose(lse.cpu().numpy(), want_lse, atol=3e-3, rtol=1e-4)
    # and the same bits every time, also once the cache has become L2-resident
    for _ in range(20):
        again, _ = fwd_kvcache_int(H.to_dev(q, dtype, device), *cache, None, scale, "k-channel", gs, bits, **kw)
        assert torch.equal(again, out)


@pytest.mark.parametrize("b,lengths", [(5, [1024, 0, 1024, 384, 2048]), (16, None), (2, [128, 2048]), (64, None)])
def test_sequences_dealt_out_by_length_give_the_same_bits(device, b, lengths):
    """More workgroups than compute units and per-sequence lengths on the device: the kernel permutes the batch
    index by rank of length (ties by index; odd batch sizes; empty sequences).  The permutation must not change a
    bit: every sequence's output equals that of a call over that sequence alone with the same split count, and
    matches the oracle."""
    from bitladder_amd import fwd_kvcache_int
    h_k, g, S, R, bits, gs = 8, 2, 2048, 40, 4, 128
    if b == 64:
        h_k, g = 2, 4
    h = h_k * g
    rng = np.random.default_rng(b)
    seqlens = np.asarray(lengths if lengths is not None else 128 * rng.integers(0, S // 128 + 1, b), dtype=np.int32)
    ns = max(2, -(-300 // (b * h_k)))                     # b * h_k * ns > 256 compute units
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=77 + b)
    cache = _pack_gpu(k, v, bits, gs, "fp16", device, S)
    qd = H.to_dev(q, "fp16", device)
    kr, vr = H.to_dev(k[:, S:], "fp16", device), H.to_dev(v[:, S:], "fp16", device)
    out = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, seqlens_k=torch.from_numpy(seqlens).to(device),
                          max_seqlen_k=S, k_residual=kr, v_residual=vr, num_splits=ns)
    for i in range(b):      # alone, with a host-side length: a grid without the permutation
        alone = fwd_kvcache_int(qd[i:i + 1], *(t[i:i + 1] for t in cache), None, SCALE, "k-channel", gs, bits,
                                seqlen_k=int(seqlens[i]), k_residual=kr[i:i + 1], v_residual=vr[i:i + 1], num_splits=ns)
        assert torch.equal(out[i:i + 1], alone), (i, int(seqlens[i]))
    qkv = O.quantize_kv_ref(k[:, :S], v[:, :S], bits, gs)
    k_hat, v_hat = O.dequantize_ref(qkv)
    want, _ = O.attend_ref(q, k_hat, v_hat, SCALE, k[:, S:], v[:, S:], seqlens_k=seqlens)
    assert np.abs(out.float().cpu().numpy() - want).max() < ATOL


@pytest.mark.parametrize("bits", [2, 4])
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_qpack_ranges_from_subnormal_to_max(device, bits, dtype):
    """Groups whose range spans 2^-24 .. 2^16 (fp16 subnormals up to +-65504), every group containing its
    exact minimum and maximum: the codes of the extremes must be 0 and 2^bits - 1, nothing may spill into
    a neighbouring field, and all bytes must equal the oracle's (which clamps explicitly)."""
    rng = np.random.default_rng(77 + bits)
    b, h_k, S, gs = 1, 2, 512, 32
    e = rng.uniform(-24, 15.9, size=(b, S // gs, 1, h_k, 128))
    lo = rng.uniform(-1, 1, size=e.shape) * 2.0 ** e
    u = rng.uniform(0, 1, size=(b, S // gs, gs, h_k, 128))
    u[:, :, 0], u[:, :, 1] = 0.0, 1.0                                   # exact extremes in every K group
    k = (lo + u * 2.0 ** e).reshape(b, S, h_k, 128)
    ev = rng.uniform(-24, 15.9, size=(b, S, h_k, 128 // gs, 1))
    lov = rng.uniform(-1, 1, size=ev.shape) * 2.0 ** ev
    uv = rng.uniform(0, 1, size=(b, S, h_k, 128 // gs, gs))
    uv[..., 0], uv[..., 1] = 0.0, 1.0
    v = (lov + uv * 2.0 ** ev).reshape(b, S, h_k, 128)
    k, v = np.clip(k, -65504, 65504).astype(np.float32), np.clip(v, -65504, 65504).astype(np.float32)
    k, v = O.round_to_storage(k, dtype), O.round_to_storage(v, dtype)
    want = O.quantize_kv_ref(k, v, bits, gs, dtype)
    assert want.k_codes.max() == (1 << bits) - 1 and want.v_codes.max() == (1 << bits) - 1
    cache = _pack_gpu(k, v, bits, gs, dtype, device, S)
    torch.cuda.synchronize()
    H.assert_cache_equals_oracle(H.cache_to_numpy(*cache), want)


@pytest.mark.parametrize("bits,gs,S,ns", [(4, 32, 4096, 1), (4, 32, 8192, 2), (4, 128, 8192, 1), (2, 64, 16384, 1),
                                        (2, 128, 16384, 1), (2, 32, 8192, 1), (2, 128, 16384, 2)])
def test_waves_with_many_units_on_cache_resident_data_are_deterministic(device, bits, gs, S, ns):
    """Each wave streams three or more units through its LDS region, and the cache is small enough to stay in
    L2 while the call is repeated: the direct-to-LDS loads of the next unit then come back fast, and must
    still not overtake the LDS reads of the current one (the kernel waits for those reads before it issues
    the loads).  Every repetition must give the same bits, and the right ones."""
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    b, h, h_k = 1, 8, 2
    q, k, v = O.make_inputs(b, h, h_k, S, 0, seed=61)
    qd, kd, vd = H.to_dev(q, "fp16", device), H.to_dev(k, "fp16", device), H.to_dev(v, "fp16", device)
    cache = H.alloc_cache(b, S, h_k, bits, gs, device)
    kvcache_pack_int(kd, cache[0], cache[1], vd, cache[2], cache[3], None, None, S, "k-channel", gs, bits)
    outs = [fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, num_splits=ns) for _ in range(200)]
    torch.cuda.synchronize()
    assert all(torch.equal(o, outs[0]) for o in outs[1:])
    qkv = O.quantize_kv_ref(k, v, bits, gs)
    k_hat, v_hat = O.dequantize_ref(qkv)
    ref, _ = O.attend_ref(q, k_hat, v_hat, SCALE)
    assert np.abs(outs[0].float().cpu().numpy() - ref).max() < 2e-3


@pytest.mark.parametrize("bits,vmax", [(2, 30000.0), (4, 30000.0), (2, 65000.0)])
def test_decode_with_v_groups_spanning_the_fp16_range(device, bits, vmax):
    """V groups whose range is close to the whole fp16 range: the V scale reaches 2 * vmax / (2^bits - 1)
    (43 000 at 2 bits), and probability x scale must still fit fp16."""
    from bitladder_amd import fwd_kvcache_int
    b, h, h_k, S, gs = 1, 8, 2, 512, 128
    q, k, v = O.make_inputs(b, h, h_k, S, 0, seed=61)
    rng = np.random.default_rng(3)
    v = O.round_to_storage((rng.uniform(-1, 1, v.shape) * vmax).astype(np.float32), "fp16")
    v[0, ::7, 0, 5], v[0, ::7, 0, 6] = vmax, -vmax
    v = O.round_to_storage(v, "fp16")
    qkv = O.quantize_kv_ref(k, v, bits, gs)
    assert qkv.v_scale.max() > (1.9 * vmax) / ((1 << bits) - 1)
    cache = _pack_gpu(k, v, bits, gs, "fp16", device, S)
    k_hat, v_hat = O.dequantize_ref(qkv)
    want, _ = O.attend_ref(q, k_hat, v_hat, SCALE)
    out = fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-channel", gs, bits).float().cpu().numpy()
    assert np.isfinite(out).all()
    # outputs are of the order of vmax / sqrt(S): the bound is relative here (2e-3 of the largest expected value)
    assert np.abs(out - want).max() < 2e-3 * np.abs(want).max(), (np.abs(out - want).max(), np.abs(want).max())


def test_device_side_lengths_and_offsets_beyond_the_buffers_are_clamped(device):
    """Per-sequence lengths and offsets are device data the host never sees: a packed length beyond the cache
    counts as the capacity, a window length beyond the window as the window, and a pack offset that is off a
    chunk boundary or past the cache writes nothing."""
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    b, h, h_k, S, R, bits, gs = 2, 8, 2, 1024, 64, 4, 128
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=62)
    cache = _pack_gpu(k, v, bits, gs, "fp16", device, S)
    kr, vr = H.to_dev(k[:, S:], "fp16", device), H.to_dev(v[:, S:], "fp16", device)
    qd = H.to_dev(q, "fp16", device)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    kw = dict(k_residual=kr, v_residual=vr, max_seqlen_k=S, max_residual_len=R)
    want = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, seqlens_k=i32([S, 512]), residual_len=i32([R, 10]), **kw)
    got = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, seqlens_k=i32([S + 4096, 512]),
                          residual_len=i32([R + 1000, 10]), **kw)
    assert torch.equal(got, want)
    neg = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, seqlens_k=i32([S, -128]), residual_len=i32([R, 10]), **kw)
    zero = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, seqlens_k=i32([S, 0]), residual_len=i32([R, 10]), **kw)
    assert torch.equal(neg, zero)
    # pack: sequence 0 at a valid offset, sequence 1 once misaligned and once past the end -> untouched
    before = [t.clone() for t in cache]
    kd, vd = H.to_dev(k[:, :128] * 0.5, "fp16", device), H.to_dev(v[:, :128] * 0.5, "fp16", device)
    for bad in (64, S):
        kvcache_pack_int(kd, cache[0], cache[1], vd, cache[2], cache[3], None, None, 128, "k-channel", gs, bits,
                         dst_offsets=i32([256, bad]))
        torch.cuda.synchronize()
        for t, t0 in zip(cache, before):
            assert torch.equal(t[1], t0[1])                  # sequence 1: nothing written
        assert not torch.equal(cache[0][0], before[0][0])    # sequence 0: its chunk was packed


@pytest.mark.parametrize("bits,gs", [(4, 128), (2, 128)])
@pytest.mark.parametrize("ns", [2, 4, 32])
def test_splits_whose_outputs_cancel_stay_within_the_bar(device, bits, gs, ns):
    """Designed inputs: the splits' own outputs are about +5 and -5 in every channel (|v| = 4 ... 6, signs that flip
    from one split to the next) with near-equal softmax weights, so the merged output is small and whatever the
    partial outputs lose on their way between workgroups shows in full against the plain 2e-3 bar.  The
    reference keeps its partial outputs in fp32 (flash_fwd_kernel.h:1280-1298)."""
    from bitladder_amd import fwd_kvcache_int
    b, h, h_k, S = 2, 8, 2, 128 * ns * 4
    rng = np.random.default_rng(1234 + ns + bits)
    q = (0.05 * rng.standard_normal((b, 1, h, 128))).astype(np.float32)      # flat softmax: weights nearly equal
    k = rng.standard_normal((b, S, h_k, 128)).astype(np.float32)
    sign_c = rng.choice([-1.0, 1.0], size=(1, 1, h_k, 128)).astype(np.float32)
    sign_s = np.where((np.arange(S) // (S // ns)) % 2 == 0, 1.0, -1.0).astype(np.float32).reshape(1, S, 1, 1)
    v = (sign_c * sign_s * (5.0 + 0.3 * rng.standard_normal((b, S, h_k, 128)))).astype(np.float32)
    q, k, v = (O.round_to_storage(x, "fp16") for x in (q, k, v))
    qkv = O.quantize_kv_ref(k, v, bits, gs)
    cache = _pack_gpu(k, v, bits, gs, "fp16", device, S)
    k_hat, v_hat = O.dequantize_ref(qkv)
    want, _ = O.attend_ref(q, k_hat, v_hat, SCALE)
    assert np.abs(want).max() < 0.5, "the designed outputs are meant to cancel"
    out = fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-channel", gs, bits, num_splits=ns)
    one = fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-channel", gs, bits, num_splits=1)
    err = np.abs(out.float().cpu().numpy() - want).max()
    err1 = np.abs(one.float().cpu().numpy() - want).max()
    assert err1 < ATOL, err1
    assert err < ATOL, (ns, err, err1)


def test_plain_call_recorded_into_a_hip_graph_has_a_workspace_of_its_own(device):
    """fwd_kvcache_int (not a plan) recorded into a HIP graph: the recorded call must not share the per-stream
    workspace cache with later eager calls.  The graph is replayed on a side stream while eager calls of the same
    shape run on the default stream, several times; every replay and every eager call reproduces its result."""
    from bitladder_amd import fwd_kvcache_int
    from bitladder_amd import interface as I
    b, h, h_k, S, bits, gs, ns = 2, 8, 2, 128 * 16, 4, 128, 4
    q, k, v = O.make_inputs(b, h, h_k, S, 0, seed=91)
    cache = _pack_gpu(k, v, bits, gs, "fp16", device, S)
    qd = H.to_dev(q, "fp16", device)
    q2 = (qd * -0.75).contiguous()
    eager1 = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, num_splits=ns).clone()
    eager2 = fwd_kvcache_int(q2, *cache, None, SCALE, "k-channel", gs, bits, num_splits=ns).clone()
    torch.cuda.synchronize()
    shared = {id(w) for w in I._WORKSPACES.values()}
    out_g = torch.empty_like(qd)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, num_splits=ns, out=out_g)
    assert {id(w) for w in I._WORKSPACES.values()} == shared, "the capture must not add to the stream workspaces"
    side = torch.cuda.Stream(device)
    for rep in range(4):
        out_g.zero_()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            graph.replay()
        outs = [fwd_kvcache_int(q2, *cache, None, SCALE, "k-channel", gs, bits, num_splits=ns) for _ in range(3)]
        torch.cuda.synchronize()
        assert torch.equal(out_g, eager1), rep
        for o in outs:
            assert torch.equal(o, eager2), rep


@pytest.mark.parametrize("bits,gs,h,h_k,ns", [(4, 128, 8, 2, 7), (2, 64, 4, 4, 32), (4, 32, 16, 2, 3)])
def test_one_workspace_over_many_launches_with_changing_queries(device, bits, gs, h, h_k, ns):
    """The two record slots of a split workspace are used in turn, and a launch sets its records of the other
    slot back to "not written".  One plan (one workspace) runs 41 launches, the query rewritten in place before each:
    every launch must give the bits that a fresh workspace gives for that query, i.e. no record of an earlier launch
    is ever taken for one of the current launch."""
    from bitladder_amd import plan_fwd_kvcache_int
    b, S = 2, 128 * 33
    q, k, v = O.make_inputs(b, h, h_k, S, 60, seed=300 + ns)
    cache = _pack_gpu(k[:, :S], v[:, :S], bits, gs, "fp16", device, S)
    kres, vres = H.to_dev(k[:, S:], "fp16", device), H.to_dev(v[:, S:], "fp16", device)
    qd = H.to_dev(q, "fp16", device)
    plan = plan_fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, k_residual=kres, v_residual=vres,
                                num_splits=ns)
    gen = torch.Generator(device=device).manual_seed(17)
    for it in range(41):
        qd.copy_(torch.randn(qd.shape, generator=gen, device=device) * (0.25 + 0.1 * (it % 9)))
        got = plan.run().clone()
        fresh = plan_fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, k_residual=kres,
                                     v_residual=vres, num_splits=ns).run()
        assert torch.equal(got, fresh), it


def test_workspace_zeroed_again_serves_another_shape(device):
    """The C ABI's rule for a caller-owned workspace: all zero before its first call and before a call with another
    (b, h, num_splits).  One buffer, sized for the larger of two shapes, serves them in turn with a fill in between;
    results equal those of workspaces of their own."""
    import ctypes
    from bitladder_amd import _lib, plan_fwd_kvcache_int
    L = _lib.lib()

    def plan_for(seed, b, h, h_k, S, bits, gs, ns):
        q, k, v = O.make_inputs(b, h, h_k, S, 0, seed=seed)
        cache = _pack_gpu(k, v, bits, gs, "fp16", device, S)
        return plan_fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-channel", gs, bits,
                                    num_splits=ns)

    plans = [plan_for(410, 1, 32, 8, 128 * 64, 4, 128, 32), plan_for(411, 3, 4, 2, 128 * 10, 2, 128, 5)]
    want = [p.run().clone() for p in plans]
    nbytes = max(L.bitdecode_fwd_workspace_bytes(p.args.b, p.args.h, p.args.num_splits) for p in plans)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    for rep in range(3):
        for p, w in zip(plans, want):
            ws.zero_()
            a = _lib.FwdArgs()
            ctypes.memmove(ctypes.byref(a), ctypes.byref(p.args), ctypes.sizeof(a))
            out = torch.full_like(p.out, float("nan"))
            a.out, a.workspace, a.workspace_bytes = out.data_ptr(), ws.data_ptr(), nbytes
            for call in range(3):      # the same shape again needs no fill
                assert L.bitdecode_fwd(ctypes.byref(a), torch.cuda.current_stream(device).cuda_stream) == 0
                torch.cuda.synchronize()
                assert torch.equal(out, w), (rep, call)


@pytest.mark.parametrize("h,h_k,m", [(8, 8, 5), (8, 2, 3), (16, 2, 2), (4, 4, 11)])
def test_several_query_rows_per_sequence(device, h, h_k, m):
    """q [b, m, h, d] with m > 1 (admitted by the reference, decode_api.cpp:341, 358-368; its Python interface
    fixes is_causal = False, bit_decode_interface.py:72-84, so every row attends every key): each row must equal
    the oracle's output for that row alone, and a call with that row alone."""
    from bitladder_amd import fwd_kvcache_int
    b, S, R, bits, gs = 2, 128 * 9, 37, 4, 64
    _, k, v = O.make_inputs(b, h, h_k, S, R, seed=700 + m)
    rng = np.random.default_rng(701 + m)
    q = O.round_to_storage(rng.standard_normal((b, m, h, 128), dtype=np.float32), "fp16")
    cache = _pack_gpu(k[:, :S], v[:, :S], bits, gs, "fp16", device, S)
    kres, vres = H.to_dev(k[:, S:], "fp16", device), H.to_dev(v[:, S:], "fp16", device)
    qd = H.to_dev(q, "fp16", device)
    out, lse = fwd_kvcache_int(qd, *cache, None, SCALE, "k-channel", gs, bits, k_residual=kres, v_residual=vres,
                               return_lse=True)
    assert out.shape == qd.shape and lse.shape == (b, m, h)
    qkv = O.quantize_kv_ref(k[:, :S], v[:, :S], bits, gs)
    k_hat, v_hat = O.dequantize_ref(qkv)
    for r in range(m):
        want, want_lse = O.attend_ref(q[:, r:r + 1], k_hat, v_hat, SCALE, k[:, S:], v[:, S:])
        assert np.abs(out[:, r:r + 1].float().cpu().numpy() - want).max() < ATOL, r
        assert np.abs(lse[:, r].cpu().numpy() - want_lse).max() < 1e-3, r
        alone = fwd_kvcache_int(qd[:, r:r + 1].contiguous(), *cache, None, SCALE, "k-channel", gs, bits,
                                k_residual=kres, v_residual=vres)
        assert (alone.float() - out[:, r:r + 1].float()).abs().max().item() < 5e-4, r
