"""`torch.library` registration of the entry points (`bitladder_amd/torch_ops.py`): schemas that declare what is
written, fake implementations that let a graph be traced without running a kernel, and on the GPU the same
results as the plain functions, also from inside a compiled function."""
import math

import pytest
import torch

from tests import helpers as H

SCALE = 1.0 / math.sqrt(128)


def _fake_inputs(device="cuda"):
    q = torch.empty((2, 1, 8, 128), dtype=torch.float16, device=device)
    kp = torch.empty((2, 64, 2, 128), dtype=torch.uint16, device=device)
    kpar = torch.empty((2, 2, 2, 128), dtype=torch.float32, device=device)
    vp = torch.empty((2, 256, 2, 32), dtype=torch.uint16, device=device)
    vpar = torch.empty((2, 1, 2, 256), dtype=torch.float32, device=device)
    return q, kp, kpar, vp, vpar


def test_operators_are_registered_with_their_mutations():
    import bitladder_amd.torch_ops  # noqa: F401
    ops = torch.ops.bitladder_amd
    pack, fwd, step = (str(getattr(ops, n).default._schema) for n in
                       ("kvcache_pack_int", "fwd_kvcache_int", "fwd_kvcache_int_append"))
    assert "Tensor(a1!) k_pack" in pack and "Tensor(a5!) v_params" in pack and pack.endswith("-> ()")
    assert "!" not in fwd and fwd.endswith("-> Tensor")
    for name in ("k_pack", "k_params", "v_pack", "v_params", "k_residual", "v_residual", "lengths"):
        assert f"!) {name}" in step, name
    assert "!) q" not in step and "!) k_new" not in step


def test_fake_implementations_trace_without_a_gpu():
    import bitladder_amd.torch_ops  # noqa: F401
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        q, kp, kpar, vp, vpar = _fake_inputs()
        out = torch.ops.bitladder_amd.fwd_kvcache_int(q, kp, kpar, vp, vpar, None, SCALE)
        assert out.shape == q.shape and out.dtype == q.dtype and out.device == q.device
        kn = torch.empty((2, 1, 2, 128), dtype=torch.float16, device="cuda")
        win = torch.empty((2, 128, 2, 128), dtype=torch.float16, device="cuda")
        lengths = torch.empty(2, dtype=torch.int32, device="cuda")
        out = torch.ops.bitladder_amd.fwd_kvcache_int_append(q, kn, kn, kp, kpar, vp, vpar, win, win, lengths, 256)
        assert out.shape == q.shape
        k = torch.empty((2, 256, 2, 128), dtype=torch.float16, device="cuda")
        assert torch.ops.bitladder_amd.kvcache_pack_int(k, kp, kpar, k, vp, vpar) is None


def test_operators_have_no_cpu_kernel():
    """There is no CPU path behind the operators either."""
    import bitladder_amd.torch_ops  # noqa: F401
    q, kp, kpar, vp, vpar = _fake_inputs("cpu")
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.bitladder_amd.fwd_kvcache_int(q, kp, kpar, vp, vpar, None, SCALE)


@pytest.mark.gpu
def test_operators_equal_the_plain_functions_also_when_compiled(device):
    import bitladder_amd.torch_ops  # noqa: F401
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    from oracle import bitdecode_oracle as O
    b, h, h_k, S, R, bits, gs = 2, 8, 2, 512, 32, 4, 128
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=13)
    qd, kd, vd = H.to_dev(q, "fp16", device), H.to_dev(k, "fp16", device), H.to_dev(v, "fp16", device)
    want_cache = H.alloc_cache(b, S, h_k, bits, gs, device)
    kvcache_pack_int(kd[:, :S], want_cache[0], want_cache[1], vd[:, :S], want_cache[2], want_cache[3], None, None, S,
                     "k-channel", gs, bits)
    want = fwd_kvcache_int(qd, *want_cache, None, SCALE, "k-channel", gs, bits, k_residual=kd[:, S:],
                           v_residual=vd[:, S:], num_splits=2)
    ops = torch.ops.bitladder_amd

    def pack_then_decode(q_, k_, v_, cache):
        ops.kvcache_pack_int(k_[:, :S], cache[0], cache[1], v_[:, :S], cache[2], cache[3], None, gs, bits)
        return ops.fwd_kvcache_int(q_ * 1.0, cache[0], cache[1], cache[2], cache[3], None, SCALE, gs, bits, None, None,
                                   k_[:, S:], v_[:, S:], None, 2) + 0.0

    for fn in (pack_then_decode, torch.compile(pack_then_decode, backend="aot_eager", fullgraph=True)):
        cache = H.alloc_cache(b, S, h_k, bits, gs, device)
        got = fn(qd, kd, vd, cache)
        assert torch.equal(got, want)
        for g_, w_ in zip(cache, want_cache):
            assert torch.equal(g_, w_)

    # the step operator against the plain step function
    from bitladder_amd import fwd_kvcache_int_append
    state = []
    for _ in range(2):
        cache = [t.clone() for t in want_cache]
        win_k = torch.zeros((b, 128, h_k, 128), dtype=torch.float16, device=device)
        win_v = torch.zeros_like(win_k)
        win_k[:, :R], win_v[:, :R] = kd[:, S:], vd[:, S:]
        state.append((cache, win_k, win_v, torch.full((b,), S + R, dtype=torch.int32, device=device)))
    kn, vn = kd[:, 5:6].contiguous(), vd[:, 7:8].contiguous()
    (c0, k0, v0, l0), (c1, k1, v1, l1) = state
    a = fwd_kvcache_int_append(qd, kn, vn, *c0, k0, v0, l0, S + R, None, SCALE, "k-channel", gs, bits, num_splits=2)
    bb = ops.fwd_kvcache_int_append(qd, kn, vn, *c1, k1, v1, l1, S + R, None, SCALE, gs, bits, 2)
    assert torch.equal(a, bb) and torch.equal(l0, l1) and torch.equal(k0, k1) and torch.equal(v0, v1)
    assert l1.tolist() == [S + R + 1] * b


@pytest.mark.gpu
def test_operators_pass_the_quantization_mode_on(device):
    """`quant_mode` is the last argument of each operator: "k-tensor" gives what the plain functions give."""
    import bitladder_amd.torch_ops  # noqa: F401
    from bitladder_amd import fwd_kvcache_int, fwd_kvcache_int_append, kvcache_pack_int
    from oracle import bitdecode_oracle as O
    b, h, h_k, S, bits, gs, mode = 2, 8, 2, 256, 4, 64, "k-tensor"
    q, k, v = O.make_inputs(b, h, h_k, S + 1, 0, seed=19)
    qd, kd, vd = H.to_dev(q, "fp16", device), H.to_dev(k, "fp16", device), H.to_dev(v, "fp16", device)
    ops = torch.ops.bitladder_amd
    caches = [H.alloc_cache(b, S + 128, h_k, bits, gs, device, k_tensor=True) for _ in range(2)]
    kvcache_pack_int(kd[:, :S], caches[0][0], caches[0][1], vd[:, :S], caches[0][2], caches[0][3], None, None, S,
                     mode, gs, bits)
    ops.kvcache_pack_int(kd[:, :S], caches[1][0], caches[1][1], vd[:, :S], caches[1][2], caches[1][3], None, gs, bits,
                         quant_mode=mode)
    for g_, w_ in zip(caches[1], caches[0]):
        assert torch.equal(g_, w_)
    held = torch.full((b,), S, dtype=torch.int32, device=device)
    want = fwd_kvcache_int(qd, *caches[0], None, SCALE, mode, gs, bits, seqlens_k=held, max_seqlen_k=S, num_splits=2)
    got = ops.fwd_kvcache_int(qd, *caches[1], None, SCALE, gs, bits, held, S, num_splits=2, quant_mode=mode)
    assert torch.equal(got, want)
    outs = []
    for i, cache in enumerate(caches):
        win_k = torch.zeros((b, 128, h_k, 128), dtype=torch.float16, device=device)
        win_v = torch.zeros_like(win_k)
        lengths = torch.full((b,), S, dtype=torch.int32, device=device)
        if i == 0:
            outs.append(fwd_kvcache_int_append(qd, kd[:, S:], vd[:, S:], *cache, win_k, win_v, lengths, S, None, SCALE,
                                               mode, gs, bits, num_splits=2))
        else:
            outs.append(ops.fwd_kvcache_int_append(qd, kd[:, S:], vd[:, S:], *cache, win_k, win_v, lengths, S, None,
                                                   SCALE, gs, bits, 2, quant_mode=mode))
        assert lengths.tolist() == [S + 1] * b
    assert torch.equal(outs[0], outs[1])
