"""Workspaces and streams: the plain entry point takes its split workspace from a per-stream cache
(nothing is allocated or filled after the first call), two streams never share one, and calls whose
workspaces differ may overlap in time without changing a bit of their results."""
import math

import numpy as np
import pytest
import torch

from oracle import bitdecode_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

SCALE = 1.0 / math.sqrt(128)


def _problem(device, seed, b=1, h=8, h_k=2, S=4096, R=128, bits=4, gs=128):
    from bitladder_amd import kvcache_pack_int
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=seed)
    kd, vd = H.to_dev(k, "fp16", device), H.to_dev(v, "fp16", device)
    cache = H.alloc_cache(b, S, h_k, bits, gs, device)
    kvcache_pack_int(kd[:, :S], cache[0], cache[1], vd[:, :S], cache[2], cache[3], None, None, S, "k-channel", gs, bits)
    return H.to_dev(q, "fp16", device), cache, kd[:, S:].contiguous(), vd[:, S:].contiguous(), (q, k, v)


def test_dropin_call_reuses_a_per_stream_workspace(device):
    from bitladder_amd import fwd_kvcache_int, interface, plan_fwd_kvcache_int
    q, cache, kr, vr, host = _problem(device, 11)
    ns = 16
    kw = dict(k_residual=kr, v_residual=vr, num_splits=ns)
    plan = plan_fwd_kvcache_int(q, *cache, None, SCALE, "k-channel", 128, 4, **kw)
    want = plan.run().clone()
    torch.cuda.synchronize()

    interface._WORKSPACES.clear()
    out1 = fwd_kvcache_int(q, *cache, None, SCALE, "k-channel", 128, 4, **kw)
    assert len(interface._WORKSPACES) == 1
    (key0, ws0), = interface._WORKSPACES.items()
    torch.cuda.synchronize()
    allocated = torch.cuda.memory_allocated(device)
    out_buf = torch.empty_like(q)
    for _ in range(5):
        out2 = fwd_kvcache_int(q, *cache, None, SCALE, "k-channel", 128, 4, out=out_buf, **kw)
        assert torch.equal(out2, want)
    torch.cuda.synchronize()
    # same buffer, nothing new allocated (the output buffer was passed in)
    assert len(interface._WORKSPACES) == 1 and interface._WORKSPACES[key0] is ws0
    assert torch.cuda.memory_allocated(device) == allocated + out_buf.numel() * 2
    assert torch.equal(out1, want)
    # the arrival counters are back at zero after every call: one 256-byte block per query head
    counters = ws0[:256 * q.shape[0] * q.shape[2]].view(torch.int32)
    assert int(counters.abs().sum()) == 0

    # another stream gets another workspace; another split count as well
    side = torch.cuda.Stream(device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        out3 = fwd_kvcache_int(q, *cache, None, SCALE, "k-channel", 128, 4, **kw)
    side.synchronize()
    assert len(interface._WORKSPACES) == 2
    ptrs = {ws.data_ptr() for ws in interface._WORKSPACES.values()}
    assert len(ptrs) == 2
    assert torch.equal(out3, want)
    fwd_kvcache_int(q, *cache, None, SCALE, "k-channel", 128, 4, k_residual=kr, v_residual=vr, num_splits=8)
    assert len(interface._WORKSPACES) == 3

    # and the result is the oracle's
    qn, kn, vn = host
    qkv = O.quantize_kv_ref(kn[:, :4096], vn[:, :4096], 4, 128)
    k_hat, v_hat = O.dequantize_ref(qkv)
    ref, _ = O.attend_ref(qn, k_hat, v_hat, SCALE, kn[:, 4096:], vn[:, 4096:])
    assert np.abs(want.float().cpu().numpy() - ref).max() < 2e-3


def test_dropin_call_finds_its_argument_block_again(device):
    """The plain call keeps the validated argument block of its last few distinct calls.  What must hold: every
    call returns a tensor of its own, new contents of the same tensors give new results, a call that differs in
    any tensor's address, strides or type is another call, and nothing keeps the caller's tensors alive."""
    import gc
    import weakref
    from bitladder_amd import fwd_kvcache_int, interface, plan_fwd_kvcache_int
    q, cache, kr, vr, host = _problem(device, 13)
    kw = dict(k_residual=kr, v_residual=vr, num_splits=8)
    args = (None, SCALE, "k-channel", 128, 4)
    interface._plan_cache().clear()
    want = plan_fwd_kvcache_int(q, *cache, *args, **kw).run().clone()
    outs = [fwd_kvcache_int(q, *cache, *args, **kw) for _ in range(4)]
    assert len(interface._plan_cache()) == 1
    assert len({o.data_ptr() for o in outs}) == 4 and all(torch.equal(o, want) for o in outs)
    # the same tensors with new contents
    q2 = torch.randn_like(q)
    want2 = plan_fwd_kvcache_int(q2, *cache, *args, **kw).run().clone()
    q.copy_(q2)
    out2, lse2 = fwd_kvcache_int(q, *cache, *args, return_lse=True, **kw)          # another call: it returns the LSE
    out3, lse3 = fwd_kvcache_int(q, *cache, *args, return_lse=True, **kw)          # found again
    assert torch.equal(out2, want2) and torch.equal(out3, want2) and torch.equal(lse2, lse3)
    assert lse2.data_ptr() != lse3.data_ptr() and not torch.equal(outs[0], want2)
    # a strided q of the same contents, and a caller-given output
    wide = torch.zeros((q.shape[0], 1, q.shape[2], 256), dtype=q.dtype, device=device)
    wide[..., :128] = q
    given = torch.empty_like(q)
    n = len(interface._plan_cache())
    assert fwd_kvcache_int(wide[..., :128], *cache, *args, out=given, **kw) is given and torch.equal(given, want2)
    assert len(interface._plan_cache()) == n + 1
    # an invalid call is still rejected although a valid one over the same cache is held
    with pytest.raises(RuntimeError):
        fwd_kvcache_int(q[:, :, :3], *cache, *args, **kw)
    # the held argument blocks do not hold the caller's tensors
    ref = weakref.ref(kr)
    del kr, kw, outs
    gc.collect()
    assert ref() is None


def test_dropin_calls_of_a_whole_model_keep_their_argument_blocks(device):
    """A decode loop makes one call per attention layer and token, each over that layer's cache: the calls of
    all layers of a deep model are kept side by side, so the second token's calls find theirs again."""
    from bitladder_amd import fwd_kvcache_int, interface, plan_fwd_kvcache_int
    layers = 80
    q, cache0, kr, vr, _ = _problem(device, 17, S=256)
    caches = [cache0] + [tuple(t.clone() for t in cache0) for _ in range(layers - 1)]
    for i, c in enumerate(caches):
        c[1].view(torch.float16)[..., :128].mul_(1.0 + i / 64.0)      # each layer its own K scales
    args = (None, SCALE, "k-channel", 128, 4)
    kw = dict(k_residual=kr, v_residual=vr, num_splits=2)
    wants = [plan_fwd_kvcache_int(q, *c, *args, **kw).run().clone() for c in caches]
    assert not torch.equal(wants[0], wants[1])
    interface._plan_cache().clear()
    for token in range(3):
        for c, want in zip(caches, wants):
            assert torch.equal(fwd_kvcache_int(q, *c, *args, **kw), want)
        assert len(interface._plan_cache()) == layers


def test_two_plans_on_two_streams_overlap_without_changing_a_bit(device):
    """Two plans (different problems, a workspace each) replayed many times on two streams at once give,
    every time, the bits they give when run alone."""
    from bitladder_amd import plan_fwd_kvcache_int
    probs = [_problem(device, 21, h=8, h_k=2, S=8192), _problem(device, 22, h=8, h_k=1, S=4096, bits=2, gs=64)]
    plans, wants = [], []
    for (q, cache, kr, vr, _), (bits, gs, ns) in zip(probs, [(4, 128, 24), (2, 64, 32)]):
        plan = plan_fwd_kvcache_int(q, *cache, None, SCALE, "k-channel", gs, bits, k_residual=kr, v_residual=vr,
                                    num_splits=ns, out=torch.empty_like(q))
        plans.append(plan)
        wants.append(plan.run().clone())
    torch.cuda.synchronize()
    assert plans[0].args.workspace != plans[1].args.workspace
    streams = [torch.cuda.Stream(device), torch.cuda.Stream(device)]
    outs = [[], []]
    for s in streams:
        s.wait_stream(torch.cuda.current_stream(device))
    for rep in range(40):
        for i in (0, 1):
            with torch.cuda.stream(streams[i]):
                plans[i].run()
                if rep % 8 == 7:
                    outs[i].append(plans[i].out.clone())
    for s in streams:
        s.synchronize()
    for i in (0, 1):
        assert len(outs[i]) == 5
        for o in outs[i]:
            assert torch.equal(o, wants[i])
