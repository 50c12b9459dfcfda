"""bitdecode_fwd_static: the decode entry point that allocates nothing (partial outputs and counters in a
device array inside the library).  Called through the C ABI and compared, bit for bit, with bitdecode_fwd
on two calls in a row, the second with a smaller input, and once more with the first."""
import copy
import ctypes
import math

import pytest
import torch

from oracle import bitdecode_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

SCALE = 1.0 / math.sqrt(128)


def _plan(device, seed, b, h, h_k, S, R, bits, gs, ns):
    from bitladder_amd import kvcache_pack_int, plan_fwd_kvcache_int
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=seed)
    kd, vd = H.to_dev(k, "fp16", device), H.to_dev(v, "fp16", device)
    cache = H.alloc_cache(b, S, h_k, bits, gs, device)
    kvcache_pack_int(kd[:, :S], cache[0], cache[1], vd[:, :S], cache[2], cache[3], None, None, S, "k-channel", gs, bits)
    return plan_fwd_kvcache_int(H.to_dev(q, "fp16", device), *cache, None, SCALE, "k-channel", gs, bits,
                                k_residual=kd[:, S:].contiguous(), v_residual=vd[:, S:].contiguous(),
                                num_splits=ns, return_lse=True)


def _run_static(plan, device, out=None, lse=None):
    """The plan's argument block with no workspace and fresh (or the given) outputs, through
    bitdecode_fwd_static on the current stream."""
    from bitladder_amd import _lib
    L = _lib.lib()
    a = _lib.FwdArgs()
    ctypes.memmove(ctypes.byref(a), ctypes.byref(plan.args), ctypes.sizeof(a))
    if out is None:
        out = torch.full_like(plan.out, float("nan"))
        lse = torch.full_like(plan.lse, float("nan"))
    a.out, a.softmax_lse = out.data_ptr(), lse.data_ptr()
    a.workspace, a.workspace_bytes = None, 0
    rc = L.bitdecode_fwd_static(ctypes.byref(a), torch.cuda.current_stream(device).cuda_stream)
    assert rc == 0, L.bitdecode_last_error()
    return out, lse


def test_static_scratch_entry_matches_the_workspace_entry(device):
    from bitladder_amd import _lib
    big = _plan(device, 31, 1, 32, 8, 8192, 128, 4, 128, 0)        # 32 splits of 8 kv heads
    small = _plan(device, 32, 2, 8, 2, 1024, 40, 2, 64, 5)         # fewer rows, fewer splits: other layout in the scratch
    single = _plan(device, 33, 1, 4, 4, 256, 0, 4, 32, 1)          # one split: no scratch at all
    assert big.num_splits > 1
    want = {}
    for name, plan in (("big", big), ("small", small), ("single", single)):
        plan.run()
        want[name] = (plan.out.clone(), plan.lse.clone())
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(device)
    for name, plan in (("big", big), ("small", small), ("big", big), ("single", single), ("small", small)):
        out, lse = _run_static(plan, device)
        torch.cuda.synchronize()
        assert torch.equal(out, want[name][0]), name
        assert torch.equal(lse, want[name][1]), name
        del out, lse
    assert torch.cuda.memory_allocated(device) == before

    # The allocator of torch does not see a hipMalloc made inside the library: the device's free memory does.
    # Outputs are allocated up front; after one warm-up call (the library looks the scratch address up once per
    # device) a run of calls, one of them on a side stream, leaves the free memory of the device where it was.
    outs = {name: (torch.full_like(plan.out, float("nan")), torch.full_like(plan.lse, float("nan")))
            for name, plan in (("big", big), ("small", small))}
    side = torch.cuda.Stream(device)
    _run_static(big, device, *outs["big"])
    with torch.cuda.stream(side):      # the runtime sets a stream's queue up at its first launch: not the library's doing
        _run_static(small, device, *outs["small"])
    side.synchronize()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(device)
    for rep in range(6):
        for name, plan in (("big", big), ("small", small)):
            _run_static(plan, device, *outs[name])
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        _run_static(small, device, *outs["small"])
    side.synchronize()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(device)
    assert free_after == free_before, (free_before, free_after)
    for name in outs:
        assert torch.equal(outs[name][0], want[name][0]) and torch.equal(outs[name][1], want[name][1]), name

    # beyond the built-in scratch: a clear error, nothing launched
    L = _lib.lib()
    wide = _plan(device, 34, 2, 32, 8, 8192, 128, 4, 128, 0)
    a = _lib.FwdArgs()
    ctypes.memmove(ctypes.byref(a), ctypes.byref(wide.args), ctypes.sizeof(a))
    a.num_splits = 512                                             # 512 x 64 rows x 264 B = 8.65 MB > 7 MiB
    rc = L.bitdecode_fwd_static(ctypes.byref(a), torch.cuda.current_stream(device).cuda_stream)
    assert rc == 3 and b"built-in scratch" in L.bitdecode_last_error()
