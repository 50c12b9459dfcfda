"""Decode step with append in one launch (`fwd_kvcache_int_append`, `BitKVCache.step`): the "residual kernel"
of the reference's figures (imgs/overview.png, imgs/scheme.png), for which its main branch has no code.
Pinned by composition: a step must equal, bit for bit, the same work done with the separately verified
entry points (store the token, `fwd_kvcache_int` over prefix + window, `kvcache_pack_int` of a full
window), and its output must match the oracle's dequantize-then-attend."""
import math

import numpy as np
import pytest
import torch

from oracle import bitdecode_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

SCALE = 1.0 / math.sqrt(128)


class _Manual:
    """The step spelled out with the plain entry points, lengths kept on the host."""

    def __init__(self, b, h_k, capacity, bits, gs, dtype, device, table=None, pool_pages=0, page=0,
                 quant_mode="k-channel"):
        self.b, self.bits, self.gs, self.device, self.table = b, bits, gs, device, table
        self.mode = quant_mode
        kt = quant_mode == "k-tensor"
        self.cache = (H.alloc_cache(pool_pages, page, h_k, bits, gs, device, k_tensor=kt) if table is not None
                      else H.alloc_cache(b, capacity, h_k, bits, gs, device, k_tensor=kt))
        self.k_res = torch.zeros((b, 128, h_k, 128), dtype=dtype, device=device)
        self.v_res = torch.zeros_like(self.k_res)
        self.capacity = capacity
        self.total = [0] * b

    def prefill(self, k, v, lengths):
        from bitladder_amd import kvcache_pack_int
        n_pack = max(lengths) // 128 * 128
        if n_pack:
            kvcache_pack_int(k[:, :n_pack], self.cache[0], self.cache[1], v[:, :n_pack], self.cache[2], self.cache[3],
                             self.table, None, n_pack, self.mode, self.gs, self.bits)
        for i, L in enumerate(lengths):
            p = L // 128 * 128
            self.k_res[i, :L - p] = k[i, p:L]
            self.v_res[i, :L - p] = v[i, p:L]
        self.total = list(lengths)

    def _i32(self, x):
        return torch.tensor(x, dtype=torch.int32, device=self.device)

    def step(self, q, k_new, v_new, ns):
        from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
        r = [t % 128 for t in self.total]
        p = [t - x for t, x in zip(self.total, r)]
        over = [x == 127 and y + 128 > self.capacity for x, y in zip(r, p)]
        k_win, v_win = self.k_res, self.v_res
        if any(over):                 # attended, not stored
            k_win, v_win = self.k_res.clone(), self.v_res.clone()
        for i in range(self.b):
            k_win[i, r[i]] = k_new[i, 0]
            v_win[i, r[i]] = v_new[i, 0]
            if not over[i] and k_win is not self.k_res:
                self.k_res[i, r[i]] = k_new[i, 0]
                self.v_res[i, r[i]] = v_new[i, 0]
        out = fwd_kvcache_int(q, *self.cache, self.table, SCALE, self.mode, self.gs, self.bits,
                              # (the host bound the step uses: the library picks the kernel variant from it)
                              seqlens_k=self._i32(p), max_seqlen_k=self.capacity, k_residual=k_win, v_residual=v_win,
                              residual_len=self._i32([x + 1 for x in r]), max_residual_len=128, num_splits=ns)
        full = [x == 127 and not o for x, o in zip(r, over)]
        if any(full):
            kvcache_pack_int(self.k_res, self.cache[0], self.cache[1], self.v_res, self.cache[2], self.cache[3],
                             self.table, None, 128, self.mode, self.gs, self.bits,
                             dst_offsets=self._i32([y if f else -1 for y, f in zip(p, full)]))
        self.total = [t if o else t + 1 for t, o in zip(self.total, over)]
        return out


def _inputs(b, h, h_k, n, dtype, device, seed):
    q, k, v = O.make_inputs(b, h, h_k, n, 0, seed=seed, dtype=dtype)
    rng = np.random.default_rng(seed + 1)
    qs = O.round_to_storage(rng.standard_normal((n, b, 1, h, 128)).astype(np.float32), dtype)
    return qs, k, v, H.to_dev(qs, dtype, device), H.to_dev(k, dtype, device), H.to_dev(v, dtype, device)


@pytest.mark.parametrize("bits,gs,dtype,ns", [(4, 128, "fp16", 2), (2, 64, "fp16", 1), (4, 32, "bf16", 3),
                                              (2, 128, "bf16", 0)])
def test_step_equals_store_decode_pack(device, bits, gs, dtype, ns):
    from bitladder_amd import BitKVCache
    b, h, h_k, steps, capacity = 3, 8, 2, 140, 640
    lengths = [120, 255, 0]
    tdt = H.torch_dtype(dtype)
    qs, k, v, qd, kd, vd = _inputs(b, h, h_k, 256 + steps, dtype, device, 17)
    cache = BitKVCache(b, h_k, capacity, num_bits=bits, group_size=gs, dtype=tdt, device=device)
    manual = _Manual(b, h_k, capacity, bits, gs, tdt, device)
    cache.prefill(kd[:, :256], vd[:, :256], lengths)
    manual.prefill(kd[:, :256], vd[:, :256], lengths)
    if ns == 0:        # the step sizes its grid for the capacity: use the same count on the other side
        from bitladder_amd import _lib
        ns_manual = _lib.lib().bitdecode_num_splits(b, h_k, capacity, 128, 0, bits, gs)
    for s in range(steps):
        t = 256 + s
        out = cache.step(qd[s], kd[:, t:t + 1], vd[:, t:t + 1], SCALE, num_splits=ns)
        want = manual.step(qd[s], kd[:, t:t + 1], vd[:, t:t + 1], ns or ns_manual)
        assert torch.equal(out, want), (s, manual.total)
    assert cache.total.tolist() == manual.total == [x + steps for x in lengths]
    assert cache.lengths == manual.total
    for got, ref in zip((cache.k_pack, cache.k_params, cache.v_pack, cache.v_params), manual.cache):
        assert torch.equal(got, ref)
    # rows of the window beyond the current length are leftovers on both sides; the live rows agree
    for i, r in enumerate(cache.res_len):
        assert torch.equal(cache.k_res[i, :r], manual.k_res[i, :r]) and torch.equal(cache.v_res[i, :r], manual.v_res[i, :r])


@pytest.mark.parametrize("bits,gs,ns", [(4, 128, 2), (4, 32, 1), (2, 128, 2)])
def test_step_with_eight_query_heads_per_kv_head(device, bits, gs, ns):
    """A full GQA group: in the 8-wave kernels every wave of the workgroup merges a head, the two that store the
    token and count the sequence included."""
    from bitladder_amd import BitKVCache
    b, h, h_k, steps, capacity = 2, 8, 1, 140, 512
    lengths = [250, 5]
    qs, k, v, qd, kd, vd = _inputs(b, h, h_k, 256 + steps, "fp16", device, 23)
    cache = BitKVCache(b, h_k, capacity, num_bits=bits, group_size=gs, dtype=torch.float16, device=device)
    manual = _Manual(b, h_k, capacity, bits, gs, torch.float16, device)
    cache.prefill(kd[:, :256], vd[:, :256], lengths)
    manual.prefill(kd[:, :256], vd[:, :256], lengths)
    for s in range(steps):
        t = 256 + s
        out = cache.step(qd[s], kd[:, t:t + 1], vd[:, t:t + 1], SCALE, num_splits=ns)
        want = manual.step(qd[s], kd[:, t:t + 1], vd[:, t:t + 1], ns)
        assert torch.equal(out, want), (s, manual.total)
    assert cache.total.tolist() == manual.total == [x + steps for x in lengths]
    for got, ref in zip((cache.k_pack, cache.k_params, cache.v_pack, cache.v_params), manual.cache):
        assert torch.equal(got, ref)


@pytest.mark.parametrize("gs,dtype,ns", [(128, "fp16", 2), (64, "bf16", 1), (32, "fp16", 3)])
def test_step_with_k_quantized_per_token(device, gs, dtype, ns):
    """quant_mode "k-tensor" through the one-launch step: the same composition, with K's parameters per token."""
    from bitladder_amd import BitKVCache
    b, h, h_k, steps, capacity, bits = 3, 8, 2, 140, 640, 4
    lengths = [120, 255, 0]
    tdt = H.torch_dtype(dtype)
    qs, k, v, qd, kd, vd = _inputs(b, h, h_k, 256 + steps, dtype, device, 31)
    cache = BitKVCache(b, h_k, capacity, num_bits=bits, group_size=gs, dtype=tdt, device=device, quant_mode="k-tensor")
    manual = _Manual(b, h_k, capacity, bits, gs, tdt, device, quant_mode="k-tensor")
    cache.prefill(kd[:, :256], vd[:, :256], lengths)
    manual.prefill(kd[:, :256], vd[:, :256], lengths)
    for s in range(steps):
        t = 256 + s
        out = cache.step(qd[s], kd[:, t:t + 1], vd[:, t:t + 1], SCALE, num_splits=ns)
        want = manual.step(qd[s], kd[:, t:t + 1], vd[:, t:t + 1], ns)
        assert torch.equal(out, want), (s, manual.total)
    assert cache.total.tolist() == manual.total == [x + steps for x in lengths]
    for got, ref in zip((cache.k_pack, cache.k_params, cache.v_pack, cache.v_params), manual.cache):
        assert torch.equal(got, ref)


@pytest.mark.parametrize("mode", ["k-channel", "k-tensor"])
def test_step_output_and_packed_window_match_the_oracle(device, mode):
    """The step that fills the window: 128 tokens attended in fp16 behind a quantized prefix, and the chunk it
    leaves in the cache is the oracle's quantization of those 128 tokens."""
    from bitladder_amd import fwd_kvcache_int_append, kvcache_pack_int
    b, h, h_k, bits, gs, S = 2, 8, 2, 4, 128, 256
    q, k, v = O.make_inputs(b, h, h_k, S + 128, 0, seed=29)
    qd, kd, vd = H.to_dev(q, "fp16", device), H.to_dev(k, "fp16", device), H.to_dev(v, "fp16", device)
    cache = H.alloc_cache(b, S + 128, h_k, bits, gs, device, k_tensor=mode == "k-tensor")
    kvcache_pack_int(kd[:, :S], cache[0], cache[1], vd[:, :S], cache[2], cache[3], None, None, S, mode, gs, bits)
    k_res = kd[:, S:S + 128].clone()
    v_res = vd[:, S:S + 128].clone()
    k_res[:, 127] = 0          # the last row arrives as the new token
    v_res[:, 127] = 0
    lengths = torch.full((b,), S + 127, dtype=torch.int32, device=device)
    out, lse = fwd_kvcache_int_append(qd, kd[:, S + 127:], vd[:, S + 127:], *cache, k_res, v_res, lengths, S + 127,
                                      None, SCALE, mode, gs, bits, return_lse=True)
    torch.cuda.synchronize()
    assert lengths.tolist() == [S + 128] * b
    assert torch.equal(k_res, kd[:, S:S + 128]) and torch.equal(v_res, vd[:, S:S + 128])
    qkv = O.quantize_kv_ref(k[:, :S], v[:, :S], bits, gs, quant_mode=mode)
    k_hat, v_hat = O.dequantize_ref(qkv)
    ref, ref_lse = O.attend_ref(q, k_hat, v_hat, SCALE, k[:, S:], v[:, S:])
    assert np.abs(out.float().cpu().numpy() - ref).max() < 2e-3
    assert np.abs(lse.cpu().numpy() - ref_lse).max() < 2e-3
    H.assert_cache_equals_oracle(H.cache_to_numpy(*cache), O.quantize_kv_ref(k, v, bits, gs, quant_mode=mode))


def test_step_leaves_a_full_sequence_unchanged(device):
    from bitladder_amd import BitKVCache
    b, h, h_k, capacity = 2, 4, 1, 256
    qs, k, v, qd, kd, vd = _inputs(b, h, h_k, 400, "fp16", device, 3)
    cache = BitKVCache(b, h_k, capacity, device=device)
    manual = _Manual(b, h_k, capacity, 4, 128, torch.float16, device)
    lengths = [capacity + 127, 100]          # sequence 0: packed to capacity and 127 tokens in its window
    # (a state only the plain entry points reach: BitKVCache itself stops at `capacity` tokens)
    from bitladder_amd import kvcache_pack_int
    kvcache_pack_int(kd[:, :256], manual.cache[0], manual.cache[1], vd[:, :256], manual.cache[2], manual.cache[3],
                     None, None, 256, "k-channel", 128, 4)       # sequence 1 ignores its share: it has no packed tokens
    manual.k_res[0, :127], manual.v_res[0, :127] = kd[0, 256:383], vd[0, 256:383]
    manual.k_res[1, :100], manual.v_res[1, :100] = kd[1, :100], vd[1, :100]
    manual.total = list(lengths)
    for dst, src in zip((cache.k_pack, cache.k_params, cache.v_pack, cache.v_params, cache.k_res, cache.v_res),
                        manual.cache + (manual.k_res, manual.v_res)):
        dst.copy_(src)
    cache.total.copy_(torch.tensor(lengths, dtype=torch.int32))
    before = [t.clone() for t in (cache.k_pack, cache.k_params, cache.v_pack, cache.v_params)]
    win0 = cache.k_res[0].clone()
    plan = cache.plan_step(qd[0], kd[:, 390:391], vd[:, 390:391], SCALE, num_splits=2)
    out = plan.run()
    want = manual.step(qd[0], kd[:, 390:391], vd[:, 390:391], 2)
    assert torch.equal(out, want)
    assert cache.total.tolist() == [capacity + 127, 101] == manual.total
    assert torch.equal(cache.k_res[0], win0)
    assert torch.equal(cache.k_res[1, 100], kd[1, 390])
    for got, ref in zip((cache.k_pack, cache.k_params, cache.v_pack, cache.v_params), before):
        assert torch.equal(got, ref)


def test_step_plan_replays_in_a_hip_graph(device):
    """One captured step, replayed token after token across a window that fills: lengths live on the device,
    so the replay needs no host work beyond refreshing the three input tensors."""
    from bitladder_amd import BitKVCache
    b, h, h_k, steps, capacity = 2, 8, 2, 40, 512
    lengths = [100, 230]
    qs, k, v, qd, kd, vd = _inputs(b, h, h_k, 256 + steps, "fp16", device, 41)
    eager = BitKVCache(b, h_k, capacity, device=device)
    graphed = BitKVCache(b, h_k, capacity, device=device)
    eager.prefill(kd[:, :256], vd[:, :256], lengths)
    graphed.prefill(kd[:, :256], vd[:, :256], lengths)
    q_in = torch.zeros_like(qd[0])
    k_in = torch.zeros_like(kd[:, :1])
    v_in = torch.zeros_like(k_in)
    out_buf = torch.zeros_like(q_in)
    plan = graphed.plan_step(q_in, k_in, v_in, SCALE, out=out_buf)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        # capture records the launch without running it: the cache does not advance here
        with torch.cuda.graph(graph, stream=side):
            plan.run()
    torch.cuda.synchronize()
    assert graphed.total.tolist() == lengths
    for s in range(steps):
        t = 256 + s
        q_in.copy_(qd[s])
        k_in.copy_(kd[:, t:t + 1])
        v_in.copy_(vd[:, t:t + 1])
        graph.replay()
        want = eager.step(qd[s], kd[:, t:t + 1], vd[:, t:t + 1], SCALE, num_splits=plan.num_splits)
        assert torch.equal(out_buf, want), s
    graphed.sync_lengths()
    assert graphed.lengths == eager.lengths == [x + steps for x in lengths]
    for got, ref in zip((graphed.k_pack, graphed.k_params, graphed.v_pack, graphed.v_params),
                        (eager.k_pack, eager.k_params, eager.v_pack, eager.v_params)):
        assert torch.equal(got, ref)


def test_step_into_a_paged_cache(device):
    from bitladder_amd import fwd_kvcache_int_append
    b, h, h_k, bits, gs, page, pages_per_seq, num_pages, steps = 2, 8, 2, 4, 128, 256, 3, 8, 150
    lengths = [250, 3]
    qs, k, v, qd, kd, vd = _inputs(b, h, h_k, 256 + steps, "fp16", device, 57)
    table = torch.tensor([[6, 1, 4], [0, 7, 2]], dtype=torch.int32, device=device)
    paged = _Manual(b, h_k, page * pages_per_seq, bits, gs, torch.float16, device, table, num_pages, page)
    flat = _Manual(b, h_k, page * pages_per_seq, bits, gs, torch.float16, device)
    paged.prefill(kd[:, :256], vd[:, :256], lengths)
    flat.prefill(kd[:, :256], vd[:, :256], lengths)
    len_p = torch.tensor(lengths, dtype=torch.int32, device=device)
    len_f = len_p.clone()
    for s in range(steps):
        t = 256 + s
        args = (qd[s], kd[:, t:t + 1], vd[:, t:t + 1])
        out_p = fwd_kvcache_int_append(*args, *paged.cache, paged.k_res, paged.v_res, len_p, 256 + s, table, SCALE,
                                       "k-channel", gs, bits, num_splits=2)
        out_f = fwd_kvcache_int_append(*args, *flat.cache, flat.k_res, flat.v_res, len_f, 256 + s, None, SCALE,
                                       "k-channel", gs, bits, num_splits=2)
        assert torch.equal(out_p, out_f), s
    assert len_p.tolist() == len_f.tolist() == [x + steps for x in lengths]
    for f, p in zip(flat.cache, paged.cache):
        fb = f.contiguous().view(torch.uint8).reshape(b, h_k, pages_per_seq, -1)
        pb = p.contiguous().view(torch.uint8).reshape(num_pages, h_k, -1)
        for i in range(b):
            for j in range((lengths[i] + steps) // page):
                assert torch.equal(pb[int(table[i, j])], fb[i, :, j]), (i, j)


def test_step_arguments_are_validated(device):
    from bitladder_amd import fwd_kvcache_int_append
    b, h, h_k = 2, 4, 2
    cache = H.alloc_cache(b, 256, h_k, 4, 128, device)
    q = torch.zeros((b, 1, h, 128), dtype=torch.float16, device=device)
    kn = torch.zeros((b, 1, h_k, 128), dtype=torch.float16, device=device)
    win = torch.zeros((b, 128, h_k, 128), dtype=torch.float16, device=device)
    lengths = torch.zeros(b, dtype=torch.int32, device=device)
    with pytest.raises(RuntimeError):        # window too small
        fwd_kvcache_int_append(q, kn, kn, *cache, win[:, :64], win[:, :64], lengths, 0)
    with pytest.raises(RuntimeError):        # lengths on the host
        fwd_kvcache_int_append(q, kn, kn, *cache, win, win, lengths.cpu(), 0)
    with pytest.raises(RuntimeError):        # new token of the wrong shape
        fwd_kvcache_int_append(q, kn[:, :, :1], kn, *cache, win, win, lengths, 0)
    with pytest.raises(RuntimeError):        # more tokens than the cache can hold
        fwd_kvcache_int_append(q, kn, kn, *cache, win, win, lengths, 1024)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("bits,gs", [(4, 128), (4, 64), (4, 32), (2, 128), (2, 64), (2, 32)])
def test_step_packs_exactly_what_the_pack_kernel_packs(device, bits, gs, dtype):
    """64 windows filled by one step: every byte of the chunks it writes equals the pack kernel's (whose codes and
    parameters are pinned against the oracle), rounding ties included."""
    from bitladder_amd import fwd_kvcache_int_append, kvcache_pack_int
    b, h, h_k = 16, 4, 4
    q, k, v = O.make_inputs(b, h, h_k, 128, 0, seed=71, dtype=dtype)
    k = O.round_to_storage(k * np.float32(0.37), dtype)           # off the grid of exactly representable ratios
    qd, kd, vd = H.to_dev(q, dtype, device), H.to_dev(k, dtype, device), H.to_dev(v, dtype, device)
    want = H.alloc_cache(b, 128, h_k, bits, gs, device)
    kvcache_pack_int(kd, want[0], want[1], vd, want[2], want[3], None, None, 128, "k-channel", gs, bits)
    got = H.alloc_cache(b, 128, h_k, bits, gs, device)
    k_res, v_res = kd.clone(), vd.clone()
    k_res[:, 127] = 0
    v_res[:, 127] = 0
    lengths = torch.full((b,), 127, dtype=torch.int32, device=device)
    fwd_kvcache_int_append(qd, kd[:, 127:], vd[:, 127:], *got, k_res, v_res, lengths, 127, None, SCALE, "k-channel",
                           gs, bits)
    assert lengths.tolist() == [128] * b
    for g_, w_ in zip(got, want):
        assert torch.equal(g_, w_)



def test_step_on_a_ragged_batch_of_sixteen(device):
    """The batch shape of the reference's batched driver (csrc/bit_decode/src/test_batch_packdecode.cu: 16
    sequences, 32 query / 8 kv heads) with ragged lengths: 128 workgroup groups share the XCD-aware block
    mapping, every sequence has eight ticket holders, and windows fill at different steps."""
    from bitladder_amd import BitKVCache
    b, h, h_k, steps, capacity = 16, 32, 8, 135, 2048 + 256
    rng = np.random.default_rng(4)
    lengths = [int(x) for x in rng.integers(1024, 2049, b)]
    qs, k, v, qd, kd, vd = _inputs(b, h, h_k, 2048 + steps, "fp16", device, 77)
    cache = BitKVCache(b, h_k, capacity, device=device)
    manual = _Manual(b, h_k, capacity, 4, 128, torch.float16, device)
    cache.prefill(kd[:, :2048], vd[:, :2048], lengths)
    manual.prefill(kd[:, :2048], vd[:, :2048], lengths)
    for s in range(steps):
        t = 2048 + s
        out = cache.step(qd[s], kd[:, t:t + 1], vd[:, t:t + 1], SCALE, num_splits=2)
        want = manual.step(qd[s], kd[:, t:t + 1], vd[:, t:t + 1], 2)
        assert torch.equal(out, want), s
    assert cache.total.tolist() == manual.total == [x + steps for x in lengths]
    for got, ref in zip((cache.k_pack, cache.k_params, cache.v_pack, cache.v_params), manual.cache):
        assert torch.equal(got, ref)       # (both sides started from the same prefill call)
    # the fused path against the oracle on the full history of one sequence
    i = int(np.argmax(lengths))
    L = lengths[i] + steps
    hist_k = np.concatenate([k[i, :lengths[i]], k[i, 2048:2048 + steps]], 0)
    hist_v = np.concatenate([v[i, :lengths[i]], v[i, 2048:2048 + steps]], 0)
    P = (L - 1) // 128 * 128
    qkv = O.quantize_kv_ref(hist_k[None, :P], hist_v[None, :P], 4, 128)
    k_hat, v_hat = O.dequantize_ref(qkv)
    ref, _ = O.attend_ref(qs[steps - 1][i:i + 1], k_hat, v_hat, SCALE, hist_k[None, P:], hist_v[None, P:])
    assert np.abs(out[i:i + 1].float().cpu().numpy() - ref).max() < 2e-3
