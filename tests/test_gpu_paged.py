"""Paged KV cache (opt_block_table): pools of pages addressed through a block table, as in the reference
(csrc/bit_decode/decode_api.cpp:328-352; test recipe csrc/bit_decode/src/test_batch_packdecode.cu:16-79:
random permutation of the pool's pages dealt to the sequences).  A paged cache must hold, page by page, the
bytes a contiguous cache holds, and decode to bit-identical results."""
import math

import numpy as np
import pytest
import torch

from oracle import bitdecode_oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

SCALE = 1.0 / math.sqrt(128)


def _pool(num_pages, page, h_k, bits, gs, device):
    return H.alloc_cache(num_pages, page, h_k, bits, gs, device, fill=0x5A5A)


def _where(got, want):
    """Which (sequence, head) rows differ, and by how much: for the message of a failed comparison."""
    d = (got.float() - want.float()).abs().amax(dim=(1, 3))
    return [(int(i), int(j), float(d[i, j])) for i, j in torch.nonzero(d)]


def _region_bytes(t, regions):
    """Flat bytes of a cache tensor, one row per (batch-or-page, kv-head) region."""
    return t.contiguous().view(torch.uint8).reshape(regions, -1)


@pytest.mark.parametrize("bits,gs,page", [(4, 128, 256), (2, 64, 512), (4, 32, 128)])
def test_paged_pack_and_decode_equal_contiguous(device, bits, gs, page):
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    b, h, h_k, S, R = 3, 8, 2, 2048, 40
    pages_per_seq = S // page
    num_pages = b * pages_per_seq + 5                     # a few pages of the pool stay unused
    q, k, v = O.make_inputs(b, h, h_k, S, R, seed=61)
    kd, vd, qd = H.to_dev(k, "fp16", device), H.to_dev(v, "fp16", device), H.to_dev(q, "fp16", device)
    g = torch.Generator().manual_seed(3)
    table = torch.randperm(num_pages, generator=g)[:b * pages_per_seq].to(torch.int32).reshape(b, pages_per_seq)
    table = table.to(device)

    flat = H.alloc_cache(b, S, h_k, bits, gs, device)
    kvcache_pack_int(kd[:, :S], flat[0], flat[1], vd[:, :S], flat[2], flat[3], None, None, S, "k-channel", gs, bits)
    pool = _pool(num_pages, page, h_k, bits, gs, device)
    kvcache_pack_int(kd[:, :S], pool[0], pool[1], vd[:, :S], pool[2], pool[3], table, None, S, "k-channel", gs, bits)
    torch.cuda.synchronize()

    # page table[i, j] of the pool holds tokens [j*page, (j+1)*page) of sequence i: same bytes as the
    # matching slice of the contiguous cache's region
    for f, p in zip(flat, pool):
        fb = _region_bytes(f, b * h_k).reshape(b, h_k, pages_per_seq, -1)
        pb = _region_bytes(p, num_pages * h_k).reshape(num_pages, h_k, -1)
        for i in range(b):
            for j in range(pages_per_seq):
                assert torch.equal(pb[int(table[i, j])], fb[i, :, j]), (i, j)

    kw = dict(k_residual=kd[:, S:], v_residual=vd[:, S:])
    seqlens = torch.tensor([S, S - 3 * 128, 640], dtype=torch.int32, device=device)
    for ns in (0, 1, 3):
        want = fwd_kvcache_int(qd, *flat, None, SCALE, "k-channel", gs, bits, num_splits=ns, **kw)
        got = fwd_kvcache_int(qd, *pool, table, SCALE, "k-channel", gs, bits, num_splits=ns, **kw)
        assert torch.equal(got, want), ns
        want = fwd_kvcache_int(qd, *flat, None, SCALE, "k-channel", gs, bits, num_splits=ns, seqlens_k=seqlens,
                               max_seqlen_k=S, **kw)
        got = fwd_kvcache_int(qd, *pool, table, SCALE, "k-channel", gs, bits, num_splits=ns, seqlens_k=seqlens,
                              max_seqlen_k=S, **kw)
        assert torch.equal(got, want), (ns, _where(got, want))
    # and the paged result is right, not merely equal
    qkv = O.quantize_kv_ref(k[:, :S], v[:, :S], bits, gs)
    k_hat, v_hat = O.dequantize_ref(qkv)
    ref, _ = O.attend_ref(q, k_hat, v_hat, SCALE, k[:, S:], v[:, S:])
    out = fwd_kvcache_int(qd, *pool, table, SCALE, "k-channel", gs, bits, **kw)
    assert np.abs(out.float().cpu().numpy() - ref).max() < 2e-3


def test_paged_append_with_per_sequence_offsets(device):
    """Append one block per sequence into a paged cache at different positions (dst_offsets), one sequence
    skipped; pages named by the table receive the data, all other pages keep their fill pattern."""
    from bitladder_amd import kvcache_pack_int
    b, h_k, page, bits, gs = 3, 2, 256, 4, 128
    pages_per_seq, num_pages = 4, 16
    _, k, v = O.make_inputs(b, h_k, h_k, 128, 0, seed=8)
    kd, vd = H.to_dev(k, "fp16", device), H.to_dev(v, "fp16", device)
    table = torch.tensor([[3, 9, 1, 12], [7, 0, 15, 4], [5, 6, 2, 8]], dtype=torch.int32, device=device)
    offsets = torch.tensor([384, -1, 0], dtype=torch.int32, device=device)       # page slot 1 (2nd half), skip, slot 0
    pool = _pool(num_pages, page, h_k, bits, gs, device)
    before = [p.clone() for p in pool]
    kvcache_pack_int(kd, pool[0], pool[1], vd, pool[2], pool[3], table, None, 128, "k-channel", gs, bits,
                     dst_offsets=offsets)
    one = H.alloc_cache(b, 128, h_k, bits, gs, device)
    kvcache_pack_int(kd, one[0], one[1], vd, one[2], one[3], None, None, 128, "k-channel", gs, bits)
    torch.cuda.synchronize()
    touched = {9: (0, 1), 5: (2, 0)}                      # page -> (sequence, chunk inside the page)
    for p, bf, o in zip(pool, before, one):
        pb = _region_bytes(p, num_pages * h_k).reshape(num_pages, h_k, 2, -1)      # two chunks per page
        bb = _region_bytes(bf, num_pages * h_k).reshape(num_pages, h_k, 2, -1)
        ob = _region_bytes(o, b * h_k).reshape(b, h_k, -1)
        for page_id in range(num_pages):
            for c in range(2):
                if page_id in touched and touched[page_id][1] == c:
                    assert torch.equal(pb[page_id, :, c], ob[touched[page_id][0]]), (page_id, c)
                else:
                    assert torch.equal(pb[page_id, :, c], bb[page_id, :, c]), (page_id, c)


def test_paged_arguments_are_validated(device):
    from bitladder_amd import fwd_kvcache_int
    from bitladder_amd._lib import BitDecodeError
    b, h, h_k, page = 2, 4, 2, 256
    pool = _pool(4, page, h_k, 4, 128, device)
    q = torch.zeros((b, 1, h, 128), dtype=torch.float16, device=device)
    table = torch.zeros((b, 2), dtype=torch.int32, device=device)
    with pytest.raises(RuntimeError):
        fwd_kvcache_int(q, *pool, table.to(torch.int64))
    with pytest.raises(RuntimeError):
        fwd_kvcache_int(q, *pool, table[:1])
    with pytest.raises(BitDecodeError):       # 3 pages' worth of tokens with a 2-column table
        fwd_kvcache_int(q, *pool, table, seqlen_k=3 * page)
