"""CPU tests: physical layout description, C-ABI exports and host-side argument checks.
No GPU compute is issued: every C-ABI call made here fails validation before any launch."""
import ctypes
import os
import re

import numpy as np
import pytest

from bitladder_amd import _lib
from bitladder_amd import layout as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("bits", [2, 4])
@pytest.mark.parametrize("gs", [32, 64, 128])
def test_layout_roundtrip_and_byte_budget(bits, gs):
    rng = np.random.default_rng(bits * 1000 + gs)
    b, S, h = 2, 256, 3
    kc = rng.integers(0, 1 << bits, (b, S, h, 128), dtype=np.uint8)
    vc = rng.integers(0, 1 << bits, (b, S, h, 128), dtype=np.uint8)
    ks = rng.integers(0, 65536, (b, S // gs, h, 128)).astype(np.uint16)
    kz = rng.integers(0, 65536, (b, S // gs, h, 128)).astype(np.uint16)
    vs = rng.integers(0, 65536, (b, S, h, 128 // gs)).astype(np.uint16)
    vz = rng.integers(0, 65536, (b, S, h, 128 // gs)).astype(np.uint16)
    phys = L.pack_physical(kc, ks, kz, vc, vs, vz, bits, gs)
    pn = 16 // bits
    # the reference's tensor contract (evaluation/test.py:76-83)
    assert phys[0].shape == (b, S // pn, h, 128) and phys[0].dtype == np.uint16
    assert phys[1].shape == (b, S // gs, h, 128) and phys[1].dtype == np.float32
    assert phys[2].shape == (b, S, h, 128 // pn) and phys[2].dtype == np.uint16
    assert phys[3].shape == (b, 128 // gs, h, S) and phys[3].dtype == np.float32
    back = L.unpack_physical(*phys, bits, gs)
    for a, c in zip((kc, ks, kz, vc, vs, vz), back):
        np.testing.assert_array_equal(a, c)


@pytest.mark.parametrize("gs", [32, 64, 128])
def test_ktensor_layout_roundtrip(gs):
    """"k-tensor" mode: K parameters per token and channel group, k_params with v_params' shape."""
    rng = np.random.default_rng(gs)
    b, S, h, bits, ncg = 2, 256, 3, 4, 128 // gs
    kc = rng.integers(0, 16, (b, S, h, 128), dtype=np.uint8)
    vc = rng.integers(0, 16, (b, S, h, 128), dtype=np.uint8)
    par = [rng.integers(0, 65536, (b, S, h, ncg)).astype(np.uint16) for _ in range(4)]
    phys = L.pack_physical(kc, par[0], par[1], vc, par[2], par[3], bits, gs, "fp16", "k-tensor")
    assert phys[1].shape == phys[3].shape == (b, ncg, h, S)
    back = L.unpack_physical(*phys, bits, gs, "fp16", "k-tensor")
    for a, c in zip((kc, par[0], par[1], vc, par[2], par[3]), back):
        np.testing.assert_array_equal(a, c)
    # the (scale, zero) pair of token n, group g sits at [half][g][tile][token] of its chunk
    raw = np.ascontiguousarray(phys[1]).reshape(-1).view(np.uint16).reshape(b, h, S // 128, 2, ncg, 4, 16, 2)
    n, g = 128 + 64 + 16 * 2 + 5, ncg - 1
    assert raw[1, 2, 1, 1, g, 2, 5, 0] == par[0][1, n, 2, g] and raw[1, 2, 1, 1, g, 2, 5, 1] == par[1][1, n, 2, g]


def test_reference_layout_converters_roundtrip_and_hand_built_group():
    """Converters to and from the reference's own 4-bit, group-128 layout (derived from qpack.h:259-294,
    dequantize.h:352-375, flash_fwd_kernel.h:939-964).  Pinned by round trips and a hand-built group only:
    no cache packed by the reference's CUDA kernels exists here (parity with one is unpinned)."""
    rng = np.random.default_rng(9)
    b, S, h = 2, 256, 3
    kc = rng.integers(0, 16, (b, S, h, 128), dtype=np.uint8)
    vc = rng.integers(0, 16, (b, S, h, 128), dtype=np.uint8)
    ks, kz = (rng.integers(0, 65536, (b, S // 128, h, 128)).astype(np.uint16) for _ in range(2))
    vs, vz = (rng.integers(0, 65536, (b, S, h, 1)).astype(np.uint16) for _ in range(2))
    ref = L.to_reference_layout(kc, ks, kz, vc, vs, vz)
    # the reference's tensor contract (evaluation/test.py:76-83)
    assert [a.shape for a in ref] == [(b, S // 4, h, 128), (b, S // 128, h, 128), (b, S, h, 32), (b, 1, h, S)]
    for a, c in zip((kc, ks, kz, vc, vs, vz), L.from_reference_layout(*ref)):
        np.testing.assert_array_equal(a, c)
    ours = L.import_reference_cache(*ref)
    for a, c in zip(ours, L.pack_physical(kc, ks, kz, vc, vs, vz, 4, 128)):
        np.testing.assert_array_equal(a, c)
    for a, c in zip(ref, L.export_reference_cache(*ours)):
        np.testing.assert_array_equal(np.ascontiguousarray(a).view(np.uint8), np.ascontiguousarray(c).view(np.uint8))
    # by hand: K word of pack row p, channel c = tokens p, p+32, p+64, p+96 of the block in nibbles 0..3;
    # V word of token n, column pc = channels pc, pc+32, pc+64, pc+96 in nibbles 0..3
    k_pack, k_params, v_pack, v_params = ref
    p_, c_ = 7, 19
    want = sum(int(kc[1, 128 + p_ + 32 * t, 2, c_]) << (4 * t) for t in range(4))
    assert int(k_pack.view(np.uint16)[1, 32 + p_, 2, c_]) == want
    n_, pc = 200, 5
    want = sum(int(vc[0, n_, 1, pc + 32 * t]) << (4 * t) for t in range(4))
    assert int(v_pack.view(np.uint16)[0, n_, 1, pc]) == want
    # parameters: 256 halves per (group, head): scale[c] then zero[c]; per 128-token block: scale[n] then zero[n]
    kh = np.ascontiguousarray(k_params).view(np.uint16).reshape(b, S // 128, h, 256)
    assert kh[1, 1, 2, c_] == ks[1, 1, 2, c_] and kh[1, 1, 2, 128 + c_] == kz[1, 1, 2, c_]
    vh = np.ascontiguousarray(v_params[:, 0]).view(np.uint16).reshape(b, h, S // 128, 256)
    assert vh[0, 1, 1, n_ - 128] == vs[0, n_, 1, 0] and vh[0, 1, 1, 128 + n_ - 128] == vz[0, n_, 1, 0]


def test_reference_word_nibble_order_from_the_packing_statement():
    """The reference packs four fragment elements jj .. jj+3 into one 16-bit word by or-ing val3, val2, val1, val0
    with a 4-bit shift in between (qpack.h:283-291), so element jj + t lands in nibble t.  Restated here literally,
    as a scalar loop over one fragment row, and compared with the converter's words.  What the statement does NOT
    say is which token (K) or channel (V) fragment element jj + t is: the converter takes them 32 apart
    (dequantize.h:352-375 read with the 32-row pack tile), and that reading is unpinned against a real CUDA cache."""
    rng = np.random.default_rng(11)
    kc = rng.integers(0, 16, (1, 128, 1, 128), dtype=np.uint8)
    vc = rng.integers(0, 16, (1, 128, 1, 128), dtype=np.uint8)
    z = np.zeros((1, 1, 1, 128), np.uint16)
    zv = np.zeros((1, 128, 1, 1), np.uint16)
    k_pack, _, v_pack, _ = L.to_reference_layout(kc, z, z, vc, zv, zv)

    def pack4(vals):                       # qpack.h:283-291, literally
        packed = 0
        packed |= int(vals[3]) & 0xF
        packed <<= 4
        packed |= int(vals[2]) & 0xF
        packed <<= 4
        packed |= int(vals[1]) & 0xF
        packed <<= 4
        packed |= int(vals[0]) & 0xF
        return packed

    for p_, c_ in ((0, 0), (31, 127), (13, 77)):
        assert int(k_pack.view(np.uint16)[0, p_, 0, c_]) == pack4([kc[0, p_ + 32 * t, 0, c_] for t in range(4)])
    for n_, pc in ((0, 0), (127, 31), (64, 9)):
        assert int(v_pack.view(np.uint16)[0, n_, 0, pc]) == pack4([vc[0, n_, 0, pc + 32 * t] for t in range(4)])


def test_bf16_parameters_are_stored_as_fp16_bits():
    """A bf16 cache keeps scale/zero as fp16 bit patterns: bf16 values inside the fp16 normal range
    survive pack -> unpack unchanged, and the stored pattern is the fp16 encoding of the value."""
    rng = np.random.default_rng(5)
    b, S, h, bits, gs = 1, 128, 2, 4, 64
    kc = rng.integers(0, 16, (b, S, h, 128), dtype=np.uint8)
    vals = rng.choice(np.array([1.0, -2.5, 0.0078125, 1000.0, -6.4849853515625e-05, 65280.0], np.float32), (b, S // gs, h, 128))
    as_bf16 = (vals.view(np.uint32) >> 16).astype(np.uint16)            # all exactly representable in bf16
    vsz = np.full((b, S, h, 128 // gs), 0x3F80, np.uint16)              # bf16 1.0
    phys = L.pack_physical(kc, as_bf16, as_bf16, kc, vsz, vsz, bits, gs, "bf16")
    stored = np.ascontiguousarray(phys[1]).reshape(-1).view(np.float16).reshape(b, h, S // gs, 2, 128)
    np.testing.assert_array_equal(stored[:, :, :, 0].transpose(0, 2, 1, 3).astype(np.float32), vals)
    assert np.ascontiguousarray(phys[3]).reshape(-1).view(np.uint16)[0] == 0x3C00   # fp16 1.0
    back = L.unpack_physical(*phys, bits, gs, "bf16")
    np.testing.assert_array_equal(back[1], as_bf16)
    np.testing.assert_array_equal(back[4], vsz)


@pytest.mark.parametrize("bits", [2, 4])
def test_code_maps_are_bijections_and_chunk_local(bits):
    for fn in (L.k_code_map, L.v_code_map):
        tok, ch = fn(bits)
        assert tok.shape == (128 * 128 * bits // 32, 32 // bits)
        pairs = set(zip(tok.ravel().tolist(), ch.ravel().tolist()))
        assert len(pairs) == 128 * 128
        assert tok.min() == 0 and tok.max() == 127 and ch.min() == 0 and ch.max() == 127


def test_k_dword_holds_one_token_and_v_dword_one_channel():
    """A K dword feeds the MFMA A operand of S^T = K Q^T (8 channels of one token); a V dword
    feeds the A operand of O^T = V^T P^T (8 tokens of one channel)."""
    for bits in (2, 4):
        tok, ch = L.k_code_map(bits)
        assert (tok == tok[:, :1]).all()
        tok, ch = L.v_code_map(bits)
        assert (ch == ch[:, :1]).all()


def test_chunks_are_independent_regions():
    """Packing two chunks at once equals packing them separately and concatenating per head:
    what lets 128 new tokens be appended without touching the rest of the cache."""
    rng = np.random.default_rng(3)
    bits, gs, b, h = 4, 128, 1, 2
    mk = lambda S: (rng.integers(0, 16, (b, S, h, 128), dtype=np.uint8),
                    rng.integers(0, 65536, (b, S // gs, h, 128)).astype(np.uint16),
                    rng.integers(0, 65536, (b, S // gs, h, 128)).astype(np.uint16),
                    rng.integers(0, 16, (b, S, h, 128), dtype=np.uint8),
                    rng.integers(0, 65536, (b, S, h, 1)).astype(np.uint16),
                    rng.integers(0, 65536, (b, S, h, 1)).astype(np.uint16))
    full = mk(256)
    whole = L.pack_physical(*full, bits, gs)
    for half in (0, 1):
        part = tuple(a[:, (half * 128 // (256 // a.shape[1])):((half + 1) * 128 // (256 // a.shape[1]))] for a in full)
        sub = L.pack_physical(*part, bits, gs)
        for w, s_ in zip(whole, sub):
            wb = w.reshape(-1).view(np.uint8).reshape(b * h, -1)
            sb = s_.reshape(-1).view(np.uint8).reshape(b * h, -1)
            n = sb.shape[1]
            np.testing.assert_array_equal(wb[:, half * n:(half + 1) * n], sb)


# ------------------------------------------------------------------ C ABI
def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "bitdecode.h")).read()
    declared = set(re.findall(r"\b(bitdecode_[a-z_0-9]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    lib = _lib.lib()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.bitdecode_abi_version() == _lib.ABI_VERSION


def test_struct_mirrors_match_header_field_order():
    header = open(os.path.join(ROOT, "include", "bitdecode.h")).read()
    for cname, cls in (("bitdecode_qpack_args", _lib.QpackArgs), ("bitdecode_fwd_args", _lib.FwdArgs),
                       ("bitdecode_fwd_append_args", _lib.FwdAppendArgs)):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cname, cname), header, re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        names = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            for part in decl.split(","):
                names.append(re.findall(r"[A-Za-z_][A-Za-z_0-9]*", part)[-1])
        assert names == [f[0] for f in cls._fields_], cname


def _fwd_args(**kw):
    a = _lib.FwdArgs()
    fake = 0x1000
    a.q = a.out = a.k_pack = a.k_params = a.v_pack = a.v_params = fake
    a.q_stride_b, a.q_stride_h = 32 * 128, 128
    a.out_stride_b, a.out_stride_h = 32 * 128, 128
    a.cache_tokens = a.seqlen_k = a.max_seqlen_k = 1024
    a.b, a.h, a.h_k, a.d = 1, 32, 8, 128
    a.bits, a.group_size, a.dtype = 4, 128, 0
    a.softmax_scale = 0.088
    a.num_splits = 1
    for k, v in kw.items():
        setattr(a, k, v)
    return a


@pytest.mark.parametrize("kw,code,text", [
    (dict(d=64), 2, "head_dim"),
    (dict(bits=3), 2, "num_bits"),
    (dict(group_size=16), 2, "group_size"),
    (dict(dtype=5), 2, "dtype"),
    (dict(h=30), 1, "multiple"),
    (dict(h=8 * 9), 2, "query heads per kv head"),
    (dict(seqlen_k=1000, max_seqlen_k=1000), 1, "multiple of 128"),
    (dict(seqlen_k=2048, max_seqlen_k=2048), 1, "exceeds cache capacity"),
    (dict(q=0), 1, "null"),
    (dict(q=0x1004), 1, "aligned"),
    (dict(q_stride_h=100), 1, "strides"),
    (dict(num_splits=4), 3, "workspace"),
    (dict(num_splits=-1), 1, "negative"),
    (dict(res_len=5), 1, "null residual"),
])
def test_fwd_rejects_bad_arguments_without_launching(kw, code, text):
    lib = _lib.lib()
    rc = lib.bitdecode_fwd(ctypes.byref(_fwd_args(**kw)), None)
    assert rc == code, lib.bitdecode_last_error()
    assert text in lib.bitdecode_last_error().decode()
    with pytest.raises(_lib.BitDecodeError):
        _lib.check(rc)


def _qpack_args(**kw):
    a = _lib.QpackArgs()
    fake = 0x1000
    a.k = a.v = a.k_pack = a.k_params = a.v_pack = a.v_params = fake
    a.k_stride_b = a.v_stride_b = 256 * 8 * 128
    a.k_stride_t = a.v_stride_t = 8 * 128
    a.k_stride_h = a.v_stride_h = 128
    a.b, a.n_tokens, a.h_k, a.d = 1, 256, 8, 128
    a.cache_tokens = 1024
    a.bits, a.group_size, a.dtype = 4, 128, 0
    for k, v in kw.items():
        setattr(a, k, v)
    return a


@pytest.mark.parametrize("kw,code,text", [
    (dict(n_tokens=100), 1, "multiple of 128"),
    (dict(cache_tokens=1000), 1, "cache_tokens"),
    (dict(dst_offset=64), 1, "dst_offset"),
    (dict(dst_offset=896), 1, "exceeds cache capacity"),
    (dict(bits=8), 2, "num_bits"),
    (dict(k=0), 1, "null"),
    (dict(k_stride_t=1020), 1, "strides"),
])
def test_qpack_rejects_bad_arguments_without_launching(kw, code, text):
    lib = _lib.lib()
    rc = lib.bitdecode_qpack(ctypes.byref(_qpack_args(**kw)), None)
    assert rc == code, lib.bitdecode_last_error()
    assert text in lib.bitdecode_last_error().decode()


def test_qpack_of_zero_tokens_is_a_no_op():
    assert _lib.lib().bitdecode_qpack(ctypes.byref(_qpack_args(n_tokens=0)), None) == 0


def test_split_choice_and_workspace_size():
    lib = _lib.lib()
    # 32K GQA config on 256 CUs: 8 kv heads x 32 splits = one workgroup per CU, one 64-token unit per wave
    assert lib.bitdecode_num_splits(1, 8, 32768, 128, 256, 4, 128) == 32
    # enough (batch x kv-head) workgroups already: no split
    assert lib.bitdecode_num_splits(64, 8, 4096, 128, 256, 4, 128) == 1
    # never more splits than there is work for: 4 units of 64 tokens -> one workgroup
    assert lib.bitdecode_num_splits(1, 1, 256, 0, 256, 4, 128) == 1
    # 48 units, at least one unit for every second of the 16 waves -> 6 splits
    assert lib.bitdecode_num_splits(1, 1, 128 * 24, 0, 256, 4, 128) == 6
    assert lib.bitdecode_num_splits(1, 1, 1024, 0, 256, 3, 128) == -1
    # per-sequence lengths on the device: a batch of 16 gets two workgroups of the 8-wave kernel per compute unit
    assert lib.bitdecode_num_splits(16, 8, 8192, 256, 256, 4, 128) == 2
    assert lib.bitdecode_num_splits_for(16, 8, 8192, 256, 256, 4, 128, 0) == 2
    assert lib.bitdecode_num_splits_for(16, 8, 8192, 256, 256, 4, 128, 1) == 4
    # ... not the 2-bit kernels (16 waves, one workgroup per unit), not one sequence, not workgroups of more than 32 units
    assert lib.bitdecode_num_splits_for(16, 8, 8192, 256, 256, 2, 128, 1) == 2
    assert lib.bitdecode_num_splits_for(1, 8, 32768, 128, 256, 4, 128, 1) == 32
    assert lib.bitdecode_num_splits_for(16, 8, 65536, 128, 256, 4, 128, 1) == 2
    # ... and not batches that need more than two splits to fill the machine anyway
    assert lib.bitdecode_num_splits_for(8, 8, 8192, 128, 256, 4, 128, 1) == lib.bitdecode_num_splits(8, 8, 8192, 128, 256, 4, 128) == 4
    assert lib.bitdecode_fwd_workspace_bytes(1, 32, 1) == 0
    # one 256-byte counter block per query head + two slots of records per split: fp16 partial outputs, as many
    # residual words, an fp32 (max, sum) pair; a slot is a whole number of 256-byte blocks
    assert lib.bitdecode_fwd_workspace_bytes(1, 32, 32) == 32 * 256 + 2 * 32 * 32 * 130 * 4
    assert lib.bitdecode_fwd_workspace_bytes(1, 3, 5) == 3 * 256 + 2 * ((3 * 5 * 130 * 4 + 255) // 256 * 256)


def test_python_entry_points_validate_before_touching_the_gpu():
    import torch
    from bitladder_amd import fwd_kvcache_int, kvcache_pack_int
    t = torch.zeros(1, 128, 2, 128, dtype=torch.float16)
    kp = torch.zeros(1, 32, 2, 128, dtype=torch.uint16)
    with pytest.raises(NotImplementedError):      # "k-tensor" is a 4-bit mode, as in the reference
        kvcache_pack_int(t, kp, kp, t, kp, kp, None, None, 128, "k-tensor", 128, 2)
    with pytest.raises(ValueError):
        kvcache_pack_int(t, kp, kp, t, kp, kp, None, None, 128, "k-token", 128, 4)
    with pytest.raises(ValueError):
        kvcache_pack_int(t, kp, kp, t, kp, kp, None, None, 128, "k-channel", 48, 4)
    with pytest.raises(ValueError):
        fwd_kvcache_int(t[:, :1], kp, kp, kp, kp, None, 1.0, "k-channel", 128, 3)
    with pytest.raises(RuntimeError):      # a block table is accepted, but like everything else not on the CPU
        fwd_kvcache_int(t[:, :1], kp, kp, kp, kp, torch.zeros(1, 1, dtype=torch.int32))
    with pytest.raises(RuntimeError):      # CPU tensors: the reference's CHECK_DEVICE
        kvcache_pack_int(t, kp, kp, t, kp, kp)


def test_drop_in_package_name_and_signatures():
    import inspect
    import bit_decode
    sig = inspect.signature(bit_decode.kvcache_pack_int)
    assert list(sig.parameters)[:12] == ["k_cache", "k_pack", "k_params", "v_cache", "v_pack", "v_params",
                                         "opt_block_table", "cu_seqlens_k", "seqlen_k", "quant_mode", "group_size",
                                         "num_bits"]
    assert sig.parameters["group_size"].default == 128 and sig.parameters["num_bits"].default == 4
    sig = inspect.signature(bit_decode.fwd_kvcache_int)
    assert list(sig.parameters)[:10] == ["q", "k_pack", "k_params", "v_pack", "v_params", "opt_block_table",
                                         "softmax_scale", "quant_mode", "group_size", "num_bits"]
    assert sig.parameters["softmax_scale"].default == 1.0       # bit_decode_interface.py:47
    assert bit_decode.__version__ == "1.0.0.post1"              # bit_decode/__init__.py:1
