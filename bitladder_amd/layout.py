"""Host-side (numpy) description of the physical packed-cache layout: converts between the
logical form (codes [b,S,h_k,128] uint8, scale/zero as raw 16-bit patterns) and the bytes of the
four cache tensors.  Mirrors bitladder_amd/csrc/layout.h.  Used to import/export caches and by
the tests to compare the pack kernel with the quantizer oracle; the decode path never calls it.
"""
from __future__ import annotations

import numpy as np

D = 128
CHUNK = 128


def _field_of_element(bits: int):
    """Position (field index inside a dword) of element e = 8*kstep_in_dword + i."""
    if bits == 4:
        i = np.arange(8)
        return i // 2 + 4 * (i % 2)
    e = np.arange(16)
    return e // 2 + 8 * (e % 2)


def k_code_map(bits: int):
    """(token, channel) of every code field of one K chunk, shape [n_dwords, fields] each,
    dwords in memory order."""
    if bits == 4:
        t, l, j, i = np.meshgrid(np.arange(8), np.arange(64), np.arange(4), np.arange(8), indexing="ij")
        m, kg = l % 16, l // 16
        tok = 16 * t + m
        ch = 32 * j + 8 * kg + i
        p = i // 2 + 4 * (i % 2)
        tok_f = np.empty((8, 64, 4, 8), np.int64)
        ch_f = np.empty_like(tok_f)
        np.put_along_axis(tok_f, p, tok, axis=3)
        np.put_along_axis(ch_f, p, ch, axis=3)
        return tok_f.reshape(-1, 8), ch_f.reshape(-1, 8)
    tp, l, tin, jj, e = np.meshgrid(np.arange(4), np.arange(64), np.arange(2), np.arange(2), np.arange(16),
                                    indexing="ij")
    m, kg = l % 16, l // 16
    tok = 16 * (2 * tp + tin) + m
    j, i = 2 * jj + e // 8, e % 8
    ch = 32 * j + 8 * kg + i
    f = e // 2 + 8 * (e % 2)
    tok_f = np.empty(tok.shape, np.int64)
    ch_f = np.empty_like(tok_f)
    np.put_along_axis(tok_f, f, tok, axis=4)
    np.put_along_axis(ch_f, f, ch, axis=4)
    return tok_f.reshape(-1, 16), ch_f.reshape(-1, 16)


def v_code_map(bits: int):
    """(token, channel) of every code field of one V chunk, dwords in memory order."""
    if bits == 4:
        sb, hf, l, x, i = np.meshgrid(np.arange(4), np.arange(2), np.arange(64), np.arange(4), np.arange(8),
                                      indexing="ij")
        c, kg = l % 16, l // 16
        ch = 16 * (4 * hf + x) + c
        tok = 32 * sb + 16 * (i // 4) + 4 * kg + i % 4
        p = i // 2 + 4 * (i % 2)
        tok_f = np.empty(tok.shape, np.int64)
        ch_f = np.empty_like(tok_f)
        np.put_along_axis(tok_f, p, tok, axis=4)
        np.put_along_axis(ch_f, p, ch, axis=4)
        return tok_f.reshape(-1, 8), ch_f.reshape(-1, 8)
    sb2, hf, l, x, e = np.meshgrid(np.arange(2), np.arange(2), np.arange(64), np.arange(4), np.arange(16),
                                   indexing="ij")
    c, kg = l % 16, l // 16
    ch = 16 * (4 * hf + x) + c
    ks, i = e // 8, e % 8
    tok = 64 * sb2 + 32 * ks + 16 * (i // 4) + 4 * kg + i % 4
    f = e // 2 + 8 * (e % 2)
    tok_f = np.empty(tok.shape, np.int64)
    ch_f = np.empty_like(tok_f)
    np.put_along_axis(tok_f, f, tok, axis=4)
    np.put_along_axis(ch_f, f, ch, axis=4)
    return tok_f.reshape(-1, 16), ch_f.reshape(-1, 16)


def v_param_token_map():
    """token-in-chunk of V-param slot [sb, q, i]."""
    sb, q, i = np.meshgrid(np.arange(4), np.arange(4), np.arange(8), indexing="ij")
    return 32 * sb + 16 * (i // 4) + 4 * q + i % 4


def _codes_to_dwords(codes_chunk: np.ndarray, tok_f, ch_f, bits: int) -> np.ndarray:
    """codes_chunk [..., 128 tok, 128 ch] uint8 -> dwords [..., n_dwords] uint32."""
    vals = codes_chunk[..., tok_f, ch_f].astype(np.uint32)           # [..., n_dwords, fields]
    shifts = (np.arange(tok_f.shape[1], dtype=np.uint32) * bits)
    return (vals << shifts).sum(axis=-1, dtype=np.uint32)


def _dwords_to_codes(dwords: np.ndarray, tok_f, ch_f, bits: int) -> np.ndarray:
    shifts = (np.arange(tok_f.shape[1], dtype=np.uint32) * bits)
    vals = ((dwords[..., None] >> shifts) & np.uint32((1 << bits) - 1)).astype(np.uint8)
    out = np.zeros(dwords.shape[:-1] + (CHUNK, D), np.uint8)
    out[..., tok_f, ch_f] = vals
    return out


def _bf16_bits_to_fp16_bits(x: np.ndarray) -> np.ndarray:
    f = (x.astype(np.uint32) << 16).view(np.float32)
    with np.errstate(over="ignore"):
        return f.astype(np.float16).view(np.uint16)


def _fp16_bits_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    # round to nearest even; exact when the fp16 value came from a bf16 inside the fp16 normal range
    u = np.ascontiguousarray(x).view(np.float16).astype(np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def pack_physical(k_codes, k_scale, k_zero, v_codes, v_scale, v_zero, bits: int, gs: int, dtype: str = "fp16",
                  quant_mode: str = "k-channel"):
    """Logical -> physical.  codes uint8 [b,S,h,128]; k_scale/k_zero uint16 bit patterns of the
    element type `dtype` [b,S/gs,h,128]; v_scale/v_zero uint16 [b,S,h,128/gs].  Returns the four
    cache tensors as numpy arrays with the reference shapes (k_pack/v_pack uint16,
    k_params/v_params float32 containers).  Parameters are stored as fp16 bits for both element
    types (bf16 values are converted, exact inside the fp16 normal range).
    With quant_mode "k-tensor" k_scale/k_zero are [b,S,h,128/gs] like V's and k_params takes
    v_params' shape; per chunk its bytes are [64-token half][channel group][16-token tile][token]
    (scale, zero) pairs, the order in which the decode kernel's score tiles need them."""
    if dtype == "bf16":
        k_scale, k_zero, v_scale, v_zero = (_bf16_bits_to_fp16_bits(np.ascontiguousarray(a))
                                            for a in (k_scale, k_zero, v_scale, v_zero))
    b, S, h, d = k_codes.shape
    assert d == D and S % CHUNK == 0
    nc, pn, ncg = S // CHUNK, 16 // bits, D // gs
    kt, kc_ = k_code_map(bits)
    vt, vc_ = v_code_map(bits)
    kch = k_codes.reshape(b, nc, CHUNK, h, d).transpose(0, 3, 1, 2, 4)       # [b,h,nc,128,128]
    vch = v_codes.reshape(b, nc, CHUNK, h, d).transpose(0, 3, 1, 2, 4)
    k_pack = _codes_to_dwords(kch, kt, kc_, bits).reshape(-1).view(np.uint16).reshape(b, S // pn, h, d)
    v_pack = _codes_to_dwords(vch, vt, vc_, bits).reshape(-1).view(np.uint16).reshape(b, S, h, d // pn)
    if quant_mode == "k-tensor":
        # K params: [b,h,chunk][half][cg][tile][token][scale, zero]
        ks = k_scale.reshape(b, nc, 2, 4, 16, h, ncg).transpose(0, 5, 1, 2, 6, 3, 4)     # [b,h,nc,half,cg,tile,tok]
        kz = k_zero.reshape(b, nc, 2, 4, 16, h, ncg).transpose(0, 5, 1, 2, 6, 3, 4)
        kp = np.stack([ks, kz], axis=-1)
        k_params = np.ascontiguousarray(kp).astype(np.uint16).reshape(-1).view(np.float32).reshape(b, d // gs, h, S)
    else:
        # K params: [b,h,group][scale 128 | zero 128]
        kp = np.stack([k_scale.transpose(0, 2, 1, 3), k_zero.transpose(0, 2, 1, 3)], axis=3)   # [b,h,G,2,128]
        k_params = np.ascontiguousarray(kp).astype(np.uint16).reshape(-1).view(np.float32).reshape(b, S // gs, h, d)
    # V params: [b,h,chunk][sb][cg][which][q][i]
    tokmap = v_param_token_map()                                               # [4,4,8]
    vs = v_scale.reshape(b, nc, CHUNK, h, ncg).transpose(0, 3, 1, 4, 2)       # [b,h,nc,cg,128]
    vz = v_zero.reshape(b, nc, CHUNK, h, ncg).transpose(0, 3, 1, 4, 2)
    vs = vs[..., tokmap]                                                       # [b,h,nc,cg,sb,q,i]
    vz = vz[..., tokmap]
    vp = np.stack([vs, vz], axis=5)                                            # [b,h,nc,cg,sb,2,q,i]
    vp = vp.transpose(0, 1, 2, 4, 3, 5, 6, 7)                                  # [b,h,nc,sb,cg,2,q,i]
    v_params = np.ascontiguousarray(vp).astype(np.uint16).reshape(-1).view(np.float32).reshape(b, d // gs, h, S)
    return k_pack, k_params, v_pack, v_params


def unpack_physical(k_pack, k_params, v_pack, v_params, bits: int, gs: int, dtype: str = "fp16",
                    quant_mode: str = "k-channel"):
    """Physical -> logical; inverse of pack_physical.  Inputs are numpy arrays with the reference
    shapes (any 16-bit / 32-bit dtype).  Returns (k_codes, k_scale, k_zero, v_codes, v_scale,
    v_zero) with scale/zero as uint16 bit patterns of the element type `dtype`."""
    b, S, h, dp = v_pack.shape
    pn = 16 // bits
    d = dp * pn
    assert d == D and S % CHUNK == 0
    nc, ncg = S // CHUNK, D // gs
    kt, kc_ = k_code_map(bits)
    vt, vc_ = v_code_map(bits)
    ndw = CHUNK * D * bits // 32
    kd = np.ascontiguousarray(k_pack).reshape(-1).view(np.uint32).reshape(b, h, nc, ndw)
    vd = np.ascontiguousarray(v_pack).reshape(-1).view(np.uint32).reshape(b, h, nc, ndw)
    k_codes = _dwords_to_codes(kd, kt, kc_, bits).transpose(0, 2, 3, 1, 4).reshape(b, S, h, d)
    v_codes = _dwords_to_codes(vd, vt, vc_, bits).transpose(0, 2, 3, 1, 4).reshape(b, S, h, d)
    if quant_mode == "k-tensor":
        kp = np.ascontiguousarray(k_params).reshape(-1).view(np.uint16).reshape(b, h, nc, 2, ncg, 4, 16, 2)
        kp = kp.transpose(0, 2, 3, 5, 6, 1, 4, 7)                                # [b,nc,half,tile,tok,h,cg,2]
        k_scale = np.ascontiguousarray(kp[..., 0]).reshape(b, S, h, ncg)
        k_zero = np.ascontiguousarray(kp[..., 1]).reshape(b, S, h, ncg)
    else:
        kp = np.ascontiguousarray(k_params).reshape(-1).view(np.uint16).reshape(b, h, S // gs, 2, d)
        k_scale = np.ascontiguousarray(kp[:, :, :, 0].transpose(0, 2, 1, 3))
        k_zero = np.ascontiguousarray(kp[:, :, :, 1].transpose(0, 2, 1, 3))
    vp = np.ascontiguousarray(v_params).reshape(-1).view(np.uint16).reshape(b, h, nc, 4, ncg, 2, 4, 8)
    tokmap = v_param_token_map()
    vs = np.zeros((b, h, nc, ncg, CHUNK), np.uint16)
    vz = np.zeros_like(vs)
    vs[..., tokmap] = vp[:, :, :, :, :, 0].transpose(0, 1, 2, 4, 3, 5, 6)
    vz[..., tokmap] = vp[:, :, :, :, :, 1].transpose(0, 1, 2, 4, 3, 5, 6)
    v_scale = np.ascontiguousarray(vs.transpose(0, 2, 4, 1, 3)).reshape(b, S, h, ncg)
    v_zero = np.ascontiguousarray(vz.transpose(0, 2, 4, 1, 3)).reshape(b, S, h, ncg)
    if dtype == "bf16":
        k_scale, k_zero, v_scale, v_zero = (_fp16_bits_to_bf16_bits(a) for a in (k_scale, k_zero, v_scale, v_zero))
    return k_codes, k_scale, k_zero, v_codes, v_scale, v_zero


# --------------------------------------------------------------------------------------------------
# The reference's own physical layout (4 bits, group size 128, "k-channel"), as far as it can be derived
# from its sources: the word packing of its quantizer (csrc/bit_decode/src/include/qpack.h:259-294), the
# consumer's nibble-to-column rule (include/dequantize.h:352-375) and the parameter stores
# (src/flash_fwd_kernel.h:939-964).  A cache packed by the reference's CUDA kernels could not be produced
# here, so these converters are pinned by round trips and a hand-built example only: parity with a real
# CUDA cache is unpinned.
#   k_pack   [b, S/4, h, 128] u16: row 32*B + p, channel c holds tokens 128*B + p + 32*t in nibble t
#   k_params [b, S/128, h, 128] f32 = 256 halves per (group, head): scale[c] (128) | zero[c] (128)
#   v_pack   [b, S, h, 32] u16: token n, column pc holds channels pc + 32*t in nibble t
#   v_params [b, 1, h, S] f32 = per head and 128-token block 256 halves: scale[n] (128) | zero[n] (128)
# --------------------------------------------------------------------------------------------------
def to_reference_layout(k_codes, k_scale, k_zero, v_codes, v_scale, v_zero):
    """Logical form (4 bits, group size 128; scale/zero as uint16 fp16 bit patterns) -> the four
    tensors in the reference's layout."""
    b, S, h, d = k_codes.shape
    assert d == D and S % CHUNK == 0 and k_scale.shape == (b, S // 128, h, d) and v_scale.shape == (b, S, h, 1)
    nb = S // 128
    sh = (np.arange(4, dtype=np.uint16) * 4)
    kc = k_codes.reshape(b, nb, 4, 32, h, d).astype(np.uint16)                  # token = 128*B + 32*t + p
    k_pack = (kc << sh[None, None, :, None, None, None]).sum(axis=2, dtype=np.uint16).reshape(b, S // 4, h, d)
    vc = v_codes.reshape(b, S, h, 4, 32).astype(np.uint16)                      # channel = 32*t + pc
    v_pack = (vc << sh[None, None, None, :, None]).sum(axis=3, dtype=np.uint16)
    kp = np.concatenate([k_scale, k_zero], axis=3).astype(np.uint16)            # [b, G, h, 256]
    k_params = np.ascontiguousarray(kp).reshape(-1).view(np.float32).reshape(b, nb, h, d)
    vs = v_scale[..., 0].reshape(b, nb, 128, h).transpose(0, 3, 1, 2)           # [b, h, B, 128]
    vz = v_zero[..., 0].reshape(b, nb, 128, h).transpose(0, 3, 1, 2)
    vp = np.concatenate([vs, vz], axis=3).astype(np.uint16)                     # [b, h, B, 256]
    v_params = np.ascontiguousarray(vp).reshape(-1).view(np.float32).reshape(b, h, 1, S).transpose(0, 2, 1, 3)
    return k_pack, k_params, v_pack, np.ascontiguousarray(v_params)


def from_reference_layout(k_pack, k_params, v_pack, v_params):
    """Inverse of to_reference_layout."""
    b, S, h, pc = v_pack.shape
    assert pc == 32 and S % CHUNK == 0
    nb = S // 128
    sh = (np.arange(4, dtype=np.uint16) * 4)
    kw = np.ascontiguousarray(k_pack).view(np.uint16).reshape(b, nb, 1, 32, h, D)
    k_codes = ((kw >> sh[None, None, :, None, None, None]) & 0xF).astype(np.uint8).reshape(b, S, h, D)
    vw = np.ascontiguousarray(v_pack).view(np.uint16).reshape(b, S, h, 1, 32)
    v_codes = ((vw >> sh[None, None, None, :, None]) & 0xF).astype(np.uint8).reshape(b, S, h, D)
    kp = np.ascontiguousarray(k_params).reshape(-1).view(np.uint16).reshape(b, nb, h, 256)
    k_scale, k_zero = np.ascontiguousarray(kp[..., :128]), np.ascontiguousarray(kp[..., 128:])
    vp = np.ascontiguousarray(np.ascontiguousarray(v_params).transpose(0, 2, 1, 3)).reshape(-1).view(np.uint16)
    vp = vp.reshape(b, h, nb, 256)
    v_scale = np.ascontiguousarray(vp[..., :128].transpose(0, 2, 3, 1)).reshape(b, S, h, 1)
    v_zero = np.ascontiguousarray(vp[..., 128:].transpose(0, 2, 3, 1)).reshape(b, S, h, 1)
    return k_codes, k_scale, k_zero, v_codes, v_scale, v_zero


def import_reference_cache(k_pack, k_params, v_pack, v_params):
    """A 4-bit, group-128 cache in the reference's layout -> the same cache in this library's layout
    (same tensor shapes)."""
    return pack_physical(*from_reference_layout(k_pack, k_params, v_pack, v_params), 4, 128)


def export_reference_cache(k_pack, k_params, v_pack, v_params):
    """This library's 4-bit, group-128 cache -> the reference's layout."""
    return to_reference_layout(*unpack_physical(k_pack, k_params, v_pack, v_params, 4, 128))
