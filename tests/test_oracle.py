"""Pins for the CPU oracle (oracle/bitdecode_oracle.py).

The reference cannot be built or imported here (CUDA/PTX + absent CUTLASS) and holds no golden
vectors for this path, so each oracle function is pinned by what the mathematics fixes: closed
forms, invariants, brute force on tiny inputs, a second independent C restatement, and the
known answers the reference's own comments state.  A plausible mistake (wrong rounding mode,
wrong grouping axis, dropped zero term, transposed GQA mapping) fails at least one test here.
"""
import itertools
import math

import numpy as np
import pytest

from oracle import bitdecode_oracle as O
from oracle import c_oracle as C

F32 = np.float32


# ------------------------------------------------------------------ quantizer: closed forms
def test_hand_computed_group_4bit():
    # x = 0..15 scaled by 0.5: range 7.5, scale_inv = 2, scale = 0.5, codes = 0..15 exactly
    x = (np.arange(16, dtype=F32) * F32(0.5) - F32(3.0)).reshape(1, 16)
    codes, scale, zero = O.quantize_group(x, 4, axis=1)
    assert codes.tolist() == [list(range(16))]
    assert scale.item() == 0.5 and zero.item() == -3.0


def test_hand_computed_group_2bit():
    x = np.array([[-1.0, 0.0, 1.0, 2.0, 0.4, 0.6]], dtype=F32)       # range 3, scale_inv 1
    codes, scale, zero = O.quantize_group(x, 2, axis=1)
    # (x - min) * 1 = 0,1,2,3,1.4,1.6 -> 0,1,2,3,1,2
    assert codes.tolist() == [[0, 1, 2, 3, 1, 2]]
    assert scale.item() == 1.0 and zero.item() == -1.0


def test_round_half_away_from_zero_not_to_even():
    # (x - min) * scale_inv lands exactly on .5 ties: roundf gives 1, 3, 5 (rint would give 0, 2, 4)
    x = np.array([[0.0, 0.5, 1.5, 2.5, 2.5, 15.0]], dtype=F32)        # range 15 -> scale_inv 1
    codes, _, _ = O.quantize_group(x, 4, axis=1)
    assert codes.tolist() == [[0, 1, 2, 3, 3, 15]]
    assert O.roundf(np.array([0.5, 1.5, 2.5, -0.5, -2.5, 0.49999997], F32)).tolist() == [1, 2, 3, -1, -3, 0]


def test_constant_group_gives_zero_scale_and_exact_dequant():
    x = np.full((3, 32), 1.7265625, dtype=F32)
    codes, scale, zero = O.quantize_group(x, 4, axis=1)
    assert not codes.any() and not scale.any()
    np.testing.assert_array_equal(codes * scale + zero, x)


@pytest.mark.parametrize("bits", [2, 4])
def test_extremes_map_to_end_codes_and_error_bound(bits):
    rng = np.random.default_rng(1)
    x = O.round_to_storage(rng.standard_normal((200, 64), dtype=F32) * F32(3), "fp16")
    codes, scale, zero = O.quantize_group(x, bits, axis=1)
    M = (1 << bits) - 1
    assert codes.min() == 0 and codes.max() == M
    assert (codes[np.arange(200), x.argmin(1)] == 0).all()
    assert (codes[np.arange(200), x.argmax(1)] == M).all()
    # |x - dequant| <= scale/2 plus the fp16 rounding of scale accumulated over M steps
    err = np.abs(codes.astype(F32) * scale + zero - x)
    bound = scale / 2 + M * np.abs(scale) * 2.0 ** -11 + 1e-6
    assert (err <= bound).all()


def test_fp16_max_range_values():
    x = np.array([[65504.0, -65504.0] + [0.0] * 30], dtype=F32)
    codes, scale, zero = O.quantize_group(x, 4, axis=1)
    assert codes[0, 0] == 15 and codes[0, 1] == 0 and zero.item() == -65504.0
    assert scale.item() == np.float16(131008.0 / 15.0)       # fits fp16 (8733.9)
    assert codes[0, 2] in (7, 8)


def test_idempotent_on_own_grid():
    """Quantizing already-dequantized values whose grid is exactly representable reproduces the codes."""
    rng = np.random.default_rng(2)
    codes0 = rng.integers(0, 16, (50, 32)).astype(np.uint8)
    codes0[:, 0], codes0[:, 1] = 0, 15
    x = codes0.astype(F32) * F32(0.25) - F32(2.0)             # scale 0.25: exact grid
    codes, scale, zero = O.quantize_group(x, 4, axis=1)
    np.testing.assert_array_equal(codes, codes0)
    assert (scale == 0.25).all() and (zero == -2.0).all()


def test_brute_force_tiny_groups_against_scalar_python():
    """Every 3-element group over a small fp16 grid, checked against a scalar restatement of
    qpack.h:243-285 written with Python floats forced through fp32."""
    vals = [F32(v) for v in (-1.5, -0.25, 0.0, 0.125, 0.5, 1.0, 2.75)]

    def scalar(group, bits):
        M = F32((1 << bits) - 1)
        mx, mn = max(group), min(group)
        rng = F32(mx - mn)
        sinv = F32(M / rng) if rng > 0 else F32(0)
        out = []
        for v in group:
            t = F32(F32(v - mn) * sinv)
            r = math.floor(abs(float(t)) + 0.5)                # exact here: t has few bits
            out.append(int(min(max(r, 0), float(M))))
        return out, (F32(0) if sinv == 0 else F32(F32(1) / sinv)), mn

    for bits in (2, 4):
        for g in itertools.product(vals, repeat=3):
            want_c, want_s, want_z = scalar(g, bits)
            codes, scale, zero = O.quantize_group(np.array([g], F32), bits, axis=1)
            assert codes[0].tolist() == want_c, (g, bits)
            assert scale.item() == np.float16(want_s) and zero.item() == want_z


# ------------------------------------------------------------------ grouping axes
def test_k_groups_run_along_tokens_and_v_groups_along_channels():
    b, S, h, d, gs = 1, 64, 1, 128, 32
    k = np.zeros((b, S, h, d), F32)
    v = np.zeros((b, S, h, d), F32)
    k[0, 5, 0, 7] = 8.0            # one large K value: affects its channel's token group only
    v[0, 9, 0, 40] = 4.0           # one large V value: affects its token's channel group only
    q = O.quantize_kv_ref(k, v, 4, gs)
    assert q.k_scale.shape == (b, S // gs, h, d) and q.v_scale.shape == (b, S, h, d // gs)
    ks = q.k_scale[0, :, 0, :]
    assert ks[0, 7] > 0 and np.count_nonzero(ks) == 1
    vs = q.v_scale[0, :, 0, :]
    assert vs[9, 1] > 0 and np.count_nonzero(vs) == 1
    assert q.k_codes[0, 5, 0, 7] == 15 and q.v_codes[0, 9, 0, 40] == 15


# ------------------------------------------------------------------ dequantize_ref, pinned directly
@pytest.mark.parametrize("bits,gs", [(4, 128), (4, 32), (2, 64)])
def test_dequantize_is_exact_on_an_exact_grid_and_inverts_the_quantizer(bits, gs):
    """Values that lie on a grid both scale and zero represent exactly come back unchanged, for K (groups
    along tokens) and V (groups along channels) separately; a transposed or mis-repeated parameter axis
    would put another group's scale or zero under a value and break the equality."""
    rng = np.random.default_rng(bits * 10 + gs)
    b, S, h, d, M = 2, 256, 2, 128, (1 << bits) - 1
    kc = rng.integers(0, M + 1, (b, S, h, d)).astype(np.uint8)
    vc = rng.integers(0, M + 1, (b, S, h, d)).astype(np.uint8)
    # every group holds both end codes, so the quantizer finds the grid again
    kc.reshape(b, S // gs, gs, h, d)[:, :, 0], kc.reshape(b, S // gs, gs, h, d)[:, :, 1] = 0, M
    vc.reshape(b, S, h, d // gs, gs)[..., 0], vc.reshape(b, S, h, d // gs, gs)[..., 1] = 0, M
    # a different power-of-two scale and a different zero for every group
    k_scale = np.exp2(rng.integers(-6, 3, (b, S // gs, h, d))).astype(F32)
    k_zero = (rng.integers(-8, 8, (b, S // gs, h, d)) * k_scale).astype(F32)
    v_scale = np.exp2(rng.integers(-6, 3, (b, S, h, d // gs))).astype(F32)
    v_zero = (rng.integers(-8, 8, (b, S, h, d // gs)) * v_scale).astype(F32)
    k = kc.astype(F32) * np.repeat(k_scale, gs, axis=1) + np.repeat(k_zero, gs, axis=1)
    v = vc.astype(F32) * np.repeat(v_scale, gs, axis=3) + np.repeat(v_zero, gs, axis=3)
    q = O.quantize_kv_ref(k, v, bits, gs)
    np.testing.assert_array_equal(q.k_codes, kc)
    np.testing.assert_array_equal(q.v_codes, vc)
    np.testing.assert_array_equal(q.k_scale, k_scale)
    np.testing.assert_array_equal(q.v_zero, v_zero)
    k_hat, v_hat = O.dequantize_ref(q)
    np.testing.assert_array_equal(k_hat, k)
    np.testing.assert_array_equal(v_hat, v)


@pytest.mark.parametrize("bits", [2, 4])
def test_dequantize_stays_within_half_a_step_of_the_input(bits):
    """dequantize_ref(quantize_kv_ref(x)) is within scale/2 of x, plus what rounding scale to fp16 can
    add over the code range, element by element with each element's own group scale."""
    gs = 64
    _, k, v = O.make_inputs(2, 2, 2, 256, 0, seed=40 + bits)
    q = O.quantize_kv_ref(k, v, bits, gs)
    k_hat, v_hat = O.dequantize_ref(q)
    M = (1 << bits) - 1
    ks = np.repeat(q.k_scale, gs, axis=1)
    vs = np.repeat(q.v_scale, gs, axis=3)
    assert (np.abs(k_hat - k) <= ks / 2 + M * ks * 2.0 ** -11 + 1e-6).all()
    assert (np.abs(v_hat - v) <= vs / 2 + M * vs * 2.0 ** -11 + 1e-6).all()
    # a group's minimum is reproduced exactly (code 0 -> zero)
    kmin = k.reshape(2, 256 // gs, gs, 2, 128).min(axis=2)
    np.testing.assert_array_equal(k_hat.reshape(2, 256 // gs, gs, 2, 128).min(axis=2), kmin)
    vmin = v.reshape(2, 256, 2, 128 // gs, gs).min(axis=4)
    np.testing.assert_array_equal(v_hat.reshape(2, 256, 2, 128 // gs, gs).min(axis=4), vmin)


def test_dequantize_axes_with_one_hot_parameters():
    """One non-zero scale: exactly the values of that group change, along tokens for K and along channels
    for V."""
    b, S, h, d, gs = 1, 128, 1, 128, 32
    z = lambda *s: np.zeros(s, F32)
    q = O.QuantKV(4, gs, "fp16", np.ones((b, S, h, d), np.uint8), z(b, S // gs, h, d), z(b, S // gs, h, d),
                  np.ones((b, S, h, d), np.uint8), z(b, S, h, d // gs), z(b, S, h, d // gs))
    q.k_scale[0, 2, 0, 17] = 3.0        # token group 2 (tokens 64..95) of channel 17
    q.v_scale[0, 70, 0, 1] = 5.0        # channel group 1 (channels 32..63) of token 70
    k_hat, v_hat = O.dequantize_ref(q)
    want_k = z(b, S, h, d)
    want_k[0, 64:96, 0, 17] = 3.0
    want_v = z(b, S, h, d)
    want_v[0, 70, 0, 32:64] = 5.0
    np.testing.assert_array_equal(k_hat, want_k)
    np.testing.assert_array_equal(v_hat, want_v)


# ------------------------------------------------------------------ "k-tensor" mode
def test_ktensor_mode_quantizes_k_like_v():
    """quant_mode "k-tensor" (qpack.h:378-470): K per token over channel groups -- the V quantizer applied to K."""
    _, k, v = O.make_inputs(2, 2, 2, 128, 0, seed=77)
    a = O.quantize_kv_ref(k, v, 4, 32, "fp16", "k-tensor")
    as_v = O.quantize_kv_ref(v, k, 4, 32)             # K in V's place
    assert a.k_scale.shape == (2, 128, 2, 4)
    np.testing.assert_array_equal(a.k_codes, as_v.v_codes)
    np.testing.assert_array_equal(a.k_scale, as_v.v_scale)
    np.testing.assert_array_equal(a.k_zero, as_v.v_zero)
    np.testing.assert_array_equal(a.v_codes, O.quantize_kv_ref(k, v, 4, 32).v_codes)     # V is untouched by the mode
    # hand-computed token: channels 0..31 hold 0, 1, ..., 15, 0, ... -> range 15, scale 1, codes = values
    k2 = np.zeros((1, 128, 1, 128), F32)
    k2[0, 5, 0, :16] = np.arange(16)
    k2[0, 5, 0, 40] = 30.0                            # another channel group of the same token: range 30, scale 2
    b_ = O.quantize_kv_ref(k2, k2, 4, 32, "fp16", "k-tensor")
    assert b_.k_codes[0, 5, 0, :16].tolist() == list(range(16)) and b_.k_scale[0, 5, 0, 0] == 1.0
    assert b_.k_codes[0, 5, 0, 40] == 15 and b_.k_scale[0, 5, 0, 1] == 2.0 and np.count_nonzero(b_.k_scale) == 2
    k_hat, _ = O.dequantize_ref(b_)
    np.testing.assert_array_equal(k_hat, k2)


def test_ktensor_dequantize_axis_with_one_hot_parameters():
    b, S, h, d, gs = 1, 128, 1, 128, 32
    z = lambda *s: np.zeros(s, F32)
    q = O.QuantKV(4, gs, "fp16", np.ones((b, S, h, d), np.uint8), z(b, S, h, d // gs), z(b, S, h, d // gs),
                  np.zeros((b, S, h, d), np.uint8), z(b, S, h, d // gs), z(b, S, h, d // gs), "k-tensor")
    q.k_scale[0, 70, 0, 2] = 3.0        # channel group 2 (channels 64..95) of token 70
    q.k_zero[0, 9, 0, 0] = -1.0
    k_hat, _ = O.dequantize_ref(q)
    want = z(b, S, h, d)
    want[0, 70, 0, 64:96] = 3.0
    want[0, 9, 0, 0:32] = -1.0
    np.testing.assert_array_equal(k_hat, want)


# ------------------------------------------------------------------ second witness (C restatement)
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("bits,gs", [(4, 128), (4, 32), (2, 64), (2, 128)])
def test_numpy_and_c_restatements_agree_bitwise(bits, gs, dtype):
    _, k, v = O.make_inputs(2, 4, 2, 256, 0, seed=bits + gs, dtype=dtype)
    k[0, :gs, 0, 3] = 0.75                       # constant group
    a = O.quantize_kv_ref(k, v, bits, gs, dtype)
    c = C.quantize_kv_c(k, v, bits, gs, dtype)
    for name in ("k_codes", "k_scale", "k_zero", "v_codes", "v_scale", "v_zero"):
        np.testing.assert_array_equal(getattr(a, name), getattr(c, name), err_msg=name)


def test_torch_oracle_matches_numpy_oracle():
    import torch
    from oracle import torch_oracle as TO
    q, k, v = O.make_inputs(1, 8, 2, 512, 64, seed=4)
    a = O.quantize_kv_ref(k[:, :512], v[:, :512], 4, 128)
    t = TO.quantize_kv(torch.from_numpy(k[:, :512]), torch.from_numpy(v[:, :512]), 4, 128, torch.float16)
    np.testing.assert_array_equal(a.k_codes, t.k_codes.numpy())
    np.testing.assert_array_equal(a.v_codes, t.v_codes.numpy())
    np.testing.assert_array_equal(a.k_scale, t.k_scale.float().numpy())
    np.testing.assert_array_equal(a.v_zero, t.v_zero.float().numpy())
    kh, vh = O.dequantize_ref(a)
    want, _ = O.attend_ref(q, kh, vh, 0.0884, k[:, 512:], v[:, 512:])
    got = TO.dequant_attend(torch.from_numpy(q), t, 0.0884, torch.from_numpy(k[:, 512:]),
                            torch.from_numpy(v[:, 512:])).numpy()
    np.testing.assert_allclose(got, want, atol=2e-6)


# ------------------------------------------------------------------ attention
def test_attend_reduces_to_textbook_softmax_and_gqa_mapping():
    """Against the reference's own three-line attention (evaluation/test.py:12-36) restated with
    einsum on repeated K/V: q head hq must use kv head hq // g (repeat 'b s h d -> b s (h g) d')."""
    rng = np.random.default_rng(5)
    b, h, hk, S, d = 2, 8, 2, 37, 128
    g = h // hk
    q = rng.standard_normal((b, 1, h, d), dtype=F32)
    k = rng.standard_normal((b, S, hk, d), dtype=F32)
    v = rng.standard_normal((b, S, hk, d), dtype=F32)
    out, lse = O.attend_ref(q, k, v, 1 / math.sqrt(d))
    krep, vrep = np.repeat(k, g, axis=2), np.repeat(v, g, axis=2)
    s = np.einsum("bthd,bshd->bhts", q / math.sqrt(d), krep).astype(np.float64)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = np.einsum("bhts,bshd->bthd", p, vrep)
    np.testing.assert_allclose(out, want, atol=3e-6)
    want_lse = np.log(np.exp(s - s.max(-1, keepdims=True)).sum(-1)) + s.max(-1)
    np.testing.assert_allclose(lse, want_lse[:, :, 0], atol=1e-5)


def test_attend_c_witness_and_masks():
    q, k, v = O.make_inputs(3, 8, 2, 256, 64, seed=6)
    qkv = O.quantize_kv_ref(k[:, :256], v[:, :256], 4, 64)
    kh, vh = O.dequantize_ref(qkv)
    seqlens = np.array([256, 128, 0], np.int32)
    reslens = np.array([64, 5, 0], np.int32)
    a, la = O.attend_ref(q, kh, vh, 0.09, k[:, 256:], v[:, 256:], seqlens, reslens)
    c, lc = C.attend_c(q, qkv, 0.09, k[:, 256:], v[:, 256:], seqlens, reslens)
    np.testing.assert_allclose(a, c, atol=3e-6)
    np.testing.assert_allclose(la[:2], lc[:2], atol=2e-5)
    assert np.isneginf(la[2]).all() and not a[2].any()            # empty row: out 0, lse -inf


def test_split_combine_is_invariant_to_split_count():
    """Splitting the keys into n parts and combining (flash_fwd_kernel.h:1217-1298) reproduces the
    unsplit attention for every n, including empty splits."""
    rng = np.random.default_rng(7)
    S, d, h = 300, 128, 4
    q = rng.standard_normal((1, 1, h, d), dtype=F32)
    k = rng.standard_normal((1, S, h, d), dtype=F32) * F32(2)
    v = rng.standard_normal((1, S, h, d), dtype=F32)
    want, want_lse = O.attend_ref(q, k, v, 0.1)
    for n in (1, 2, 3, 7, 128):
        per = -(-S // n)
        outs, lses = [], []
        for i in range(n):
            sl = slice(min(S, i * per), min(S, (i + 1) * per))
            if sl.start == sl.stop:
                outs.append(np.zeros((1, 1, h, d), F32))
                lses.append(np.full((1, h), -np.inf, F32))
            else:
                o, l = O.attend_ref(q, k[:, sl], v[:, sl], 0.1)
                outs.append(o)
                lses.append(l)
        o, l = O.lse_combine_ref(np.stack([x[:, 0] for x in outs]), np.stack(lses))
        np.testing.assert_allclose(o, want[:, 0], atol=2e-6, err_msg=str(n))
        np.testing.assert_allclose(l, want_lse, atol=2e-5)


def test_combine_all_empty_gives_zero_and_plus_inf():
    o, l = O.lse_combine_ref(np.zeros((3, 2, 128), F32), np.full((3, 2), -np.inf, F32))
    assert not o.any() and np.isposinf(l).all()


# ------------------------------------------------------------------ split heuristic known answers
def test_num_splits_heuristic_known_answers():
    # decode_api.cpp:228-233: 48 blocks on 108 SMs -> 2 splits (efficiency 0.89), not 3 (0.67)
    assert O.num_splits_heuristic_ref(48, 108, 64, 128) == 2
    # decode_api.cpp:236: enough blocks to almost fill the SMs -> 1
    assert O.num_splits_heuristic_ref(87, 108, 64, 128) == 1
    # never more splits than key blocks
    assert O.num_splits_heuristic_ref(1, 216, 3, 128) <= 3
    # the reference's own call for its S=4096 MHA test on a 108-SM part: b*h = 32, 2*SMs, 32 n-blocks
    n = O.num_splits_heuristic_ref(32, 216, 32, 128)
    assert 1 <= n <= 32 and (32 * n / 216) / math.ceil(32 * n / 216) >= 0.85 * 0.89


def test_algorithmic_bytes_match_published_table():
    # published figures for the four fixed-shape benchmark configurations: 19 939 328, 36 192 256, 84 426 752, 306 446 336
    assert O.algorithmic_bytes(1, 32, 32, 4096, 128, 4, 128) == 19_939_328
    assert O.algorithmic_bytes(1, 32, 8, 32768, 128, 4, 128) == 36_192_256
    assert O.algorithmic_bytes(1, 32, 8, 131072, 128, 2, 64) == 84_426_752
    assert O.algorithmic_bytes(8, 64, 8, 8 * 65536, 8 * 128, 2, 128) == 306_446_336


def test_roundf_equals_floor_of_biased_sum_for_nonnegative_values():
    """The pack kernel computes roundf(t), t >= 0, as floor(t + 0.49999997f) in fp32.  Checked against
    round-half-away for every float in [0.25, 16.5] and a sweep of smaller ones."""
    c = np.nextafter(np.float32(0.5), np.float32(0))
    assert c == np.float32(0.49999997)
    lo, hi = np.float32(0.25).view(np.uint32), np.float32(16.5).view(np.uint32)
    for start in range(int(lo), int(hi) + 1, 1 << 24):
        t = np.arange(start, min(start + (1 << 24), int(hi) + 1), dtype=np.uint32).view(np.float32)
        fl = np.floor(t)
        want = fl + ((t - fl) >= np.float32(0.5))
        np.testing.assert_array_equal(np.floor((t + c).astype(np.float32)), want)
        np.testing.assert_array_equal(want, O.roundf(t))
    small = np.arange(0, int(lo), 4099, dtype=np.uint32).view(np.float32)
    np.testing.assert_array_equal(np.floor((small + c).astype(np.float32)), np.zeros_like(small))


def test_zero_minimum_takes_the_sign_of_a_negative_zero():
    """A group whose minimum is zero and that holds a -0 stores zero = -0 whatever the order of its
    elements (numpy and C restatements agree); value, scale and codes do not depend on the sign."""
    x = np.array([[0.0, 1.0, -0.0, 3.0], [-0.0, 1.0, 0.0, 3.0], [0.0, 1.0, 0.0, 3.0]], np.float32)
    codes, scale, zero = O.quantize_group(x, 4, axis=1)
    assert np.signbit(zero[:, 0]).tolist() == [True, True, False]
    np.testing.assert_array_equal(codes, np.tile(np.array([0, 5, 0, 15], np.uint8), (3, 1)))
    k = np.zeros((1, 128, 1, 128), np.float32)
    k[0, :, 0, :] = np.linspace(0, 2, 128, dtype=np.float32)[:, None]
    k[0, 5, 0, 3] = -0.0
    k[0, 0, 0, 3] = 0.0
    k = O.round_to_storage(k, "fp16")
    a = O.quantize_kv_ref(k, k, 4, 128)
    c = C.quantize_kv_c(k, k, 4, 128, "fp16")
    assert np.signbit(a.k_zero[0, 0, 0, 3]) and not np.signbit(a.k_zero[0, 0, 0, 4])
    np.testing.assert_array_equal(np.signbit(a.k_zero), np.signbit(c.k_zero))
    np.testing.assert_array_equal(np.signbit(a.v_zero), np.signbit(c.v_zero))


def test_round_to_bf16_equals_the_library_conversion():
    """round_to_bf16 (the oracle's storage rounding for bf16 inputs, scales and zeros) against an independent
    implementation: torch's fp32 -> bf16 conversion (round to nearest, ties to even), on random values over
    the whole exponent range, on exact ties with an even and an odd neighbour below, on values around the
    largest finite bf16, on subnormals, zeros and infinities."""
    import torch
    rng = np.random.default_rng(5)
    bits = rng.integers(0, 1 << 32, size=1 << 20, dtype=np.uint64).astype(np.uint32)
    rand = bits.view(np.float32)
    rand = rand[np.isfinite(rand)]
    # exact ties: upper 16 bits arbitrary, lower 16 bits = 0x8000; both parities of bit 16 occur
    hi = rng.integers(0, 1 << 16, size=1 << 16, dtype=np.uint64).astype(np.uint32)
    ties = ((hi << 16) | np.uint32(0x8000)).view(np.float32)
    ties = ties[np.isfinite(ties)]
    near = (((hi << 16) | np.uint32(0x7FFF)).view(np.float32), ((hi << 16) | np.uint32(0x8001)).view(np.float32))
    edge = np.array([0.0, -0.0, np.inf, -np.inf, 3.3895314e38, 3.4e38, -3.4e38, 1e-40, -1e-40, 1.0, 1.00390625,
                     1.01171875, 65504.0, 6.1e-5], dtype=np.float32)
    x = np.concatenate([rand, ties, near[0][np.isfinite(near[0])], near[1][np.isfinite(near[1])], edge])
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).to(torch.float32).numpy()
    got = O.round_to_bf16(x)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.isnan(O.round_to_bf16(np.array([np.nan], np.float32))[0])
