"""Pins the CPU oracle against closed forms, invariants and the literal
vectors the reference's own tests and docstrings hold."""
from fractions import Fraction

import numpy as np
import pytest

from oracle import marlin_oracle as mo


# ---------------------------------------------------------------- ScalarType
def test_scalar_type_ids_closed_form():
    # exponent[0:8] mantissa[8:16] signed[16] bias[17:49] finite[49] nan_repr[50:58]
    assert mo.UINT4B8_ID == (4 << 8) | (8 << 17) | (1 << 50) == 1125899907892224
    assert mo.UINT4_ID == (4 << 8) | (1 << 50) == 1125899906843648
    assert mo.UINT8B128_ID == (8 << 8) | (128 << 17) | (1 << 50) == 1125899923621888


@pytest.mark.parametrize("mant,signed,bias,lo,hi", [
    # rows of tests/test_scalartype.py:10-25 that are integer types
    (4, False, 0, 0, 15),      # uint4
    (4, False, 8, -8, 7),      # uint4b8
    (8, False, 128, -128, 127),  # uint8b128
    (3, True, 0, -8, 7),       # int4
    (7, True, 0, -128, 127),   # int8
])
def test_scalar_type_min_max(mant, signed, bias, lo, hi):
    assert mo.scalar_type_min_max(mant, signed, bias) == (lo, hi)


# ---------------------------------------------------------------- packings
def _brute_pack_rows(q):
    k, n = q.shape
    out = [[0] * n for _ in range(k // 8)]
    for kk in range(k):
        for nn in range(n):
            out[kk // 8][nn] |= int(q[kk, nn]) << (4 * (kk % 8))
    return np.array(out, dtype=np.uint32).view(np.int32)


def _brute_awq_pack(q):
    k, n = q.shape
    order = [0, 2, 4, 6, 1, 3, 5, 7]
    out = [[0] * (n // 8) for _ in range(k)]
    for kk in range(k):
        for w in range(n // 8):
            for p in range(8):
                out[kk][w] |= int(q[kk, 8 * w + order[p]]) << (4 * p)
    return np.array(out, dtype=np.uint32).view(np.int32)


def test_packings_brute_force_and_inverse():
    rng = np.random.default_rng(0)
    q = rng.integers(0, 16, size=(32, 64), dtype=np.int32)
    assert np.array_equal(mo.pack_rows(q), _brute_pack_rows(q))
    assert np.array_equal(mo.awq_pack(q), _brute_awq_pack(q))
    assert np.array_equal(mo.unpack_rows(mo.pack_rows(q)), q)
    assert np.array_equal(mo.unpack_cols(mo.pack_cols(q)), q)
    assert np.array_equal(mo.awq_unpack(mo.awq_pack(q)), q)
    # top nibble set: sign bit of the int32 word must survive
    q[:] = 15
    assert np.array_equal(mo.unpack_rows(mo.pack_rows(q)), q)
    assert mo.pack_rows(q).dtype == np.int32 and mo.pack_rows(q)[0, 0] == -1


# ---------------------------------------------------------------- Marlin layout
def test_weight_perm_is_bijection():
    perm = mo.marlin_weight_perm_recipe()
    assert perm.shape == (1024,)
    assert np.array_equal(np.sort(perm), np.arange(1024))


@pytest.mark.parametrize("k,n", [(16, 64), (32, 128), (128, 256), (1024, 448)])
def test_marlin_layout_two_derivations_agree(k, n):
    rng = np.random.default_rng(k * 131 + n)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    a = mo.marlin_pack_recipe(q)
    b = mo.marlin_pack_closed_form(q)
    assert a.shape == (k // 16, 2 * n) and a.dtype == np.int32
    assert np.array_equal(a, b)
    assert np.array_equal(mo.marlin_unpack(a, k, n), q)


def test_marlin_layout_single_nibble_positions():
    """One-hot inputs: the nibble of W[r][c] lands exactly where the closed
    form of the layout says (word lane*4+j, lane = 4*(c%8) + (r%8)//2, slot from
    {r%2, r//8, (c%16)//8})."""
    k, n = 16, 64
    for r in range(16):
        for c in range(64):
            q = np.zeros((k, n), dtype=np.int32)
            q[r, c] = 0xF
            w = mo.marlin_pack_recipe(q).view(np.uint32).ravel()
            (idx,) = np.nonzero(w)
            assert idx.size == 1
            j, cc = divmod(c, 16)
            lane = 4 * (cc % 8) + (r % 8) // 2
            slot = (r // 8) + 2 * (cc // 8) + 4 * (r % 2)
            assert idx[0] == lane * 4 + j
            assert w[idx[0]] == 0xF << (4 * slot)


def test_repack_identities():
    rng = np.random.default_rng(5)
    k, n = 256, 192
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    g = mo.gptq_marlin_repack(mo.gptq_pack(q), None, k, n)
    a = mo.awq_marlin_repack(mo.awq_pack(q), k, n)
    assert np.array_equal(g, a)
    perm = rng.permutation(k).astype(np.int32)
    with_perm = mo.gptq_marlin_repack(mo.gptq_pack(q), perm, k, n)
    pre_perm = mo.gptq_marlin_repack(mo.gptq_pack(q[perm]), None, k, n)
    assert np.array_equal(with_perm, pre_perm)
    assert np.array_equal(mo.gptq_marlin_repack(mo.gptq_pack(q), np.empty(0, np.int32), k, n), g)


# ---------------------------------------------------------------- scale / zp / bias
def test_scale_perm_tables():
    assert list(mo.SCALE_PERM[:10]) == [0, 8, 16, 24, 32, 40, 48, 56, 1, 9]
    assert list(mo.SCALE_PERM_SINGLE[:10]) == [0, 1, 8, 9, 16, 17, 24, 25, 2, 3]
    assert np.array_equal(np.sort(mo.SCALE_PERM), np.arange(64))
    assert np.array_equal(np.sort(mo.SCALE_PERM_SINGLE), np.arange(32))


def test_scale_zp_bias_round_trip():
    rng = np.random.default_rng(7)
    k, n, g = 512, 256, 128
    s = rng.uniform(1e-3, 1e-2, size=(k // g, n)).astype(np.float32)
    sp = mo.marlin_permute_scales(s, k, n, g)
    # 8x8 transpose inside every 64 columns
    assert sp[1, 8 * 3 + 5] == s[1, 3 + 8 * 5]
    assert np.array_equal(mo.marlin_unpermute_scales(sp, k, n, g), s)
    s1 = s[:1]
    sp1 = mo.marlin_permute_scales(s1, k, n, -1)
    assert sp1[0, 1] == s1[0, 1] and sp1[0, 2] == s1[0, 8]
    assert np.array_equal(mo.marlin_unpermute_scales(sp1, k, n, -1), s1)
    b = rng.standard_normal(n).astype(np.float32)
    assert np.array_equal(mo.marlin_unpermute_bias(mo.marlin_permute_bias(b)), b)
    zp = rng.integers(0, 16, size=(k // g, n), dtype=np.int32)
    zpp = mo.marlin_zero_points(zp, k // g, n)
    assert zpp.shape == (k // g, n // 8) and zpp.dtype == np.int32
    assert np.array_equal(mo.marlin_unpack_zero_points(zpp, k // g, n), zp)
    assert np.array_equal(mo.awq_to_marlin_zero_points(mo.awq_pack(zp), k // g, n), zpp)


def test_zero_point_slot_closed_form():
    """Column nl of a 64-column block sits in word nl%8 of the block at slot
    [0,4,1,5,2,6,3,7][nl//8] (derived from scale_perm then the 8-interleave)."""
    inv = [0, 4, 1, 5, 2, 6, 3, 7]
    for nl in range(64):
        zp = np.zeros((1, 64), dtype=np.int32)
        zp[0, nl] = 0xF
        w = mo.marlin_zero_points(zp, 1, 64).view(np.uint32).ravel()
        (idx,) = np.nonzero(w)
        assert idx.size == 1 and idx[0] == nl % 8
        assert w[idx[0]] == 0xF << (4 * inv[nl // 8])


# ---------------------------------------------------------------- gfx950 layout
@pytest.mark.parametrize("k,n", [(32, 64), (128, 128), (4096, 256)])
def test_gfx950_layout_round_trip(k, n):
    rng = np.random.default_rng(k + n)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    p = mo.gfx950_pack(q)
    assert p.size == k * n // 8
    assert np.array_equal(mo.gfx950_unpack(p, k, n), q)
    assert np.array_equal(mo.marlin_to_gfx950(mo.marlin_pack(q), k, n), p)


def test_gfx950_layout_word_positions():
    k, n = 64, 128
    for (r, c) in [(0, 0), (1, 0), (7, 15), (8, 16), (31, 63), (32, 64), (45, 101), (63, 127)]:
        q = np.zeros((k, n), dtype=np.int32)
        q[r, c] = 0xF
        w = mo.gfx950_pack(q).view(np.uint32)
        (idx,) = np.nonzero(w)
        assert idx.size == 1
        strip, cl = divmod(c, 64)
        chunk, rl = divmod(r, 32)
        j, l = divmod(cl, 16)
        kb, t = divmod(rl, 8)
        lane = 16 * kb + l
        assert idx[0] == ((strip * (k // 32) + chunk) * 64 + lane) * 4 + j
        slot = (t // 2) + 4 * (t % 2)
        assert w[idx[0]] == 0xF << (4 * slot)


# ---------------------------------------------------------------- dequant
def _rne_fraction_to(dtype, value: Fraction) -> float:
    """Exact rational -> nearest-even representable value of dtype, by
    searching the two neighbours around the float64 approximation."""
    if value == 0:
        return 0.0
    mant_bits = 10 if dtype == "fp16" else 7
    min_exp = -14 if dtype == "fp16" else -126
    sign = -1 if value < 0 else 1
    v = abs(value)
    import math
    e = math.floor(math.log2(float(v)))
    while Fraction(2) ** e > v:
        e -= 1
    while Fraction(2) ** (e + 1) <= v:
        e += 1
    e = max(e, min_exp)
    ulp = Fraction(2) ** (e - mant_bits)
    qf = v / ulp
    lo = qf.numerator // qf.denominator
    rem = qf - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    return sign * float(lo * ulp)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_dequant_exhaustive_against_exact_rationals(dtype):
    rng = np.random.default_rng(11)
    raw = np.concatenate([
        rng.uniform(1e-3, 1e-2, 64), rng.uniform(1e-6, 1.0, 32),
        np.array([0.0, 1.0, 2.0 ** -14, 2.0 ** -20, 3.0e-5, 0.333, 100.0])])
    s = mo.round_to_dtype(raw.astype(np.float32), dtype)
    q = np.tile(np.arange(16, dtype=np.int32)[:, None], (1, s.size))
    w = mo.dequantize(q, s[None, :], -1, dtype)
    zeros = np.full((1, s.size), 3, dtype=np.int32)
    wz = mo.dequantize(q, s[None, :], -1, dtype, zeros=zeros)
    for j, sv in enumerate(s):
        for code in range(16):
            want = _rne_fraction_to(dtype, Fraction(code - 8) * Fraction(float(sv)))
            assert w[code, j] == np.float32(want), (dtype, code, sv)
            want = _rne_fraction_to(dtype, Fraction(code - 3) * Fraction(float(sv)))
            assert wz[code, j] == np.float32(want)
    assert np.all(w[8] == 0)           # code 8 is zero for uint4b8
    assert np.all(w[:, s == 0] == 0)   # zero scale (tile padding) gives zero


def test_bf16_rounding_ties_to_even():
    # 1 + 2^-8 is exactly between 1.0 and 1 + 2^-7 -> even mantissa (1.0)
    x = np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, -(1.0 + 2.0 ** -8)], dtype=np.float32)
    assert list(mo.round_to_dtype(x, "bf16")) == [1.0, 1.0 + 2.0 ** -6, -1.0]
    assert mo.f32_to_bf16_bits(np.array([1.0], np.float32))[0] == 0x3F80


def test_dequant_grouping_and_act_order():
    layer = mo.make_layer(3, 256, 64, 128, "fp16", act_order=True)
    w = mo.dequantize(layer["q"], layer["scales"], 128, "fp16", g_idx=layer["g_idx"])
    k = 17
    g = layer["g_idx"][k]
    want = mo.round_to_dtype((layer["q"][k] - 8).astype(np.float32) * layer["scales"][g], "fp16")
    assert np.array_equal(w[k], want)
    # sorting rows by group and using contiguous groups is the same matrix, permuted
    gs, order = mo.stable_sort_g_idx(layer["g_idx"])
    w_sorted = mo.dequantize(layer["q"][order], layer["scales"], 128, "fp16")
    assert np.array_equal(w_sorted, w[order])
    assert np.array_equal(gs, np.arange(256) // 128)


# ---------------------------------------------------------------- GEMM reference
def test_gemm_reference_special_cases():
    k, n, m = 128, 64, 3
    a = mo.make_activations(1, m, k, "fp16")
    # all codes 9, scale 1: W == 1 -> every output column is the row sum of A
    q = np.full((k, n), 9, dtype=np.int32)
    w = mo.dequantize(q, np.ones((1, n), np.float32), -1, "fp16")
    out = mo.gemm_reference(a, w)
    assert np.allclose(out, a.sum(axis=1, keepdims=True).repeat(n, 1), rtol=1e-6, atol=1e-5)
    # a single non-zero row of W picks one column of A
    q = np.full((k, n), 8, dtype=np.int32)
    q[5, :] = 10
    w = mo.dequantize(q, np.full((1, n), 0.5, np.float32), -1, "fp16")
    out = mo.gemm_reference(a, w)
    assert np.allclose(out, a[:, 5:6].repeat(n, 1), rtol=1e-6)
    ok, _, _ = mo.gemm_tolerance_ok(out, out)
    assert ok
    ok, _, _ = mo.gemm_tolerance_ok(out * 1.05, out)
    assert not ok


# ---------------------------------------------------------------- MoE routing
def test_moe_align_docstring_example():
    # fused_moe/moe_align_block_size.py:60-73 (expert ids 1..4 -> 5 experts, 0 unused)
    topk_ids = np.array([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]])
    sorted_ids, expert_ids, post = mo.moe_align_block_size(topk_ids, 4, 5)
    assert list(sorted_ids[:16]) == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert list(expert_ids[:4]) == [1, 2, 3, 4]
    assert post[0] == 16


@pytest.mark.parametrize("m,topk,e,bs", [(1, 2, 8, 8), (16, 2, 8, 8), (133, 3, 12, 16), (64, 2, 8, 64)])
def test_moe_align_invariants(m, topk, e, bs):
    rng = np.random.default_rng(m)
    topk_ids = np.stack([rng.permutation(e)[:topk] for _ in range(m)])
    sorted_ids, expert_ids, post = mo.moe_align_block_size(topk_ids, bs, e)
    numel = m * topk
    assert post[0] % bs == 0
    valid = sorted_ids[:post[0]][sorted_ids[:post[0]] < numel]
    assert np.array_equal(np.sort(valid), np.arange(numel))
    assert np.all(sorted_ids[post[0]:] == numel)
    for b in range(post[0] // bs):
        ids = sorted_ids[b * bs:(b + 1) * bs]
        ids = ids[ids < numel]
        assert ids.size > 0
        assert np.all(topk_ids.reshape(-1)[ids] == expert_ids[b])
    blocks = expert_ids[:post[0] // bs]
    assert np.all(np.diff(blocks) >= 0)
    expect_len = numel + e * (bs - 1)
    if numel < e:
        expect_len = min(numel * bs, expect_len)
    assert sorted_ids.size == expect_len


def test_moe_block_size_rule():
    assert mo.moe_block_size_rule(16, 2, 8) == 8
    assert mo.moe_block_size_rule(4096, 2, 8) == 64
    assert mo.moe_block_size_rule(64, 2, 8) == 32  # 16/8=2, 16/16=1, 16/32=.5


# ---------------------------------------------------------------- 8-bit weights (W8A16)
def test_packings8_brute_force_and_inverse():
    rng = np.random.default_rng(8)
    q = rng.integers(0, 256, size=(16, 5), dtype=np.int32)
    q[3, 2] = 255        # top byte of a word set: sign handling
    p = mo.pack_rows8(q)
    assert p.dtype == np.int32 and p.shape == (4, 5)
    for k in range(16):
        for n in range(5):
            assert ((int(p.view(np.uint32)[k // 4, n]) >> (8 * (k % 4))) & 0xFF) == q[k, n]
    assert np.array_equal(mo.unpack_rows8(p), q)


@pytest.mark.parametrize("k,n", [(16, 64), (64, 128), (128, 320)])
def test_marlin8_layout_two_derivations_agree(k, n):
    rng = np.random.default_rng(k + n)
    q = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    a, b = mo.marlin_pack8_recipe(q), mo.marlin_pack8_closed_form(q)
    assert a.shape == (k // 16, 4 * n) and np.array_equal(a, b)
    assert np.array_equal(mo.marlin_unpack8(a, k, n), q)
    perm = mo.marlin_weight_perm_recipe8()
    assert sorted(perm.tolist()) == list(range(1024))


def test_marlin8_layout_single_byte_positions():
    """One code set at a time: word lane*8 + 2j + half of its tile, byte i with
    row 2*(lane%4) + {0,8,1,9}[i] (gptq_marlin_repack.cu:216-236)."""
    for (row, col) in [(0, 0), (1, 0), (8, 0), (9, 0), (5, 8), (15, 63), (6, 37)]:
        q = np.zeros((16, 64), dtype=np.int32)
        q[row, col] = 0xAB
        u = mo.marlin_pack8(q).view(np.uint32).ravel()
        (word,) = np.nonzero(u)[0]
        j, c16 = col // 16, col % 16
        lane = 4 * (c16 % 8) + (row % 8) // 2
        assert word == lane * 8 + 2 * j + c16 // 8
        byte = [b for b in range(4) if (int(u[word]) >> (8 * b)) & 0xFF][0]
        assert row == 2 * (lane % 4) + (0, 8, 1, 9)[byte]


def test_repack8_identities():
    rng = np.random.default_rng(5)
    k, n = 64, 128
    q = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    packed = mo.pack_rows8(q)
    assert np.array_equal(mo.gptq_marlin_repack8(packed, None, k, n), mo.marlin_pack8(q))
    perm = rng.permutation(k).astype(np.int32)
    assert np.array_equal(mo.gptq_marlin_repack8(packed, perm, k, n), mo.marlin_pack8(q[perm]))


@pytest.mark.parametrize("k,n", [(32, 64), (96, 192)])
def test_gfx950_layout8_round_trip_and_positions(k, n):
    rng = np.random.default_rng(k)
    q = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    g = mo.gfx950_pack8(q)
    assert g.size == k * n // 4
    assert np.array_equal(mo.gfx950_unpack8(g, k, n), q)
    assert np.array_equal(mo.marlin8_to_gfx950(mo.marlin_pack8(q), k, n), g)
    # word ((strip*chunks + c)*2 + h)*256 + lane*4 + j, byte GFX950_BYTE[t]
    u = g.view(np.uint32)
    chunks = k // 32
    for (kk, nn) in [(0, 0), (5, 17), (31, 63), (k - 1, n - 1), (13, 40)]:
        strip, j, l16 = nn // 64, (nn % 64) // 16, nn % 16
        c, r = kk // 32, kk % 32
        kb, h, t = r // 8, (r % 8) // 4, r % 4
        word = ((strip * chunks + c) * 2 + h) * 256 + (16 * kb + l16) * 4 + j
        assert (int(u[word]) >> (8 * int(mo.GFX950_BYTE[t]))) & 0xFF == q[kk, nn]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_dequant8_exhaustive_against_exact_rationals(dtype):
    rng = np.random.default_rng(12)
    raw = np.concatenate([rng.uniform(1e-4, 1e-2, 24), np.array([0.0, 1.0, 2.0 ** -14, 3.0e-5, 0.333])])
    s = mo.round_to_dtype(raw.astype(np.float32), dtype)
    q = np.tile(np.arange(256, dtype=np.int32)[:, None], (1, s.size))
    w = mo.dequantize(q, s[None, :], -1, dtype, num_bits=8)
    for j, sv in enumerate(s):
        for code in range(256):
            want = _rne_fraction_to(dtype, Fraction(code - 128) * Fraction(float(sv)))
            assert w[code, j] == np.float32(want), (dtype, code, sv)
    assert np.all(w[128] == 0)


# ---------------------------------------------------------------- fp8 weights (float8_e4m3fn)
def test_fp8_type_id_and_value_table():
    import torch
    assert mo.FLOAT8_E4M3FN_ID == 4 | (3 << 8) | (1 << 16) | (1 << 49) | (2 << 50) == 2814749767172868
    v = mo.fp8_e4m3fn_values()
    # torch's own conversion of the 254 finite codes (the two NaN codes aside)
    t = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    finite = np.isfinite(t)
    assert finite.sum() == 254 and not finite[0x7F] and not finite[0xFF]
    assert np.array_equal(v[finite], t[finite])
    assert np.array_equal(np.signbit(v[finite]), np.signbit(t[finite]))   # 0x80 is -0
    # hand values: 1, the largest (1.75 * 2^8), the smallest subnormal, the smallest normal, -2
    assert v[0x38] == 1.0 and v[0x7E] == 448.0 and v[0x01] == 2.0 ** -9 and v[0x08] == 2.0 ** -6 and v[0xC0] == -2.0
    assert v[0x7F] == 480.0 and v[0xFF] == -480.0   # what the bit trick makes of the NaN codes


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_fp8_kernel_recipe_equals_value_times_scale(dtype):
    """The code read as a 16-bit float is value * 2^-8 / 2^-120 for every code,
    and the recipe (that reading times the scale with the bias folded in) is
    round-to-nearest-even of value * scale in exact arithmetic."""
    v = mo.fp8_e4m3fn_values()
    shift = mo.FP8_EXPONENT_BIAS_SHIFT[dtype]
    as16 = mo.fp8_code_as_16bit_float(np.arange(256), dtype)
    assert all(Fraction(float(as16[c])) * Fraction(2) ** shift == Fraction(float(v[c])) for c in range(256))
    rng = np.random.default_rng(13)
    raw = np.concatenate([rng.uniform(1e-4, 1e-2, 24), np.array([1.0, 2.0 ** -10, 3.0e-5, 0.333, 0.0])])
    s = mo.round_to_dtype(raw.astype(np.float32), dtype)
    fused = mo.fp8_fuse_exponent_bias(s, dtype)
    assert all(Fraction(float(f)) == Fraction(float(x)) * Fraction(2) ** shift for f, x in zip(fused, s))
    codes = np.tile(np.arange(256, dtype=np.int32)[:, None], (1, s.size))
    w = mo.dequantize_fp8(codes, fused[None, :], -1, dtype)
    for j, sv in enumerate(s):
        for code in range(256):
            want = _rne_fraction_to(dtype, Fraction(float(v[code])) * Fraction(float(sv)))
            assert w[code, j] == np.float32(want), (dtype, code, sv)
    assert np.all(w[0] == 0) and np.all(w[0x80] == 0)


def test_fp8_dequant_groups():
    rng = np.random.default_rng(14)
    codes = rng.integers(0, 256, size=(256, 8), dtype=np.int32)
    s = mo.round_to_dtype(rng.uniform(1e-3, 1e-2, size=(2, 8)).astype(np.float32), "fp16")
    w = mo.dequantize_fp8(codes, mo.fp8_fuse_exponent_bias(s, "fp16"), 128, "fp16")
    v = mo.fp8_e4m3fn_values()
    assert np.array_equal(w[:128], mo.round_to_dtype(v[codes[:128]] * s[0], "fp16"))
    assert np.array_equal(w[128:], mo.round_to_dtype(v[codes[128:]] * s[1], "fp16"))


# ---------------------------------------------------------------- MXFP4 weights (float4_e2m1f, e8m0 scales)
def test_fp4_type_id_values_and_scales():
    import torch
    assert mo.FLOAT4_E2M1F_ID == 2 | (1 << 8) | (1 << 16) | (1 << 49) == 562949953487106
    v = mo.fp4_e2m1_values()
    # the list of the OCP microscaling format, codes 0..7, and its negatives for 8..15
    assert v[:8].tolist() == [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    assert v[8:].tolist() == [-0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0] and np.signbit(v[8])
    # the reference's test recipe (marlin_utils_fp4.py:720-727): sign and the three other bits at
    # the top of a float8_e4m3fn byte, torch's conversion, times 2^6
    code = torch.arange(16, dtype=torch.uint8) << 4
    as_fp8 = ((code & 0x80) | ((code & 0x70) >> 2)).view(torch.float8_e4m3fn).float() * 64
    assert np.array_equal(v, as_fp8.numpy())
    # the kernel's reading: sign at bit 15, the other three bits at bits 11-9 of an fp16, times 2^14
    c = np.arange(16, dtype=np.uint16)
    h = (((c & 8) << 12) | ((c & 7) << 9)).astype(np.uint16).view(np.float16).astype(np.float64)
    assert np.array_equal(h * 2.0 ** 14, v.astype(np.float64))
    e = np.arange(255, dtype=np.uint8)
    t = torch.from_numpy(e).view(torch.float8_e8m0fnu).float().numpy()
    assert np.array_equal(mo.mx_scale_values(e), t)
    assert mo.mx_scale_values(np.array([127, 120, 0]))[:2].tolist() == [1.0, 2.0 ** -7]


def test_mxfp4_dequant_and_scale_reorder():
    rng = np.random.default_rng(15)
    codes = rng.integers(0, 16, size=(64, 8), dtype=np.int32)
    e = rng.integers(100, 130, size=(2, 8)).astype(np.uint8)
    w = mo.dequantize_mxfp4(codes, e)
    v = mo.fp4_e2m1_values()
    for k in (0, 31, 32, 63):
        for n in (0, 7):
            assert w[k, n] == v[codes[k, n]] * 2.0 ** (int(e[k // 32, n]) - 127)
    x = np.arange(16).reshape(2, 8)
    y = mo.mxfp4_process_scales(x)
    assert y[0].tolist() == [0, 2, 1, 3, 4, 6, 5, 7] and np.array_equal(mo.mxfp4_process_scales(y), x)


# ---------------------------------------------------------------- NVFP4 weights (float4_e2m1f, e4m3 scales, global scale)
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_nvfp4_scale_bytes_against_both_kernel_readings(dtype):
    """Every non-negative float8_e4m3fn scale (torch's own conversion on the CPU)
    through nvfp4_process_scales and back through the kernel-side reading of a
    byte (dequant.h:520-549): scale * scale_factor * 2^7, or 0 below 2."""
    import torch
    from fractions import Fraction
    codes = torch.arange(0, 0x7F, dtype=torch.uint8)                 # 0 .. 448, no NaN
    scales = codes.view(torch.float8_e4m3fn).float().numpy().reshape(1, -1)
    scales = np.concatenate([scales, np.zeros((1, 1), np.float32)], axis=1)      # 128 columns
    b, sf = mo.nvfp4_process_scales(scales, dtype)
    assert sf == 1.0   # the largest scale is 448 already
    back = mo.nvfp4_scale_bytes_as_16bit_float(b, dtype).astype(np.float64)
    back = back.reshape(-1, 4)[:, [0, 2, 1, 3]].reshape(back.shape)   # the reorder is its own inverse
    want = np.where(scales.astype(np.float64) * 128 < 2, 0.0, scales.astype(np.float64) * 128)
    assert np.array_equal(back, want)
    # the byte is bits 14..7 of the half-precision number: hand values
    one = mo.nvfp4_process_scales(np.full((1, 4), 1.0, np.float32), "fp16")[0]
    assert int(one[0, 0]) == (int(np.float16(128.0).view(np.uint16)) >> 7)    # 128.0 = 0x5800 -> 0xB0
    assert int(one[0, 0]) == 0xB0
    # kernel scales: value * 2^-bias, exact in the activation type
    ks = mo.nvfp4_kernel_scales(b, dtype)
    bias = mo.NVFP4_EXPONENT_BIAS[dtype]
    assert np.array_equal(ks.astype(np.float64), want * 2.0 ** -bias)
    assert np.array_equal(mo.round_to_dtype(ks, dtype), ks)
    # the whole chain in exact arithmetic: value(code) * kernel scale * processed global scale
    # == value(code) * scale * global scale, for every code and a sample of scales
    g = 0.3712158203125
    pg = mo.nvfp4_process_global_scale(g, dtype, sf)
    assert Fraction(float(pg)) == Fraction(float(np.float32(g))) * Fraction(2) ** (bias - 7)
    v = mo.fp4_e2m1_values()
    for col in (8, 9, 57, 100, 126):
        if want[0, col] == 0:
            continue
        for code in range(16):
            w = mo.dequantize_nvfp4(np.full((16, 128), code), ks, dtype)[0, col]
            assert Fraction(float(w)) * Fraction(float(pg)) == \
                Fraction(float(v[code])) * Fraction(float(scales[0, col])) * Fraction(float(np.float32(g)))


def test_nvfp4_scale_factor_and_small_scales():
    """marlin_utils_fp4.py:37-58, 112-114: bf16 lifts small scales by a power of two
    so that the largest is just below 448 (fp16 never does); what stays below
    2^-6 after that is cut to zero."""
    s = np.array([[0.5, 0.001953125, 3.0, 0.0]], dtype=np.float32)          # 2^-9 is the smallest e4m3 number
    b16, sf16 = mo.nvfp4_process_scales(s, "fp16")
    assert sf16 == 1.0
    back = mo.nvfp4_scale_bytes_as_16bit_float(b16, "fp16")[0, [0, 2, 1, 3]]
    assert back.tolist() == [64.0, 0.0, 384.0, 0.0]                          # 2^-9 * 128 = 0.25 < 2: cut
    b, sf = mo.nvfp4_process_scales(s, "bf16")
    assert sf == 128.0                                                        # 448 / 3 = 149.3 -> 2^7
    back = mo.nvfp4_scale_bytes_as_16bit_float(b, "bf16")[0, [0, 2, 1, 3]]
    assert back.tolist() == [64.0 * 128, 0.25 * 128, 384.0 * 128, 0.0]
    assert mo.nvfp4_scale_factor(np.array([448.0], np.float32), "bf16") == 1.0
    assert float(mo.nvfp4_process_global_scale(2.0, "bf16", 128.0)) == 2.0 * 2.0 ** 119 / 128
    assert float(mo.nvfp4_process_global_scale(2.0, "fp16")) == 2.0 * 2.0 ** 7


def test_moe_activation_closed_forms_and_limits():
    """oracle.moe_activation against values that follow from the formulas without evaluating
    them the same way: alpha = 0 turns every sigmoid into 1/2; a gate or an up value beyond the
    limit gives what the limit gives (gate clamped from above only, up from both sides); the
    +1 of swigluoai and the beta of the clamped SiLU make u = -1 / u = -beta a zero; the
    interleaved order of swigluoai against the packed order of swigluoai_uninterleave with
    alpha 1.702, beta 1; SITU with a huge beta is SiLU; relu2 of a negative is 0."""
    x = np.array([[2.0, -3.0, 0.5, 4.0,    1.5, 2.0, -1.0, 0.25]], dtype=np.float32)       # gate | up
    for dtype in ("fp16", "bf16"):
        half = mo.moe_activation("swigluoai_uninterleave", x, dtype, clamp_limit=100.0, alpha=0.0, beta=0.0)
        assert np.array_equal(half, mo.round_to_dtype(mo.round_to_dtype(x[:, :4] / 2, dtype) * x[:, 4:], dtype))
        with_beta = mo.moe_activation("swigluoai_uninterleave", x, dtype, clamp_limit=100.0, alpha=0.0, beta=1.0)
        assert with_beta[0, 2] == 0.0 and with_beta[0, 0] == 2.5                          # (u + 1): -1 -> 0; 1 * 2.5
        # clamps: gate 9 acts as gate 3 (limit 3) but gate -9 stays; up +-9 act as +-3
        big = np.array([[9.0, -9.0, 1.0, 1.0,   1.0, 1.0, 9.0, -9.0]], dtype=np.float32)
        lim = np.array([[3.0, -9.0, 1.0, 1.0,   1.0, 1.0, 3.0, -3.0]], dtype=np.float32)
        for name, kw in (("silu", dict(clamp_limit=3.0)),
                         ("swigluoai_uninterleave", dict(clamp_limit=3.0, alpha=1.702, beta=1.0))):
            assert np.array_equal(mo.moe_activation(name, big, dtype, **kw), mo.moe_activation(name, lim, dtype, **kw))
        assert not np.array_equal(mo.moe_activation("silu", big, dtype, clamp_limit=3.0),
                                  mo.moe_activation("silu", big, dtype))
        # SILU with a clamp no value reaches is plain SILU
        assert np.array_equal(mo.moe_activation("silu", x, dtype, clamp_limit=50.0), mo.moe_activation("silu", x, dtype))
        # swigluoai: pairs alternate; the same numbers packed, alpha 1.702, beta 1, limit 7: one rounding
        # less in the interleaved kernel, so compare within an ulp
        inter = np.empty_like(x)
        inter[:, 0::2], inter[:, 1::2] = x[:, :4], x[:, 4:]
        a = mo.moe_activation("swigluoai", inter, dtype)
        b = mo.moe_activation("swigluoai_uninterleave", x, dtype, clamp_limit=7.0, alpha=1.702, beta=1.0)
        ulp = 2.0 ** (-9 if dtype == "fp16" else -6)
        assert np.all(np.abs(a - b) <= ulp * np.abs(b)) and a[0, 2] == 0.0
        g = np.float64(2.0)
        assert a[0, 0] == mo.round_to_dtype(np.array([2.5 * g / (1 + np.exp(-1.702 * g))], np.float32), dtype)[0]
        # limits of swigluoai: gate 9 -> 7, up -9 -> -7 (so u + 1 = -6)
        lim7 = mo.moe_activation("swigluoai", np.array([[9.0, -9.0]], np.float32), dtype)
        assert lim7[0, 0] == mo.round_to_dtype(np.array([-6.0 * 7.0 / (1 + np.exp(-1.702 * 7.0))], np.float32), dtype)[0]
        # SITU: beta -> infinity is SiLU(gate) * up in one rounding; linear_beta bounds the up half
        situ = mo.moe_activation("situ", x, dtype, situ_beta=1e6)
        one = mo.round_to_dtype((x[:, :4].astype(np.float64) / (1 + np.exp(-x[:, :4].astype(np.float64)))
                                 * x[:, 4:]).astype(np.float32), dtype)
        assert np.array_equal(situ, one)
        bounded = mo.moe_activation("situ", np.array([[1.0, 50.0]], np.float32), dtype, situ_beta=1e6, situ_linear_beta=2.0)
        assert bounded[0, 0] == mo.round_to_dtype(np.array([2.0 / (1 + np.exp(-1.0))], np.float32), dtype)[0]
        # swiglustep: silu(gate) capped at 7, up within +-7
        step = mo.moe_activation("swiglustep", np.array([[20.0, 1.0, 9.0, -9.0]], np.float32), dtype)
        assert step[0, 0] == 49.0 and step[0, 1] == mo.round_to_dtype(np.array([-7.0 / (1 + np.exp(-1.0))], np.float32), dtype)[0]
        # gelu: 0 -> 0, large -> identity; the tanh form agrees with erf to 1e-3
        ge = mo.moe_activation("gelu", np.array([[0.0, 8.0, 1.0, 1.0, 3.0, 0.5, 1.0, 1.0]], np.float32), dtype)
        assert ge[0, 0] == 0.0 and ge[0, 1] == 4.0
        assert abs(float(mo.moe_activation("gelu_tanh", x, dtype)[0, 0]) - float(mo.moe_activation("gelu", x, dtype)[0, 0])) < 1e-2
        # no gate
        r2 = mo.moe_activation("relu2_no_mul", np.array([[-2.0, 3.0]], np.float32), dtype)
        assert r2.tolist() == [[0.0, 9.0]]
        assert mo.moe_activation("silu_no_mul", np.array([[0.0]], np.float32), dtype)[0, 0] == 0.0


def test_moe_gemm_reference_against_per_slot_brute_force():
    """moe_gemm_reference (the oracle of the grouped GEMM) follows sorted_ids / expert_ids
    block by block.  Brute force from the routing itself, slot by slot, without any of
    that bookkeeping: C[t * top_k + j] = A[t] @ W[topk_ids[t][j]], rounded, times the
    rounded routing weight, rounded.  Integer-valued matrices keep every product and sum
    exact in fp32, so the two must agree exactly; a wrong row index (id % top_k for
    id // top_k), a wrong expert, a dropped rounding of the weight or a block that is
    skipped or written twice all show."""
    rng = np.random.default_rng(11)
    m, e, top_k, k, n, bs = 13, 5, 3, 16, 8, 4
    a = rng.integers(-4, 5, size=(m, k)).astype(np.float32)
    w = [rng.integers(-3, 4, size=(k, n)).astype(np.float32) for _ in range(e)]
    topk_ids = np.stack([rng.permutation(e)[:top_k] for _ in range(m)]).astype(np.int32)
    weights = rng.random((m, top_k)).astype(np.float32)
    sorted_ids, expert_ids, past = mo.moe_align_block_size(topk_ids, bs, e)
    for dtype in ("fp16", "bf16"):
        for tw in (None, weights):
            got = mo.moe_gemm_reference(a, w, sorted_ids, expert_ids, int(past[0]), bs, top_k, m, tw, dtype)
            want = np.zeros((m * top_k, n), dtype=np.float32)
            for t in range(m):
                for j in range(top_k):
                    row = np.zeros(n, dtype=np.float32)
                    for col in range(n):
                        acc = 0.0
                        for kk in range(k):
                            acc += float(a[t, kk]) * float(w[topk_ids[t, j]][kk, col])
                        row[col] = acc
                    row = mo.round_to_dtype(row, dtype)
                    if tw is not None:
                        wt = mo.round_to_dtype(np.array([tw[t, j]], dtype=np.float32), dtype)[0]
                        row = mo.round_to_dtype(row * wt, dtype)
                    want[t * top_k + j] = row
            assert np.array_equal(got, want), (dtype, tw is None)
    # a block whose expert is not on this rank (-1) and slots past the padded total write nothing
    expert_ids2 = expert_ids.copy()
    expert_ids2[0] = -1
    got = mo.moe_gemm_reference(a, w, sorted_ids, expert_ids2, int(past[0]), bs, top_k, m, None, "fp16")
    dropped = sorted_ids[:bs]
    dropped = dropped[dropped < m * top_k]
    assert np.all(got[dropped] == 0) and dropped.size > 0
    kept = np.setdiff1d(np.arange(m * top_k), dropped)
    full = mo.moe_gemm_reference(a, w, sorted_ids, expert_ids, int(past[0]), bs, top_k, m, None, "fp16")
    assert np.array_equal(got[kept], full[kept])


# ------------------------------------------------- 8-bit activations (W4A8)
@pytest.mark.parametrize("k,n", [(32, 64), (96, 128), (160, 192)])
def test_marlin_a8_layout_two_derivations_agree(k, n):
    rng = np.random.default_rng(k + n)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    recipe = mo.marlin_pack_recipe_a8(q)
    closed = mo.marlin_pack_closed_form_a8(q)
    assert recipe.shape == (k // 16, 2 * n)
    assert np.array_equal(recipe, closed)
    assert np.array_equal(mo.marlin_unpack_a8(closed, k, n), q)
    # a different order from the 16-bit one (a mix-up of the two would pass nothing above)
    assert not np.array_equal(closed, mo.marlin_pack(q))
    # the gather table is a permutation of the 1024 tile elements
    perm = mo.marlin_weight_perm_recipe_a8()
    assert sorted(perm.tolist()) == list(range(1024))


def test_marlin_a8_layout_single_positions():
    # one code set at (k, n): the word and nibble the repack kernel's arithmetic gives by hand:
    # tile (k/32, n/32), lane 4*(n%8) + (k%16)/4, warp (n%32)/8, slot 2*(k%4) + (k%32)/16
    for k, n in [(0, 0), (5, 9), (17, 31), (40, 70), (63, 127)]:
        q = np.zeros((64, 128), dtype=np.int32)
        q[k, n] = 15
        w = mo.marlin_pack_a8(q).view(np.uint32).reshape(-1)
        idx = np.nonzero(w)[0]
        assert idx.size == 1
        tile = (k // 32) * (128 // 32) + n // 32
        lane = 4 * (n % 8) + (k % 16) // 4
        warp = (n % 32) // 8
        slot = 2 * (k % 4) + (k % 32) // 16
        assert idx[0] == tile * 128 + lane * 4 + warp
        assert w[idx[0]] == 15 << (4 * slot)


def test_repack_a8_identities_and_gfx950():
    rng = np.random.default_rng(3)
    q = rng.integers(0, 16, size=(64, 128), dtype=np.int32)
    m = mo.marlin_pack_a8(q)
    assert np.array_equal(mo.gptq_marlin_repack_a8(mo.pack_rows(q), 64, 128), m)
    assert np.array_equal(mo.awq_marlin_repack_a8(mo.awq_pack(q), 64, 128), m)
    assert np.array_equal(mo.marlin_a8_to_gfx950(m, 64, 128), mo.gfx950_pack(q))


def test_scales_and_zero_points_a8():
    rng = np.random.default_rng(4)
    s = rng.uniform(1, 2, size=(4, 128)).astype(np.float32)
    p = mo.marlin_permute_scales_a8(s, 512, 128, 128)
    # always the single permutation: equal to the 16-bit channelwise one row by row
    for g in range(4):
        assert np.array_equal(p[g:g + 1], mo.marlin_permute_scales(s[g:g + 1], 128, 128, -1))
    assert np.array_equal(mo.marlin_unpermute_scales_a8(p, 512, 128, 128), s)
    zp = rng.integers(0, 16, size=(4, 128), dtype=np.int32)
    packed = mo.marlin_zero_points_a8(zp, 4, 128)
    assert np.array_equal(mo.marlin_unpack_zero_points_a8(packed, 4, 128), zp)
    # column n of a 64 block: word n % 8, nibble n / 8 (the transpose, no interleave)
    one = np.zeros((1, 64), dtype=np.int32)
    one[0, 19] = 7
    w = mo.marlin_zero_points_a8(one, 1, 64).view(np.uint32).reshape(-1)
    assert w[19 % 8] == 7 << (4 * (19 // 8)) and np.count_nonzero(w) == 1
    assert np.array_equal(mo.awq_to_marlin_zero_points_a8(mo.awq_pack(zp), 4, 128), packed)


def test_int4_fp8_preprocess_formulas_and_inverse():
    # the two formulas of tests/kernels/quantization/test_marlin_gemm.py:148-188
    q = np.arange(16, dtype=np.int32).reshape(16, 1)
    assert mo.int4_fp8_preprocess(q).reshape(-1).tolist() == \
        [15, 14, 13, 12, 11, 10, 9, 8, 0, 1, 2, 3, 4, 5, 6, 7]
    assert np.array_equal(mo.int4_fp8_preprocess_inverse(mo.int4_fp8_preprocess(q)), q)
    rng = np.random.default_rng(5)
    qq = rng.integers(0, 16, size=(64, 8), dtype=np.int32)
    zz = rng.integers(0, 16, size=(2, 8), dtype=np.int32)
    want = qq - np.repeat(zz, 32, axis=0)
    want[want < 0] = (15 - qq)[want < 0]
    assert np.array_equal(mo.int4_fp8_preprocess(qq, zz, 32), want)
    # sign and magnitude: the kernel reads nibble p as -(8 - q) = -((p & 7) + 1) when p >= 8
    p = mo.int4_fp8_preprocess(q).reshape(-1)
    value = np.where(p < 8, p, -((p & 7) + 1))
    assert np.array_equal(value, np.arange(16) - 8)


def test_per_token_quant_int8_hand_values_and_bound():
    x = np.array([[127.0, -63.5, 0.4, -0.5], [1e-12, 0, 0, 0], [2.0, 1.0, -1.0, 0.5]], dtype=np.float32)
    codes, scale = mo.per_token_quant_int8(x)
    assert codes[0].tolist() == [127, -64, 0, -1]          # halves round away from zero
    assert np.isclose(scale[0, 0], 1.0)
    assert scale[1, 0] == np.float32(1e-10) / np.float32(127)  # the floor of absmax
    assert codes[2].tolist() == [127, 64, -64, 32]          # 63.5 -> 64, 31.75 -> 32
    rng = np.random.default_rng(6)
    y = rng.normal(size=(8, 256)).astype(np.float32)
    c, s = mo.per_token_quant_int8(y)
    assert np.all(np.abs(y - c.astype(np.float32) * s) <= s * 0.5001)
    assert np.all(np.max(np.abs(c), axis=1) == 127)


def test_marlin_act_int8_process_scales():
    s = np.array([[0.5, 1.0], [0.25, 0.1234]], dtype=np.float32)
    ints, factor = mo.marlin_act_int8_process_scales(s)
    assert ints.tolist() == [[2048, 4096], [1024, 505]]     # 0.1234 * 4096 = 505.4
    assert factor == np.float32(1.0 / 4096)


@pytest.mark.parametrize("group_size,zp", [(-1, False), (32, False), (64, True), (128, True)])
def test_gemm_w4a8_int8_against_python_loop(group_size, zp):
    rng = np.random.default_rng(7 + (group_size % 97))
    m, k, n = 3, 128, 8
    a = rng.integers(-127, 128, size=(m, k)).astype(np.int8)
    a_s = rng.uniform(1e-6, 2e-6, size=(m, 1)).astype(np.float32) * (1e3 if group_size == -1 else 1)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    gs = k if group_size == -1 else group_size
    groups = k // gs
    zeros = rng.integers(0, 16, size=(groups, n), dtype=np.int32) if zp else None
    if group_size == -1:
        scales = mo.round_to_dtype(rng.uniform(1e-3, 1e-2, size=(1, n)).astype(np.float32), "fp16")
    else:
        scales = rng.integers(1, 4097, size=(groups, n)).astype(np.int16)
    got = mo.gemm_w4a8_int8(a, a_s, q, group_size, scales, "fp16", zeros)
    for mm in range(m):
        for nn in range(n):
            total = 0
            for g in range(groups):
                part = 0
                for kk in range(g * gs, (g + 1) * gs):
                    z = 8 if zeros is None else int(zeros[g, nn])
                    part += int(a[mm, kk]) * (int(q[kk, nn]) - z)
                total += part * (int(scales[g, nn]) if group_size != -1 else 1)
            want = np.float32(total) * a_s[mm, 0]
            if group_size == -1:
                want = want * scales[0, nn]
            assert np.isfinite(got[mm, nn]) and got[mm, nn] != 0
            assert got[mm, nn] == np.float32(want).astype(np.float16).astype(np.float32)


def test_moe_gemm_w4a8_int8_against_per_slot_loop():
    """moe_gemm_w4a8_int8 (the checker of the grouped W4A8 GPU tests) walks sorted_ids /
    expert_ids block by block.  The same result from the routing alone, one routed slot at a
    time in plain Python integers: C[t * top_k + j] = (sum_g s[e][g][n] * sum_{k in g}
    a[t][k] * (q[e][k][n] - z)) * a_scale[t] for e = topk_ids[t][j], rounded, times the rounded
    routing weight, rounded.  A wrong row (id % top_k for id // top_k), a wrong expert, the
    activation scale of another row, a block skipped or written twice, or the routing weight
    applied before the rounding all fail it."""
    rng = np.random.default_rng(21)
    m, e, top_k, k, n, bs, gs = 9, 4, 2, 64, 8, 8, 32
    a = rng.integers(-127, 128, size=(m, k)).astype(np.int8)
    a_s = rng.uniform(1e-6, 2e-6, size=(m, 1)).astype(np.float32)
    experts = []
    for _ in range(e):
        experts.append(dict(q=rng.integers(0, 16, size=(k, n), dtype=np.int32), group_size=gs,
                            scales=rng.integers(1, 4097, size=(k // gs, n)).astype(np.int16),
                            zeros=rng.integers(0, 16, size=(k // gs, n), dtype=np.int32), bias32=None))
    topk_ids = np.stack([rng.permutation(e)[:top_k] for _ in range(m)]).astype(np.int32)
    weights = rng.uniform(0.1, 1.0, size=(m, top_k)).astype(np.float32)
    sorted_ids, expert_ids, past = mo.moe_align_block_size(topk_ids, bs, e)
    for dtype in ("fp16", "bf16"):
        for tw in (None, weights):
            got = mo.moe_gemm_w4a8_int8(a, a_s, experts, sorted_ids, expert_ids, int(past[0]), bs, top_k, tw, dtype)
            for t in range(m):
                for j in range(top_k):
                    ex = experts[int(topk_ids[t, j])]
                    for col in range(n):
                        total = 0
                        for g in range(k // gs):
                            part = sum(int(a[t, kk]) * (int(ex["q"][kk, col]) - int(ex["zeros"][g, col]))
                                       for kk in range(g * gs, (g + 1) * gs))
                            total += part * int(ex["scales"][g, col])
                        assert -2 ** 31 <= total < 2 ** 31          # no wrap in this case
                        want = mo.round_to_dtype(np.array([np.float32(total) * a_s[t, 0]], np.float32), dtype)[0]
                        if tw is not None:
                            wt = mo.round_to_dtype(np.array([tw[t, j]], np.float32), dtype)[0]
                            want = mo.round_to_dtype(np.array([want * wt], np.float32), dtype)[0]
                        assert want != 0 and got[t * top_k + j, col] == want, (dtype, t, j, col)
    # a block of an expert held elsewhere (-1) writes nothing
    skipped = expert_ids.copy()
    skipped[0] = -1
    got = mo.moe_gemm_w4a8_int8(a, a_s, experts, sorted_ids, skipped, int(past[0]), bs, top_k, None, "fp16")
    dropped = sorted_ids[:bs]
    dropped = dropped[dropped < m * top_k]
    assert dropped.size > 0 and np.all(got[dropped] == 0)


def test_gemm_w4a8_limit_cases():
    # all integer group scales equal to c: the result is c * (a @ (q - 8)), the textbook product
    rng = np.random.default_rng(8)
    a = rng.integers(-127, 128, size=(4, 64)).astype(np.int8)
    q = rng.integers(0, 16, size=(64, 16), dtype=np.int32)
    ones = np.ones((4, 1), dtype=np.float32)
    got = mo.gemm_w4a8_int8(a, ones, q, 32, np.full((2, 16), 3, dtype=np.int16), "bf16")
    want = mo.round_to_dtype((3 * (a.astype(np.int64) @ (q.astype(np.int64) - 8))).astype(np.float32), "bf16")
    assert np.array_equal(got, want)
    # 32-bit wrap-around of the integer accumulator is part of the definition
    big = mo.gemm_w4a8_int8(np.full((1, 128), 127, dtype=np.int8), np.ones((1, 1), np.float32),
                            np.full((128, 1), 15, dtype=np.int32), 64,
                            np.full((2, 1), -1, dtype=np.int16), "bf16")  # -1 is read as 65535
    wrapped = (2 * 127 * 7 * 64 * 65535 + 2**31) % 2**32 - 2**31
    assert wrapped != 2 * 127 * 7 * 64 * 65535
    assert big[0, 0] == mo.round_to_dtype(np.array([wrapped], dtype=np.float32), "bf16")[0]
    # fp8 activations: equal to the dequantised matmul
    af = rng.integers(-8, 9, size=(2, 64)).astype(np.float32)
    s = rng.uniform(0.5, 1, size=(2, 16)).astype(np.float32)
    w = (q - 8) * np.repeat(s, 32, axis=0)
    assert np.allclose(mo.gemm_w4a8_fp8(af, np.ones((2, 1), np.float32), q, 32, s), af @ w, rtol=1e-6)


def test_marlin8_a8_layout_two_derivations_agree():
    rng = np.random.default_rng(21)
    q = rng.integers(0, 256, size=(96, 128), dtype=np.int32)
    recipe, closed = mo.marlin_pack8_recipe_a8(q), mo.marlin_pack8_closed_form_a8(q)
    assert recipe.shape == (6, 512) and np.array_equal(recipe, closed)
    assert np.array_equal(mo.gptq_marlin_repack8_a8(mo.pack_rows8(q), 96, 128), closed)
    assert not np.array_equal(closed, mo.marlin_pack8_closed_form(q))     # not the 16-bit order
    # one code at (k, n): tile (k/32, n/32), lane 4*(n%8) + (k%16)/4, warp (n%32)/8, half (k%32)/16, byte k%4
    for k, n in [(0, 0), (21, 13), (63, 127)]:
        one = np.zeros((64, 128), dtype=np.int32)
        one[k, n] = 255
        w = mo.marlin_pack8_closed_form_a8(one).view(np.uint32).reshape(-1)
        idx = np.nonzero(w)[0]
        tile = (k // 32) * 4 + n // 32
        assert idx.tolist() == [tile * 256 + (4 * (n % 8) + (k % 16) // 4) * 8 + 2 * ((n % 32) // 8) + (k % 32) // 16]
        assert w[idx[0]] == 255 << (8 * (k % 4))


def test_fp4_code_as_fp8_byte_is_value_times_2_pow_minus_6():
    """The byte the 8-bit-activation kernels make of a float4_e2m1f code, decoded as float8_e4m3fn,
    is 2^-6 times the code's value for all 16 codes; the scale bytes carry the 6."""
    codes = np.arange(16)
    got = mo.fp8_e4m3fn_value(mo.fp4_code_as_fp8_byte(codes))
    assert np.array_equal(got * np.float32(64.0), mo.fp4_e2m1_values())
    # the float8_e4m3fn decoder itself, against torch's
    import torch
    every = np.array([b for b in range(256) if b & 0x7f != 0x7f], dtype=np.uint8)
    assert np.array_equal(mo.fp8_e4m3fn_value(every),
                          torch.from_numpy(every).view(torch.float8_e4m3fn).float().numpy())
    b = np.array([[10, 100], [121, 240]], dtype=np.uint8)
    assert np.array_equal(mo.mxfp4_process_scales_a8(b), b + 6)
    assert np.array_equal(mo.mx_scale_values(mo.mxfp4_process_scales_a8(b)) / 64, mo.mx_scale_values(b))
    with pytest.raises(AssertionError):
        mo.mxfp4_process_scales_a8(np.array([250], dtype=np.uint8))


def test_gemm_w4a8_fp4_against_dequantised_matmul():
    rng = np.random.default_rng(5)
    k, n, m = 64, 8, 3
    codes = rng.integers(0, 16, size=(k, n))
    e = rng.integers(120, 130, size=(k // 32, n)).astype(np.uint8)
    a = rng.standard_normal((m, k)).astype(np.float32)
    a_s = rng.uniform(0.5, 2, size=m).astype(np.float32)
    want = (a.astype(np.float64) @ mo.dequantize_mxfp4(codes, e, "bf16").astype(np.float64)) * a_s[:, None]
    assert np.allclose(mo.gemm_w4a8_fp4(a, a_s, codes, e), want, rtol=1e-6)
