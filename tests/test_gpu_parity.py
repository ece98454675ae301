"""GPU parity: HIP kernels, called through the C ABI, against the CPU oracle.
Integer results are compared bit for bit; GEMM outputs with the tolerance
max|err| <= 1e-2*max|ref| and |err| <= 1e-2*max|ref| + 1e-2*|ref|."""
import os

import numpy as np
import pytest
import torch

from oracle import marlin_oracle as mo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gu():
    from tests import gpu_util
    return gpu_util


# reference repack tests use K = 128*{8,5,11}, N = {64,256}*{4,7,13}
REPACK_SHAPES = [(128 * 8, 64 * 4), (128 * 5, 64 * 7), (128 * 11, 256 * 13), (128, 64), (4096, 4096)]


@pytest.mark.parametrize("k,n", REPACK_SHAPES)
@pytest.mark.parametrize("act_order", [False, True])
def test_gptq_marlin_repack_bit_exact(gu, k, n, act_order):
    rng = np.random.default_rng(k + n)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    perm = rng.permutation(k).astype(np.int32) if act_order else None
    out = gu.gptq_repack(gu.dev_i32(mo.gptq_pack(q)), gu.dev_i32(perm) if act_order else None, k, n)
    want = mo.gptq_marlin_repack(mo.gptq_pack(q), perm, k, n)
    assert out.shape == (k // 16, 2 * n)
    assert np.array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("k,n", REPACK_SHAPES)
def test_awq_marlin_repack_bit_exact(gu, k, n):
    rng = np.random.default_rng(k * 3 + n)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    out = gu.awq_repack(gu.dev_i32(mo.awq_pack(q)), k, n)
    assert np.array_equal(out.cpu().numpy(), mo.awq_marlin_repack(mo.awq_pack(q), k, n))


@pytest.mark.parametrize("k,n", [(32, 64), (640, 448), (4096, 11008), (14336, 4096)])
def test_gfx950_retile_bit_exact_and_round_trip(gu, k, n):
    rng = np.random.default_rng(k + 7 * n)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    marlin = gu.dev_i32(mo.marlin_pack(q))
    native = gu.to_gfx950(marlin, k, n)
    assert np.array_equal(native.cpu().numpy(), mo.gfx950_pack(q))
    back = gu.from_gfx950(native, k, n)
    assert torch.equal(back.view(-1), marlin.view(-1))


DEQUANT_CASES = [
    # k, n, group, zero_points
    (256, 128, 128, False), (256, 128, 64, False), (256, 128, 32, True), (512, 192, -1, False),
    (512, 192, -1, True), (4096, 4096, 128, False), (4096, 11008, 128, True),
]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("k,n,g,zp", DEQUANT_CASES)
def test_in_kernel_dequant_bit_exact(gu, dtype, k, n, g, zp):
    layer = gu.DeviceLayer(11, k, n, g, dtype, zero_points=zp)
    w = layer.dequant()
    got = w.view(torch.int16).cpu().numpy().view(np.uint16)
    want = mo.to_bits16(layer.w_ref, dtype)
    # +0 and -0 are both "zero times scale"; compare as values where the oracle has a zero
    same = (got == want) | ((layer.w_ref == 0) & ((got & 0x7FFF) == 0))
    assert bool(same.all()), f"{(~same).sum()} of {same.size} dequantised values differ"


def test_dequant_extreme_scales_bit_exact(gu):
    """Scales far outside the usual range (tiny, large, zero) still give
    round((v - z) * s) exactly."""
    k, n = 128, 64
    for dtype in ("fp16", "bf16"):
        layer = gu.DeviceLayer(5, k, n, 32, dtype, zero_points=True)
        rng = np.random.default_rng(1)
        s = np.concatenate([rng.uniform(1e-6, 1e-4, 64), rng.uniform(0.5, 100.0, 64),
                            np.zeros(16), rng.uniform(1e-3, 1e-2, 112)]).astype(np.float32)
        s = mo.round_to_dtype(s.reshape(4, 64), dtype)
        layer.scales = gu.dev_bits16(mo.marlin_permute_scales(s, k, n, 32), dtype)
        want = mo.dequantize(layer.layer["q"], s, 32, dtype, zeros=layer.layer["zeros"])
        got = gu.host_f32(layer.dequant())
        assert np.array_equal(got, want)


GEMM_CASES = [
    # m, k, n, group, zp, act_order, bias
    (1, 128, 64, 128, False, False, False),
    (16, 4096, 4096, 128, False, False, False),      # benchmark config 1
    (1, 256, 128, 32, False, False, False),
    (26, 1024, 256, 64, False, False, True),
    (7, 640, 448, -1, False, False, False),
    (33, 512, 192, 128, True, False, False),
    (64, 2048, 1024, 128, True, False, True),
    (1, 4096, 11008, 128, False, True, False),       # act-order, benchmark config 4
    (1, 4096, 11008, 128, True, False, False),       # AWQ, benchmark config 4
    (48, 1024, 512, 32, False, True, False),
    (65, 512, 256, 128, False, False, False),
    (257, 1280, 320, 128, False, False, True),
    (8, 96, 64, 32, False, False, False),            # K % 64 != 0
    (3, 14336, 4096, 128, False, False, False),
    (5, 4096, 28672, 128, False, False, False),
    (2, 4096, 6144, 128, False, False, False),
    (2, 14336, 6144, 128, False, False, False),      # more than four activation slices per wavefront
    (11, 4096, 512, 128, True, False, True),
    # 17..128 rows on a matrix with at least 64 short strips: one launch of the
    # 16-row kernel with a block of rows per workgroup
    (33, 512, 4096, 128, False, False, True),
    (100, 1024, 4224, 128, True, False, False),
    (128, 256, 4096, -1, False, False, False),
    (64, 4096, 6144, 128, False, False, False),
    (17, 384, 8192, 128, True, False, True),
    # more than 128 rows where that is at most four workgroups of 32 rows per compute unit
    (200, 512, 4096, 128, False, False, True),
    (300, 1024, 4224, 128, True, False, False),
    (512, 256, 4096, -1, False, False, False),
    # the same with strips shared between workgroups (partial tiles per block of rows)
    (33, 14336, 1024, 128, False, False, True),
    (64, 2048, 512, 128, True, False, False),
    (40, 4096, 640, -1, False, False, False),
    # 65..128 rows on a long K: 128-row tiles of the wide tile kernel, K in ranges
    (72, 8192, 1280, 128, True, False, False),
    (128, 14336, 768, 128, False, False, True),
    (65, 11008, 512, -1, False, False, False),
    # 33..64 rows on more strips than half the compute units: two workgroups of two blocks of rows per strip
    (40, 1024, 8320, 128, True, False, True),
    (64, 512, 16384, -1, False, False, False),
    (33, 2048, 8448, 128, False, False, True),
    (49, 256, 8256, 256, True, False, False),
    # up to 16 rows on more strips than compute units: workgroups of four wavefronts, with one, two and four
    # groups per 128 rows
    (9, 256, 16448, 128, True, False, False),
    (16, 256, 16448, 64, False, False, True),
    (13, 512, 16448, 64, True, False, False),
    (16, 256, 16448, 32, False, False, False),
    (5, 512, 16448, 32, True, False, True),
    # K = 320 is not a whole number of the decode kernel's 128-row units: the general kernel with zero points,
    # one, two and three blocks of 16 rows
    (7, 320, 192, 64, True, False, False),
    (20, 320, 192, -1, True, False, True),
    (40, 320, 192, 64, True, False, False),
]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m,k,n,g,zp,act,bias", GEMM_CASES)
def test_marlin_gemm_within_tolerance(gu, dtype, m, k, n, g, zp, act, bias):
    layer = gu.DeviceLayer(21 + m, k, n, g, dtype, zero_points=zp, act_order=act, bias=bias)
    a32 = mo.make_activations(m * 7 + 1, m, k, dtype)
    a = gu.dev_bits16(a32, dtype)
    c = layer.gemm(a, m)
    torch.cuda.synchronize()
    ref = mo.gemm_reference(a32, layer.w_ref, layer.bias32)
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), ref)
    assert ok, f"max_err={max_err} max_ref={max_ref}"
    assert int(layer.workspace.abs().sum().item()) == 0, "workspace must return to zero"
    # a second call on the same workspace gives the same bits (fixed reduction order)
    c2 = layer.gemm(a, m)
    assert torch.equal(c.view(torch.int16), c2.view(torch.int16))


@pytest.mark.parametrize("m,k,n", [(9, 512, 256), (37, 512, 4096), (50, 1024, 256), (300, 512, 512)])
def test_gemm_row_strided_activations(gu, m, k, n):
    layer = gu.DeviceLayer(3, k, n, 128, "fp16")
    big32 = mo.make_activations(5, m, k + 64, "fp16")
    big = gu.dev_bits16(big32, "fp16")
    a = big[:, 32:32 + k]   # row stride k + 64, 64-byte offset
    c = layer.gemm(a, m)
    ref = mo.gemm_reference(big32[:, 32:32 + k], layer.w_ref)
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), ref)
    assert ok, (max_err, max_ref)


@pytest.mark.parametrize("m,n", [(32, 2048), (300, 2048),
                                 # the same window through the decode kernel (one block of rows, and blocks of
                                 # rows on 64 strips) and through 256-row tiles
                                 (9, 2048), (16, 4096), (40, 4096), (2100, 4096)])
def test_gemm_subset_input_like_the_reference(gu, m, n):
    """tests/kernels/quantization/test_marlin_gemm.py:494-537: A is the window
    [8:m+8, 8:k+8] of a matrix twice as large (row stride 2k, 16-byte offset)."""
    k = 1024
    layer = gu.DeviceLayer(8, k, n, 128, "fp16")
    big32 = mo.make_activations(6, 2 * m, 2 * k, "fp16")
    a = gu.dev_bits16(big32, "fp16")[8:m + 8, 8:k + 8]
    assert not a.is_contiguous() and a.data_ptr() % 16 == 0
    c = layer.gemm(a, m)
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), mo.gemm_reference(big32[8:m + 8, 8:k + 8], layer.w_ref))
    assert ok, (max_err, max_ref)


def test_gemm_special_cases_reduce_to_row_sums(gu):
    """All codes 9, scale 1: W == 1, so C[m][n] is the row sum of A; and M = 0
    leaves the output untouched."""
    m, k, n = 4, 256, 128
    layer = gu.DeviceLayer(1, k, n, 128, "fp16")
    q = np.full((k, n), 9, dtype=np.int32)
    layer.native = gu.to_gfx950(gu.gptq_repack(gu.dev_i32(mo.gptq_pack(q)), None, k, n), k, n)
    layer.scales = gu.dev_bits16(np.ones((2, n), np.float32), "fp16")
    a32 = mo.make_activations(2, m, k, "fp16")
    c = gu.host_f32(layer.gemm(gu.dev_bits16(a32, "fp16"), m))
    want = a32.sum(axis=1, keepdims=True).repeat(n, 1)
    assert np.allclose(c, want, rtol=2e-3, atol=2e-2)
    empty = layer.gemm(torch.empty((0, k), dtype=torch.float16, device=gu.DEV), 0)
    assert empty.shape == (0, n)


def test_error_paths(gu):
    from sonar_amd import _lib
    lib = _lib.load()
    t = torch.zeros(1024, dtype=torch.int32, device=gu.DEV)
    with pytest.raises(_lib.SonarMarlinError, match="size_k"):
        _lib.check(lib.sonar_gptq_marlin_repack(gu.ptr(t), None, gu.ptr(t), 24, 64, 4, gu.stream()))
    with pytest.raises(_lib.SonarMarlinError, match="size_n"):
        _lib.check(lib.sonar_awq_marlin_repack(gu.ptr(t), gu.ptr(t), 32, 96, 4, gu.stream()))
    with pytest.raises(NotImplementedError):   # 8-bit AWQ weights
        _lib.check(lib.sonar_awq_marlin_repack(gu.ptr(t), gu.ptr(t), 32, 64, 8, gu.stream()))
    layer = gu.DeviceLayer(1, 128, 64, 128, "fp16")
    a = torch.zeros((1, 128), dtype=torch.float16, device=gu.DEV)
    layer.b_type = 1125899906844672  # uint8: 8-bit codes with zero points
    with pytest.raises(NotImplementedError):
        layer.gemm(a, 1)
    layer.b_type = _lib.TYPE_UINT4  # uint4 needs zero points
    with pytest.raises(_lib.SonarMarlinError, match="has_zp"):
        layer.gemm(a, 1)
    layer.b_type = _lib.TYPE_UINT4B8
    layer.workspace = torch.zeros(4, dtype=torch.int32, device=gu.DEV)
    with pytest.raises(_lib.SonarMarlinError, match="workspace"):
        layer.gemm(a, 1)
    # act-order with zero points: the reference generates no such kernel (generate_kernels.py:66-72) and
    # fails with "Unsupported shapes" (marlin.cu:509-519)
    layer = gu.DeviceLayer(2, 256, 64, 128, "fp16", zero_points=True, act_order=True)
    with pytest.raises(NotImplementedError, match="Unsupported shapes"):
        layer.gemm(torch.zeros((1, 256), dtype=torch.float16, device=gu.DEV), 1)


TILE_CASES = [
    # m, k, n, group, zp, act_order, bias   (more than 64 rows: the MFMA-tiled kernel)
    (65, 512, 256, 128, False, False, False),
    (256, 4096, 4096, 128, False, False, False),
    (257, 1280, 320, 128, False, False, True),
    (300, 1024, 448, 32, True, False, False),
    (512, 4096, 11008, 128, False, True, False),     # act-order, benchmark config 4
    (512, 4096, 11008, 128, True, False, False),     # AWQ, benchmark config 4
    (1000, 2048, 64, -1, False, False, True),
    (129, 14336, 4096, 128, False, False, False),
    (600, 1024, 768, 64, True, False, True),
    (520, 512, 192, 32, True, False, False),         # groups of 32 rows: two scale rows per K step
    (1000, 2048, 1024, 32, False, False, True),
    # 9 x 29 = 261 tiles: 256 whole ones, then the last 5 split six ways along K
    (2200, 3072, 7360, 128, True, False, True),
    # K of five steps: not a whole number of the wide kernel's passes of four, the eight-wavefront kernel
    (600, 320, 512, 64, False, False, True),
]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m,k,n,g,zp,act,bias", TILE_CASES)
def test_marlin_gemm_tiled_within_tolerance(gu, dtype, m, k, n, g, zp, act, bias):
    layer = gu.DeviceLayer(31 + m, k, n, g, dtype, zero_points=zp, act_order=act, bias=bias)
    a32 = mo.make_activations(m * 3 + 1, m, k, dtype, std=0.5)
    a = gu.dev_bits16(a32, dtype)
    c = layer.gemm(a, m)
    ref = mo.gemm_reference(a32, layer.w_ref, layer.bias32)
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), ref)
    assert ok, f"max_err={max_err} max_ref={max_ref}"
    c2 = layer.gemm(a, m)
    assert torch.equal(c.view(torch.int16), c2.view(torch.int16))


WIDE_TILE_CASES = [
    # m, k, n, group, zp, bias: the forms of the one-wavefront-per-SIMD tile kernel (K a multiple of 256,
    # groups of 32 or 64 * 2^i rows or one group).  At most 128 tiles of 256 rows: 128-row tiles
    (300, 256, 256, 64, False, False),        # one pass of the four-step loop
    (300, 1024, 768, 128, True, True),        # 9 tiles of 128 rows, two ranges of K
    (520, 2048, 512, 256, False, True),       # groups of four steps
    (1100, 512, 1024, -1, True, False),       # channelwise, zero points, no split
    (140, 8192, 256, 128, False, False),      # long K, eight ranges
    # more than 128 tiles of 256 rows: 256-row tiles
    (2100, 256, 4096, 64, True, True),        # 144 tiles, one pass of the loop
    (2100, 1024, 4096, 128, False, False),
    (2304, 512, 3840, -1, False, True),       # 9 x 15 tiles, the last column tile full
    (2050, 1024, 4160, 128, True, False),     # a ragged last column tile (one strip) and a ragged last row tile
    # K = 10240 > 8192 keeps 256-row tiles although there are few
    (300, 10240, 512, 128, False, True),
    # K ranges that are not a multiple of four steps: padded with steps of zeros
    (2100, 2880, 4096, 64, False, True),      # 45 steps, one range
    (520, 1344, 5120, 64, True, False),       # 21 steps in two ranges of 11 and 10 (128-row tiles)
    # 65..128 rows with a long K: the tile kernel (256-row tiles, K split) instead of 64-row slabs
    (100, 8192, 512, 128, False, True),
    (128, 14336, 256, 128, True, False),
    # 97..128 rows on more strips than compute units: 128-row tiles, K in two ranges
    (128, 512, 16640, 128, False, True),
    (100, 1024, 16448, -1, True, False),
    # groups of 32 rows: a row of scales (and zero points) per k block
    (300, 1024, 768, 32, True, True),         # 128-row tiles, two ranges of K
    (2100, 512, 4096, 32, False, False),      # 144 tiles of 256 rows
    (1030, 2048, 4160, 32, True, False),      # ragged both ways, K split
    (600, 1216, 512, 32, False, True),        # 19 steps: the eight-wavefront kernel
    (2100, 256, 4160, 32, True, True),        # 153 tiles of 256 rows with zero points, ragged both ways
]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m,k,n,g,zp,bias", WIDE_TILE_CASES)
def test_wide_tile_kernel_forms_within_tolerance(gu, dtype, m, k, n, g, zp, bias):
    layer = gu.DeviceLayer(77 + m + k, k, n, g, dtype, zero_points=zp, act_order=False, bias=bias)
    a32 = mo.make_activations(m + 3, m, k, dtype, std=0.5)
    a = gu.dev_bits16(a32, dtype)
    c = layer.gemm(a, m)
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), mo.gemm_reference(a32, layer.w_ref, layer.bias32))
    assert ok, f"max_err={max_err} max_ref={max_ref}"
    c2 = layer.gemm(a, m)
    assert torch.equal(c.view(torch.int16), c2.view(torch.int16))   # split K is summed in a fixed order


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m,k,n", [(1, 4096, 11008), (16, 512, 256), (48, 1024, 512), (512, 4096, 1024)])
def test_act_order_with_permuted_copy_of_a(gu, dtype, m, k, n):
    """With size_m * size_k * 2 bytes more scratch an act-order call permutes A
    once and runs the plain kernels; it must agree with the gathering path."""
    layer = gu.DeviceLayer(77 + m, k, n, 128, dtype, act_order=True)
    a32 = mo.make_activations(m + 5, m, k, dtype, std=0.5)
    a = gu.dev_bits16(a32, dtype)
    fast = layer.gemm(a, m, extra_scratch=m * k * 2)
    ref = mo.gemm_reference(a32, layer.w_ref)
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(fast), ref)
    assert ok, f"max_err={max_err} max_ref={max_ref}"
    gathered = layer.gemm(a, m)
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(fast), gu.host_f32(gathered))
    assert ok, f"max_err={max_err} max_ref={max_ref}"


def _random_cases(count=int(os.environ.get("SONAR_RANDOM_CASES", "56"))):
    """Seeded draws over the dispatcher's decision variables: rows around the
    kernel boundaries, short and long strips, narrow and wide matrices, every
    group size, zero points, act-order, bias."""
    rng = np.random.default_rng(2024)
    ms = [1, 2, 15, 16, 17, 31, 32, 33, 48, 64, 65, 100, 128, 129, 200, 256, 300, 520]
    ks = [32, 64, 96, 128, 256, 384, 512, 1024, 2048, 4096]
    ns = [64, 128, 192, 320, 1024, 4096, 4160, 8192]
    cases = []
    while len(cases) < count:
        m, k, n = int(rng.choice(ms)), int(rng.choice(ks)), int(rng.choice(ns))
        g = int(rng.choice([32, 64, 128, -1]))
        if g != -1 and (k % g != 0 or g > k):
            continue
        if m * k * n > 3e9:
            continue
        zp = bool(rng.integers(0, 2))
        act = (not zp) and g != -1 and k // g > 1 and bool(rng.integers(0, 3) == 0)
        cases.append((m, k, n, g, zp, act, bool(rng.integers(0, 2)), "fp16" if rng.integers(0, 2) else "bf16"))
    return cases


@pytest.mark.parametrize("m,k,n,g,zp,act,bias,dtype", _random_cases())
def test_random_shapes_against_oracle(gu, m, k, n, g, zp, act, bias, dtype):
    layer = gu.DeviceLayer(m + k + n, k, n, g, dtype, zero_points=zp, act_order=act, bias=bias)
    a32 = mo.make_activations(m, m, k, dtype, std=0.5)
    a = gu.dev_bits16(a32, dtype)
    c = layer.gemm(a, m, extra_scratch=m * k * 2 if act and m % 2 else 0)   # with and without the permuted copy
    torch.cuda.synchronize()
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), mo.gemm_reference(a32, layer.w_ref, layer.bias32))
    assert ok, f"max_err={max_err} max_ref={max_ref}"
    assert int(layer.workspace.abs().sum().item()) == 0


def _layer8(gu, seed, k, n, g, dtype, act_order=False):
    """An 8-bit (uint8b128) layer on the device: GPTQ packing -> repack op ->
    streaming order, plus the oracle's dequantised matrix."""
    from sonar_amd import _lib
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    groups = 1 if g in (-1, k) else k // g
    scales = mo.round_to_dtype(rng.uniform(1e-4, 1e-3, size=(groups, n)).astype(np.float32), dtype)
    g_idx = perm = None
    order = None
    if act_order:
        g_idx_np = (rng.permutation(k) // g).astype(np.int32)
        g_sorted, order = mo.stable_sort_g_idx(g_idx_np)
        g_idx, perm = gu.dev_i32(g_sorted), gu.dev_i32(order)
        w_ref = mo.dequantize(q, scales, g, dtype, g_idx=g_idx_np, num_bits=8)
    else:
        w_ref = mo.dequantize(q, scales, g, dtype, num_bits=8)
    lib = _lib.load()
    marlin = torch.empty((k // 16, 4 * n), dtype=torch.int32, device=gu.DEV)
    _lib.check(lib.sonar_gptq_marlin_repack(gu.ptr(gu.dev_i32(mo.pack_rows8(q))), gu.ptr(perm), gu.ptr(marlin),
                                            k, n, 8, gu.stream()))
    native = torch.empty_like(marlin)
    _lib.check(lib.sonar_marlin8_to_gfx950(gu.ptr(marlin), gu.ptr(native), k, n, gu.stream()))
    s_dev = gu.dev_bits16(mo.marlin_permute_scales(scales, k, n, -1 if groups == 1 else g), dtype)
    return dict(q=q, order=order, marlin=marlin, native=native, scales=s_dev, groups=groups, w_ref=w_ref,
                g_idx=g_idx, perm=perm)


@pytest.mark.parametrize("k,n", [(128, 64), (640, 448), (4096, 1024)])
@pytest.mark.parametrize("act_order", [False, True])
def test_repack8_and_layout_bit_exact(gu, k, n, act_order):
    from sonar_amd import _lib
    L = _layer8(gu, k + n, k, n, 128, "fp16", act_order)
    torch.cuda.synchronize()
    q_rows = L["q"] if L["order"] is None else L["q"][L["order"]]
    assert np.array_equal(L["marlin"].cpu().numpy(), mo.marlin_pack8(q_rows).reshape(k // 16, 4 * n))
    assert np.array_equal(L["native"].cpu().numpy().ravel(), mo.gfx950_pack8(q_rows))
    back = torch.empty_like(L["marlin"])
    _lib.check(_lib.load().sonar_gfx950_to_marlin8(gu.ptr(L["native"]), gu.ptr(back), k, n, gu.stream()))
    assert torch.equal(back, L["marlin"])


W8_CASES = [
    # m, k, n, g, act_order, bias
    (1, 128, 64, 128, False, False),
    (7, 512, 256, 128, False, True),
    (16, 4096, 1024, 128, False, False),
    (33, 1024, 320, 64, False, False),
    (64, 256, 4096, -1, False, True),
    (100, 1024, 512, 128, False, False),
    (13, 1024, 256, 128, True, False),
    (300, 512, 192, 32, False, False),
    # more than 128 rows on enough K steps or tiles: the MFMA tile kernel's 8-bit form
    (300, 2048, 512, 128, False, True),      # K split over workgroups
    (1024, 1024, 832, 128, False, False),    # a last column of tiles that is not full
    (260, 1024, 4160, -1, False, False),     # one group
    (512, 2048, 320, 32, False, True),       # groups of 32 rows
    (300, 2048, 512, 128, True, False),      # act-order through the permuted copy of A
    (520, 2048, 512, 256, False, True),      # few tiles: 128-row tiles, groups of four steps
    (1100, 512, 1024, -1, False, False),     # ... one group, no K split
    (1024, 1024, 832, 32, False, False),     # groups of 32 rows, whole tiles over all of K
    (700, 1280, 4160, 32, False, True),      # ... K ranges of 20 steps, ragged tiles both ways
    (300, 1216, 512, 32, False, False),      # ... 19 steps: not a multiple of four (the eight-wavefront kernel)
    (2100, 512, 4160, 128, False, True),     # more than 128 tiles of 256 rows: 256-row tiles, ragged both ways
]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m,k,n,g,act,bias", W8_CASES)
def test_w8a16_dequant_bit_exact_and_gemm_within_tolerance(gu, dtype, m, k, n, g, act, bias):
    """uint8b128 weights through the same entry points (generate_kernels.py:80-86,
    dequant.h: code - 128, then the scale)."""
    from sonar_amd import _lib
    lib = _lib.load()
    L = _layer8(gu, 3 * m + k, k, n, g, dtype, act)
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    w = torch.empty((k, n), dtype=tdt, device=gu.DEV)
    _lib.check(lib.sonar_marlin_dequant(gu.ptr(L["native"]), _lib.LAYOUT_GFX950, gu.ptr(L["scales"]), None,
                                        gu.ptr(L["g_idx"]), gu.ptr(w), gu.dtype_code(dtype), _lib.TYPE_UINT8B128,
                                        n, k, L["groups"], 1, gu.stream()))
    torch.cuda.synchronize()
    want = L["w_ref"] if L["order"] is None else L["w_ref"][L["order"]]
    assert np.array_equal(gu.host_f32(w), want)

    bias32 = bias_dev = None
    if bias:
        bias32 = mo.round_to_dtype(np.random.default_rng(m).standard_normal(n).astype(np.float32), dtype)
        bias_dev = gu.dev_bits16(mo.marlin_permute_bias(bias32), dtype)
    a32 = mo.make_activations(m + 1, m, k, dtype, std=0.5)
    a = gu.dev_bits16(a32, dtype)
    c = torch.empty((m, n), dtype=tdt, device=gu.DEV)
    workspace = torch.zeros(torch.cuda.get_device_properties(0).multi_processor_count, dtype=torch.int32,
                            device=gu.DEV)
    nbytes = lib.sonar_marlin_gemm_scratch_bytes(m, n, k) + (m * k * 2 if act else 0)
    scratch = torch.empty(nbytes, dtype=torch.uint8, device=gu.DEV)
    _lib.check(lib.sonar_marlin_gemm(
        gu.ptr(a), k, gu.ptr(c), gu.ptr(L["native"]), _lib.LAYOUT_GFX950, gu.ptr(bias_dev), gu.ptr(L["scales"]), None,
        gu.ptr(L["g_idx"]), gu.ptr(L["perm"]), gu.ptr(workspace), workspace.numel(), gu.ptr(scratch), scratch.numel(),
        gu.dtype_code(dtype), _lib.TYPE_UINT8B128, m, n, k, L["groups"], 1, 0, 1, gu.stream()))
    torch.cuda.synchronize()
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), mo.gemm_reference(a32, L["w_ref"], bias32))
    assert ok, f"max_err={max_err} max_ref={max_ref}"


def _layer_fp8(gu, seed, k, n, g, dtype, all_codes=False):
    """A float8_e4m3fn layer on the device: the codes packed four to a word along
    K -> repack op (num_bits = 8) -> streaming order; scales permuted, with the
    exponent bias folded in; plus the oracle's dequantised matrix."""
    from sonar_amd import _lib
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    if all_codes:
        codes[:256, 0] = np.arange(256)   # every code, the two NaN codes included, in one column
    else:
        codes[(codes & 0x7F) == 0x7F] = 0x3C
    groups = 1 if g in (-1, k) else k // g
    scales = mo.round_to_dtype(rng.uniform(2e-4, 2e-3, size=(groups, n)).astype(np.float32), dtype)
    fused = mo.fp8_fuse_exponent_bias(scales, dtype)
    w_ref = mo.dequantize_fp8(codes, fused, g, dtype)
    lib = _lib.load()
    marlin = torch.empty((k // 16, 4 * n), dtype=torch.int32, device=gu.DEV)
    _lib.check(lib.sonar_gptq_marlin_repack(gu.ptr(gu.dev_i32(mo.pack_rows8(codes))), None, gu.ptr(marlin),
                                            k, n, 8, gu.stream()))
    native = torch.empty_like(marlin)
    _lib.check(lib.sonar_marlin8_to_gfx950(gu.ptr(marlin), gu.ptr(native), k, n, gu.stream()))
    s_dev = gu.dev_bits16(mo.marlin_permute_scales(fused, k, n, -1 if groups == 1 else g), dtype)
    return dict(codes=codes, native=native, scales=s_dev, groups=groups, w_ref=w_ref)


FP8_CASES = [
    # m, k, n, g, bias
    (1, 128, 64, 128, False),
    (7, 512, 256, -1, True),
    (16, 4096, 1024, 128, False),
    (33, 1024, 320, 128, True),
    (64, 256, 4096, -1, False),
    (100, 1024, 512, 128, False),
    (300, 512, 192, -1, True),
    (1, 4096, 4096, 128, False),
    (16, 1024, 256, 32, False),       # groups of 32 rows: MXFP8
    (100, 512, 192, 32, True),
    (20, 512, 192, 32, False),        # ... two blocks of 16 rows
    # the MFMA tile kernel's form for 8-bit floating-point codes
    (300, 2048, 512, 128, True),
    (1024, 1024, 832, -1, False),
    (512, 2048, 320, 32, True),
    (520, 2048, 512, 128, True),      # few tiles: 128-row tiles
    (1100, 512, 1024, -1, False),     # ... one group, no K split
    (1024, 1024, 832, 32, False),     # groups of 32 rows, whole tiles over all of K
    (700, 1280, 4160, 32, True),      # ... K ranges of 20 steps, ragged tiles both ways
    (300, 1216, 512, 32, False),      # ... 19 steps: not a multiple of four (the eight-wavefront kernel)
    (2100, 512, 4160, -1, True),      # more than 128 tiles of 256 rows: 256-row tiles, ragged both ways
]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m,k,n,g,bias", FP8_CASES)
def test_fp8_weights_dequant_bit_exact_and_gemm_within_tolerance(gu, dtype, m, k, n, g, bias):
    """float8_e4m3fn weights through the same entry points (generate_kernels.py:
    87-93; dequant.h:320-380: the code read as a 16-bit float, times the scale
    with the exponent bias folded in)."""
    from sonar_amd import _lib
    lib = _lib.load()
    L = _layer_fp8(gu, 5 * m + k, k, n, g, dtype, all_codes=k >= 256)
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    w = torch.empty((k, n), dtype=tdt, device=gu.DEV)
    _lib.check(lib.sonar_marlin_dequant(gu.ptr(L["native"]), _lib.LAYOUT_GFX950, gu.ptr(L["scales"]), None,
                                        None, gu.ptr(w), gu.dtype_code(dtype), _lib.TYPE_FLOAT8_E4M3FN,
                                        n, k, L["groups"], 1, gu.stream()))
    torch.cuda.synchronize()
    got = w.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got, mo.to_bits16(L["w_ref"], dtype))   # bits: the code 0x80 gives -0

    bias32 = bias_dev = None
    if bias:
        bias32 = mo.round_to_dtype(np.random.default_rng(m).standard_normal(n).astype(np.float32), dtype)
        bias_dev = gu.dev_bits16(mo.marlin_permute_bias(bias32), dtype)
    a32 = mo.make_activations(m + 1, m, k, dtype, std=0.5)
    a = gu.dev_bits16(a32, dtype)
    c = torch.empty((m, n), dtype=tdt, device=gu.DEV)
    workspace = torch.zeros(torch.cuda.get_device_properties(0).multi_processor_count, dtype=torch.int32,
                            device=gu.DEV)
    scratch = torch.empty(max(lib.sonar_marlin_gemm_scratch_bytes(m, n, k), 16), dtype=torch.uint8, device=gu.DEV)
    _lib.check(lib.sonar_marlin_gemm(
        gu.ptr(a), k, gu.ptr(c), gu.ptr(L["native"]), _lib.LAYOUT_GFX950, gu.ptr(bias_dev), gu.ptr(L["scales"]), None,
        None, None, gu.ptr(workspace), workspace.numel(), gu.ptr(scratch), scratch.numel(),
        gu.dtype_code(dtype), _lib.TYPE_FLOAT8_E4M3FN, m, n, k, L["groups"], 1, 0, 1, gu.stream()))
    torch.cuda.synchronize()
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), mo.gemm_reference(a32, L["w_ref"], bias32))
    assert ok, f"max_err={max_err} max_ref={max_ref}"


def test_fp8_weights_rejected_configurations(gu):
    """Groups other than 128 rows and act-order do not exist for fp8 weights
    (generate_kernels.py:87-93: group_blocks -1 and 8 only)."""
    from sonar_amd import _lib
    lib = _lib.load()
    k, n = 256, 64
    L = _layer_fp8(gu, 1, k, n, 128, "fp16")
    w = torch.empty((k, n), dtype=torch.float16, device=gu.DEV)
    idx = torch.zeros(k, dtype=torch.int32, device=gu.DEV)

    def dequant(groups, g_idx):
        return lib.sonar_marlin_dequant(gu.ptr(L["native"]), _lib.LAYOUT_GFX950, gu.ptr(L["scales"]), None,
                                        gu.ptr(g_idx), gu.ptr(w), 0, _lib.TYPE_FLOAT8_E4M3FN, n, k, groups, 1,
                                        gu.stream())
    assert dequant(2, None) == 0
    assert dequant(4, None) != 0 and "128" in lib.sonar_marlin_last_error().decode()
    assert dequant(2, idx) != 0 and "act-order" in lib.sonar_marlin_last_error().decode()
    torch.cuda.synchronize()


def _layer_mxfp4(gu, seed, k, n):
    """An MXFP4 layer on the device: float4_e2m1f codes in GPTQ words -> repack op
    -> streaming order; the block scales 2^(e - 127) as bf16 in
    marlin_permute_scales order (what the C entry points take); plus the
    oracle's dequantised matrix."""
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    codes[:16, 0] = np.arange(16)                      # every code in one column
    e = rng.integers(108, 122, size=(k // 32, n)).astype(np.uint8)
    w_ref = mo.dequantize_mxfp4(codes, e)
    marlin = gu.gptq_repack(gu.dev_i32(mo.gptq_pack(codes)), None, k, n)
    native = gu.to_gfx950(marlin, k, n)
    s_dev = gu.dev_bits16(mo.marlin_permute_scales(mo.mx_scale_values(e), k, n, 32), "bf16")
    return dict(codes=codes, e=e, native=native, scales=s_dev, groups=k // 32, w_ref=w_ref)


MXFP4_CASES = [
    # m, k, n, bias
    (1, 128, 64, False),
    (7, 512, 256, True),
    (16, 4096, 1024, False),
    (33, 1024, 320, True),
    (64, 256, 4096, False),
    (100, 1024, 512, False),
    (300, 512, 192, True),
    (1, 2880, 5760, False),     # gpt-oss expert shape: K is 90 groups of 32 rows
    (1024, 2880, 5760, True),   # the same through the tile kernel (K = 45 steps of 64 rows)
    (4096, 4096, 1024, False),  # tile kernel, several rounds of tiles
    (2100, 512, 4160, True),    # ... 153 tiles of 256 rows, ragged both ways
    (16, 256, 16448, False),    # more strips than compute units: the decode kernel's workgroups of four wavefronts
]


@pytest.mark.parametrize("m,k,n,bias", MXFP4_CASES)
def test_mxfp4_weights_dequant_bit_exact_and_gemm_within_tolerance(gu, m, k, n, bias):
    """float4_e2m1f weights with power-of-two scales per 32 rows, bf16 activations
    (generate_kernels.py:102-110; dequant.h:397-470)."""
    from sonar_amd import _lib
    lib = _lib.load()
    L = _layer_mxfp4(gu, 7 * m + k, k, n)
    w = torch.empty((k, n), dtype=torch.bfloat16, device=gu.DEV)
    _lib.check(lib.sonar_marlin_dequant(gu.ptr(L["native"]), _lib.LAYOUT_GFX950, gu.ptr(L["scales"]), None,
                                        None, gu.ptr(w), gu.dtype_code("bf16"), _lib.TYPE_FLOAT4_E2M1F,
                                        n, k, L["groups"], 1, gu.stream()))
    torch.cuda.synchronize()
    got = w.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got, mo.to_bits16(L["w_ref"], "bf16"))   # bits: the code 8 gives -0

    bias32 = bias_dev = None
    if bias:
        bias32 = mo.round_to_dtype(1e-2 * np.random.default_rng(m).standard_normal(n).astype(np.float32), "bf16")
        bias_dev = gu.dev_bits16(mo.marlin_permute_bias(bias32), "bf16")
    a32 = mo.make_activations(m + 1, m, k, "bf16", std=0.5)
    a = gu.dev_bits16(a32, "bf16")
    c = torch.empty((m, n), dtype=torch.bfloat16, device=gu.DEV)
    workspace = torch.zeros(torch.cuda.get_device_properties(0).multi_processor_count, dtype=torch.int32,
                            device=gu.DEV)
    scratch = torch.empty(max(lib.sonar_marlin_gemm_scratch_bytes(m, n, k), 16), dtype=torch.uint8, device=gu.DEV)
    _lib.check(lib.sonar_marlin_gemm(
        gu.ptr(a), k, gu.ptr(c), gu.ptr(L["native"]), _lib.LAYOUT_GFX950, gu.ptr(bias_dev), gu.ptr(L["scales"]), None,
        None, None, gu.ptr(workspace), workspace.numel(), gu.ptr(scratch), scratch.numel(),
        gu.dtype_code("bf16"), _lib.TYPE_FLOAT4_E2M1F, m, n, k, L["groups"], 1, 0, 1, gu.stream()))
    torch.cuda.synchronize()
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), mo.gemm_reference(a32, L["w_ref"], bias32))
    assert ok, f"max_err={max_err} max_ref={max_ref}"


def _layer_nvfp4(gu, seed, k, n, dtype):
    """An NVFP4 layer on the device: float4_e2m1f codes in GPTQ words -> repack op ->
    streaming order; float8_e4m3fn block scales per 16 rows through the reference's
    chain (marlin_permute_scales, nvfp4_marlin_process_scales) and back to the
    numbers of the activation type the C entry points take; a processed global
    scale; plus the oracle's dequantised matrix (without the global scale)."""
    import torch
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    codes[:16, 0] = np.arange(16)                      # every code in one column
    e4m3 = torch.from_numpy(rng.integers(0x20, 0x7F, size=(k // 16, n)).astype(np.uint8))   # 2^-3 .. 448
    scales = e4m3.view(torch.float8_e4m3fn).float().numpy()
    scales[0, :4] = [0.0, 2.0 ** -9, 448.0, 1.0]       # zero, the smallest number (cut to zero for fp16), the largest
    permuted = mo.marlin_permute_scales(scales, k, n, 16)
    scale_bytes, sf = mo.nvfp4_process_scales(permuted, dtype)
    kernel_scales = mo.nvfp4_kernel_scales(scale_bytes, dtype)
    w_ref = mo.dequantize_nvfp4(codes, mo.marlin_unpermute_scales(kernel_scales, k, n, 16), dtype)
    global_scale = mo.nvfp4_process_global_scale(0.0123, dtype, sf)
    marlin = gu.gptq_repack(gu.dev_i32(mo.gptq_pack(codes)), None, k, n)
    return dict(native=gu.to_gfx950(marlin, k, n), marlin=marlin, scales=gu.dev_bits16(kernel_scales, dtype),
                scale_bytes=scale_bytes, groups=k // 16, w_ref=w_ref, global_scale=float(global_scale),
                gs_dev=torch.tensor([float(global_scale)], dtype=torch.float32, device=gu.DEV))


NVFP4_CASES = [
    # m, k, n, bias
    (1, 128, 64, False),
    (7, 512, 256, True),
    (16, 4096, 1024, False),
    (33, 1024, 320, True),
    (64, 256, 4096, False),
    (100, 1024, 512, False),      # 64-row slabs of the streaming kernel (few tiles)
    (300, 512, 192, True),
    (600, 2048, 1536, True),      # tile kernel, K split, partial tiles summed by the second kernel
    (4096, 4096, 1024, False),    # tile kernel, whole tiles
    (2100, 512, 4160, True),      # ... 153 tiles, ragged both ways
    (300, 1216, 512, False),      # ... 19 steps: not a multiple of four (the eight-wavefront kernel)
]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m,k,n,bias", NVFP4_CASES)
def test_nvfp4_weights_dequant_bit_exact_and_gemm_within_tolerance(gu, m, k, n, bias, dtype):
    """float4_e2m1f weights with float8_e4m3fn scales per 16 rows and a global scale,
    either activation type (generate_kernels.py:94-100; dequant.h:397-470, 518-549;
    marlin_template.h:1661-1665)."""
    from sonar_amd import _lib
    lib = _lib.load()
    L = _layer_nvfp4(gu, 11 * m + k, k, n, dtype)
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    w = torch.empty((k, n), dtype=tdt, device=gu.DEV)
    _lib.check(lib.sonar_marlin_dequant(gu.ptr(L["native"]), _lib.LAYOUT_GFX950, gu.ptr(L["scales"]), None,
                                        None, gu.ptr(w), gu.dtype_code(dtype), _lib.TYPE_FLOAT4_E2M1F,
                                        n, k, L["groups"], 1, gu.stream()))
    torch.cuda.synchronize()
    got = w.view(torch.int16).cpu().numpy().view(np.uint16)
    want = mo.to_bits16(L["w_ref"], dtype)
    # every bit but the sign of a zero (a negative code times a zero scale is +0 here, -0 in the oracle)
    assert np.array_equal(np.where((got & 0x7FFF) == 0, 0, got), np.where((want & 0x7FFF) == 0, 0, want))

    bias32 = bias_dev = None
    if bias:
        bias32 = mo.round_to_dtype(1e-2 * np.random.default_rng(m).standard_normal(n).astype(np.float32), dtype)
        bias_dev = gu.dev_bits16(mo.marlin_permute_bias(bias32), dtype)
    a32 = mo.make_activations(m + 1, m, k, dtype, std=0.5)
    a = gu.dev_bits16(a32, dtype)
    c = torch.full((m, n), float("nan"), dtype=tdt, device=gu.DEV)
    workspace = torch.zeros(torch.cuda.get_device_properties(0).multi_processor_count, dtype=torch.int32,
                            device=gu.DEV)
    scratch = torch.empty(max(lib.sonar_marlin_gemm_scratch_bytes(m, n, k), 16), dtype=torch.uint8, device=gu.DEV)
    _lib.check(lib.sonar_marlin_gemm_nvfp4(
        gu.ptr(a), k, gu.ptr(c), gu.ptr(L["native"]), _lib.LAYOUT_GFX950, gu.ptr(bias_dev), gu.ptr(L["scales"]),
        gu.ptr(L["gs_dev"]), gu.ptr(workspace), workspace.numel(), gu.ptr(scratch), scratch.numel(),
        gu.dtype_code(dtype), m, n, k, L["groups"], gu.stream()))
    torch.cuda.synchronize()
    ref = mo.gemm_reference(a32, L["w_ref"]).astype(np.float64) * L["global_scale"]
    if bias:
        ref = ref + bias32
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), ref.astype(np.float32))
    assert ok, f"max_err={max_err} max_ref={max_ref}"
    assert int(workspace.abs().sum().item()) == 0


def test_nvfp4_rejected_configurations(gu):
    """NVFP4 takes one scale per 16 rows and needs its global scale."""
    from sonar_amd import _lib
    lib = _lib.load()
    k, n, m = 256, 128, 4
    L = _layer_nvfp4(gu, 3, k, n, "bf16")
    a = gu.dev_bits16(mo.make_activations(1, m, k, "bf16"), "bf16")
    c = torch.empty((m, n), dtype=torch.bfloat16, device=gu.DEV)
    workspace = torch.zeros(torch.cuda.get_device_properties(0).multi_processor_count, dtype=torch.int32,
                            device=gu.DEV)
    scratch = torch.empty(max(lib.sonar_marlin_gemm_scratch_bytes(m, n, k), 16), dtype=torch.uint8, device=gu.DEV)

    def call(groups, gs):
        return lib.sonar_marlin_gemm_nvfp4(
            gu.ptr(a), k, gu.ptr(c), gu.ptr(L["native"]), _lib.LAYOUT_GFX950, None, gu.ptr(L["scales"]), gs,
            gu.ptr(workspace), workspace.numel(), gu.ptr(scratch), scratch.numel(), gu.dtype_code("bf16"), m, n, k,
            groups, gu.stream())
    assert call(k // 32, gu.ptr(L["gs_dev"])) != 0 and "16 rows" in lib.sonar_marlin_last_error().decode()
    assert call(k // 16, None) != 0 and "global_scale" in lib.sonar_marlin_last_error().decode()
    assert call(k // 16, gu.ptr(L["gs_dev"])) == 0
    torch.cuda.synchronize()


def test_mxfp4_weights_rejected_configurations(gu):
    """MXFP4 exists for bfloat16 activations and groups of 32 rows only
    (generate_kernels.py:102-110), without act-order."""
    from sonar_amd import _lib
    lib = _lib.load()
    k, n = 256, 64
    L = _layer_mxfp4(gu, 1, k, n)
    w = torch.empty((k, n), dtype=torch.bfloat16, device=gu.DEV)
    idx = torch.zeros(k, dtype=torch.int32, device=gu.DEV)

    def dequant(dtype, groups, g_idx):
        return lib.sonar_marlin_dequant(gu.ptr(L["native"]), _lib.LAYOUT_GFX950, gu.ptr(L["scales"]), None,
                                        gu.ptr(g_idx), gu.ptr(w), dtype, _lib.TYPE_FLOAT4_E2M1F, n, k, groups, 1,
                                        gu.stream())
    assert dequant(1, 8, None) == 0
    assert dequant(0, 8, None) != 0 and "bfloat16" in lib.sonar_marlin_last_error().decode()
    assert dequant(1, 2, None) != 0 and "32 rows" in lib.sonar_marlin_last_error().decode()
    assert dequant(1, 8, idx) != 0 and "act-order" in lib.sonar_marlin_last_error().decode()
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m", [1, 16, 40, 100, 300])
def test_act_order_shard_without_whole_groups(gu, dtype, m):
    """A row-parallel shard of an act-order matrix (is_k_full = False,
    marlin.cu:343-351,763-769): the shard's rows lie in all groups, no group is
    whole, every row finds its scale through g_idx.  Dequantised values bit
    for bit, GEMM within the tolerance."""
    from sonar_amd import _lib
    k_full, n, g = 1024, 320, 128
    full = mo.make_layer(91, k_full, n, g, dtype, act_order=True)
    lo, hi = 256, 768
    k = hi - lo
    q, g_idx, scales = full["q"][lo:hi], full["g_idx"][lo:hi], full["scales"]
    assert len(np.unique(g_idx)) == k_full // g and np.bincount(g_idx).max() < g
    w_ref = mo.dequantize(q, scales, g, dtype, g_idx=g_idx)
    g_sorted, order = mo.stable_sort_g_idx(g_idx)
    perm, g_dev = gu.dev_i32(order), gu.dev_i32(g_sorted)
    native = gu.to_gfx950(gu.gptq_repack(gu.dev_i32(mo.gptq_pack(q)), perm, k, n), k, n)
    s_dev = gu.dev_bits16(mo.marlin_permute_scales(scales, k_full, n, g), dtype)
    lib = _lib.load()
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16

    w = torch.empty((k, n), dtype=tdt, device=gu.DEV)
    _lib.check(lib.sonar_marlin_dequant(gu.ptr(native), _lib.LAYOUT_GFX950, gu.ptr(s_dev), None, gu.ptr(g_dev),
                                        gu.ptr(w), gu.dtype_code(dtype), _lib.TYPE_UINT4B8, n, k, k_full // g, 0,
                                        gu.stream()))
    torch.cuda.synchronize()
    assert np.array_equal(gu.host_f32(w), w_ref[order])      # weight rows are in sorted-group order

    a32 = mo.make_activations(m, m, k, dtype, std=0.5)
    a = gu.dev_bits16(a32, dtype)
    c = torch.empty((m, n), dtype=tdt, device=gu.DEV)
    workspace = torch.zeros(torch.cuda.get_device_properties(0).multi_processor_count, dtype=torch.int32,
                            device=gu.DEV)
    base = lib.sonar_marlin_gemm_scratch_bytes(m, n, k)

    def call(scratch_bytes):
        scratch = torch.empty(scratch_bytes, dtype=torch.uint8, device=gu.DEV)
        return lib.sonar_marlin_gemm(
            gu.ptr(a), k, gu.ptr(c), gu.ptr(native), _lib.LAYOUT_GFX950, None, gu.ptr(s_dev), None, gu.ptr(g_dev),
            gu.ptr(perm), gu.ptr(workspace), workspace.numel(), gu.ptr(scratch), scratch.numel(),
            gu.dtype_code(dtype), _lib.TYPE_UINT4B8, m, n, k, k_full // g, 0, 0, 1, gu.stream())

    _lib.check(call(base + m * k * 2))
    torch.cuda.synchronize()
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), mo.gemm_reference(a32, w_ref))
    assert ok, f"max_err={max_err} max_ref={max_ref}"
    # without room for the permuted copy of A the call is refused, not mis-computed
    assert call(base) != 0 and b"more scratch" in lib.sonar_marlin_last_error()


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m", [1, 40, 200])
def test_act_order_shard_without_whole_groups_8bit(gu, dtype, m):
    """The same for uint8b128 codes (the reference's test grid runs GPTQ-INT8
    with act-order and is_k_full = False, test_marlin_gemm.py:86-91,304-333)."""
    from sonar_amd import _lib
    k_full, n, g = 1024, 192, 128
    lo, hi = 128, 640
    k = hi - lo
    rng = np.random.default_rng(5 + m)
    q = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    scales = mo.round_to_dtype(rng.uniform(1e-4, 1e-3, size=(k_full // g, n)).astype(np.float32), dtype)
    g_idx = (rng.permutation(k_full) // g).astype(np.int32)[lo:hi]
    assert np.bincount(g_idx, minlength=k_full // g).max() < g
    w_ref = mo.dequantize(q, scales, g, dtype, g_idx=g_idx, num_bits=8)
    g_sorted, order = mo.stable_sort_g_idx(g_idx)
    perm, g_dev = gu.dev_i32(order), gu.dev_i32(g_sorted)
    lib = _lib.load()
    marlin = torch.empty((k // 16, 4 * n), dtype=torch.int32, device=gu.DEV)
    _lib.check(lib.sonar_gptq_marlin_repack(gu.ptr(gu.dev_i32(mo.pack_rows8(q))), gu.ptr(perm), gu.ptr(marlin), k, n, 8,
                                            gu.stream()))
    native = torch.empty_like(marlin)
    _lib.check(lib.sonar_marlin8_to_gfx950(gu.ptr(marlin), gu.ptr(native), k, n, gu.stream()))
    s_dev = gu.dev_bits16(mo.marlin_permute_scales(scales, k_full, n, g), dtype)
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    w = torch.empty((k, n), dtype=tdt, device=gu.DEV)
    _lib.check(lib.sonar_marlin_dequant(gu.ptr(native), _lib.LAYOUT_GFX950, gu.ptr(s_dev), None, gu.ptr(g_dev),
                                        gu.ptr(w), gu.dtype_code(dtype), _lib.TYPE_UINT8B128, n, k, k_full // g, 0,
                                        gu.stream()))
    torch.cuda.synchronize()
    assert np.array_equal(gu.host_f32(w), w_ref[order])
    a32 = mo.make_activations(m, m, k, dtype, std=0.5)
    a = gu.dev_bits16(a32, dtype)
    c = torch.empty((m, n), dtype=tdt, device=gu.DEV)
    workspace = torch.zeros(torch.cuda.get_device_properties(0).multi_processor_count, dtype=torch.int32,
                            device=gu.DEV)
    scratch = torch.empty(lib.sonar_marlin_gemm_scratch_bytes(m, n, k) + m * k * 2, dtype=torch.uint8, device=gu.DEV)
    _lib.check(lib.sonar_marlin_gemm(
        gu.ptr(a), k, gu.ptr(c), gu.ptr(native), _lib.LAYOUT_GFX950, None, gu.ptr(s_dev), None, gu.ptr(g_dev),
        gu.ptr(perm), gu.ptr(workspace), workspace.numel(), gu.ptr(scratch), scratch.numel(),
        gu.dtype_code(dtype), _lib.TYPE_UINT8B128, m, n, k, k_full // g, 0, 0, 1, gu.stream()))
    torch.cuda.synchronize()
    ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), mo.gemm_reference(a32, w_ref))
    assert ok, f"max_err={max_err} max_ref={max_ref}"


@pytest.mark.parametrize("dtype,m,k,n", [("fp16", 4096, 4096, 4096), ("bf16", 8192, 4096, 6144),
                                          ("fp16", 1024, 14336, 4096), ("fp16", 256, 4096, 28672),
                                          ("fp16", 4096, 4096, 6144)])   # 384 tiles: the last 128 split in two
def test_full_size_tile_gemm_agrees_with_streamed_rows(gu, dtype, m, k, n):
    """At the benchmark's prefill sizes the CPU oracle is too slow, so the tile
    kernels (without split K, with every tile split, with the last round of
    tiles split) are checked through a size-independent
    property: any subset of rows of A gives the same rows of C, and 16 rows go
    through the decode kernel, which is checked against the oracle elsewhere."""
    layer = gu.DeviceLayer(5, k, n, 128, dtype)
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    gen = torch.Generator(device=gu.DEV).manual_seed(m + n)
    a = (torch.randn((m, k), device=gu.DEV, generator=gen) * 0.5).to(tdt)
    c = layer.gemm(a, m)
    assert bool(torch.isfinite(c.float()).all())
    scale = float(c.float().abs().max())
    for start in (0, m // 2 - 8, m - 16):
        rows = layer.gemm(a[start:start + 16].contiguous(), 16)
        err = float((rows.float() - c[start:start + 16].float()).abs().max())
        assert err <= 1e-2 * scale, (start, err, scale)
    # and against the oracle on a few output columns: w_ref is already on hand
    cols = np.array([0, 1, 63, 64, n // 2 + 5, n - 1])
    a_rows = a[:4].float().cpu().numpy()
    want = a_rows @ layer.w_ref[:, cols]
    got = c[:4].float().cpu().numpy()[:, cols]
    assert np.all(np.abs(got - want) <= 1e-2 * scale)
