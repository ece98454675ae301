"""The committed fixtures of tests/golden (written by tests/golden/make_fixtures.py
from the oracle) against the oracle as it is now (CPU) and against the HIP
kernels through the C ABI (GPU)."""
from __future__ import annotations

import os

import numpy as np
import pytest

from oracle import marlin_oracle as mo


def U32(x):
    return np.ascontiguousarray(x).view(np.uint32)

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
LAYERS = [("gptq_fp16_k128_n128_g64.npz", "fp16"), ("awq_bf16_k128_n64_g32.npz", "bf16"),
          ("actorder_fp16_k256_n64_g128.npz", "fp16")]


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


@pytest.mark.parametrize("name,dtype", LAYERS)
def test_oracle_reproduces_layer_fixture(name, dtype):
    f = load(name)
    k, n, g = int(f["size_k"]), int(f["size_n"]), int(f["group_size"])
    q = f["q"].astype(np.int64)
    assert np.array_equal(mo.gptq_pack(q), f["gptq_packed"])
    assert np.array_equal(mo.awq_pack(q), f["awq_packed"])
    perm = f["perm"] if "perm" in f.files else None
    assert np.array_equal(mo.gptq_marlin_repack(f["gptq_packed"], perm, k, n), f["marlin"])
    if perm is None:
        assert np.array_equal(mo.awq_marlin_repack(f["awq_packed"], k, n), f["marlin"])
    else:
        g_sorted, order = mo.stable_sort_g_idx(f["g_idx"])
        assert np.array_equal(order, perm) and np.array_equal(g_sorted, f["g_idx_sorted"])
    assert np.array_equal(mo.marlin_to_gfx950(f["marlin"], k, n), f["gfx950"])
    scales = mo.from_bits16(f["scales_bits"], dtype)
    gs = g if g < k else -1
    assert np.array_equal(mo.to_bits16(mo.marlin_permute_scales(scales, k, n, gs), dtype), f["scales_marlin_bits"])
    zeros = f["zeros"].astype(np.int64) if "zeros" in f.files else None
    if zeros is not None:
        assert np.array_equal(mo.marlin_zero_points(zeros, k // g, n), f["zeros_marlin"])
    w = mo.dequantize(q, scales, g, dtype, zeros=zeros, g_idx=f["g_idx"] if perm is not None else None)
    assert np.array_equal(mo.to_bits16(w, dtype), f["dequant_bits"])
    a = mo.from_bits16(f["a_bits"], dtype)
    assert np.allclose(mo.gemm_reference(a, w), f["c_ref"], rtol=1e-6, atol=1e-6)


def test_oracle_reproduces_moe_align_and_dequant_tables():
    f = load("moe_align_example.npz")
    s, e, p = mo.moe_align_block_size(f["topk_ids"], int(f["block_size"]), int(f["num_experts"]))
    assert np.array_equal(s, f["sorted_ids"]) and np.array_equal(e, f["expert_ids"]) and p[0] == f["num_post_pad"][0]
    assert s[:16].tolist() == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    for dtype in ("fp16", "bf16"):
        t = load(f"dequant_table_{dtype}.npz")
        scales = mo.from_bits16(t["scales_bits"], dtype)
        for z in range(16):
            q = np.arange(16, dtype=np.int64)[:, None].repeat(scales.size, 1)     # [16 rows][S columns]
            w = mo.dequantize(q, scales[None, :], 16, dtype, zeros=np.full((1, scales.size), z, dtype=np.int64))
            assert np.array_equal(mo.to_bits16(w, dtype), t["table_bits"][z])


@pytest.mark.gpu
@pytest.mark.parametrize("name,dtype", LAYERS)
def test_hip_kernels_reproduce_layer_fixture(name, dtype):
    import torch

    from sonar_amd import _lib
    from tests import gpu_util as gu
    f = load(name)
    k, n, g, m = int(f["size_k"]), int(f["size_n"]), int(f["group_size"]), int(f["size_m"])
    has_perm = "perm" in f.files
    has_zp = "zeros" in f.files
    perm = gu.dev_i32(f["perm"]) if has_perm else None
    marlin = gu.gptq_repack(gu.dev_i32(f["gptq_packed"]), perm, k, n)
    assert np.array_equal(marlin.cpu().numpy().view(np.uint32), U32(f["marlin"]))
    if not has_perm:
        awq = gu.awq_repack(gu.dev_i32(f["awq_packed"]), k, n)
        assert np.array_equal(awq.cpu().numpy().view(np.uint32), U32(f["marlin"]))
    native = gu.to_gfx950(marlin, k, n)
    assert np.array_equal(native.cpu().numpy().view(np.uint32), U32(f["gfx950"].reshape(-1)))
    assert np.array_equal(gu.from_gfx950(native, k, n).cpu().numpy().view(np.uint32), U32(f["marlin"]))

    lib = _lib.load()
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    scales = torch.from_numpy(f["scales_marlin_bits"].view(np.int16).copy()).to(gu.DEV).view(tdt)
    zeros = gu.dev_i32(f["zeros_marlin"]) if has_zp else None
    b_type = _lib.TYPE_UINT4 if has_zp else _lib.TYPE_UINT4B8
    groups = k // g
    # in-kernel dequantised values, bit for bit.  With act-order the kernel sees
    # the rows in sorted-group order: row i of its matrix is row perm[i] of W.
    w = torch.empty((k, n), dtype=tdt, device=gu.DEV)
    _lib.check(lib.sonar_marlin_dequant(gu.ptr(native), _lib.LAYOUT_GFX950, gu.ptr(scales), gu.ptr(zeros), None,
                                        gu.ptr(w), gu.dtype_code(dtype), b_type, n, k, groups, 1, gu.stream()))
    want = f["dequant_bits"][f["perm"]] if has_perm else f["dequant_bits"]
    assert np.array_equal(w.view(torch.int16).cpu().numpy().view(np.uint16), want)

    a = torch.from_numpy(f["a_bits"].view(np.int16).copy()).to(gu.DEV).view(tdt)
    c = torch.empty((m, n), dtype=tdt, device=gu.DEV)
    ws = torch.zeros(torch.cuda.get_device_properties(0).multi_processor_count, dtype=torch.int32, device=gu.DEV)
    nbytes = lib.sonar_marlin_gemm_scratch_bytes(m, n, k)
    scratch = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=gu.DEV)
    g_idx = gu.dev_i32(f["g_idx_sorted"]) if has_perm else None
    _lib.check(lib.sonar_marlin_gemm(gu.ptr(a), k, gu.ptr(c), gu.ptr(native), _lib.LAYOUT_GFX950, None,
                                     gu.ptr(scales), gu.ptr(zeros), gu.ptr(g_idx), gu.ptr(perm), gu.ptr(ws),
                                     ws.numel(), gu.ptr(scratch), scratch.numel(), gu.dtype_code(dtype), b_type,
                                     m, n, k, groups, 1, 0, 1, gu.stream()))
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(c), f["c_ref"])
    assert ok, worst


def test_oracle_reproduces_8bit_fixture():
    f = load("gptq8_bf16_k128_n64_g64.npz")
    k, n, g = int(f["size_k"]), int(f["size_n"]), int(f["group_size"])
    q = f["q"].astype(np.int64)
    assert np.array_equal(mo.pack_rows8(q), f["gptq_packed"])
    assert np.array_equal(mo.gptq_marlin_repack8(f["gptq_packed"], None, k, n), f["marlin"])
    assert np.array_equal(mo.marlin_pack8_recipe(q), f["marlin"])
    assert np.array_equal(mo.marlin8_to_gfx950(f["marlin"], k, n), f["gfx950"])
    scales = mo.from_bits16(f["scales_bits"], "bf16")
    assert np.array_equal(mo.to_bits16(mo.marlin_permute_scales(scales, k, n, g), "bf16"), f["scales_marlin_bits"])
    w = mo.dequantize(q, scales, g, "bf16", num_bits=8)
    assert np.array_equal(mo.to_bits16(w, "bf16"), f["dequant_bits"])
    assert np.allclose(mo.gemm_reference(mo.from_bits16(f["a_bits"], "bf16"), w), f["c_ref"], rtol=1e-6, atol=1e-6)


@pytest.mark.gpu
def test_hip_kernels_reproduce_8bit_fixture():
    import torch

    from sonar_amd import _lib
    from tests import gpu_util as gu
    f = load("gptq8_bf16_k128_n64_g64.npz")
    k, n, g, m = int(f["size_k"]), int(f["size_n"]), int(f["group_size"]), int(f["size_m"])
    lib = _lib.load()
    marlin = torch.empty((k // 16, 4 * n), dtype=torch.int32, device=gu.DEV)
    _lib.check(lib.sonar_gptq_marlin_repack(gu.ptr(gu.dev_i32(f["gptq_packed"])), None, gu.ptr(marlin), k, n, 8,
                                            gu.stream()))
    assert np.array_equal(marlin.cpu().numpy().view(np.uint32), U32(f["marlin"]))
    native = torch.empty_like(marlin)
    _lib.check(lib.sonar_marlin8_to_gfx950(gu.ptr(marlin), gu.ptr(native), k, n, gu.stream()))
    assert np.array_equal(native.cpu().numpy().view(np.uint32).ravel(), U32(f["gfx950"].reshape(-1)))
    scales = torch.from_numpy(f["scales_marlin_bits"].view(np.int16).copy()).to(gu.DEV).view(torch.bfloat16)
    w = torch.empty((k, n), dtype=torch.bfloat16, device=gu.DEV)
    _lib.check(lib.sonar_marlin_dequant(gu.ptr(native), _lib.LAYOUT_GFX950, gu.ptr(scales), None, None, gu.ptr(w),
                                        gu.dtype_code("bf16"), _lib.TYPE_UINT8B128, n, k, k // g, 1, gu.stream()))
    assert np.array_equal(w.view(torch.int16).cpu().numpy().view(np.uint16), f["dequant_bits"])
    a = torch.from_numpy(f["a_bits"].view(np.int16).copy()).to(gu.DEV).view(torch.bfloat16)
    c = torch.empty((m, n), dtype=torch.bfloat16, device=gu.DEV)
    ws = torch.zeros(torch.cuda.get_device_properties(0).multi_processor_count, dtype=torch.int32, device=gu.DEV)
    scratch = torch.empty(lib.sonar_marlin_gemm_scratch_bytes(m, n, k), dtype=torch.uint8, device=gu.DEV)
    _lib.check(lib.sonar_marlin_gemm(gu.ptr(a), k, gu.ptr(c), gu.ptr(native), _lib.LAYOUT_GFX950, None,
                                     gu.ptr(scales), None, None, None, gu.ptr(ws), ws.numel(), gu.ptr(scratch),
                                     scratch.numel(), gu.dtype_code("bf16"), _lib.TYPE_UINT8B128, m, n, k, k // g,
                                     1, 0, 1, gu.stream()))
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(c), f["c_ref"])
    assert ok, worst


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_oracle_reproduces_fp8_and_mxfp4_tables(dtype):
    t = load(f"fp8_dequant_table_{dtype}.npz")
    fused = mo.from_bits16(t["fused_scales_bits"], dtype)
    w = mo.dequantize_fp8(t["codes"].astype(np.int32), fused, -1, dtype)
    assert np.array_equal(mo.to_bits16(w, dtype), t["dequant_bits"])
    if dtype == "bf16":
        f = load("mxfp4_dequant_k128_n64.npz")
        codes = f["codes"].astype(np.int32)
        assert np.array_equal(mo.gptq_pack(codes), f["gptq_packed"])
        assert np.array_equal(mo.to_bits16(mo.dequantize_mxfp4(codes, f["exponent_bytes"]), "bf16"), f["dequant_bits"])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_hip_kernels_reproduce_fp8_and_mxfp4_tables(dtype):
    """In-kernel dequantised values of the floating-point weight types, bit for
    bit: all 256 fp8 codes under 64 channel scales; MXFP4 codes under block
    scales that include the exponent bytes 0, 1 and 250."""
    import torch

    from sonar_amd import _lib
    from tests import gpu_util as gu
    lib = _lib.load()
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    t = load(f"fp8_dequant_table_{dtype}.npz")
    k, n = t["codes"].shape
    marlin = torch.empty((k // 16, 4 * n), dtype=torch.int32, device=gu.DEV)
    _lib.check(lib.sonar_gptq_marlin_repack(gu.ptr(gu.dev_i32(mo.pack_rows8(t["codes"].astype(np.int32)))), None,
                                            gu.ptr(marlin), k, n, 8, gu.stream()))
    native = torch.empty_like(marlin)
    _lib.check(lib.sonar_marlin8_to_gfx950(gu.ptr(marlin), gu.ptr(native), k, n, gu.stream()))
    fused = mo.from_bits16(t["fused_scales_bits"], dtype)
    scales = gu.dev_bits16(mo.marlin_permute_scales(fused, k, n, -1), dtype)
    w = torch.empty((k, n), dtype=tdt, device=gu.DEV)
    _lib.check(lib.sonar_marlin_dequant(gu.ptr(native), _lib.LAYOUT_GFX950, gu.ptr(scales), None, None, gu.ptr(w),
                                        gu.dtype_code(dtype), _lib.TYPE_FLOAT8_E4M3FN, n, k, 1, 1, gu.stream()))
    assert np.array_equal(w.view(torch.int16).cpu().numpy().view(np.uint16), t["dequant_bits"])
    if dtype != "bf16":
        return
    f = load("mxfp4_dequant_k128_n64.npz")
    k, n = f["codes"].shape
    native = gu.to_gfx950(gu.gptq_repack(gu.dev_i32(f["gptq_packed"]), None, k, n), k, n)
    scales = gu.dev_bits16(mo.marlin_permute_scales(mo.mx_scale_values(f["exponent_bytes"]), k, n, 32), "bf16")
    w = torch.empty((k, n), dtype=torch.bfloat16, device=gu.DEV)
    _lib.check(lib.sonar_marlin_dequant(gu.ptr(native), _lib.LAYOUT_GFX950, gu.ptr(scales), None, None, gu.ptr(w),
                                        gu.dtype_code("bf16"), _lib.TYPE_FLOAT4_E2M1F, n, k, k // 32, 1, gu.stream()))
    assert np.array_equal(w.view(torch.int16).cpu().numpy().view(np.uint16), f["dequant_bits"])


def test_oracle_reproduces_w4a8_fixture():
    f = load("w4a8_int8_fp16_k256_n128_g64.npz")
    k, n, g = int(f["size_k"]), int(f["size_n"]), int(f["group_size"])
    q, zeros = f["q"].astype(np.int32), f["zeros"].astype(np.int32)
    assert np.array_equal(mo.gptq_marlin_repack_a8(f["gptq_packed"], k, n), f["marlin_a8"])
    assert np.array_equal(mo.awq_marlin_repack_a8(f["awq_packed"], k, n), f["marlin_a8"])
    assert np.array_equal(mo.marlin_pack_recipe_a8(q), f["marlin_a8"])
    assert np.array_equal(mo.marlin_a8_to_gfx950(f["marlin_a8"], k, n), f["gfx950"])
    assert np.array_equal(mo.gfx950_pack(q), f["gfx950"])        # the same stream as for 16-bit activations
    assert np.array_equal(mo.int4_fp8_preprocess(q), f["fp8_preprocessed"])
    assert np.array_equal(mo.marlin_zero_points_a8(zeros, k // g, n), f["zeros_marlin_a8"])
    assert np.array_equal(mo.marlin_permute_scales_a8(f["int_scales"], k, n, g), f["int_scales_marlin_a8"])
    a_q, a_s = mo.per_token_quant_int8(f["x"])
    assert np.array_equal(a_q, f["a_q"])
    for zp, key in ((None, "c_bits"), (zeros, "c_zp_bits")):
        c = mo.gemm_w4a8_int8(f["a_q"], f["a_scales"], q, g, f["int_scales"], "fp16", zp)
        assert np.array_equal(mo.to_bits16(c, "fp16"), f[key])


@pytest.mark.gpu
def test_hip_kernels_reproduce_w4a8_fixture():
    import torch

    from sonar_amd import _lib
    from tests import gpu_util as gu
    f = load("w4a8_int8_fp16_k256_n128_g64.npz")
    k, n, g, m = int(f["size_k"]), int(f["size_n"]), int(f["group_size"]), int(f["size_m"])
    lib = _lib.load()
    marlin = torch.empty((k // 16, 2 * n), dtype=torch.int32, device=gu.DEV)
    src = gu.dev_i32(f["gptq_packed"])
    _lib.check(lib.sonar_gptq_marlin_repack_a8(gu.ptr(src), gu.ptr(marlin), k, n, 4, gu.stream()))
    assert np.array_equal(marlin.cpu().numpy().view(np.uint32), U32(f["marlin_a8"]))
    native = torch.empty(k * n // 8, dtype=torch.int32, device=gu.DEV)
    _lib.check(lib.sonar_marlin_a8_to_gfx950(gu.ptr(marlin), gu.ptr(native), k, n, gu.stream()))
    assert np.array_equal(native.cpu().numpy().view(np.uint32), U32(f["gfx950"].reshape(-1)))
    x = torch.from_numpy(f["x"]).to(gu.DEV)
    a_q = torch.empty((m, k), dtype=torch.int8, device=gu.DEV)
    a_s = torch.empty(m, dtype=torch.float32, device=gu.DEV)
    _lib.check(lib.sonar_per_token_quant_int8(gu.ptr(x), _lib.DTYPE_F32, k, gu.ptr(a_q), gu.ptr(a_s), m, k,
                                              gu.stream()))
    assert np.array_equal(a_q.cpu().numpy(), f["a_q"])
    scales = torch.from_numpy(f["int_scales_marlin_a8"].copy()).to(gu.DEV)
    a_scales = torch.from_numpy(f["a_scales"].reshape(-1).copy()).to(gu.DEV)
    zeros = gu.dev_i32(f["zeros_marlin_a8"])
    for zp, b_type, key in ((None, _lib.TYPE_UINT4B8, "c_bits"), (zeros, _lib.TYPE_UINT4, "c_zp_bits")):
        c = torch.empty((m, n), dtype=torch.float16, device=gu.DEV)
        _lib.check(lib.sonar_marlin_gemm_a8(gu.ptr(a_q), k, _lib.ADTYPE_INT8, gu.ptr(c), gu.ptr(native),
                                            _lib.LAYOUT_GFX950, None, gu.ptr(scales), gu.ptr(a_scales), gu.ptr(zp),
                                            None, 0, _lib.DTYPE_F16, b_type, m, n, k, k // g, gu.stream()))
        assert np.array_equal(c.view(torch.int16).cpu().numpy().view(np.uint16), f[key])
