"""CPU tests: the C ABI library loads and exports what the header declares,
the torch ops exist with the reference's schemas, and the host-side tensor
preparation agrees with the oracle.  No kernel is launched here."""
import os
import re

import numpy as np
import pytest
import torch

from oracle import marlin_oracle as mo

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_c_abi_exports_every_declared_symbol():
    from sonar_amd import _lib
    header = open(os.path.join(ROOT, "include", "sonar_marlin.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(sonar_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 11
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert declared == set(_lib.PROTOTYPES), "ctypes prototypes out of step with the header"
    assert lib.sonar_marlin_version().startswith(b"sonar-marlin-gfx950")


def test_type_id_constants_match_header_and_oracle():
    from sonar_amd import _lib
    from sonar_amd.scalar_type import scalar_types
    header = open(os.path.join(ROOT, "include", "sonar_marlin.h")).read()
    assert int(re.search(r"SONAR_TYPE_UINT4B8 (\d+)LL", header).group(1)) == mo.UINT4B8_ID
    assert int(re.search(r"SONAR_TYPE_UINT4 (\d+)LL", header).group(1)) == mo.UINT4_ID
    assert scalar_types.uint4b8.id == mo.UINT4B8_ID == _lib.TYPE_UINT4B8
    assert scalar_types.uint4.id == mo.UINT4_ID == _lib.TYPE_UINT4
    assert scalar_types.uint8b128.id == mo.UINT8B128_ID == _lib.TYPE_UINT8B128
    assert int(re.search(r"SONAR_TYPE_FLOAT8_E4M3FN (\d+)LL", header).group(1)) == mo.FLOAT8_E4M3FN_ID
    assert scalar_types.float8_e4m3fn.id == mo.FLOAT8_E4M3FN_ID == _lib.TYPE_FLOAT8_E4M3FN
    assert int(re.search(r"SONAR_TYPE_FLOAT4_E2M1F (\d+)LL", header).group(1)) == mo.FLOAT4_E2M1F_ID
    assert scalar_types.float4_e2m1f.id == mo.FLOAT4_E2M1F_ID == _lib.TYPE_FLOAT4_E2M1F
    assert str(scalar_types.float4_e2m1f) == "float4_e2m1f" and scalar_types.float4_e2m1f.size_bits == 4
    assert str(scalar_types.float8_e4m3fn) == "float8_e4m3fn" and scalar_types.float8_e4m3fn.size_bits == 8
    assert str(scalar_types.uint8b128) == "uint8b128" and str(scalar_types.int4) == "int4"
    # tests/test_scalartype.py:10-25 of the reference
    for lo, hi, t in [(-8, 7, scalar_types.int4), (0, 15, scalar_types.uint4),
                      (-8, 7, scalar_types.uint4b8), (-128, 127, scalar_types.uint8b128),
                      (-128, 127, scalar_types.int8), (0, 255, scalar_types.uint8)]:
        assert (t.min(), t.max()) == (lo, hi)


def test_torch_ops_have_the_reference_schemas():
    import sonar_amd.ops  # noqa: F401
    s = str(torch.ops._C.marlin_gemm.default._schema)
    assert s == ("_C::marlin_gemm(Tensor a, Tensor? c_or_none, Tensor b_q_weight, Tensor? b_bias_or_none, "
                 "Tensor b_scales, Tensor? a_scales, Tensor? global_scale, Tensor? b_zeros_or_none, "
                 "Tensor? g_idx_or_none, Tensor? perm_or_none, Tensor workspace, int b_type_id, "
                 "SymInt size_m, SymInt size_n, SymInt size_k, bool is_k_full, bool use_atomic_add, "
                 "bool use_fp32_reduce, bool is_zp_float) -> Tensor")
    assert str(torch.ops._C.gptq_marlin_gemm.default._schema) == s.replace("marlin_gemm", "gptq_marlin_gemm")
    assert str(torch.ops._C.gptq_marlin_repack.default._schema) == (
        "_C::gptq_marlin_repack(Tensor b_q_weight, Tensor perm, SymInt size_k, SymInt size_n, "
        "int num_bits, bool is_a_8bit) -> Tensor")
    assert str(torch.ops._C.awq_marlin_repack.default._schema) == (
        "_C::awq_marlin_repack(Tensor b_q_weight, SymInt size_k, SymInt size_n, int num_bits, "
        "bool is_a_8bit) -> Tensor")
    m = str(torch.ops._moe_C.moe_wna16_marlin_gemm.default._schema)
    assert m.startswith("_moe_C::moe_wna16_marlin_gemm(Tensor($0! -> ) a, Tensor? c_or_none, Tensor($1! -> ) b_q_weight")
    names = re.findall(r"(\w+)(?:,|\))", m)
    assert names[:4] == ["a", "c_or_none", "b_q_weight", "b_bias_or_none"] and len(names) == 29
    assert m.endswith("bool is_zp_float, int thread_k, int thread_n, int blocks_per_sm) -> Tensor")


def test_fake_impls_give_reference_shapes():
    from sonar_amd import ops
    from sonar_amd.scalar_type import scalar_types
    meta = dict(device="meta")
    qw = torch.empty((4096 // 8, 11008), dtype=torch.int32, **meta)
    out = ops.gptq_marlin_repack(qw, torch.empty(0, dtype=torch.int32, **meta), 4096, 11008, 4)
    assert out.shape == (256, 22016) and out.dtype == torch.int32
    aw = torch.empty((4096, 11008 // 8), dtype=torch.int32, **meta)
    assert ops.awq_marlin_repack(aw, 4096, 11008, 4).shape == (256, 22016)
    a = torch.empty((7, 4096), dtype=torch.bfloat16, **meta)
    s = torch.empty((32, 11008), dtype=torch.bfloat16, **meta)
    ws = torch.empty(256, dtype=torch.int32, **meta)
    c = ops.marlin_gemm(a, None, out, None, s, None, None, None, None, None, ws, scalar_types.uint4b8,
                        7, 11008, 4096)
    assert c.shape == (7, 11008) and c.dtype == torch.bfloat16
    w3 = torch.empty((8, 256, 57344), dtype=torch.int32, **meta)
    s3 = torch.empty((8, 32, 28672), dtype=torch.bfloat16, **meta)
    ids = torch.empty(88, dtype=torch.int32, **meta)
    c = ops.moe_wna16_marlin_gemm(a, None, w3, None, s3, None, None, None, None, None, ws, ids, ids, ids,
                                  torch.empty((7, 2), **meta), 8, 2, False, scalar_types.uint4b8, 7, 28672,
                                  4096, True, False, True, False)
    assert c.shape == (14, 28672)


def test_host_layouts_match_oracle():
    from sonar_amd import marlin_utils as mu
    rng = np.random.default_rng(3)
    k, n, g = 512, 256, 128
    s = rng.standard_normal((k // g, n)).astype(np.float32)
    for gs in (g, -1):
        src = s if gs == g else s[:1]
        got = mu.marlin_permute_scales(torch.from_numpy(src), k, n, gs).numpy()
        assert np.array_equal(got, mo.marlin_permute_scales(src, k, n, gs))
    b = rng.standard_normal(n).astype(np.float32)
    assert np.array_equal(mu.marlin_permute_bias(torch.from_numpy(b)).numpy(), mo.marlin_permute_bias(b))
    zp = rng.integers(0, 16, size=(k // g, n), dtype=np.int32)
    zp[0, :8] = 15  # top nibble of a word set: sign handling
    got = mu.marlin_zero_points(torch.from_numpy(zp), k // g, n, 4).numpy()
    assert got.dtype == np.int32 and np.array_equal(got, mo.marlin_zero_points(zp, k // g, n))
    packed = mu.pack_cols(torch.from_numpy(zp), 4, k // g, n)
    assert np.array_equal(packed.numpy(), mo.pack_cols(zp))
    assert np.array_equal(mu.unpack_cols(packed, 4, k // g, n).numpy(), zp)
    awq = mo.awq_pack(zp)
    got = mu.awq_to_marlin_zero_points(torch.from_numpy(awq), k // g, n, 4).numpy()
    assert np.array_equal(got, mo.awq_to_marlin_zero_points(awq, k // g, n))
    g_idx = torch.from_numpy(rng.permutation(k).astype(np.int32) // g)
    sorted_g, order = mu.marlin_sort_g_idx(g_idx)
    assert order.dtype == torch.int32 and torch.equal(sorted_g, g_idx[order.long()])
    assert bool((sorted_g[1:] >= sorted_g[:-1]).all())


ODD = [(1, 1), (65, 129), (200, 208), (100, 300), (4000, 11000)]
ALIGNED = [(64, 128), (128, 64), (256, 256), (4608, 4096)]


def _aligned(n, k):
    return (n % 64 == 0 and k % 128 == 0) or (n % 128 == 0 and k % 64 == 0)


@pytest.mark.parametrize("shape", ODD + ALIGNED)
@pytest.mark.parametrize("group_size", [-1, 16, 32, 64, 128])
def test_marlin_padded_nk(shape, group_size):
    """Same properties the reference checks
    (tests/kernels/quantization/test_marlin_tile_padding.py:62-100)."""
    from sonar_amd import marlin_utils as mu
    size_n, size_k = shape
    pn, pk = mu.marlin_padded_nk(size_n, size_k, group_size)
    assert pn >= size_n and pk >= size_k and _aligned(pn, pk)
    if group_size > 0:
        assert pk % group_size == 0
    if _aligned(size_n, size_k) and (group_size <= 0 or size_k % group_size == 0):
        assert (pn, pk) == (size_n, size_k)
    if pn * pk <= 300 * 400:
        for cn in range(size_n, pn + 1):
            for ck in range(size_k, pk + 1):
                if _aligned(cn, ck) and (group_size <= 0 or ck % group_size == 0):
                    assert cn * ck >= pn * pk
    repacked = torch.empty((pk // 16, pn * 16 // 8), device="meta")
    assert mu.marlin_repacked_nk(repacked, 4) == (pn, pk)


def test_pad_helpers_shapes():
    from sonar_amd import marlin_utils as mu
    size_n, size_k, group = 200, 208, 16
    pn, pk = mu.marlin_padded_nk(size_n, size_k, group)
    assert mu.marlin_pad_qweight(torch.zeros(size_k // 8, size_n, dtype=torch.int32), size_n, size_k, pn,
                                 pk).shape == (pk // 8, pn)
    padded = mu.marlin_pad_scales(torch.ones(size_k // group, size_n), size_n, size_k, pn, pk, group)
    assert padded.shape == (pk // group, pn) and padded[:, size_n:].abs().sum() == 0
    assert mu.marlin_pad_scales(torch.ones(1, size_n), size_n, size_k, pn, pk, -1).shape == (1, pn)


def test_marlin_linear_kernel_gates():
    from sonar_amd.marlin_linear import MarlinLinearKernel, MPLinearLayerConfig
    from sonar_amd.scalar_type import scalar_types as st
    ok = MPLinearLayerConfig((4096, 4096), (4096, 4096), st.uint4b8, torch.float16, 128, False, False)
    assert MarlinLinearKernel.can_implement(ok) == (True, None)
    eight_bit = MPLinearLayerConfig((4096, 4096), (4096, 4096), st.uint8b128, torch.float16, 128, False, False)
    assert MarlinLinearKernel.can_implement(eight_bit) == (True, None)
    bad_type = MPLinearLayerConfig((4096, 4096), (4096, 4096), st.uint8, torch.float16, 128, True, False)
    assert not MarlinLinearKernel.can_implement(bad_type)[0]
    bad_group = MPLinearLayerConfig((4096, 4096), (4096, 4096), st.uint4b8, torch.float16, 100, False, False)
    assert not MarlinLinearKernel.can_implement(bad_group)[0]
    zp_needs_uint4 = MPLinearLayerConfig((4096, 4096), (4096, 4096), st.uint4b8, torch.float16, 128, True, False)
    assert not MarlinLinearKernel.can_implement(zp_needs_uint4)[0]
    act_order_odd = MPLinearLayerConfig((4096, 4000), (4096, 4000), st.uint4b8, torch.float16, 128, False, True)
    assert not MarlinLinearKernel.can_implement(act_order_odd)[0]
    straddle = MPLinearLayerConfig((4096, 4096), (1000, 4096), st.uint4b8, torch.float16, 128, False, False)
    assert not MarlinLinearKernel.can_implement(straddle)[0]


# ---------------------------------------------------------------- MoE routing (torch mirror)
@pytest.mark.parametrize("m,topk,e,bs", [(4, 3, 5, 4), (1, 2, 8, 8), (33, 2, 8, 16), (257, 2, 4, 64),
                                         (5, 6, 64, 16), (100, 1, 3, 48)])
def test_torch_moe_align_block_size_matches_oracle(m, topk, e, bs):
    import torch

    from sonar_amd import fused_moe
    rng = np.random.default_rng(m * 31 + e)
    ids = np.stack([rng.permutation(e)[:topk] for _ in range(m)]).astype(np.int32)
    want = mo.moe_align_block_size(ids, bs, e)
    got = fused_moe.moe_align_block_size(torch.from_numpy(ids), bs, e)
    past = int(want[2][0])
    assert int(got[2][0]) == past and got[2].dtype == torch.int32
    assert got[0].shape[0] == want[0].shape[0] and got[1].shape[0] == want[1].shape[0]
    assert np.array_equal(got[0].numpy()[:past], want[0][:past])
    assert np.all(got[0].numpy()[past:] == ids.size)
    assert np.array_equal(got[1].numpy(), want[1])


def test_torch_moe_align_docstring_example_and_expert_map():
    import torch

    from sonar_amd import fused_moe
    ids = torch.tensor([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], dtype=torch.int32)
    s, e, p = fused_moe.moe_align_block_size(ids, 4, 5)
    assert s[:16].tolist() == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert e[:4].tolist() == [1, 2, 3, 4] and int(p) == 16
    # experts 1 and 3 live on this rank as local experts 0 and 1
    emap = torch.tensor([-1, 0, -1, 1, -1], dtype=torch.int32)
    s2, e2, p2 = fused_moe.moe_align_block_size(ids, 4, 5, emap, ignore_invalid_experts=True)
    assert int(p2) == 8 and e2[:2].tolist() == [0, 1] and s2[:8].tolist() == [3, 6, 9, 12, 1, 7, 11, 12]
    assert (e2[2:] == -1).all() and (s2[8:] == 12).all()
    s3, e3, p3 = fused_moe.moe_align_block_size(ids, 4, 5, emap, ignore_invalid_experts=False)
    assert int(p3) == 16 and e3[:4].tolist() == [0, -1, 1, -1] and torch.equal(s3, s)


def test_moe_block_size_and_silu_and_mul():
    import torch

    from sonar_amd import fused_moe
    for m, topk, e in [(16, 2, 8), (4096, 2, 8), (1, 2, 8), (64, 6, 64), (300, 2, 8)]:
        assert fused_moe.moe_block_size(m, topk, e) == mo.moe_block_size_rule(m, topk, e)
    x = torch.randn(5, 8)
    out = torch.empty(5, 4)
    fused_moe.silu_and_mul(out, x)
    assert torch.allclose(out, x[:, :4] / (1 + torch.exp(-x[:, :4])) * x[:, 4:], atol=1e-6)


def test_kernels_with_hand_counted_waits_do_not_spill():
    """The LDS-DMA kernels wait for their copies with hand-counted
    `s_waitcnt vmcnt(N)`; a register spill adds scratch loads and stores to the
    same counter and would silently weaken those waits."""
    import re
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    watched = [("gemm_tile.hip", "marlin_tile_async_kernel"), ("gemm_tile.hip", "marlin_tile_wide_kernel"),
               ("gemm_stream.hip", "marlin_stream_fast_kernel")]
    for src, kernel in watched:
        out = subprocess.run(
            [hipcc, "-O3", "--offload-arch=gfx950", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops", "-I", os.path.join(root, "include"), "-I", os.path.join(root, "sonar_amd", "csrc"),
             "-c", "--offload-device-only", "-Rpass-analysis=kernel-resource-usage",
             os.path.join(root, "sonar_amd", "csrc", src), "-o", os.devnull],
            capture_output=True, text=True, timeout=600)
        assert out.returncode == 0, out.stderr[-2000:]
        name = None
        seen = 0
        for line in out.stderr.splitlines():
            m = re.search(r"Function Name: (\S+)", line)
            if m:
                name = m.group(1)
            m = re.search(r"VGPRs Spill: (\d+)", line)
            if m and name and kernel in name:
                seen += 1
                assert int(m.group(1)) == 0, f"{name} spills {m.group(1)} VGPRs"
        assert seen >= 4, f"no resource report for {kernel}"


KERNEL_FORMS = {
    "awq_to_marlin_kernel": 1, "gfx950_to_marlin_kernel": 1, "gptq8_to_marlin_a8_kernel": 1,
    "gptq8_to_marlin_kernel": 2, "gptq_to_marlin_kernel": 2, "int4_fp8_preprocess_kernel": 1,
    "marlin8_gfx950_kernel": 2, "marlin_a8_finish_kernel": 9, "marlin_a8_kernel": 68,
    "marlin_a8_tile_kernel": 48, "marlin_a8_to_gfx950_kernel": 1, "marlin_dequant8_kernel": 4,
    "marlin_dequant_kernel": 7, "marlin_fixup_kernel": 8, "marlin_moe8_kernel": 40, "marlin_moe_a8_kernel": 68,
    "marlin_moe_kernel": 52, "marlin_stream8_kernel": 40, "marlin_stream_fast_kernel": 68,
    "marlin_stream_kernel": 44, "marlin_tile_async_kernel": 38, "marlin_tile_kernel": 6,
    "marlin_tile_wide_kernel": 60, "marlin_to_gfx950_kernel": 1, "moe_activation_kernel": 12,
    "moe_align_count_kernel": 1, "moe_align_place_kernel": 1, "moe_permute_rows_kernel": 1,
    "moe_sum_kernel": 2, "moe_tile_reduce_kernel": 2, "moe_tile_table_kernel": 1, "per_token_quant_kernel": 6,
    "permute_columns_kernel": 1, "silu_and_mul_kernel": 2, "tile_reduce_kernel": 2, "to_marlin_a8_kernel": 3,
}


def test_library_holds_the_kernel_forms_the_gpu_tests_launch():
    """The instantiations of every __global__ function in the built library,
    counted from its host-side launch stubs.  Each of the forms counted here is
    launched by at least one GPU parity case (compared against a kernel trace of
    the whole GPU suite); a count that changes means a form was added or dropped:
    give a new form a parity case before raising the number."""
    import collections
    import re
    import shutil
    import subprocess
    from sonar_amd import _lib
    nm = shutil.which("nm") or shutil.which("llvm-nm")
    if nm is None:
        pytest.skip("nm not available")
    _lib.load()
    syms = subprocess.run([nm, _lib._LIB_PATH], capture_output=True, text=True, timeout=120).stdout
    seen = collections.Counter(m.group(1) for m in re.finditer(r"__device_stub__\d*([a-z_0-9]+kernel)", syms))
    assert dict(seen) == KERNEL_FORMS


def test_awq_checkpoint_conversion_matches_gptq_packing():
    """AutoAWQ tensors through convert_awq_to_standard_format give what packing the
    same codes the GPTQ way gives (layers/quantization/auto_awq.py:93-153)."""
    import types
    from sonar_amd.marlin_linear import convert_awq_to_standard_format
    rng = np.random.default_rng(12)
    k, n, g = 256, 192, 64
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    zp = rng.integers(0, 16, size=(k // g, n), dtype=np.int32)
    q[:, :8] = 15       # top nibble of a word set: sign handling
    zp[:, -8:] = 15
    layer = types.SimpleNamespace(qweight=torch.from_numpy(mo.awq_pack(q)), qzeros=torch.from_numpy(mo.awq_pack(zp)))
    convert_awq_to_standard_format(layer)
    assert layer.qweight.dtype == torch.int32 and layer.qweight.shape == (k // 8, n)
    assert np.array_equal(layer.qweight.numpy(), mo.pack_rows(q))
    assert layer.qzeros.shape == (n // 8, k // g)
    assert np.array_equal(layer.qzeros.numpy(), mo.pack_rows(np.ascontiguousarray(zp.T)))
    # and the converted zero points unpack to the codes again (pack_cols form, transposed)
    assert np.array_equal(mo.unpack_cols(np.ascontiguousarray(layer.qzeros.numpy().T)), zp)


def test_support_checks_follow_the_reference_rules():
    """marlin_utils.py:111-203, 284-359 of the reference: type / group-size
    gate, shape gate (N % 64, K % 128, groups dividing the shard), layer gates
    and the MoE intermediate-size helpers, on values worked out by hand."""
    from types import SimpleNamespace as NS
    from sonar_amd import marlin_utils as mu
    from sonar_amd.scalar_type import scalar_types as st
    assert mu.check_marlin_supported(st.uint4b8, 128)
    assert mu.check_marlin_supported(st.uint8b128, -1)
    assert mu.check_marlin_supported(st.uint4, 64, has_zp=True)
    assert not mu.check_marlin_supported(st.uint4, 64, has_zp=False)
    assert not mu.check_marlin_supported(st.uint4b8, 100)
    assert not mu.check_marlin_supported(st.uint8, 128, has_zp=True)   # 8-bit codes with zero points: not built
    mu.verify_marlin_supported(st.uint4b8, 32)
    with pytest.raises(ValueError, match="group_size = 256"):
        mu.verify_marlin_supported(st.uint4b8, 256)
    with pytest.raises(ValueError, match="weight_bits"):
        mu.verify_marlin_supported(st.uint8, 128, has_zp=True)
    mu.verify_marlin_supports_shape(4096, 4096, 4096, 128)
    with pytest.raises(ValueError, match="min_thread_n"):
        mu.verify_marlin_supports_shape(4000, 4096, 4096, 128)
    with pytest.raises(ValueError, match="min_thread_k"):
        mu.verify_marlin_supports_shape(4096, 4160, 8320, 128)
    # a row-parallel shard of 1408 rows (11 groups of 128) passes, one of 1344 rows does not
    layer = NS(output_size=4096, input_size=5632, output_size_per_partition=4096, input_size_per_partition=1408)
    assert mu.check_marlin_supports_layer(layer, 128)
    layer.input_size_per_partition = 1344
    assert not mu.check_marlin_supports_layer(layer, 128)
    assert not mu.check_marlin_supports_layer(layer, 128, allow_tile_padding=True)   # a group straddles the shard
    assert mu.check_marlin_supports_layer(layer, 64, allow_tile_padding=True)
    assert mu.check_marlin_supports_layer(layer, -1, allow_tile_padding=True)
    # MoE: lcm(64, group) granularity
    assert mu.marlin_moe_padded_intermediate(1408, 128) == 1408
    assert mu.marlin_moe_padded_intermediate(1000, 128) == 1024
    assert mu.marlin_moe_padded_intermediate(1000, -1) == 1024
    assert mu.marlin_moe_padded_intermediate(100, 32) == 128
    moe = NS(hidden_size=2048, apply_router_weight_on_input=False,
             moe_config=NS(intermediate_size_per_partition_unpadded=1408))
    assert mu.check_moe_marlin_supports_layer(moe, 128)
    assert mu.check_moe_marlin_supports_layer(moe, 64)
    assert not mu.check_moe_marlin_supports_layer(moe, 256)
    moe.moe_config.intermediate_size_per_partition_unpadded = 1376      # 43 * 32
    assert not mu.check_moe_marlin_supports_layer(moe, 32)
    assert mu.check_moe_marlin_supports_layer(moe, 32, allow_tile_padding=True)
    moe.apply_router_weight_on_input = True
    assert not mu.check_moe_marlin_supports_layer(moe, 32, allow_tile_padding=True)
    w2 = torch.zeros((4, 1408 // 16, 2048 * 2), dtype=torch.int32)
    assert mu.marlin_moe_intermediate_size(None, w2) == 1408


def test_moe_packed_zero_points_match_oracle():
    """Zero points packed eight to a word along the columns, in plain order,
    per expert: unpack, then the op's layout (marlin_utils.py:538-559)."""
    from sonar_amd import marlin_utils as mu
    rng = np.random.default_rng(12)
    experts, groups, n = 3, 4, 128
    zp = rng.integers(0, 16, size=(experts, groups, n)).astype(np.int32)
    packed = np.stack([mo.pack_cols(zp[e]) for e in range(experts)])
    got = mu.moe_packed_to_marlin_zero_points(torch.from_numpy(packed.view(np.int32)), groups, n, 4)
    want = np.stack([mo.marlin_zero_points(zp[e], groups, n) for e in range(experts)])
    assert np.array_equal(got.numpy().view(np.uint32), want.view(np.uint32))


def test_batched_moe_align_matches_docstring_example_and_oracle():
    """The literal example of moe_align_block_size.py:129-162 (5 batches of 8
    rows, blocks of 4, 2 / 3 / 0 / 6 / 8 valid rows).  Its expert_ids line lists
    experts 5, which five batches cannot have; the kernel
    (moe_align_sum_kernels.cu:70-81) gives a block the id of its batch, hence
    0 1 3 3 4 4.  Then the torch version against the oracle on random counts."""
    from sonar_amd.fused_moe import batched_moe_align_block_size
    counts = [2, 3, 0, 6, 8]
    want_ids = [0, 1, 40, 40, 8, 9, 10, 40, 24, 25, 26, 27, 28, 29, 40, 40, 32, 33, 34, 35, 36, 37, 38, 39] + [40] * 16
    want_experts = [0, 1, 3, 3, 4, 4, -1, -1, -1, -1]
    for fn in (mo.batched_moe_align_block_size,
               lambda m, b, c: [t.numpy() for t in batched_moe_align_block_size(m, b, torch.tensor(c, dtype=torch.int32))]):
        ids, experts, past = fn(8, 4, counts)
        assert ids.tolist() == want_ids and experts.tolist() == want_experts and past.tolist() == [24]
    rng = np.random.default_rng(3)
    for _ in range(40):
        batches = int(rng.integers(1, 12))
        max_tokens = int(rng.integers(1, 70))
        bs = int(rng.choice([4, 8, 16, 32, 48, 64]))
        counts = rng.integers(0, max_tokens + 1, size=batches).astype(np.int32)
        got = batched_moe_align_block_size(max_tokens, bs, torch.from_numpy(counts))
        want = mo.batched_moe_align_block_size(max_tokens, bs, counts)
        for g, w in zip(got, want):
            assert g.dtype == torch.int32 and np.array_equal(g.numpy(), w), (batches, max_tokens, bs, counts)


def test_marlin_test_utils_match_the_oracle_layout():
    """get_weight_perm / marlin_weights (marlin_utils_test.py:31-121) against the
    oracle's restatement of the same recipe and its closed form, 4 and 8 bits;
    gptq_pack / awq_pack against the oracle's packings."""
    from tests import marlin_utils_for_tests as mt
    from tests import quant_utils as qu
    assert np.array_equal(mt.get_weight_perm(4).numpy(), mo.marlin_weight_perm_recipe())
    assert np.array_equal(mt.get_weight_perm(8).numpy(), mo.marlin_weight_perm_recipe8())
    rng = np.random.default_rng(0)
    q = rng.integers(0, 16, size=(128, 192)).astype(np.int32)
    got = mt.marlin_weights(torch.from_numpy(q), 128, 192, 4, mt.get_weight_perm(4)).numpy()
    assert np.array_equal(got.view(np.uint32).ravel(), mo.marlin_pack_closed_form(q).view(np.uint32).ravel())
    q8 = rng.integers(0, 256, size=(64, 128)).astype(np.int32)
    got = mt.marlin_weights(torch.from_numpy(q8), 64, 128, 8, mt.get_weight_perm(8)).numpy()
    assert np.array_equal(got.view(np.uint32).ravel(), mo.marlin_pack8_closed_form(q8).view(np.uint32).ravel())
    assert np.array_equal(qu.gptq_pack(torch.from_numpy(q), 4, 128, 192).numpy(), mo.gptq_pack(q))
    assert np.array_equal(qu.awq_pack(torch.from_numpy(q), 4, 128, 192).numpy(), mo.awq_pack(q))
    assert np.array_equal(qu.gptq_pack(torch.from_numpy(q8), 8, 64, 128).numpy(), mo.pack_rows8(q8))


def test_quantize_weights_on_hand_worked_groups():
    """quant_utils.py:588-679 on columns whose answer is known: a symmetric
    group spanning [-8, 7] has scale 1 and codes value + 8; an asymmetric group
    spanning [-3, 12] has scale 1 and zero point 3; and in general the codes
    are in range, w_ref = (code - zero) * scale and |w - w_ref| <= scale / 2."""
    from tests import quant_utils as qu
    from sonar_amd.scalar_type import scalar_types as st
    col = torch.tensor([-8.0, 7.0, 0.0, 3.0, -1.0, 2.0, -5.0, 6.0]).repeat(4)      # one group of 32 rows
    w = torch.stack([col, 0.5 * col], dim=1)
    w_ref, q, s, zp = qu.quantize_weights(w, st.uint4b8, 32)
    assert zp is None and s.tolist() == [[1.0, 0.5]]
    assert torch.equal(q[:, 0], (col + 8).int()) and torch.equal(q[:, 1], (col + 8).int())
    assert torch.equal(w_ref, w)
    col = torch.tensor([-3.0, 12.0, 0.0, 5.0]).repeat(8)
    w_ref, q, s, zp = qu.quantize_weights(col.view(-1, 1), st.uint4, 32, zero_points=True)
    assert s.item() == 1.0 and zp.item() == 3 and torch.equal(q[:, 0], (col + 3).int())
    assert torch.equal(w_ref[:, 0], col)
    gen = torch.Generator().manual_seed(1)
    w = torch.randn((256, 64), generator=gen)
    for qt, zero in ((st.uint4b8, False), (st.uint8b128, False), (st.uint4, True)):
        w_ref, q, s, zp = qu.quantize_weights(w, qt, 64, zero_points=zero)
        top = 2 ** qt.size_bits - 1
        assert q.min() >= 0 and q.max() <= top and s.shape == (4, 64)
        z = zp.repeat_interleave(64, 0) if zero else (top + 1) // 2
        assert torch.allclose(w_ref, (q - z).float() * s.repeat_interleave(64, 0))
        inside = (q > 0) & (q < top)        # not clamped
        assert ((w - w_ref).abs()[inside] <= 0.5 * s.repeat_interleave(64, 0)[inside] + 1e-6).all()
    # act-order: rows permuted, g_idx names the group each row came from; sorting restores runs of groups
    w_ref, q, s, g_idx, rand_perm = qu.gptq_quantize_weights(w, st.uint4b8, 64, True)
    assert torch.equal(g_idx, (rand_perm // 64).int())
    q_sorted, g_sorted, sort_indices = qu.sort_weights(q, g_idx)
    assert torch.equal(g_sorted, torch.arange(256).int() // 64) and torch.equal(q_sorted, q[sort_indices.long()])


def test_marlin_post_load_preserves_runtime_tensor_addresses(monkeypatch):
    """tests/model_executor/model_loader/test_reload.py:158-258 of the reference:
    loading new checkpoint tensors into a layer and running
    process_weights_after_loading again keeps the workspace and the sort
    indices at their addresses (zeroed / refilled in place), so a recorded
    graph keeps reading live tensors."""
    import types
    from sonar_amd import marlin_linear, marlin_utils, ops
    from sonar_amd.scalar_type import scalar_types
    size_k, size_n, group = 128, 64, 64
    monkeypatch.setattr(marlin_utils, "num_compute_units", lambda _=None: 4)
    monkeypatch.setattr(ops, "gptq_marlin_repack",
                        lambda w, perm, size_k, size_n, num_bits, is_a_8bit=False:
                        torch.zeros(size_k // 16, size_n * 2, dtype=torch.int32))
    cfg = marlin_linear.MPLinearLayerConfig((size_k, size_n), (size_k, size_n), scalar_types.uint4b8,
                                            torch.float16, group, False, True)
    kernel = marlin_linear.MarlinLinearKernel(cfg, w_zp_param_name=None, w_gidx_param_name="g_idx")
    gen = torch.Generator().manual_seed(0)
    layer = types.SimpleNamespace()

    def load(g_idx):
        layer.qweight = torch.zeros(size_k // 8, size_n, dtype=torch.int32)
        layer.scales = torch.ones(size_k // group, size_n, dtype=torch.float16)
        layer.g_idx = g_idx.clone()

    first = torch.randint(0, size_k // group, (size_k,), dtype=torch.int32, generator=gen)
    second = torch.randint(0, size_k // group, (size_k,), dtype=torch.int32, generator=gen)
    load(first)
    kernel.process_weights_after_loading(layer)
    workspace_ptr = kernel.workspace.data_ptr()
    sort_ptr = layer.g_idx_sort_indices.data_ptr()
    kernel.workspace.fill_(3)           # a reload must hand the workspace back zeroed
    load(second)
    kernel.process_weights_after_loading(layer)
    assert kernel.workspace.data_ptr() == workspace_ptr and torch.all(kernel.workspace == 0)
    assert layer.g_idx_sort_indices.data_ptr() == sort_ptr
    assert torch.equal(layer.g_idx_sort_indices.data, marlin_utils.marlin_sort_g_idx(second)[1])
    assert isinstance(layer.g_idx_sort_indices, torch.nn.Parameter)


def test_fp8_host_helpers():
    """marlin_utils_fp8.py:35-46, 366-378 of the reference: the exponent-bias
    factor (2^8 / 2^120) and the packing of four consecutive K to a word, on
    values worked out by hand; fp8 joins the supported types without zero points."""
    from sonar_amd import marlin_utils as mu
    from sonar_amd import marlin_utils_fp8 as f8
    from sonar_amd.scalar_type import scalar_types as st
    s = torch.tensor([[0.5, 3.0]], dtype=torch.float16)
    assert torch.equal(f8.fp8_fused_exponent_bias_into_scales(s), torch.tensor([[128.0, 768.0]], dtype=torch.float16))
    s = torch.tensor([[2.0 ** -10]], dtype=torch.bfloat16)
    assert f8.fp8_fused_exponent_bias_into_scales(s).float().item() == 2.0 ** 110
    with pytest.raises(TypeError):
        f8.fp8_fused_exponent_bias_into_scales(torch.ones(1))
    # (K, N) = (8, 2): word [k/4][n] holds codes k%4 = 0..3 from the low byte up
    codes = torch.arange(16, dtype=torch.uint8).view(8, 2)
    words = f8.pack_fp8_to_int32(codes.view(torch.float8_e4m3fn), size_k_first=True)
    assert words.shape == (2, 2) and words.dtype == torch.int32
    assert words[0, 0].item() == 0 | (2 << 8) | (4 << 16) | (6 << 24)
    assert words[1, 1].item() == 9 | (11 << 8) | (13 << 16) | (15 << 24)
    by_n = f8.pack_fp8_to_int32(codes.T.contiguous().view(torch.float8_e4m3fn), size_k_first=False)
    assert torch.equal(by_n.T, words)
    assert np.array_equal(words.numpy().view(np.uint32), mo.pack_rows8(codes.numpy().astype(np.int32)).view(np.uint32))
    assert mu.check_marlin_supported(st.float8_e4m3fn, 128) and mu.check_marlin_supported(st.float8_e4m3fn, -1)
    assert not mu.check_marlin_supported(st.float8_e4m3fn, 128, has_zp=True)
    assert st.float8_e4m3fn not in mu.query_marlin_supported_quant_types(False, include_fp_type=False)
    assert f8.is_fp8_marlin_supported()


def test_mxfp4_host_helpers():
    """marlin_utils_fp4.py:123-135 of the reference: the scale rows with every
    four neighbours in the order 0, 2, 1, 3, as exponent bytes; float4_e2m1f
    joins the supported types without zero points."""
    from sonar_amd import marlin_utils as mu
    from sonar_amd import marlin_utils_fp4 as f4
    from sonar_amd.scalar_type import scalar_types as st
    e = torch.tensor([[120, 121, 122, 123, 124, 125, 126, 127]], dtype=torch.uint8)
    s = e.view(torch.float8_e8m0fnu).to(torch.bfloat16)
    assert s[0, 7].item() == 1.0 and s[0, 0].item() == 2.0 ** -7
    out = f4.mxfp4_marlin_process_scales(s)
    assert out.dtype == torch.float8_e8m0fnu
    assert out.view(torch.uint8).tolist() == [[120, 122, 121, 123, 124, 126, 125, 127]]
    assert np.array_equal(out.view(torch.uint8).numpy(), mo.mxfp4_process_scales(e.numpy()))
    a8 = f4.mxfp4_marlin_process_scales(s, input_dtype=torch.float8_e4m3fn)   # in place, plus 6
    assert a8.dtype == torch.float8_e8m0fnu
    assert a8.view(torch.uint8).tolist() == [[v + 6 for v in e.view(-1).tolist()]]
    assert np.array_equal(a8.view(torch.uint8).numpy(), mo.mxfp4_process_scales_a8(e.numpy()))
    from sonar_amd import marlin_utils_fp8 as f8   # MXFP8: the same reorder (marlin_utils_fp8.py:381-386)
    assert torch.equal(f8.mxfp8_marlin_process_scales(s).view(torch.uint8), out.view(torch.uint8))
    assert mu.check_marlin_supported(st.float4_e2m1f, 32)
    assert not mu.check_marlin_supported(st.float4_e2m1f, 32, has_zp=True)
    assert f4.is_fp4_marlin_supported()


def test_marlin_experts_configuration_logic():
    """MarlinExpertsBase (marlin_moe.py:568-704): the weight type from the configuration flags,
    the problem size from the packed tensors, the workspaces of both activation formats, the
    activations it accepts."""
    import torch
    from sonar_amd import marlin_experts as me
    from sonar_amd.scalar_type import scalar_types
    moe = me.ExpertsMoeConfig()
    ids = {
        "use_int4_w4a16": scalar_types.uint4b8.id, "use_int8_w8a16": scalar_types.uint8b128.id,
        "use_fp8_w8a16": scalar_types.float8_e4m3fn.id, "use_mxfp4_w4a16": scalar_types.float4_e2m1f.id,
        "use_nvfp4_w4a16": scalar_types.float4_e2m1f.id,
    }
    for flag, want in ids.items():
        assert me.MarlinExperts(moe, me.ExpertsQuantConfig(**{flag: True})).quant_type_id == want
    zp = me.ExpertsQuantConfig(use_int4_w4a16=True, w1_zp=torch.zeros(1, dtype=torch.int32))
    assert me.MarlinExperts(moe, zp).quant_type_id == scalar_types.uint4.id
    with pytest.raises(AssertionError, match="Supports only"):
        me.MarlinExperts(moe, me.ExpertsQuantConfig())
    q = me.ExpertsQuantConfig(use_int4_w4a16=True, gemm1_clamp_limit=7.0, gemm1_alpha=1.702)
    ex = me.MarlinExperts(moe, q)
    assert (ex.gemm1_clamp_limit, ex.gemm1_alpha, ex.gemm1_beta) == (7.0, 1.702, 0.0)
    # (E, K / 16, 2 * 2N) and (E, N / 16, 2K) packed tensors
    e, k, n, m, topk = 8, 4096, 14336, 5, 2
    w1 = torch.empty((e, k // 16, 4 * n), dtype=torch.int32, device="meta")
    w2 = torch.empty((e, n // 16, 2 * k), dtype=torch.int32, device="meta")
    a = torch.empty((m, k), dtype=torch.float16, device="meta")
    ti = torch.empty((m, topk), dtype=torch.int32, device="meta")
    assert ex.moe_problem_size(a, w1, w2, ti) == (e, m, n, k, topk)
    assert ex.moe_problem_size(torch.empty((e, 9, k), device="meta"), w1, w2, ti) == (e, 9, n, k, topk)
    # marlin_moe.py:741-744: swapped against fused_marlin_moe's intermediate caches
    assert ex.workspace_shapes(m, n, k, topk, e, e, None, "silu") == \
        ((m * topk, max(n, k)), (m * topk * max(2 * n, k),), (m, k))
    b = me.BatchedMarlinExperts(moe, q, max_num_tokens=32, num_dispatchers=2)
    assert b.workspace_shapes(m, n, k, topk, e, e, None, "silu") == \
        ((e * 64, max(k, 2 * n)), (e * 64, n), (e, 64, k))
    assert ex.activation_format() == "standard" and b.activation_format() == "batched_experts"
    for name in ("silu", "gelu", "gelu_tanh", "situ", "swigluoai", "swigluoai_uninterleave", "swiglustep",
                 "silu_no_mul", "gelu_no_mul", "gelu_tanh_no_mul", "relu2_no_mul"):
        assert ex._supports_activation(name), name
    assert not ex._supports_activation("relu")
    assert ex._supports_no_act_and_mul()
