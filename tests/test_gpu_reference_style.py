"""The reference's own Marlin tests, re-stated on this repository's host
mirror (tests/kernels/quantization/test_marlin_gemm.py:188-600 of the
reference): real-valued random weights are quantised by `quantize_weights`,
laid out in Marlin order by the index recipe of `marlin_utils_test.py`
(independent of the repack kernels), and
  * the repack ops must reproduce that layout bit for bit
    (test_gptq_marlin_repack, test_awq_marlin_repack), and
  * `marlin_gemm` must agree with `torch.matmul(a, w_ref)` under the
    reference's criterion mean|out - ref| / mean|ref| < 0.04 (test_marlin_gemm,
    test_marlin_gemm_with_bias), over the reference's grid of shapes, group
    sizes, weight types (integer, fp8, MXFP4), act-order and is_k_full, for 16-bit
    activations and for int8 / float8_e4m3fn activations with 4-bit weights.
No oracle here: the expected values come from torch on the GPU, as in the
reference."""
from __future__ import annotations

import itertools

import pytest
import torch

from sonar_amd.scalar_type import scalar_types

pytestmark = pytest.mark.gpu

MARLIN_K_CHUNKS = [128]
MARLIN_N_CHUNKS = [64, 256]
MARLIN_REPACK_NK_FACTORS = [(4, 8), (7, 5), (13, 11)]
MNK_FACTORS = [(1, 1, 1), (1, 4, 8), (26, 37, 13), (257, 13, 11)]
DENSE_CONFIGS = [
    {"b_type": scalar_types.uint4, "group_blocks": [-1, 2, 4, 8]},                                # AWQ int4
    {"b_type": scalar_types.uint4b8, "support_act_order": True, "group_blocks": [-1, 2, 4, 8]},   # GPTQ int4
    {"b_type": scalar_types.uint8b128, "support_act_order": True, "group_blocks": [-1, 2, 4, 8]}, # GPTQ int8
    {"b_type": scalar_types.float8_e4m3fn, "group_blocks": [-1, 8]},                              # FP8
    {"b_type": scalar_types.float4_e2m1f, "a_type": [torch.bfloat16], "group_blocks": [2]},       # MXFP4
    {"a_quant": torch.int8, "b_type": scalar_types.uint4, "group_blocks": [-1, 2, 4, 8]},         # AWQ int4, int8 A
    {"a_quant": torch.int8, "b_type": scalar_types.uint4b8, "group_blocks": [-1, 2, 4, 8]},       # GPTQ int4, int8 A
    {"a_quant": torch.float8_e4m3fn, "b_type": scalar_types.uint4b8, "group_blocks": [-1, 2, 4, 8]},  # fp8 A
    {"a_quant": torch.float8_e4m3fn, "b_type": scalar_types.uint4, "group_blocks": [-1, 2, 4, 8]},
    {"a_quant": torch.float8_e4m3fn, "b_type": scalar_types.float4_e2m1f, "a_type": [torch.bfloat16],
     "group_blocks": [2]},                                                                      # MXFP4, fp8 A
]


def compute_max_diff(output, output_ref):
    return torch.mean(torch.abs(output - output_ref)) / torch.mean(torch.abs(output_ref))


def rand_data(shape, dtype=torch.float16):
    return torch.randn(shape, dtype=dtype, device="cuda")


@pytest.mark.parametrize("n_chunk", MARLIN_N_CHUNKS)
@pytest.mark.parametrize("quant_type", [scalar_types.uint4b8, scalar_types.uint8b128], ids=str)
@pytest.mark.parametrize("act_order", [False, True])
@pytest.mark.parametrize("is_a_8bit", [True, False])
@pytest.mark.parametrize("nk_factors", MARLIN_REPACK_NK_FACTORS)
def test_gptq_marlin_repack(n_chunk, quant_type, act_order, is_a_8bit, nk_factors):
    from sonar_amd import ops
    from tests.marlin_utils_for_tests import get_weight_perm, marlin_weights
    from tests.quant_utils import gptq_pack, gptq_quantize_weights, sort_weights
    n_factor, k_factor = nk_factors
    size_k, size_n, group_size = 128 * k_factor, n_chunk * n_factor, 128
    if act_order and is_a_8bit:
        return   # the reference's filter (test_marlin_gemm.py:205-212)
    b_weight = rand_data((size_k, size_n))
    w_ref, q_w, s, g_idx, rand_perm = gptq_quantize_weights(b_weight, quant_type, group_size, act_order)
    q_w_gptq = gptq_pack(q_w, quant_type.size_bits, size_k, size_n)
    sort_indices = torch.empty(0, dtype=torch.int, device=b_weight.device)
    if act_order:
        q_w, g_idx, sort_indices = sort_weights(q_w, g_idx)
    expected = marlin_weights(q_w, size_k, size_n, quant_type.size_bits,
                              get_weight_perm(quant_type.size_bits, is_a_8bit), is_a_8bit)
    got = ops.gptq_marlin_repack(q_w_gptq, sort_indices, size_k, size_n, quant_type.size_bits, is_a_8bit)
    torch.cuda.synchronize()
    assert torch.equal(expected, got)


@pytest.mark.parametrize("n_chunk", MARLIN_N_CHUNKS)
@pytest.mark.parametrize("is_a_8bit", [True, False])
@pytest.mark.parametrize("nk_factors", MARLIN_REPACK_NK_FACTORS)
def test_awq_marlin_repack(n_chunk, is_a_8bit, nk_factors):
    from sonar_amd import ops
    from tests.marlin_utils_for_tests import get_weight_perm, marlin_weights
    from tests.quant_utils import awq_pack, quantize_weights
    quant_type = scalar_types.uint4
    n_factor, k_factor = nk_factors
    size_k, size_n = 128 * k_factor, n_chunk * n_factor
    b_weight = rand_data((size_k, size_n))
    w_ref, q_w, s, zp = quantize_weights(b_weight, quant_type, 128, zero_points=True)
    q_w_awq = awq_pack(q_w, 4, size_k, size_n)
    expected = marlin_weights(q_w, size_k, size_n, 4, get_weight_perm(4, is_a_8bit), is_a_8bit)
    got = ops.awq_marlin_repack(q_w_awq, size_k, size_n, 4, is_a_8bit)
    torch.cuda.synchronize()
    assert torch.equal(expected, got)


def _gemm_cases():
    """The reference's filter (test_marlin_gemm.py:304-333) for 16-bit activations:
    group sizes that divide K and are smaller than it, act-order only with
    groups, is_k_full = True only together with act-order, fp32 reduce."""
    cases = []
    for cfg, (mf, nf, kf), n_chunk, act_order, is_k_full in itertools.product(
            DENSE_CONFIGS, MNK_FACTORS, MARLIN_N_CHUNKS, [False, True], [False, True]):
        size_m, size_n, size_k = mf, nf * n_chunk, kf * 128
        if act_order and not cfg.get("support_act_order", False):
            continue
        for dtype, group_blocks in itertools.product(cfg.get("a_type", [torch.float16, torch.bfloat16]),
                                                     cfg["group_blocks"]):
            group_size = group_blocks if group_blocks <= 0 else group_blocks * 16
            if group_size > 0 and size_k % group_size != 0:
                continue
            if act_order and group_size in (-1, size_k):
                continue
            if group_size == size_k:
                continue
            if not act_order and is_k_full:
                continue
            cases.append((cfg.get("a_quant"), cfg["b_type"], dtype, group_size, size_m, size_n, size_k, act_order,
                          is_k_full))
    return cases


@pytest.mark.parametrize("a_quant,b_type,dtype,group_size,size_m,size_n,size_k,act_order,is_k_full", _gemm_cases(),
                         ids=lambda v: str(v).replace("torch.", ""))
def test_marlin_gemm(a_quant, b_type, dtype, group_size, size_m, size_n, size_k, act_order, is_k_full):
    from sonar_amd import ops
    from sonar_amd.marlin_utils import marlin_make_workspace_new
    from sonar_amd.marlin_utils_fp4 import rand_marlin_weight_mxfp4_like
    from sonar_amd.marlin_utils_fp8 import marlin_quant_fp8_torch
    from tests.marlin_utils_for_tests import awq_marlin_quantize, marlin_quantize
    a_input = rand_data((size_m, size_k), dtype=dtype)
    b_weight = rand_data((size_k, size_n), dtype=dtype)
    from sonar_amd.marlin_utils import per_token_quant_fp8, per_token_quant_int8
    if b_type == scalar_types.uint4:
        w_ref, marlin_q_w, marlin_s, marlin_zp = awq_marlin_quantize(b_weight, b_type, group_size,
                                                                     input_dtype=a_quant)
        g_idx = sort_indices = None
    elif b_type == scalar_types.float8_e4m3fn:
        w_ref, marlin_q_w, marlin_s = marlin_quant_fp8_torch(b_weight.T.contiguous(), group_size)
        g_idx = sort_indices = marlin_zp = None
    elif b_type == scalar_types.float4_e2m1f:
        w_ref, marlin_q_w, marlin_s = rand_marlin_weight_mxfp4_like(b_weight.T, group_size, input_dtype=a_quant)
        g_idx = sort_indices = marlin_zp = None
    else:
        w_ref, marlin_q_w, marlin_s, g_idx, sort_indices, _ = marlin_quantize(b_weight, b_type, group_size, act_order,
                                                                              input_dtype=a_quant)
        marlin_zp = None
    workspace = marlin_make_workspace_new(w_ref.device)
    a_scales, a_input_ref = None, a_input
    if a_quant == torch.int8:                      # test_marlin_gemm.py:446-455
        a_input, a_scales = per_token_quant_int8(a_input)
        a_input_ref = (a_input.to(a_scales.dtype) * a_scales.view(-1, 1)).to(dtype)
        if group_size != -1:
            a_scales = (a_scales / 4096 * marlin_s.max()).float()
            marlin_s = (marlin_s / marlin_s.max() * 4096).round().to(torch.int16).view(dtype)
    elif a_quant == torch.float8_e4m3fn:           # test_marlin_gemm.py:456-459
        a_input, a_scales = per_token_quant_fp8(a_input)
        a_input_ref = (a_input.to(a_scales.dtype) * a_scales.view(-1, 1)).to(dtype)
    output = torch.empty((size_m, size_n), dtype=dtype, device=a_input.device)
    output = ops.marlin_gemm(a_input, output, marlin_q_w, None, marlin_s, a_scales, None, marlin_zp, g_idx,
                             sort_indices, workspace, b_type, a_input.shape[0], b_weight.shape[1], a_input.shape[1],
                             is_k_full=is_k_full, use_atomic_add=False, use_fp32_reduce=True, is_zp_float=False)
    output_ref = torch.matmul(a_input_ref, w_ref)
    torch.cuda.synchronize()
    assert compute_max_diff(output, output_ref) < 0.04


@pytest.mark.parametrize("size_m", [1, 256])
def test_marlin_gemm_with_bias(size_m):
    from sonar_amd import ops
    from sonar_amd.marlin_utils import marlin_make_empty_g_idx, marlin_make_workspace_new, marlin_permute_bias
    from tests.marlin_utils_for_tests import marlin_quantize
    quant_type, group_size = scalar_types.uint4b8, 128
    size_k, size_n = 1024, 2048
    a_input = rand_data((size_m, size_k))
    b_weight = rand_data((size_k, size_n))
    b_bias = rand_data((size_n,)) * 10
    marlin_bias = marlin_permute_bias(b_bias)
    w_ref, marlin_q_w, marlin_s, g_idx, sort_indices, _ = marlin_quantize(b_weight, quant_type, group_size, False)
    marlin_zp = marlin_make_empty_g_idx(marlin_s.device)
    workspace = marlin_make_workspace_new(a_input.device)
    output = ops.marlin_gemm(a_input, None, marlin_q_w, marlin_bias, marlin_s, None, None, marlin_zp, g_idx,
                             sort_indices, workspace, quant_type, a_input.shape[0], b_weight.shape[1],
                             a_input.shape[1], is_k_full=True, use_atomic_add=False, use_fp32_reduce=True,
                             is_zp_float=False)
    output_ref = torch.matmul(a_input, w_ref) + b_bias.view(1, -1)
    torch.cuda.synchronize()
    assert compute_max_diff(output, output_ref) < 0.04


# ---------------------------------------------------------------------------
# tests/kernels/moe/test_moe.py:129-143, 688-1010 of the reference: the fused
# Marlin MoE layer against a plain torch mixture of experts on the dequantised
# weights, atol 4e-2, over the reference's scenarios for integer, fp8 and MXFP4 weights.
MOE_CONFIGS = [
    {"b_type": scalar_types.uint4, "group_blocks": [-1, 2, 4, 8]},
    {"b_type": scalar_types.uint4b8, "support_act_order": True, "group_blocks": [-1, 2, 4, 8]},
    {"b_type": scalar_types.uint8b128, "support_act_order": True, "group_blocks": [-1, 2, 4, 8]},
    {"b_type": scalar_types.float8_e4m3fn, "group_blocks": [-1, 8]},
    {"b_type": scalar_types.float4_e2m1f, "a_type": torch.bfloat16, "group_blocks": [2]},
    {"a_quant": torch.int8, "b_type": scalar_types.uint4, "group_blocks": [-1, 2, 4, 8]},
    {"a_quant": torch.int8, "b_type": scalar_types.uint4b8, "group_blocks": [-1, 2, 4, 8]},
    {"a_quant": torch.float8_e4m3fn, "b_type": scalar_types.uint4b8, "group_blocks": [-1, 2, 4, 8]},
    {"a_quant": torch.float8_e4m3fn, "b_type": scalar_types.uint4, "group_blocks": [-1, 2, 4, 8]},
    {"a_quant": torch.float8_e4m3fn, "b_type": scalar_types.float4_e2m1f, "a_type": torch.bfloat16,
     "group_blocks": [2]},
]
MARLIN_MOE_SCENARIOS = [
    # (m, n, k, e, topk, ep_size, act_order, is_k_full)
    (1, 128, 256, 5, 2, 1, False, True),
    (1, 1024, 2048, 5, 2, 1, False, True),
    (133, 256, 256, 5, 2, 1, False, True),
    (133, 1024, 2048, 12, 3, 1, False, True),
    (128, 256, 256, 5, 2, 1, False, True),
    (128, 1024, 2048, 12, 3, 1, False, True),
    (64, 1024, 2048, 12, 3, 4, False, True),
    (1, 1024, 2048, 5, 2, 1, True, True),
    (133, 256, 256, 5, 2, 1, True, False),
]


def _moe_cases():
    cases = []
    for cfg in MOE_CONFIGS:
        for group_blocks in cfg["group_blocks"]:
            group_size = group_blocks if group_blocks <= 0 else group_blocks * 16
            for (m, n, k, e, topk, ep_size, act_order, is_k_full) in MARLIN_MOE_SCENARIOS:
                if act_order and not cfg.get("support_act_order", False):
                    continue
                if group_size > 0 and k % group_size != 0:
                    continue
                if act_order and group_size in (-1, k, n):
                    continue
                if group_size in (k, n):
                    continue
                cases.append((cfg.get("a_quant"), cfg["b_type"], cfg.get("a_type", torch.float16), group_size, m, n, k,
                              e, topk, ep_size, act_order, is_k_full))
    # beyond the reference's list: act-order shards (is_k_full = False) of 8-bit experts on routing blocks of
    # 8, 32, 48 and 64 slots, either activation type
    for dtype in (torch.float16, torch.bfloat16):
        for m in (1, 40, 90, 133):
            cases.append((None, scalar_types.uint8b128, dtype, 64, m, 256, 256, 5, 2, 1, True, False))
    return cases


def _marlin_moe_weights(w, quant_type, group_size, act_order, bias=None, input_dtype=None):
    """MarlinMoEWeightData.make (test_moe.py:774-892): every expert's (N, K)
    matrix quantised and laid out on its own, then stacked."""
    from sonar_amd.marlin_utils import marlin_permute_bias
    from sonar_amd.marlin_utils_fp4 import rand_marlin_weight_mxfp4_like, rand_marlin_weight_nvfp4_like
    from sonar_amd.marlin_utils_fp8 import marlin_quant_fp8_torch
    from tests.marlin_utils_for_tests import awq_marlin_quantize, marlin_quantize
    k = w.shape[-1]
    out = {"w_ref": [], "qweight": [], "scales": [], "zeros": [], "g_idx": [], "sort_indices": [], "bias": [],
           "global_scale": []}
    for i in range(w.shape[0]):
        if quant_type == scalar_types.uint4:
            w_ref, qweight, scales, zeros = awq_marlin_quantize(w[i].transpose(1, 0), quant_type, group_size,
                                                                input_dtype=input_dtype)
            out["zeros"].append(zeros)
        elif quant_type == scalar_types.float8_e4m3fn:
            w_ref, qweight, scales = marlin_quant_fp8_torch(w[i].contiguous(), group_size)
        elif quant_type == scalar_types.float4_e2m1f and group_size == 16:      # NVFP4 (test_moe.py:806-816)
            w_ref, qweight, scales, global_scale = rand_marlin_weight_nvfp4_like(w[i], group_size,
                                                                                 input_dtype=input_dtype)
            out["global_scale"].append(global_scale.reshape(()))
        elif quant_type == scalar_types.float4_e2m1f:
            w_ref, qweight, scales = rand_marlin_weight_mxfp4_like(w[i], group_size, input_dtype=input_dtype)
        else:
            w_ref, qweight, scales, g_idx, sort_indices, _ = marlin_quantize(
                w[i].transpose(1, 0), quant_type, group_size, act_order, torch.randperm(k), input_dtype=input_dtype)
            out["g_idx"].append(g_idx)
            out["sort_indices"].append(sort_indices)
        out["w_ref"].append(w_ref.T)
        out["qweight"].append(qweight)
        out["scales"].append(scales)
        if bias is not None:
            out["bias"].append(marlin_permute_bias(bias[i]))
    res = {name: (torch.stack(v).contiguous() if v else None) for name, v in out.items()}
    res["a_scales_factor"] = None
    if input_dtype == torch.int8 and group_size != -1:        # test_moe.py:876-880
        scales = res["scales"]
        res["a_scales_factor"] = 1 / 4096 * scales.max().float()
        res["scales"] = (scales / scales.max() * 4096).round().to(torch.int16).view(w.dtype)
    return res


def _torch_experts(a, w1, w2, topk_weight, topk_ids, expert_map=None, b1=None, b2=None, quant_dtype=None,
                   activation=None):
    """Plain mixture of experts on (E, 2N, K) / (E, K, N) matrices: for every
    token and routed expert silu(x W1_gate^T) * (x W1_up^T) through W2^T, summed
    with the routing weights; experts mapped to -1 contribute nothing.  With
    `quant_dtype` (int8 / float8_e4m3fn) the input of either product is quantised per row
    and dequantised first (torch_experts with quant_input_only, tests/kernels/utils.py:845-893)."""
    from sonar_amd.marlin_utils import marlin_quant_input

    def through_quant(x):
        if quant_dtype is None:
            return x
        q, s = marlin_quant_input(x, quant_dtype)
        return (q.float() * s.view(-1, 1)).to(x.dtype)

    m, k = a.shape
    n = w2.shape[-1]
    out = torch.zeros((m, k), dtype=torch.float32, device=a.device)
    a32 = through_quant(a).float()
    for ex in torch.unique(topk_ids).tolist():
        local = ex if expert_map is None else int(expert_map[ex])
        if local < 0:
            continue
        rows, slot = torch.nonzero(topk_ids == ex, as_tuple=True)
        h = a32[rows] @ w1[local].float().T
        if b1 is not None:
            h = h + b1[local].float()
        h = h.to(a.dtype).float()
        if activation is None:
            act = (torch.nn.functional.silu(h[:, :n]) * h[:, n:]).to(a.dtype)
        else:      # any other activation of the layer, in plain fp32 torch arithmetic
            act = activation(h).to(a.dtype)
        act = through_quant(act).float()
        y = act @ w2[local].float().T
        if b2 is not None:
            y = y + b2[local].float()
        out.index_add_(0, rows, y.to(a.dtype).float() * topk_weight[rows, slot].float().unsqueeze(1))
    return out.to(a.dtype)


@pytest.mark.parametrize("a_quant,b_type,dtype,group_size,m,n,k,e,topk,ep_size,act_order,is_k_full", _moe_cases(),
                         ids=lambda v: str(v).replace("torch.", ""))
def test_fused_marlin_moe(a_quant, b_type, dtype, group_size, m, n, k, e, topk, ep_size, act_order, is_k_full):
    from sonar_amd.fused_moe import fused_marlin_moe
    torch.manual_seed(1)
    a = torch.randn((m, k), device="cuda", dtype=dtype) / 10
    w1 = torch.randn((e, 2 * n, k), device="cuda", dtype=dtype) / 10
    w2 = torch.randn((e, k, n), device="cuda", dtype=dtype) / 10
    e_map = None
    if ep_size > 1:
        local_e = e // ep_size
        e_ids = torch.randperm(e, device="cuda")[:local_e]
        e_map = torch.full((e,), -1, device="cuda", dtype=torch.int32)
        e_map[e_ids] = torch.arange(local_e, device="cuda", dtype=torch.int32)
        w1, w2 = w1[e_ids], w2[e_ids]
    d1 = _marlin_moe_weights(w1, b_type, group_size, act_order, input_dtype=a_quant)
    d2 = _marlin_moe_weights(w2, b_type, group_size, act_order, input_dtype=a_quant)
    score = torch.randn((m, e), device="cuda", dtype=dtype)
    topk_weights, topk_ids = torch.topk(torch.softmax(score, dim=-1, dtype=torch.float32), topk)
    want = _torch_experts(a, d1["w_ref"], d2["w_ref"], topk_weights, topk_ids, e_map, quant_dtype=a_quant)
    got = fused_marlin_moe(a, d1["qweight"], d2["qweight"], None, None, d1["scales"], d2["scales"], topk_weights,
                           topk_ids.to(torch.int32), global_num_experts=e, expert_map=e_map, g_idx1=d1["g_idx"],
                           g_idx2=d2["g_idx"], input_global_scale1=d1["a_scales_factor"],
                           input_global_scale2=d2["a_scales_factor"], sort_indices1=d1["sort_indices"],
                           sort_indices2=d2["sort_indices"], w1_zeros=d1["zeros"], w2_zeros=d2["zeros"],
                           input_dtype=a_quant, quant_type_id=b_type.id, is_k_full=is_k_full)
    torch.cuda.synchronize()
    torch.testing.assert_close(got, want, atol=4e-2, rtol=0)
    # and this build's own bar for two chained GEMMs: 2e-2 of the largest reference value; twice that
    # with 8-bit activations, where an intermediate value that differs in its last bit can land in
    # the next quantisation step (1 / 16 of its size for float8_e4m3fn)
    bar = 2e-2 if a_quant is None else 4e-2
    assert float((got.float() - want.float()).abs().max()) <= bar * float(want.float().abs().max())


def _swigluoai_packed(h, limit=7.0, alpha=1.702, beta=1.0):
    n = h.shape[1] // 2
    g = h[:, :n].clamp(max=limit)
    u = h[:, n:].clamp(-limit, limit)
    return g * torch.sigmoid(alpha * g) * (u + beta)


MOE_ACTIVATIONS = {
    # name -> (keywords of fused_marlin_moe, fp32 torch form on the first GEMM's output, gated)
    "swigluoai_uninterleave": (dict(clamp_limit=7.0, gemm1_alpha=1.702, gemm1_beta=1.0), _swigluoai_packed, True),
    "silu+clamp": (dict(clamp_limit=0.5), lambda h: _swigluoai_packed(h, 0.5, 1.0, 0.0), True),
    "gelu": (dict(), lambda h: torch.nn.functional.gelu(h[:, :h.shape[1] // 2]) * h[:, h.shape[1] // 2:], True),
    "swiglustep": (dict(), lambda h: torch.nn.functional.silu(h[:, :h.shape[1] // 2]).clamp(max=7.0)
                   * h[:, h.shape[1] // 2:].clamp(-7.0, 7.0), True),
    "relu2_no_mul": (dict(), lambda h: torch.relu(h) ** 2, False),
    "silu_no_mul": (dict(), torch.nn.functional.silu, False),
}


@pytest.mark.parametrize("name", list(MOE_ACTIVATIONS))
@pytest.mark.parametrize("b_type,group_size,dtype", [(scalar_types.uint4b8, 128, torch.half),
                                                     (scalar_types.float4_e2m1f, 32, torch.bfloat16)],
                         ids=["uint4b8", "mxfp4"])
def test_fused_marlin_moe_other_activations(name, b_type, group_size, dtype):
    """The layer with the reference's other activations (marlin_moe.py:74-75, 93-94, 163-174;
    tests/kernels/moe/test_moe.py:1087-1161 for the one without a gate): the clamped SwiGLU of
    gpt-oss on MXFP4 experts among them, against a torch mixture of experts with that
    activation in fp32.  Activations whose values are scaled up here so that the clamps bite."""
    from sonar_amd.fused_moe import fused_marlin_moe
    kwargs, torch_form, gated = MOE_ACTIVATIONS[name]
    torch.manual_seed(3)
    m, n, k, e, topk = 33, 512, 256, 6, 2
    a = torch.randn((m, k), device="cuda", dtype=dtype)
    w1 = torch.randn((e, (2 if gated else 1) * n, k), device="cuda", dtype=dtype) / 4
    w2 = torch.randn((e, k, n), device="cuda", dtype=dtype) / 16
    d1 = _marlin_moe_weights(w1, b_type, group_size, False)
    d2 = _marlin_moe_weights(w2, b_type, group_size, False)
    score = torch.randn((m, e), device="cuda", dtype=dtype)
    topk_weights, topk_ids = torch.topk(torch.softmax(score, dim=-1, dtype=torch.float32), topk)
    want = _torch_experts(a, d1["w_ref"], d2["w_ref"], topk_weights, topk_ids, activation=torch_form)
    got = fused_marlin_moe(a, d1["qweight"], d2["qweight"], None, None, d1["scales"], d2["scales"], topk_weights,
                           topk_ids.to(torch.int32), global_num_experts=e, quant_type_id=b_type.id,
                           activation=name.split("+")[0], **kwargs)
    torch.cuda.synchronize()
    assert float((got.float() - want.float()).abs().max()) <= 2e-2 * float(want.float().abs().max())
    if name == "silu+clamp" and b_type == scalar_types.uint4b8:   # the clamp bites: the unclamped layer is elsewhere
        plain = fused_marlin_moe(a, d1["qweight"], d2["qweight"], None, None, d1["scales"], d2["scales"],
                                 topk_weights, topk_ids.to(torch.int32), global_num_experts=e,
                                 quant_type_id=b_type.id)
        assert float((plain.float() - want.float()).abs().max()) > 5e-2 * float(want.float().abs().max())


@pytest.mark.parametrize("m", [1, 64, 256])
@pytest.mark.parametrize("n,k", [(1024, 1024), (2048, 2048)])
@pytest.mark.parametrize("e,topk", [(8, 2), (64, 4)])
def test_fused_marlin_moe_non_gated(m, n, k, e, topk):
    """tests/kernels/moe/test_moe.py:1083-1161: NVFP4 experts (groups of 16, a global scale per
    expert) with relu2_no_mul, whose w1 is (e, n, k) and not (e, 2n, k); atol 1e-1."""
    from sonar_amd.fused_moe import fused_marlin_moe
    torch.manual_seed(42)
    quant_type, dtype = scalar_types.float4_e2m1f, torch.bfloat16
    a = torch.randn((m, k), device="cuda", dtype=dtype) / 10
    w1 = torch.randn((e, n, k), device="cuda", dtype=dtype) / 10
    w2 = torch.randn((e, k, n), device="cuda", dtype=dtype) / 10
    d1 = _marlin_moe_weights(w1, quant_type, 16, False)
    d2 = _marlin_moe_weights(w2, quant_type, 16, False)
    score = torch.randn((m, e), device="cuda", dtype=dtype)
    topk_weights, topk_ids = torch.topk(torch.softmax(score, dim=-1, dtype=torch.float32), topk)
    want = _torch_experts(a, d1["w_ref"], d2["w_ref"], topk_weights, topk_ids,
                          activation=lambda h: torch.relu(h) ** 2)
    got = fused_marlin_moe(a, d1["qweight"], d2["qweight"], None, None, d1["scales"], d2["scales"], topk_weights,
                           topk_ids.to(torch.int32), global_num_experts=e, expert_map=None,
                           global_scale1=d1["global_scale"], global_scale2=d2["global_scale"],
                           quant_type_id=quant_type.id, is_k_full=True, activation="relu2_no_mul")
    torch.cuda.synchronize()
    torch.testing.assert_close(got, want, atol=1e-1, rtol=0)


@pytest.mark.parametrize("m", [1, 256])
def test_fused_marlin_moe_with_bias(m):
    """test_moe.py:1013-1090: 32 experts, top 4, N = K = 2048, biases on both GEMMs."""
    from sonar_amd.fused_moe import fused_marlin_moe
    torch.manual_seed(0)
    e, topk, n, k, group_size = 32, 4, 2048, 2048, 128
    dtype = torch.half
    a = torch.randn((m, k), device="cuda", dtype=dtype) / 10
    w1 = torch.randn((e, 2 * n, k), device="cuda", dtype=dtype) / 10
    w2 = torch.randn((e, k, n), device="cuda", dtype=dtype) / 10
    b_bias1 = torch.randn((e, 2 * n), device="cuda", dtype=dtype) / 10
    b_bias2 = torch.randn((e, k), device="cuda", dtype=dtype) / 10
    d1 = _marlin_moe_weights(w1, scalar_types.uint4b8, group_size, False, b_bias1)
    d2 = _marlin_moe_weights(w2, scalar_types.uint4b8, group_size, False, b_bias2)
    score = torch.randn((m, e), device="cuda", dtype=dtype)
    topk_weights, topk_ids = torch.topk(torch.softmax(score, dim=-1, dtype=torch.float32), topk)
    want = _torch_experts(a, d1["w_ref"], d2["w_ref"], topk_weights, topk_ids, None, b_bias1, b_bias2)
    got = fused_marlin_moe(a, d1["qweight"], d2["qweight"], d1["bias"], d2["bias"], d1["scales"], d2["scales"],
                           topk_weights, topk_ids.to(torch.int32), global_num_experts=e, expert_map=None,
                           quant_type_id=scalar_types.uint4b8.id, is_k_full=True)
    torch.cuda.synchronize()
    torch.testing.assert_close(got, want, atol=4e-2, rtol=0)
