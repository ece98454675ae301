"""torch.library.opcheck on the four ops of the boundary, as the reference's kernel
tests run it (tests/kernels/utils.py:978-992, used by
tests/kernels/quantization/test_marlin_gemm.py:238,280 and the GEMM tests): schema,
autograd registration, fake-tensor implementation and dynamic-shape AOT dispatch must
agree with what the op really does."""
import numpy as np
import pytest
import torch

from oracle import marlin_oracle as mo

pytestmark = pytest.mark.gpu

OPCHECK_TEST_UTILS = ("test_schema", "test_autograd_registration", "test_faketensor", "test_aot_dispatch_dynamic")
DEV = "cuda:0"


def opcheck(op, args, c_given=False):
    """With `c_or_none` given the op writes into that tensor and returns it
    (marlin.cu:694-708, moe/marlin_moe_wna16/ops.cu:693-706), which the reference's schema
    (copied verbatim: `Tensor? c_or_none, ... -> Tensor`, no alias annotation) does not
    declare, so the schema check must report exactly that aliasing and nothing else; the
    other checks must pass.  The reference's own tests only run opcheck with c = None."""
    if not c_given:
        return torch.library.opcheck(op, args, test_utils=OPCHECK_TEST_UTILS, raise_exception=True)
    res = torch.library.opcheck(op, args, test_utils=OPCHECK_TEST_UTILS, raise_exception=False)
    assert "not defined to alias output" in str(res["test_schema"]), res
    assert res["test_autograd_registration"] == "SUCCESS", res
    # the fake implementation mirrors the reference's (_custom_ops.py:1518-1543: a new empty
    # tensor whatever c is), so the only difference it may show is that aliasing
    for name in ("test_faketensor", "test_aot_dispatch_dynamic"):
        assert res[name] == "SUCCESS" or "alias" in str(res[name]), res
    return res


@pytest.fixture(scope="module")
def layer():
    from sonar_amd import marlin_utils, ops  # noqa: F401  (registers the ops and their fake implementations)
    k, n, g = 256, 128, 128
    made = mo.make_layer(5, k, n, g, "fp16")
    q = made["q"]
    empty = torch.empty(0, dtype=torch.int32, device=DEV)
    qw = torch.from_numpy(mo.gptq_pack(q)).to(DEV)
    marlin = ops.gptq_marlin_repack(qw, empty, k, n, 4)
    scales = marlin_utils.marlin_permute_scales(torch.from_numpy(made["scales"]).to(DEV).half(), k, n, g)
    ws = marlin_utils.marlin_make_workspace_new(torch.device(DEV), 4)
    return dict(k=k, n=n, g=g, q=q, qw=qw, marlin=marlin, scales=scales, ws=ws, empty=empty)


def test_opcheck_gptq_marlin_repack(layer):
    opcheck(torch.ops._C.gptq_marlin_repack, (layer["qw"], layer["empty"], layer["k"], layer["n"], 4, False))
    perm = torch.randperm(layer["k"], device=DEV).to(torch.int32)
    opcheck(torch.ops._C.gptq_marlin_repack, (layer["qw"], perm, layer["k"], layer["n"], 4, False))


def test_opcheck_awq_marlin_repack(layer):
    qa = torch.from_numpy(mo.awq_pack(layer["q"])).to(DEV)
    opcheck(torch.ops._C.awq_marlin_repack, (qa, layer["k"], layer["n"], 4, False))


@pytest.mark.parametrize("with_c", [False, True])
def test_opcheck_marlin_gemm(layer, with_c):
    from sonar_amd.scalar_type import scalar_types
    m = 8
    a = torch.randn((m, layer["k"]), device=DEV, dtype=torch.float16)
    c = torch.empty((m, layer["n"]), device=DEV, dtype=torch.float16) if with_c else None
    args = (a, c, layer["marlin"], None, layer["scales"], None, None, layer["empty"], layer["empty"], layer["empty"],
            layer["ws"], scalar_types.uint4b8.id, m, layer["n"], layer["k"], True, False, True, False)
    opcheck(torch.ops._C.marlin_gemm, args, c_given=with_c)
    opcheck(torch.ops._C.gptq_marlin_gemm, args, c_given=with_c)
    assert int(layer["ws"].abs().sum().item()) == 0


@pytest.mark.parametrize("with_c", [False, True])
def test_opcheck_moe_wna16_marlin_gemm(layer, with_c):
    from sonar_amd import fused_moe
    from sonar_amd.scalar_type import scalar_types
    m, e, top_k, bs = 12, 4, 2, 8
    k, n = layer["k"], layer["n"]
    w = layer["marlin"].unsqueeze(0).repeat(e, 1, 1).contiguous()
    s = layer["scales"].unsqueeze(0).repeat(e, 1, 1).contiguous()
    a = torch.randn((m, k), device=DEV, dtype=torch.float16)
    topk_ids = torch.stack([torch.randperm(e, device=DEV)[:top_k] for _ in range(m)]).to(torch.int32)
    topk_w = torch.rand((m, top_k), device=DEV, dtype=torch.float32)
    sorted_ids, expert_ids, past = fused_moe.moe_align_block_size(topk_ids, bs, e)
    c = torch.empty((m * top_k, n), device=DEV, dtype=torch.float16) if with_c else None
    args = (a, c, w, None, s, None, None, None, None, None, layer["ws"], sorted_ids, expert_ids, past, topk_w, bs,
            top_k, False, scalar_types.uint4b8.id, m, n, k, True, False, True, False, -1, -1, -1)
    opcheck(torch.ops._moe_C.moe_wna16_marlin_gemm, args, c_given=with_c)


def test_opcheck_w4a8_ops(layer):
    """The ops of the 8-bit-activation path: repack with is_a_8bit, marlin_int4_fp8_preprocess
    (out of place, as the schema promises no mutation) and marlin_gemm with int8 / fp8 `a`."""
    from sonar_amd import marlin_utils
    from sonar_amd.scalar_type import scalar_types
    k, n = layer["k"], layer["n"]
    opcheck(torch.ops._C.gptq_marlin_repack, (layer["qw"], layer["empty"], k, n, 4, True))
    qa = torch.from_numpy(mo.awq_pack(layer["q"])).to(DEV)
    opcheck(torch.ops._C.awq_marlin_repack, (qa, k, n, 4, True))
    marlin8 = torch.ops._C.gptq_marlin_repack(layer["qw"], layer["empty"], k, n, 4, True)
    opcheck(torch.ops._C.marlin_int4_fp8_preprocess, (marlin8, None, False))
    scales = marlin_utils.marlin_permute_scales(
        torch.rand((k // 128, n), device=DEV, dtype=torch.float16) * 1e-2, k, n, 128, is_a_8bit=True)
    int_scales, _ = marlin_utils.marlin_act_int8_process_scales(scales)
    m = 8
    x = torch.randn((m, k), device=DEV, dtype=torch.float16)
    for quant, s in ((marlin_utils.per_token_quant_int8, int_scales), (marlin_utils.per_token_quant_fp8, scales)):
        a, a_s = quant(x)
        args = (a, None, marlin8, None, s, a_s, None, layer["empty"], layer["empty"], layer["empty"], layer["ws"],
                scalar_types.uint4b8.id, m, n, k, True, False, True, False)
        if a.dtype == torch.int8:
            opcheck(torch.ops._C.marlin_gemm, args)
        else:
            # the schema check perturbs its inputs with arithmetic torch does not have for float8_e4m3fn
            torch.library.opcheck(torch.ops._C.marlin_gemm, args, test_utils=OPCHECK_TEST_UTILS[1:],
                                  raise_exception=True)
    opcheck(torch.ops.sonar_amd.per_token_quant_int8, (x,))
    opcheck(torch.ops.sonar_amd.per_token_quant_fp8, (x,))
