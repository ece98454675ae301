"""Python op wrappers with the names and signatures of the reference's
aphrodite/_custom_ops.py (:1363-1461 repack, :1472-1543 marlin_gemm,
:3046-3141 moe_wna16_marlin_gemm).  Importing this module loads the HIP library
and the torch op registration layer; it raises if either is missing."""
from __future__ import annotations

import os

import torch

from . import _lib
from .scalar_type import ScalarType

_OPS_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libsonar_marlin_torch.so")


def _load_ops() -> None:
    if hasattr(torch.ops._C, "marlin_gemm") and hasattr(torch.ops._C, "marlin_to_gfx950"):
        return
    _lib.load()  # raises with build instructions when the HIP library is missing
    if not os.path.exists(_OPS_PATH):
        raise ImportError(f"{_OPS_PATH} is missing: build it with `python -m sonar_amd.build`")
    torch.ops.load_library(_OPS_PATH)


_load_ops()


def _register_fakes() -> None:
    reg = torch.library.register_fake

    @reg("_C::gptq_marlin_repack")
    def _(b_q_weight, perm, size_k, size_n, num_bits, is_a_8bit=False):
        pack_factor = 32 // num_bits
        return torch.empty((size_k // 16, size_n * 16 // pack_factor), dtype=b_q_weight.dtype,
                           device=b_q_weight.device)

    @reg("_C::awq_marlin_repack")
    def _(b_q_weight, size_k, size_n, num_bits, is_a_8bit=False):
        pack_factor = 32 // num_bits
        return torch.empty((size_k // 16, size_n * 16 // pack_factor), dtype=b_q_weight.dtype,
                           device=b_q_weight.device)

    @reg("_C::marlin_int4_fp8_preprocess")
    def _(qweight, qzeros_or_none=None, inplace=False):
        return torch.empty_like(qweight)

    def quant_fake(code_dtype):
        def fake(x):
            return (torch.empty(x.shape, dtype=code_dtype, device=x.device),
                    torch.empty(x.shape[:-1] + (1,), dtype=torch.float32, device=x.device))
        return fake

    reg("sonar_amd::per_token_quant_int8")(quant_fake(torch.int8))
    reg("sonar_amd::per_token_quant_fp8")(quant_fake(torch.float8_e4m3fn))

    @reg("_C::marlin_to_gfx950")
    def _(b_q_weight, size_k, size_n):
        return torch.empty_like(b_q_weight)

    def gemm_fake(a, c, b_q_weight, b_bias, b_scales, a_scales, global_scale, b_zeros, g_idx, perm,
                  workspace, b_q_type_id, size_m, size_n, size_k, is_k_full=True, use_atomic_add=False,
                  use_fp32_reduce=False, is_zp_float=False):
        dtype = a.dtype
        if dtype not in (torch.half, torch.bfloat16):
            dtype = b_scales.dtype
        return torch.empty((size_m, size_n), device=a.device, dtype=dtype)

    reg("_C::marlin_gemm")(gemm_fake)
    reg("_C::gptq_marlin_gemm")(gemm_fake)

    @reg("_moe_C::moe_wna16_marlin_gemm")
    def _(input, output, b_qweight, b_bias, b_scales, a_scales, global_scale, b_qzeros, g_idx, perm,
          workspace, sorted_token_ids, expert_ids, num_tokens_past_padded, topk_weights, moe_block_size,
          top_k, mul_topk_weights, b_q_type, size_m, size_n, size_k, is_k_full, use_atomic_add,
          use_fp32_reduce, is_zp_float, thread_k=-1, thread_n=-1, blocks_per_sm=-1):
        return torch.empty((size_m * top_k, size_n), dtype=input.dtype, device=input.device)


try:
    _register_fakes()
except RuntimeError:
    # already registered by another import of the same ops (e.g. the reference's own wrappers)
    pass


def gptq_marlin_repack(b_q_weight: torch.Tensor, perm: torch.Tensor, size_k: int, size_n: int,
                       num_bits: int, is_a_8bit: bool = False) -> torch.Tensor:
    return torch.ops._C.gptq_marlin_repack(b_q_weight, perm, size_k, size_n, num_bits, is_a_8bit)


def awq_marlin_repack(b_q_weight: torch.Tensor, size_k: int, size_n: int, num_bits: int,
                      is_a_8bit: bool = False) -> torch.Tensor:
    return torch.ops._C.awq_marlin_repack(b_q_weight, size_k, size_n, num_bits, is_a_8bit)


def gptq_marlin_moe_repack(b_q_weight: torch.Tensor, perm: torch.Tensor, size_k: int, size_n: int,
                           num_bits: int, is_a_8bit: bool = False) -> torch.Tensor:
    num_experts = b_q_weight.shape[0]
    assert size_k % 16 == 0
    output = torch.empty((num_experts, size_k // 16, size_n * (num_bits // 2)),
                         device=b_q_weight.device, dtype=b_q_weight.dtype)
    for e in range(num_experts):
        output[e] = torch.ops._C.gptq_marlin_repack(b_q_weight[e], perm[e], size_k, size_n, num_bits, is_a_8bit)
    return output


def awq_marlin_moe_repack(b_q_weight: torch.Tensor, perm: torch.Tensor, size_k: int, size_n: int,
                          num_bits: int, is_a_8bit: bool = False) -> torch.Tensor:
    num_experts = b_q_weight.shape[0]
    assert size_k % 16 == 0
    output = torch.empty((num_experts, size_k // 16, size_n * (num_bits // 2)),
                         device=b_q_weight.device, dtype=b_q_weight.dtype)
    for e in range(num_experts):
        output[e] = torch.ops._C.awq_marlin_repack(b_q_weight[e], size_k, size_n, num_bits, is_a_8bit)
    return output


def marlin_int4_fp8_preprocess(qweight: torch.Tensor, qzeros_or_none: torch.Tensor | None = None,
                               inplace: bool = False) -> torch.Tensor:
    """aphrodite/_custom_ops.py:1464-1469: 4-bit codes -> sign and magnitude of code - zero
    point, the form the fp8-activation kernels read."""
    return torch.ops._C.marlin_int4_fp8_preprocess(qweight, qzeros_or_none, inplace)


def per_token_quant_int8(x: torch.Tensor):
    """One scale per row, max(absmax, 1e-10) / 127, and int8 codes rounded half away from zero
    (the reference's Triton kernel, layers/quantization/utils/int8_utils.py:70-120).  Returns
    (int8 of x's shape, float32 (..., 1))."""
    return torch.ops.sonar_amd.per_token_quant_int8(x)


def per_token_quant_fp8(x: torch.Tensor):
    """Dynamic per-token float8_e4m3fn quantisation (QuantFP8(False, GroupShape.PER_TOKEN),
    layers/quantization/input_quant_fp8.py:188-204): scale = max(absmax / 448, 1 / (448 * 512))."""
    return torch.ops.sonar_amd.per_token_quant_fp8(x)


def marlin_gemm(a: torch.Tensor, c: torch.Tensor | None, b_q_weight: torch.Tensor,
                b_bias: torch.Tensor | None, b_scales: torch.Tensor, a_scales: torch.Tensor | None,
                global_scale: torch.Tensor | None, b_zeros: torch.Tensor | None,
                g_idx: torch.Tensor | None, perm: torch.Tensor | None, workspace: torch.Tensor,
                b_q_type: ScalarType, size_m: int, size_n: int, size_k: int, is_k_full: bool = True,
                use_atomic_add: bool = False, use_fp32_reduce: bool = False,
                is_zp_float: bool = False) -> torch.Tensor:
    return torch.ops._C.marlin_gemm(a, c, b_q_weight, b_bias, b_scales, a_scales, global_scale, b_zeros,
                                    g_idx, perm, workspace, b_q_type.id, size_m, size_n, size_k,
                                    is_k_full, use_atomic_add, use_fp32_reduce, is_zp_float)


gptq_marlin_gemm = marlin_gemm  # the op's older name


def moe_wna16_marlin_gemm(input: torch.Tensor, output: torch.Tensor | None, b_qweight: torch.Tensor,
                          b_bias: torch.Tensor | None, b_scales: torch.Tensor,
                          a_scales: torch.Tensor | None, global_scale: torch.Tensor | None,
                          b_qzeros: torch.Tensor | None, g_idx: torch.Tensor | None,
                          perm: torch.Tensor | None, workspace: torch.Tensor,
                          sorted_token_ids: torch.Tensor, expert_ids: torch.Tensor,
                          num_tokens_past_padded: torch.Tensor, topk_weights: torch.Tensor,
                          moe_block_size: int, top_k: int, mul_topk_weights: bool,
                          b_q_type: ScalarType, size_m: int, size_n: int, size_k: int, is_k_full: bool,
                          use_atomic_add: bool, use_fp32_reduce: bool, is_zp_float: bool,
                          thread_k: int = -1, thread_n: int = -1, blocks_per_sm: int = -1) -> torch.Tensor:
    return torch.ops._moe_C.moe_wna16_marlin_gemm(
        input, output, b_qweight, b_bias, b_scales, a_scales, global_scale, b_qzeros, g_idx, perm,
        workspace, sorted_token_ids, expert_ids, num_tokens_past_padded, topk_weights, moe_block_size,
        top_k, mul_topk_weights, b_q_type.id, size_m, size_n, size_k, is_k_full, use_atomic_add,
        use_fp32_reduce, is_zp_float, thread_k, thread_n, blocks_per_sm)


def marlin_to_gfx950(b_q_weight: torch.Tensor, size_k: int, size_n: int) -> torch.Tensor:
    """Marlin tile order -> the order the gfx950 kernels stream (no reference counterpart)."""
    return torch.ops._C.marlin_to_gfx950(b_q_weight, size_k, size_n)


def marlin_weight_cache_clear() -> int:
    """Drops the converted weight copies the GEMM ops keep; returns how many there were."""
    return torch.ops._C.marlin_weight_cache_clear()


def marlin_weight_cache_invalidate(t: torch.Tensor) -> int:
    """Drops the converted copies made from the memory of `t` (a Marlin weight tensor or a
    tensor of float8_e8m0fnu block scales); returns how many.  Needed after the bytes of `t`
    were rewritten in place in a way its version counter does not show (`t.data.copy_(...)`,
    any write to an inference-mode tensor).  Weights that come out of the repack ops, and
    in-place ops on `t` itself, need no call."""
    return torch.ops._C.marlin_weight_cache_invalidate(t)
