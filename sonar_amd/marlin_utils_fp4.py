"""4-bit floating-point weights (float4_e2m1f codes) through the Marlin ops.
Mirrors aphrodite/model_executor/layers/quantization/utils/marlin_utils_fp4.py
of the reference for dense layers and experts of both formats: :34-151,
153-290, 325-448, 556-649, 652-753.  The checkpoint bytes (two codes each, low nibble
first along K) are GPTQ words as they stand and go through gptq_marlin_repack
with num_bits = 4.  MXFP4: one power-of-two scale per 32 rows (exponent bytes e,
value 2^(e - 127)), bf16 activations; the scales are permuted as for any Marlin
layer, every four neighbours are put in the order 0, 2, 1, 3, and they travel
as float8_e8m0fnu.  NVFP4: one float8_e4m3fn scale per 16 rows and an fp32
global scale, fp16 or bf16 activations; the scales travel as bytes of the
reference's special 8-bit format (nvfp4_marlin_process_scales) and the global
scale carries the exponent bias of the kernel-side reading.
"""
from __future__ import annotations

import torch

from . import ops
from .marlin_utils import (USE_FP32_REDUCE_DEFAULT, get_marlin_input_dtype, marlin_make_workspace_new,
                           marlin_pad_dim, marlin_pad_qweight, marlin_pad_scales, marlin_padded_nk,
                           marlin_permute_bias, marlin_permute_scales, marlin_quant_input, marlin_repacked_nk,
                           marlin_unpad_output, should_use_atomic_add_reduce)
from .scalar_type import scalar_types

MXFP4_GROUP_SIZE = 32
FP4_MARLIN_SUPPORTED_GROUP_SIZES = [16]   # marlin_utils_fp4.py:29 (NVFP4)


def is_fp4_marlin_supported() -> bool:
    """marlin_utils_fp4.py:34-35; one target here, which runs MXFP4."""
    return True


def mxfp4_marlin_process_scales(marlin_scales: torch.Tensor, input_dtype: torch.dtype | None = None) -> torch.Tensor:
    """marlin_utils_fp4.py:123-135: for 16-bit activations (0, 2, 1, 3) inside every four, then
    the exponent bytes; for float8_e4m3fn activations the bytes in place, plus 6 (the fp4 codes
    enter the fp8 matrix instruction as value * 2^-6)."""
    if input_dtype is None or input_dtype.itemsize == 2:
        marlin_scales = marlin_scales.view(-1, 4)[:, [0, 2, 1, 3]].view(marlin_scales.size(0), -1)
    marlin_scales = marlin_scales.to(torch.float8_e8m0fnu)
    if input_dtype == torch.float8_e4m3fn:
        as_bytes = marlin_scales.view(torch.uint8)
        assert as_bytes.max() <= 249
        marlin_scales = (as_bytes + 6).view(torch.float8_e8m0fnu)   # exponent bias fp4 -> fp8: 2^3 - 2^1
    return marlin_scales


def _nvfp4_compute_scale_factor(marlin_scales: torch.Tensor, a_dtype: torch.dtype | None = None) -> float:
    """marlin_utils_fp4.py:37-58: the power of two (>= 1) after which the largest
    scale times 2^7 is just below 448 * 2^7; 1 for half activations."""
    if a_dtype is not None and a_dtype == torch.half:
        return 1.0
    ws_float = marlin_scales.float() * (2 ** 7)
    nonzero = ws_float > 0
    if nonzero.any():
        max_val = ws_float[nonzero].max()
        if max_val < 448 * (2 ** 7):
            return (448 * (2 ** 7) / max_val).log2().floor().exp2().item()
    return 1.0


def nvfp4_marlin_process_scales(marlin_scales: torch.Tensor, scale_factor: float | None = None,
                                a_dtype: torch.dtype | None = None) -> tuple[torch.Tensor, float]:
    """marlin_utils_fp4.py:61-120: the (non-negative) block scales, already in
    marlin_permute_scales order, as bytes of the special format the kernel
    reads: (0, 2, 1, 3) inside every four, times the scale factor, times 2^7,
    what is below 2 to zero, then bits 14..7 of the half-precision number.
    Returns (bytes as float8_e4m3fn, scale_factor)."""
    marlin_scales = marlin_scales.to(torch.half)
    marlin_scales = marlin_scales.view(-1, 4)[:, [0, 2, 1, 3]].view(marlin_scales.size(0), -1)
    if scale_factor is None:
        scale_factor = _nvfp4_compute_scale_factor(marlin_scales, a_dtype)
    if scale_factor > 1.0:
        marlin_scales = (marlin_scales.float() * scale_factor).to(torch.half)
    marlin_scales = marlin_scales * (2 ** 7)
    marlin_scales[marlin_scales < 2] = 0
    marlin_scales = marlin_scales.view(torch.int16) << 1
    marlin_scales = marlin_scales.view(torch.float8_e4m3fn)
    return marlin_scales[:, 1::2].contiguous(), scale_factor


def nvfp4_marlin_process_global_scale(global_scale: torch.Tensor, a_dtype: torch.dtype | None = None) -> torch.Tensor:
    """marlin_utils_fp4.py:138-151: times 2^(exponent bias of the code read as a
    16-bit float, minus the 7 the block scales carry)."""
    if a_dtype is None:
        a_dtype = global_scale.dtype
    assert a_dtype in [torch.half, torch.bfloat16]
    target_exponent = 5 if a_dtype == torch.half else 8
    exponent_bias = 2 ** (target_exponent - 1) - 2 ** (2 - 1)
    return global_scale * (2.0 ** (exponent_bias - 7))


def apply_fp4_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                            weight_global_scale: torch.Tensor | None, workspace: torch.Tensor, size_n: int,
                            size_k: int, bias: torch.Tensor | None = None, input_dtype: torch.dtype | None = None,
                            use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT) -> torch.Tensor:
    """marlin_utils_fp4.py:153-214; with a global scale the weights are NVFP4."""
    x = input.reshape(-1, input.shape[-1])
    out_shape = input.shape[:-1] + (size_n,)
    padded_n, padded_k = marlin_repacked_nk(weight, num_bits=4)
    x = marlin_pad_dim(x, size_k, padded_k)
    use_atomic_add = should_use_atomic_add_reduce(m=x.size(0), n=padded_n, k=padded_k, device=input.device,
                                                  dtype=input.dtype)
    a_scales, c = None, None
    if input_dtype is not None and input_dtype.itemsize == 1:   # marlin_utils_fp4.py:185-191
        if weight_global_scale is not None:
            raise RuntimeError("NVFP4 weight + INT8/FP8 activation is not supported.")
        if input_dtype != torch.float8_e4m3fn:
            raise RuntimeError("MXFP4 weight + INT8 activation is not supported.")
        # the op takes the output type from c in this mode (marlin.cu:576-590); the reference passes
        # c = None here, which its op refuses
        c = torch.empty((x.size(0), padded_n), dtype=input.dtype, device=input.device)
        x, a_scales = marlin_quant_input(x, torch.float8_e4m3fn)
    out = ops.marlin_gemm(a=x, c=c, b_q_weight=weight, b_bias=bias, b_scales=weight_scale, a_scales=a_scales,
                          global_scale=weight_global_scale, b_zeros=None, g_idx=None, perm=None,
                          workspace=workspace,
                          b_q_type=scalar_types.float4_e2m1f, size_m=x.size(0), size_n=padded_n, size_k=padded_k,
                          use_atomic_add=use_atomic_add, use_fp32_reduce=use_fp32_reduce)
    return marlin_unpad_output(out, size_n, padded_n).reshape(out_shape)


def _set(layer, name: str, value: torch.Tensor) -> None:
    setattr(layer, name, torch.nn.Parameter(value, requires_grad=False)
            if isinstance(layer, torch.nn.Module) else value)


def prepare_fp4_layer_for_marlin(layer, input_dtype: torch.dtype | None = None) -> None:
    """marlin_utils_fp4.py:217-290.  The layer holds `weight` (N, K/2) uint8,
    `params_dtype`, `output_size_per_partition`, `input_size_per_partition`,
    optionally `bias`, and either `weight_scale` (N, K/32) exponent bytes
    (MXFP4, bfloat16) or `weight_scale` (N, K/16) float8_e4m3fn with
    `weight_global_scale` (NVFP4)."""
    is_nvfp4 = hasattr(layer, "weight_global_scale")
    is_a_8bit = input_dtype is not None and input_dtype.itemsize == 1
    if is_a_8bit:
        if is_nvfp4:
            raise RuntimeError("NVFP4 weight + INT8/FP8 activation is not supported.")
        if input_dtype != torch.float8_e4m3fn:
            raise RuntimeError("MXFP4 weight + INT8 activation is not supported.")
    group_size = 16 if is_nvfp4 else MXFP4_GROUP_SIZE
    part_n, part_k = layer.output_size_per_partition, layer.input_size_per_partition
    padded_n, padded_k = marlin_padded_nk(part_n, part_k, group_size)
    param_dtype = layer.params_dtype
    assert layer.weight.shape == (part_n, part_k // 2)
    device = layer.weight.device
    layer.workspace = marlin_make_workspace_new(device)
    perm = torch.empty(0, dtype=torch.int, device=device)
    qweight = marlin_pad_qweight(layer.weight.view(torch.int32).T.contiguous(), part_n, part_k, padded_n, padded_k)
    _set(layer, "weight", ops.gptq_marlin_repack(qweight, perm, padded_k, padded_n, 4, is_a_8bit))

    scales = layer.weight_scale.T.contiguous()
    if not is_nvfp4:
        scales = scales.view(torch.float8_e8m0fnu)
    scales = scales.to(param_dtype)
    scales = marlin_pad_scales(scales, part_n, part_k, padded_n, padded_k, group_size)
    scales = marlin_permute_scales(scales, padded_k, padded_n, group_size, is_a_8bit=is_a_8bit)
    if is_nvfp4:
        scales, scale_factor = nvfp4_marlin_process_scales(scales, a_dtype=param_dtype)
        _set(layer, "weight_scale", scales)
        global_scale = nvfp4_marlin_process_global_scale(layer.weight_global_scale.to(torch.float32), param_dtype)
        _set(layer, "weight_global_scale", global_scale / scale_factor)
    else:
        _set(layer, "weight_scale", mxfp4_marlin_process_scales(scales, input_dtype=input_dtype))

    if getattr(layer, "bias", None) is not None:
        assert layer.bias.shape == (part_n,)
        _set(layer, "bias", marlin_permute_bias(marlin_pad_dim(layer.bias, part_n, padded_n)))


def prepare_moe_mxfp4_layer_for_marlin(layer, w13: torch.Tensor, w2: torch.Tensor, w13_scale: torch.Tensor,
                                       w2_scale: torch.Tensor, w13_bias: torch.Tensor | None,
                                       w2_bias: torch.Tensor | None):
    """marlin_utils_fp4.py:556-649.  w13 (E, 2N, K/2), w2 (E, K, N/2) uint8; scales
    (E, 2N, K/32), (E, K, N/32) exponent bytes; `layer.params_dtype` is the
    activation type.  Returns (w13, w2, w13_scale, w2_scale, w13_bias, w2_bias)
    for fused_marlin_moe; nothing on the layer changes.  The activation type of the GEMM comes from
    get_marlin_input_dtype(): float8_e4m3fn gives the 8-bit-activation layouts."""
    input_dtype = get_marlin_input_dtype()
    if input_dtype is not None and input_dtype.itemsize == 1 and input_dtype != torch.float8_e4m3fn:
        raise RuntimeError("MXFP4 weight + INT8 activation is not supported.")
    is_a_8bit = input_dtype is not None and input_dtype.itemsize == 1
    e, n, k = w13.shape[0], w13.shape[1] // 2, w13.shape[2] * 2
    perm = torch.empty(0, dtype=torch.int, device=w13.device)

    def repack(weight: torch.Tensor, size_n: int, size_k: int) -> torch.Tensor:
        assert weight.shape == (e, size_n, size_k // 2)
        return torch.stack([ops.gptq_marlin_repack(weight[i].view(torch.int32).T.contiguous(), perm, size_k, size_n, 4,
                                                   is_a_8bit) for i in range(e)])

    def permute(scales: torch.Tensor, size_n: int, size_k: int) -> torch.Tensor:
        scales = scales.view(torch.float8_e8m0fnu).to(layer.params_dtype)
        return torch.stack([mxfp4_marlin_process_scales(
            marlin_permute_scales(scales[i].T, size_k, size_n, MXFP4_GROUP_SIZE, is_a_8bit=is_a_8bit),
            input_dtype=input_dtype) for i in range(e)])

    def permute_bias(bias: torch.Tensor | None) -> torch.Tensor | None:
        if bias is None:
            return None
        bias = bias.to(layer.params_dtype)
        return torch.stack([marlin_permute_bias(bias[i]) for i in range(e)])

    return (repack(w13, 2 * n, k), repack(w2, k, n), permute(w13_scale, 2 * n, k), permute(w2_scale, k, n),
            permute_bias(w13_bias), permute_bias(w2_bias))


def prepare_nvfp4_moe_layer_for_marlin(layer, w13: torch.Tensor, w13_scale: torch.Tensor, w13_scale_2: torch.Tensor,
                                       w2: torch.Tensor, w2_scale: torch.Tensor, w2_scale_2: torch.Tensor,
                                       is_act_and_mul: bool = True):
    """marlin_utils_fp4.py:325-448.  w13 (E, shards * N, K/2), w2 (E, K, N/2) uint8;
    block scales (E, shards * N, K/16), (E, K, N/16) float8_e4m3fn; global scales
    (E,) fp32; `layer` holds num_experts, hidden_size,
    intermediate_size_per_partition and params_dtype.  N is padded to the tile
    size with zero rows / columns.  All experts of a matrix share one scale
    factor.  Returns (w13, w13_scale, w13_scale_2, w2, w2_scale, w2_scale_2)."""
    group_size = 16
    e, k, n = layer.num_experts, layer.hidden_size, layer.intermediate_size_per_partition
    shards = 2 if is_act_and_mul else 1
    if k % 128 == 0:
        padded_n = (n + 63) // 64 * 64
    else:
        assert k % 64 == 0, f"hidden_size = {k} unsupported by Marlin tiles"
        padded_n = (n + 127) // 128 * 128
    param_dtype = layer.params_dtype
    device = w13.device

    def pad_w13(x: torch.Tensor) -> torch.Tensor:
        if padded_n == n:
            return x
        x = torch.nn.functional.pad(x.view(e, shards, n, x.size(-1)), (0, 0, 0, padded_n - n))
        return x.reshape(e, shards * padded_n, -1)

    def pad_w2(x: torch.Tensor, packing: int) -> torch.Tensor:
        return x if padded_n == n else torch.nn.functional.pad(x, (0, (padded_n - n) // packing))

    layer.workspace = marlin_make_workspace_new(device, 4)
    perm = torch.empty(0, dtype=torch.int, device=device)

    def repack(weight: torch.Tensor, is_w13: bool) -> torch.Tensor:
        if is_w13:
            assert weight.shape == (e, n * shards, k // 2)
            weight, size_n, size_k = pad_w13(weight), padded_n * shards, k
        else:
            assert weight.shape == (e, k, n // 2)
            weight, size_n, size_k = pad_w2(weight, 2), k, padded_n
        return torch.stack([ops.gptq_marlin_repack(weight[i].contiguous().view(torch.int32).T.contiguous(), perm,
                                                   size_k, size_n, 4) for i in range(e)])

    def permute_scales(scales: torch.Tensor, g_scales: torch.Tensor, is_w13: bool):
        scales = scales.to(param_dtype)
        if is_w13:
            scales, size_n, size_k = pad_w13(scales), padded_n * shards, k
        else:
            scales, size_n, size_k = pad_w2(scales, group_size), k, padded_n
        factor = _nvfp4_compute_scale_factor(scales, param_dtype)   # one for all experts: they share the processing
        out = [nvfp4_marlin_process_scales(marlin_permute_scales(scales[i].T, size_k, size_n, group_size),
                                           scale_factor=factor, a_dtype=param_dtype)[0] for i in range(e)]
        g_scales = nvfp4_marlin_process_global_scale(g_scales.to(torch.float32), param_dtype) / factor
        return torch.stack(out), g_scales

    mw13, mw2 = repack(w13, True), repack(w2, False)
    s13, g13 = permute_scales(w13_scale, w13_scale_2, True)
    s2, g2 = permute_scales(w2_scale, w2_scale_2, False)
    return mw13, s13, g13, mw2, s2, g2


def rand_marlin_weight_mxfp4_like(weight: torch.Tensor, group_size: int, input_dtype: torch.dtype | None = None):
    """The reference's test helper (marlin_utils_fp4.py:701-753): random codes of
    the shape of `weight` (N, K) and random exponents 110..119; returns
    (dequantised reference (K, N), Marlin weight, Marlin scales)."""
    is_a_8bit = input_dtype is not None and input_dtype.itemsize == 1
    if is_a_8bit:
        assert input_dtype == torch.float8_e4m3fn, "MXFP4 weight + INT8 activation is not supported."
    assert group_size > 0
    size_n, size_k = weight.shape
    device = weight.device
    scales = torch.randint(110, 120, (size_n, size_k // group_size), dtype=torch.uint8, device=device)
    scales = scales.view(torch.float8_e8m0fnu)
    codes = torch.randint(0, 256, (size_n, size_k // 2), dtype=torch.uint8, device=device)

    def values(nibble_high: torch.Tensor) -> torch.Tensor:
        # sign and the three other bits at the top of a byte: as float8_e4m3fn that is value * 2^-6
        as_fp8 = (nibble_high & 0b10000000) | ((nibble_high & 0b01110000) >> 2)
        return as_fp8.view(torch.float8_e4m3fn).to(weight.dtype) * (2 ** 6)

    odd, even = values(codes), values(codes << 4)   # k odd: high nibble; k even: low nibble
    weight_ref = torch.cat([even.unsqueeze(2), odd.unsqueeze(2)], 2).view(size_n, size_k)
    weight_ref = weight_ref * scales.repeat_interleave(group_size, 1).to(weight.dtype)
    perm = torch.empty(0, dtype=torch.int, device=device)
    marlin_qweight = ops.gptq_marlin_repack(codes.view(torch.int32).T.contiguous(), perm, size_k, size_n, 4,
                                            is_a_8bit)
    marlin_scales = marlin_permute_scales(scales.T.to(weight.dtype), size_k, size_n, group_size,
                                          is_a_8bit=is_a_8bit)
    return weight_ref.T, marlin_qweight, mxfp4_marlin_process_scales(marlin_scales, input_dtype=input_dtype)


def rand_marlin_weight_nvfp4_like(weight: torch.Tensor, group_size: int, input_dtype: torch.dtype | None = None):
    """The reference's test helper (marlin_utils_fp4.py:652-698): block scales
    from the magnitudes of `weight` (N, K), global scale max / 448, random codes;
    returns (dequantised reference (K, N), Marlin weight, Marlin scale bytes,
    processed global scale)."""
    assert input_dtype is None or input_dtype.itemsize != 1, "NVFP4 weight + INT8/FP8 activation is not supported."
    assert group_size > 0
    size_n, size_k = weight.shape
    device = weight.device
    scales = weight.view(size_n, -1, group_size).abs().max(-1)[0] / 6
    global_scale = scales.max() / 448
    scales = (scales / global_scale).to(torch.float8_e4m3fn)
    codes = torch.randint(0, 256, (size_n, size_k // 2), dtype=torch.uint8, device=device)

    def values(nibble_high: torch.Tensor) -> torch.Tensor:
        # sign and the three other bits at the top of a byte: as float8_e4m3fn that is value * 2^-6
        as_fp8 = (nibble_high & 0b10000000) | ((nibble_high & 0b01110000) >> 2)
        return as_fp8.view(torch.float8_e4m3fn).to(weight.dtype) * (2 ** 6)

    odd, even = values(codes), values(codes << 4)   # k odd: high nibble; k even: low nibble
    weight_ref = torch.cat([even.unsqueeze(2), odd.unsqueeze(2)], 2).view(size_n, size_k)
    weight_ref = weight_ref * global_scale.to(weight.dtype) * scales.repeat_interleave(group_size, 1).to(weight.dtype)
    perm = torch.empty(0, dtype=torch.int, device=device)
    marlin_qweight = ops.gptq_marlin_repack(codes.view(torch.int32).T.contiguous(), perm, size_k, size_n, 4)
    marlin_scales = marlin_permute_scales(scales.T.to(weight.dtype), size_k, size_n, group_size)
    marlin_scales, scale_factor = nvfp4_marlin_process_scales(marlin_scales)
    global_scale = nvfp4_marlin_process_global_scale(global_scale).to(torch.float32)
    return weight_ref.T, marlin_qweight, marlin_scales, global_scale / scale_factor
