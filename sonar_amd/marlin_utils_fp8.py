"""Weight-only FP8 (float8_e4m3fn weights, fp16 / bf16 activations) through the
Marlin ops.  Mirrors aphrodite/model_executor/layers/quantization/utils/
marlin_utils_fp8.py:31-631 of the reference: the bytes of the fp8
weights travel as 8-bit codes (packed four to an int32 along K, then
gptq_marlin_repack with num_bits = 8); the scales are permuted as for any Marlin
layer and multiplied by 2^8 (fp16) or 2^120 (bf16), the difference between the
exponent biases, because the kernels read a code as the 16-bit number with the
same exponent field.  MXFP8 (exponent-byte scales per 32 rows) is at the end.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import ops
from .marlin_utils import (USE_FP32_REDUCE_DEFAULT, marlin_make_workspace_new, marlin_moe_padded_intermediate,
                           marlin_pad_dim, marlin_pad_qweight, marlin_pad_scales, marlin_padded_nk,
                           marlin_permute_bias, marlin_permute_scales, marlin_repacked_nk, marlin_unpad_output,
                           should_use_atomic_add_reduce)
from .scalar_type import scalar_types


def is_fp8_marlin_supported() -> bool:
    """marlin_utils_fp8.py:31-32; one target here, which runs it."""
    return True


def fp8_fused_exponent_bias_into_scales(scales: torch.Tensor) -> torch.Tensor:
    """scales * 2^(2^(e-1) - 2^3) with e the exponent bits of the scales' type
    (marlin_utils_fp8.py:35-46): 2^8 for fp16, 2^120 for bf16."""
    if scales.dtype == torch.half:
        target_exponent = 5
    elif scales.dtype == torch.bfloat16:
        target_exponent = 8
    else:
        raise TypeError(f"scales must be float16 or bfloat16, not {scales.dtype}")
    exponent_bias = 2 ** (target_exponent - 1) - 2 ** 3
    return scales * torch.full_like(scales, 2.0) ** exponent_bias


def pack_fp8_to_int32(fp8_tensor: torch.Tensor, size_k_first: bool = True) -> torch.Tensor:
    """(K, N) (size_k_first) or (N, K) fp8 -> four consecutive K to an int32:
    (K/4, N) resp. (N, K/4)  (marlin_utils_fp8.py:366-378)."""
    assert fp8_tensor.dtype == torch.float8_e4m3fn and fp8_tensor.ndim == 2
    by_n = (fp8_tensor.T if size_k_first else fp8_tensor).contiguous()
    words = by_n.view(torch.int32)
    return words.T.contiguous() if size_k_first else words


def apply_fp8_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                            workspace: torch.Tensor, size_n: int, size_k: int, bias: torch.Tensor | None,
                            input_dtype: torch.dtype | None = None,
                            use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT) -> torch.Tensor:
    """marlin_utils_fp8.py:49-104."""
    if input_dtype is not None and input_dtype.itemsize == 1:
        raise RuntimeError("Marlin W8A8 is not supported.")
    x = input.reshape(-1, input.shape[-1])
    out_shape = input.shape[:-1] + (size_n,)
    padded_n, padded_k = marlin_repacked_nk(weight, num_bits=8)
    x = marlin_pad_dim(x, size_k, padded_k)
    use_atomic_add = should_use_atomic_add_reduce(m=x.size(0), n=padded_n, k=padded_k, device=input.device,
                                                  dtype=input.dtype)
    out = ops.marlin_gemm(a=x, c=None, b_q_weight=weight, b_bias=bias, b_scales=weight_scale, a_scales=None,
                          global_scale=None, b_zeros=None, g_idx=None, perm=None, workspace=workspace,
                          b_q_type=scalar_types.float8_e4m3fn, size_m=x.size(0), size_n=padded_n, size_k=padded_k,
                          use_atomic_add=use_atomic_add, use_fp32_reduce=use_fp32_reduce)
    return marlin_unpad_output(out, size_n, padded_n).reshape(out_shape)


def _set(layer, name: str, value: torch.Tensor) -> None:
    setattr(layer, name, torch.nn.Parameter(value, requires_grad=False)
            if isinstance(layer, torch.nn.Module) else value)


def _channel_scales(scales: torch.Tensor, size_n: int, logical_widths) -> torch.Tensor:
    """Per-tensor, per-shard or per-channel scales -> (1, size_n)
    (marlin_utils_fp8.py:164-190)."""
    count = scales.nelement()
    if count == 1:
        return scales.view(1, 1).repeat_interleave(size_n, 1)
    if count == len(logical_widths):
        assert sum(logical_widths) == size_n, (
            f"Sum of logical_widths ({sum(logical_widths)}) must be equal to part_size_n ({size_n})")
        widths = scales.new_tensor(logical_widths, dtype=torch.int64)
        return scales.view(1, -1).repeat_interleave(widths, dim=1)
    if count != size_n:
        assert size_n % count == 0
        return scales.view(1, count).repeat_interleave(size_n // count, 1)
    return scales.view(1, size_n)


def prepare_fp8_layer_for_marlin(layer, size_k_first: bool = True,
                                 input_dtype: torch.dtype | None = None) -> None:
    """marlin_utils_fp8.py:107-212.  The layer holds `weight` (fp8, (K, N) when
    size_k_first else (N, K)), `weight_scale` or `weight_scale_inv`, `orig_dtype`,
    `output_size_per_partition`, `input_size_per_partition`, optionally
    `weight_block_size` = [block_n, block_k], `logical_widths`, `bias`."""
    if input_dtype is not None and input_dtype.itemsize == 1:
        raise RuntimeError("Marlin W8A8 is not supported.")
    part_n, part_k = layer.output_size_per_partition, layer.input_size_per_partition
    block = getattr(layer, "weight_block_size", None)
    group_size = -1 if block is None else block[1]
    padded_n, padded_k = marlin_padded_nk(part_n, part_k, group_size)
    assert layer.weight.shape == ((part_k, part_n) if size_k_first else (part_n, part_k))
    device = layer.weight.device
    layer.workspace = marlin_make_workspace_new(device)

    qweight = pack_fp8_to_int32(layer.weight, size_k_first)
    if not size_k_first:
        qweight = qweight.T.contiguous()
    qweight = marlin_pad_qweight(qweight, part_n, part_k, padded_n, padded_k)
    perm = torch.empty(0, dtype=torch.int, device=device)
    _set(layer, "weight", ops.gptq_marlin_repack(qweight, perm, padded_k, padded_n, 8))

    scale_name = "weight_scale" if hasattr(layer, "weight_scale") else "weight_scale_inv"
    scales = getattr(layer, scale_name).to(layer.orig_dtype)
    if block is None:
        scales = _channel_scales(scales, part_n, getattr(layer, "logical_widths", []))
    else:   # one scale per block_n x block_k block -> one per column and group of block_k rows
        if not size_k_first:
            scales = scales.T.contiguous()
        scales = scales.repeat_interleave(block[0], 1)[:, :part_n]
    scales = marlin_pad_scales(scales, part_n, part_k, padded_n, padded_k, group_size)
    scales = marlin_permute_scales(scales, padded_k, padded_n, group_size)
    _set(layer, scale_name, fp8_fused_exponent_bias_into_scales(scales))

    if getattr(layer, "bias", None) is not None:
        assert layer.bias.shape == (part_n,)
        _set(layer, "bias", marlin_permute_bias(marlin_pad_dim(layer.bias, part_n, padded_n)))


def prepare_fp8_moe_layer_for_marlin(layer, w13_weight: torch.Tensor, w2_weight: torch.Tensor,
                                     w13_weight_scale: torch.Tensor, w2_weight_scale: torch.Tensor):
    """marlin_utils_fp8.py:234-363.  w13_weight (E, 2N, K), w2_weight (E, K, N) in
    fp8; scales per tensor (E), per shard, per channel, or per block when the
    layer has `weight_block_size` ((E, rows / block_n, cols / block_k)).  Returns
    the Marlin weights and scales of fused_marlin_moe; adds `workspace` to the
    layer."""
    e, k, n = layer.num_experts, layer.hidden_size, layer.intermediate_size_per_partition
    w13_n = w13_weight.size(1)
    block = getattr(layer, "weight_block_size", None)
    group_size = -1 if block is None else block[1]
    padded_n = marlin_moe_padded_intermediate(n, group_size)
    if padded_n != n:   # the code 0 is 0.0: padded weights add nothing
        rest = w13_weight.shape[2:]
        w13_weight = F.pad(w13_weight.view(torch.uint8).view(e, 2, n, *rest), (0, 0, 0, padded_n - n)) \
            .reshape(e, 2 * padded_n, *rest).view(torch.float8_e4m3fn)
        w2_weight = F.pad(w2_weight.view(torch.uint8), (0, padded_n - n)).view(torch.float8_e4m3fn)
    device = w13_weight.device
    layer.workspace = marlin_make_workspace_new(device, 4)
    perm = torch.empty(0, dtype=torch.int, device=device)

    def repack(weight: torch.Tensor) -> torch.Tensor:
        size_n, size_k = weight.size(1), weight.size(2)
        return torch.stack([ops.gptq_marlin_repack(pack_fp8_to_int32(weight[i], size_k_first=False).T.contiguous(),
                                                   perm, size_k, size_n, 8) for i in range(e)])

    def permute(scales: torch.Tensor, is_w13: bool) -> torch.Tensor:
        scales = scales.to(layer.orig_dtype)
        size_n, size_k = (w13_n, k) if is_w13 else (k, n)
        if block is None:
            count = scales.nelement()
            if count == e:
                scales = scales.view(e, 1, 1).repeat_interleave(size_n, 2)
            elif count != e * size_n:
                assert (e * size_n) % count == 0
                per = count // e
                scales = scales.view(e, 1, per).repeat_interleave(size_n // per, 2)
            else:
                scales = scales.view(e, 1, size_n)
        else:
            scales = scales.permute(0, 2, 1).repeat_interleave(block[0], 2)[..., :size_n].contiguous()
        if padded_n != n:
            if is_w13:
                g = scales.size(1)
                scales = F.pad(scales.view(e, g, 2, n), (0, padded_n - n)).reshape(e, g, 2 * padded_n)
                size_n = 2 * padded_n
            else:
                if group_size > 0:
                    scales = F.pad(scales, (0, 0, 0, (padded_n - n) // group_size))
                size_k = padded_n
        out = torch.stack([marlin_permute_scales(scales[i], size_k, size_n, group_size) for i in range(e)])
        return fp8_fused_exponent_bias_into_scales(out)

    return repack(w13_weight), repack(w2_weight), permute(w13_weight_scale, True), permute(w2_weight_scale, False)


def marlin_quant_fp8_torch(weight: torch.Tensor, group_size: int, input_dtype: torch.dtype | None = None):
    """The reference's test helper (marlin_utils_fp8.py:591-631): quantise an
    (N, K) weight to fp8 with one scale per row of N and group of K (amax / 448),
    and return (dequantised reference (K, N), Marlin weight, Marlin scales)."""
    assert input_dtype is None or input_dtype.itemsize != 1, "8-bit activations are not built"
    size_n, size_k = weight.shape
    span = size_k if group_size == -1 else group_size
    scales = weight.view(size_n, -1, span).abs().max(-1)[0] / 448
    repeated = scales.repeat_interleave(span, 1)
    fp8_weight = (weight / repeated).to(torch.float8_e4m3fn)
    weight_ref = fp8_weight.to(weight.dtype) * repeated
    packed = pack_fp8_to_int32(fp8_weight, False).T.contiguous()
    perm = torch.empty(0, dtype=torch.int, device=weight.device)
    marlin_qweight = ops.gptq_marlin_repack(packed, perm, size_k, size_n, 8)
    marlin_scales = marlin_permute_scales(scales.T, size_k, size_n, group_size)
    return weight_ref.T, marlin_qweight, fp8_fused_exponent_bias_into_scales(marlin_scales)


# ---------------------------------------------------------------- MXFP8
# float8_e4m3fn weights with one power-of-two scale (an exponent byte) per 32
# rows, bfloat16 activations (marlin_utils_fp8.py:381-588 of the reference).
MXFP8_GROUP_SIZE = 32


def mxfp8_marlin_process_scales(marlin_scales: torch.Tensor) -> torch.Tensor:
    """marlin_utils_fp8.py:381-386: every four neighbours of the permuted scale
    rows in the order 0, 2, 1, 3, then the exponent bytes."""
    reordered = marlin_scales.view(-1, 4)[:, [0, 2, 1, 3]].view(marlin_scales.size(0), -1)
    return reordered.to(torch.float8_e8m0fnu)


def apply_mxfp8_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                              workspace: torch.Tensor, size_n: int, size_k: int, bias: torch.Tensor | None = None,
                              use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT) -> torch.Tensor:
    """marlin_utils_fp8.py:389-434: the fp8 call with float8_e8m0fnu scales."""
    return apply_fp8_marlin_linear(input, weight, weight_scale, workspace, size_n, size_k, bias,
                                   use_fp32_reduce=use_fp32_reduce)


def _mx_scales_for_marlin(exponent_bytes: torch.Tensor, size_n: int, size_k: int, padded_n: int, padded_k: int,
                          dtype: torch.dtype) -> torch.Tensor:
    """(N, K/32) exponent bytes -> permuted, reordered float8_e8m0fnu (K/32, N)."""
    scales = exponent_bytes[:size_n, :size_k // MXFP8_GROUP_SIZE].contiguous()
    scales = scales.view(torch.float8_e8m0fnu).to(dtype).T.contiguous()
    scales = marlin_pad_scales(scales, size_n, size_k, padded_n, padded_k, MXFP8_GROUP_SIZE)
    return mxfp8_marlin_process_scales(marlin_permute_scales(scales, padded_k, padded_n, MXFP8_GROUP_SIZE))


def prepare_mxfp8_layer_for_marlin(layer) -> None:
    """marlin_utils_fp8.py:437-496.  The layer holds `weight` (N, K) fp8,
    `weight_scale` (N, K/32) exponent bytes, `output_size_per_partition`,
    `input_size_per_partition`, optionally `bias`."""
    part_n, part_k = layer.output_size_per_partition, layer.input_size_per_partition
    padded_n, padded_k = marlin_padded_nk(part_n, part_k, MXFP8_GROUP_SIZE)
    device = layer.weight.device
    layer.workspace = marlin_make_workspace_new(device)
    perm = torch.empty(0, dtype=torch.int, device=device)
    qweight = pack_fp8_to_int32(layer.weight, size_k_first=False).T.contiguous()
    qweight = marlin_pad_qweight(qweight, part_n, part_k, padded_n, padded_k)
    _set(layer, "weight", ops.gptq_marlin_repack(qweight, perm, padded_k, padded_n, 8))
    _set(layer, "weight_scale", _mx_scales_for_marlin(layer.weight_scale.data, part_n, part_k, padded_n, padded_k,
                                                      torch.bfloat16))
    if getattr(layer, "bias", None) is not None:
        assert layer.bias.shape == (part_n,)
        _set(layer, "bias", marlin_permute_bias(marlin_pad_dim(layer.bias, part_n, padded_n)))


def prepare_mxfp8_moe_layer_for_marlin(layer, w13: torch.Tensor, w2: torch.Tensor, w13_scale: torch.Tensor,
                                       w2_scale: torch.Tensor):
    """marlin_utils_fp8.py:499-588.  w13 (E, 2N, K), w2 (E, K, N) fp8; scales
    (E, 2N, K/32), (E, K, N/32) exponent bytes.  Returns the Marlin weights and
    scales of fused_marlin_moe; adds `workspace` to the layer."""
    g = MXFP8_GROUP_SIZE
    e, k, n = w13.shape[0], w13.shape[2], w2.shape[2]
    padded_n = marlin_moe_padded_intermediate(n, g)
    if padded_n != n:   # the code 0 is 0.0: padded weights add nothing, whatever their scales
        pad = padded_n - n
        w13 = F.pad(w13.view(torch.uint8).view(e, 2, n, k), (0, 0, 0, pad)).reshape(e, 2 * padded_n, k) \
            .view(torch.float8_e4m3fn)
        w13_scale = F.pad(w13_scale.view(e, 2, n, -1), (0, 0, 0, pad)).reshape(e, 2 * padded_n, -1)
        w2 = F.pad(w2.view(torch.uint8), (0, pad)).view(torch.float8_e4m3fn)
        w2_scale = F.pad(w2_scale, (0, pad // g))
        n = padded_n
    w13_n = w13.shape[1]
    device = w13.device
    layer.workspace = marlin_make_workspace_new(device, 4)
    perm = torch.empty(0, dtype=torch.int, device=device)

    def repack(weight: torch.Tensor, size_n: int, size_k: int) -> torch.Tensor:
        assert weight.shape == (e, size_n, size_k)
        return torch.stack([ops.gptq_marlin_repack(pack_fp8_to_int32(weight[i], size_k_first=False).T.contiguous(),
                                                   perm, size_k, size_n, 8) for i in range(e)])

    def permute(scales: torch.Tensor, size_n: int, size_k: int) -> torch.Tensor:
        return torch.stack([_mx_scales_for_marlin(scales[i], size_n, size_k, size_n, size_k, torch.bfloat16)
                            for i in range(e)])

    return repack(w13, w13_n, k), repack(w2, k, n), permute(w13_scale, w13_n, k), permute(w2_scale, k, n)
