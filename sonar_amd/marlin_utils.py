"""Host-side tensor preparation for the Marlin ops: the counterpart of the
reference's aphrodite/model_executor/layers/quantization/utils/marlin_utils.py
(:30-40 constants, :111-203 and :284-359 support checks, :206-281 padding,
:362-559 workspace / scale / zero-point / bias layouts, :636-700
apply_gptq_marlin_linear) and of pack_cols / unpack_cols
in quant_utils.py:749-803.  Same names, arguments and results; implemented
with torch index ops so tensors stay on their device."""
from __future__ import annotations

import math
import os

import torch

from . import ops
from .scalar_type import ScalarType, scalar_types

GPTQ_MARLIN_TILE = 16
GPTQ_MARLIN_MIN_THREAD_N = 64
GPTQ_MARLIN_MIN_THREAD_K = 128
GPTQ_MARLIN_MAX_PARALLEL = 16
MARLIN_SUPPORTED_GROUP_SIZES = [-1, 32, 64, 128]
USE_FP32_REDUCE_DEFAULT = True

_INTERLEAVE_4BIT = [0, 2, 4, 6, 1, 3, 5, 7]


def round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


def query_marlin_supported_quant_types(has_zp: bool | None = None, include_fp_type: bool = True):
    """uint4 with zero points; uint4b8, uint8b128 and (with include_fp_type)
    float8_e4m3fn and float4_e2m1f without (marlin_utils.py:64-82 of the
    reference; of the float4_e2m1f formats MXFP4 is built, NVFP4 is not)."""
    without = [scalar_types.uint4b8, scalar_types.uint8b128]
    if include_fp_type:
        without += [scalar_types.float8_e4m3fn, scalar_types.float4_e2m1f]
    if has_zp is None:
        return without + [scalar_types.uint4]
    return [scalar_types.uint4] if has_zp else without


def check_marlin_supports_shape(output_size_per_partition: int, input_size_per_partition: int,
                                input_size: int, group_size: int) -> tuple[bool, str | None]:
    if output_size_per_partition % GPTQ_MARLIN_MIN_THREAD_N != 0:
        return False, (f"Weight output_size_per_partition = {output_size_per_partition} is not "
                       f"divisible by  min_thread_n = {GPTQ_MARLIN_MIN_THREAD_N}. ")
    if input_size_per_partition % GPTQ_MARLIN_MIN_THREAD_K != 0:
        return False, (f"Weight input_size_per_partition = {input_size_per_partition} is not "
                       f"divisible by min_thread_k = {GPTQ_MARLIN_MIN_THREAD_K}. ")
    if group_size < input_size and input_size_per_partition % group_size != 0:
        return False, (f"Weight input_size_per_partition = {input_size_per_partition} is not "
                       f"divisible by group_size = {group_size}.")
    return True, None


def _check_marlin_supported(quant_type: ScalarType, group_size: int | None, has_zp: bool):
    supported = query_marlin_supported_quant_types(has_zp, True)
    if quant_type not in supported:
        return False, (f"Marlin does not support weight_bits = {quant_type}. Only types = {supported} "
                       f"are supported (for group_size = {group_size}, zp = {has_zp}).")
    if group_size is None or group_size not in MARLIN_SUPPORTED_GROUP_SIZES:
        return False, (f"Marlin does not support group_size = {group_size}. "
                       f"Only group_sizes = {MARLIN_SUPPORTED_GROUP_SIZES} are supported.")
    return True, None


def check_marlin_supported(quant_type: ScalarType, group_size: int, has_zp: bool = False,
                           device_capability: int | None = None) -> bool:
    """marlin_utils.py:142-149.  `device_capability` is accepted for the
    reference's callers and ignored: there is one target, gfx950."""
    return _check_marlin_supported(quant_type, group_size, has_zp)[0]


def verify_marlin_supported(quant_type: ScalarType, group_size: int, has_zp: bool = False) -> None:
    ok, why = _check_marlin_supported(quant_type, group_size, has_zp)
    if not ok:
        raise ValueError(why)


def verify_marlin_supports_shape(output_size_per_partition: int, input_size_per_partition: int,
                                 input_size: int, group_size: int) -> None:
    """Raises ValueError where check_marlin_supports_shape returns False
    (marlin_utils.py:159-190)."""
    ok, why = check_marlin_supports_shape(output_size_per_partition, input_size_per_partition,
                                          input_size, group_size)
    if not ok:
        raise ValueError(why)


def check_marlin_supports_layer(layer, group_size: int, allow_tile_padding: bool = False) -> bool:
    """marlin_utils.py:284-300: `layer` has output_size / input_size and, when
    sharded, the *_per_partition sizes.  With tile padding only a group that
    straddles the shard boundary stays unsupported."""
    out_part = getattr(layer, "output_size_per_partition", None) or layer.output_size
    in_part = getattr(layer, "input_size_per_partition", None) or layer.input_size
    if allow_tile_padding:
        return group_size == -1 or group_size >= layer.input_size or in_part % group_size == 0
    return check_marlin_supports_shape(out_part, in_part, layer.input_size, group_size)[0]


def marlin_moe_padded_intermediate(intermediate_size: int, group_size: int = -1) -> int:
    """Smallest intermediate size >= the given one that the grouped op takes
    (a multiple of 64 and of the group size; marlin_utils.py:303-321).  The
    padding is zero scales, so padded channels contribute nothing."""
    return round_up(intermediate_size, math.lcm(64, group_size if group_size > 0 else 1))


def check_moe_marlin_supports_layer(layer, group_size: int, allow_tile_padding: bool = False) -> bool:
    """Shape rule of marlin_utils.py:324-350 (hidden % 128, intermediate a
    multiple of max(64, group), no router weight on the input).  The reference
    answers False on ROCm before looking at the shape; with this library loaded
    that early return is the line a maintainer removes."""
    hidden = layer.hidden_size
    inter = layer.moe_config.intermediate_size_per_partition_unpadded
    if allow_tile_padding:
        shape_ok = hidden % 128 == 0 and (group_size <= 0 or inter % group_size == 0)
    else:
        shape_ok = hidden % 128 == 0 and inter % max(64, group_size) == 0
    return shape_ok and group_size in (-1, 32, 64, 128) and not layer.apply_router_weight_on_input


def marlin_moe_intermediate_size(w1_packed: torch.Tensor, w2_packed: torch.Tensor) -> int:
    """Intermediate size from the packed down-projection [E, K / 16, ...]
    (marlin_utils.py:353-359)."""
    return w2_packed.size(1) * GPTQ_MARLIN_TILE


# ---------------------------------------------------------------- packing
def get_pack_factor(num_bits: int) -> int:
    assert 32 % num_bits == 0, f"Unsupported num_bits = {num_bits}"
    return 32 // num_bits


def pack_cols(q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    assert q_w.shape == (size_k, size_n)
    pack_factor = get_pack_factor(num_bits)
    assert size_n % pack_factor == 0
    v = q_w.to(torch.int64).reshape(size_k, size_n // pack_factor, pack_factor)
    shifts = torch.arange(pack_factor, device=q_w.device, dtype=torch.int64) * num_bits
    packed = (v << shifts).sum(dim=-1)
    packed = torch.where(packed >= 2 ** 31, packed - 2 ** 32, packed)
    return packed.to(torch.int32).contiguous()


def unpack_cols(packed_q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    pack_factor = get_pack_factor(num_bits)
    assert size_n % pack_factor == 0
    assert packed_q_w.shape == (size_k, size_n // pack_factor), (
        f"packed_q_w.shape = {tuple(packed_q_w.shape)} size_k = {size_k}, size_n = {size_n} "
        f"pack_Factor = {pack_factor}")
    u = packed_q_w.to(torch.int64) & 0xFFFFFFFF
    shifts = torch.arange(pack_factor, device=packed_q_w.device, dtype=torch.int64) * num_bits
    vals = (u.unsqueeze(-1) >> shifts) & ((1 << num_bits) - 1)
    return vals.reshape(size_k, size_n).to(torch.int32).contiguous()


# ---------------------------------------------------------------- padding helpers
def marlin_padded_nk(size_n: int, size_k: int, group_size: int = -1) -> tuple[int, int]:
    group = group_size if group_size > 0 else 1
    candidates = ((round_up(size_n, 64), round_up(size_k, math.lcm(128, group))),
                  (round_up(size_n, 128), round_up(size_k, math.lcm(64, group))))
    return min(candidates, key=lambda nk: (nk[0] * nk[1], nk[0] + nk[1]))


def marlin_repacked_nk(qweight: torch.Tensor, num_bits: int) -> tuple[int, int]:
    pack_factor = 32 // num_bits
    size_k = qweight.size(0) * GPTQ_MARLIN_TILE
    size_n = qweight.size(1) * pack_factor // GPTQ_MARLIN_TILE
    return size_n, size_k


def marlin_pad_qweight(qweight: torch.Tensor, size_n: int, size_k: int, padded_n: int,
                       padded_k: int) -> torch.Tensor:
    if (padded_n, padded_k) == (size_n, size_k):
        return qweight
    pack_factor = size_k // qweight.size(0)
    return torch.nn.functional.pad(qweight, (0, padded_n - size_n, 0, (padded_k - size_k) // pack_factor))


def marlin_pad_scales(scales: torch.Tensor, size_n: int, size_k: int, padded_n: int, padded_k: int,
                      group_size: int) -> torch.Tensor:
    if (padded_n, padded_k) == (size_n, size_k):
        return scales
    pad_rows = padded_k // group_size - scales.size(0) if group_size > 0 else 0
    assert pad_rows >= 0
    return torch.nn.functional.pad(scales, (0, padded_n - size_n, 0, pad_rows))


def marlin_pad_dim(x: torch.Tensor, size: int, padded: int) -> torch.Tensor:
    if padded == size:
        return x
    return torch.nn.functional.pad(x, (0, padded - size))


def marlin_unpad_output(output: torch.Tensor, size_n: int, padded_n: int) -> torch.Tensor:
    if padded_n == size_n:
        return output
    return output[..., :size_n].contiguous()


# ---------------------------------------------------------------- workspace, g_idx
def num_compute_units(device_index: int | None = None) -> int:
    return torch.cuda.get_device_properties(device_index or 0).multi_processor_count


def marlin_make_workspace_new(device: torch.device, max_blocks_per_sm: int = 1,
                              existing: torch.Tensor | None = None) -> torch.Tensor:
    size = num_compute_units(device.index) * max_blocks_per_sm
    if existing is not None:
        if existing.device != device or existing.dtype != torch.int or existing.numel() != size:
            raise ValueError(
                f"Existing Marlin workspace is incompatible (device={existing.device}, "
                f"dtype={existing.dtype}, numel={existing.numel()}; expected device={device}, "
                f"dtype={torch.int}, numel={size}).")
        return existing.zero_()
    return torch.zeros(size, dtype=torch.int, device=device, requires_grad=False)


def marlin_is_k_full(act_order: bool, is_row_parallel: bool) -> bool:
    return (not act_order) or (act_order and not is_row_parallel)


def marlin_repeat_scales_on_all_ranks(act_order: bool, group_size: int, is_row_parallel: bool) -> bool:
    return act_order or (group_size == -1 and is_row_parallel)


def marlin_make_empty_g_idx(device: torch.device) -> torch.Tensor:
    return torch.nn.Parameter(torch.empty(0, dtype=torch.int, device=device), requires_grad=False)


def marlin_sort_g_idx(g_idx: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    g_idx_sort_indices = torch.argsort(g_idx).to(torch.int)
    return g_idx[g_idx_sort_indices], g_idx_sort_indices


# ---------------------------------------------------------------- scale / zp / bias layouts
def get_scale_perms():
    scale_perm = [i + 8 * j for i in range(8) for j in range(8)]
    scale_perm_single = [2 * i + j for i in range(4) for j in (0, 1, 8, 9, 16, 17, 24, 25)]
    return scale_perm, scale_perm_single


def marlin_permute_scales(s: torch.Tensor, size_k: int, size_n: int, group_size: int,
                          is_a_8bit: bool = False) -> torch.Tensor:
    scale_perm, scale_perm_single = get_scale_perms()
    if group_size < size_k and group_size != -1 and not is_a_8bit:
        s = s.reshape((-1, len(scale_perm)))[:, scale_perm]
    else:
        s = s.reshape((-1, len(scale_perm_single)))[:, scale_perm_single]
    return s.reshape((-1, size_n)).contiguous()


def marlin_permute_bias(s: torch.Tensor) -> torch.Tensor:
    origin_shape = s.shape
    _, scale_perm_single = get_scale_perms()
    s = s.reshape((-1, len(scale_perm_single)))[:, scale_perm_single]
    return s.reshape(*origin_shape).contiguous()


def marlin_act_int8_process_scales(s: torch.Tensor):
    """Group scales for int8 activations (marlin_utils.py:436-440): 16-bit integers
    round(s / max * 4096) stored in a tensor of the scales' dtype, and the factor
    max / 4096 that the caller multiplies into the activation scales."""
    a_scales_scale_factor = 1 / 4096 * s.max().float()
    s = s / s.max() * 4096
    s = s.round().to(torch.int16).view(s.dtype)
    return s, a_scales_scale_factor


def marlin_moe_permute_scales(s: torch.Tensor, size_k: int, size_n: int, group_size: int,
                              is_a_8bit: bool = False) -> torch.Tensor:
    output = torch.empty_like(s)
    for e in range(s.shape[0]):
        output[e] = marlin_permute_scales(s[e], size_k, size_n, group_size, is_a_8bit)
    return output


def marlin_zero_points(zp: torch.Tensor, size_k: int, size_n: int, num_bits: int,
                       is_a_8bit: bool = False) -> torch.Tensor:
    """`size_k` here is the number of groups (rows of zp), as in the reference."""
    assert num_bits == 4
    scale_perm, _ = get_scale_perms()
    zp = zp.reshape((-1, len(scale_perm)))[:, scale_perm]
    if not is_a_8bit:   # the column interleave of the 16-bit dequantiser (marlin_utils.py:472-473)
        zp = zp.reshape((-1, 8))[:, _INTERLEAVE_4BIT]
    zp = zp.reshape((-1, size_n)).contiguous()
    return pack_cols(zp, num_bits, size_k, size_n)


def awq_to_marlin_zero_points(q_zp_packed: torch.Tensor, size_k: int, size_n: int, num_bits: int,
                              is_a_8bit: bool = False) -> torch.Tensor:
    assert num_bits == 4
    q_zp = unpack_cols(q_zp_packed, num_bits, size_k, size_n)
    undo = sorted(range(8), key=lambda i: _INTERLEAVE_4BIT[i])
    q_zp = q_zp.reshape((-1, 8))[:, undo].reshape((-1, size_n)).contiguous()
    return marlin_zero_points(q_zp, size_k, size_n, num_bits, is_a_8bit)


def moe_awq_to_marlin_zero_points(q_zp_packed: torch.Tensor, size_k: int, size_n: int, num_bits: int,
                                  is_a_8bit: bool = False) -> torch.Tensor:
    output = torch.empty_like(q_zp_packed)
    for e in range(q_zp_packed.shape[0]):
        output[e] = awq_to_marlin_zero_points(q_zp_packed[e], size_k, size_n, num_bits, is_a_8bit)
    return output


def moe_packed_to_marlin_zero_points(q_zp_packed: torch.Tensor, size_k: int, size_n: int, num_bits: int,
                                     is_a_8bit: bool = False) -> torch.Tensor:
    """Per-expert zero points packed along columns in plain order (the
    compressed-tensors format, no AWQ interleave) to the op's layout
    (marlin_utils.py:538-559)."""
    out = torch.empty_like(q_zp_packed)
    for e in range(q_zp_packed.shape[0]):
        out[e] = marlin_zero_points(unpack_cols(q_zp_packed[e], num_bits, size_k, size_n), size_k, size_n,
                                    num_bits, is_a_8bit)
    return out


def should_use_atomic_add_reduce(m: int, n: int, k: int, device: torch.device, dtype: torch.dtype) -> bool:
    """The reference turns atomic-add reduction on only behind an environment
    flag for n < 2048, k >= 2048; the gfx950 kernels always reduce in a fixed
    order, so the answer here is always False."""
    return False


# ---------------------------------------------------------------- 8-bit activations
def per_token_quant_int8(x: torch.Tensor):
    """int8_utils.py:95-120: (int8 of x's shape, float32 scales (..., 1))."""
    return ops.per_token_quant_int8(x)


def per_token_quant_fp8(x: torch.Tensor):
    """What get__quant_fp8_method()(x) returns in the reference (marlin_utils.py:596-603)."""
    return ops.per_token_quant_fp8(x)


def get_marlin_input_dtype(prefix: str | None = None):
    """The activation type the environment asks for (marlin_utils.py:606-623):
    APHRODITE_MARLIN_INPUT_DTYPE = int8 | fp8, else None (16-bit).  The reference lets
    fp8 through only where the tensor cores have it (SM 8.9 / 12.x); gfx950 has fp8 matrix
    cores, so it is allowed here."""
    want = os.environ.get("APHRODITE_MARLIN_INPUT_DTYPE")
    if want is None:
        return None
    if want.lower() == "int8":
        return torch.int8
    if want.lower() == "fp8":
        return torch.float8_e4m3fn
    return None


def marlin_quant_input(x: torch.Tensor, quant_dtype: torch.dtype):
    """marlin_utils.py:626-633."""
    x = x.reshape(-1, x.shape[-1])
    if quant_dtype == torch.int8:
        return per_token_quant_int8(x)
    if quant_dtype == torch.float8_e4m3fn:
        return per_token_quant_fp8(x)
    raise ValueError(f"unsupported quant_dtype {quant_dtype}")


# ---------------------------------------------------------------- the linear call
def apply_gptq_marlin_linear(input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
                             weight_zp: torch.Tensor, g_idx: torch.Tensor,
                             g_idx_sort_indices: torch.Tensor, workspace: torch.Tensor,
                             wtype: ScalarType, output_size_per_partition: int,
                             input_size_per_partition: int, is_k_full: bool,
                             input_global_scale: torch.Tensor | None = None,
                             bias: torch.Tensor | None = None,
                             use_fp32_reduce: bool = USE_FP32_REDUCE_DEFAULT,
                             input_dtype: torch.dtype | None = None) -> torch.Tensor:
    reshaped_x = input.reshape(-1, input.shape[-1])
    out_shape = input.shape[:-1] + (output_size_per_partition,)
    padded_n, padded_k = marlin_repacked_nk(weight, wtype.size_bits)
    reshaped_x = marlin_pad_dim(reshaped_x, input_size_per_partition, padded_k)
    use_atomic_add = should_use_atomic_add_reduce(reshaped_x.size(0), padded_n, padded_k, input.device,
                                                  input.dtype)
    a_scales = None
    if input_dtype == torch.int8:      # marlin_utils.py:671-680
        assert wtype == scalar_types.uint4b8, "W8A8-INT8 is not supported by marlin kernel."
        reshaped_x, a_scales = marlin_quant_input(reshaped_x, input_dtype)
        if input_global_scale is not None:
            a_scales = a_scales * input_global_scale
    elif input_dtype == torch.float8_e4m3fn:
        assert wtype == scalar_types.uint4b8, "INT8 weight + FP8 activation is not supported."
        reshaped_x, a_scales = marlin_quant_input(reshaped_x, input_dtype)
    output = ops.marlin_gemm(reshaped_x, None, weight, bias, weight_scale, a_scales, None, weight_zp, g_idx,
                             g_idx_sort_indices, workspace, wtype, size_m=reshaped_x.shape[0],
                             size_n=padded_n, size_k=padded_k, is_k_full=is_k_full,
                             use_atomic_add=use_atomic_add, use_fp32_reduce=use_fp32_reduce,
                             is_zp_float=False)
    output = marlin_unpad_output(output, output_size_per_partition, padded_n)
    return output.reshape(out_shape)
