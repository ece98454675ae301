"""Dense caller of the Marlin ops: repack at load, GEMM at apply.  Follows the
reference's MarlinLinearKernel
(aphrodite/model_executor/kernels/linear/mixed_precision/marlin.py:35-235) and
its config (MPLinearKernel.py:26-90), with plain tensors in a namespace-like
`layer` instead of the reference's parameter classes.

Checkpoint layouts taken (as the reference's GPTQ path provides them,
layers/quantization/auto_gptq.py:304-430): qweight (K/8, N) int32 packed along
K, scales (K/G, N), qzeros (N/8-packed per group, given here already unpacked
to (K/G, N) codes, packed (K/G, N/8) along N, or that transposed), g_idx (K)
int32.  AutoAWQ checkpoints go through convert_awq_to_standard_format first."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import ops
from .marlin_utils import (MARLIN_SUPPORTED_GROUP_SIZES, apply_gptq_marlin_linear,
                           check_marlin_supports_shape, marlin_act_int8_process_scales, marlin_is_k_full, marlin_make_empty_g_idx,
                           marlin_make_workspace_new, marlin_pad_dim, marlin_pad_qweight,
                           marlin_pad_scales, marlin_padded_nk, marlin_permute_bias,
                           marlin_permute_scales, marlin_sort_g_idx, marlin_zero_points,
                           query_marlin_supported_quant_types, unpack_cols)
from .scalar_type import ScalarType, scalar_types


_AWQ_SLOT_OF_COLUMN = (0, 4, 1, 5, 2, 6, 3, 7)   # nibble slot of column j of an AWQ-packed int32


def convert_awq_to_standard_format(layer, w_q_name: str = "qweight", w_zp_name: str = "qzeros",
                                   size_bits: int = 4) -> None:
    """AutoAWQ checkpoint tensors -> the GPTQ-like ones MarlinLinearKernel takes
    (the reference's `_convert_awq_to_standard_format`,
    layers/quantization/auto_awq.py:93-153): qweight (K, N/8), packed along N
    with AWQ's interleaved nibble order, becomes (K/8, N) packed along K in
    plain order; qzeros (G, N/8) in the same AWQ packing becomes (N/8, G),
    packed along N in plain order and transposed."""
    if size_bits != 4:
        raise NotImplementedError("AWQ conversion: 4-bit only")
    qw = getattr(layer, w_q_name)
    shifts = 4 * torch.tensor(_AWQ_SLOT_OF_COLUMN, dtype=torch.int32, device=qw.device)
    plain = 4 * torch.arange(8, dtype=torch.int32, device=qw.device)

    def codes(packed: torch.Tensor) -> torch.Tensor:       # (R, N/8) -> (R, N), column order restored
        return ((packed.unsqueeze(-1) >> shifts) & 0xF).reshape(packed.shape[0], -1)

    def pack_dim0(q: torch.Tensor) -> torch.Tensor:        # (8 R, C) -> (R, C): row 8 r + t in nibble t
        q = q.reshape(q.shape[0] // 8, 8, q.shape[1]).to(torch.int32)
        return (q << plain[None, :, None]).sum(dim=1, dtype=torch.int32).contiguous()

    setattr(layer, w_q_name, pack_dim0(codes(qw)))
    setattr(layer, w_zp_name, pack_dim0(codes(getattr(layer, w_zp_name)).t().contiguous()))


@dataclass
class MPLinearLayerConfig:
    full_weight_shape: tuple[int, int]       # (in_features, out_features)
    partition_weight_shape: tuple[int, int]
    weight_type: ScalarType
    act_type: torch.dtype
    group_size: int
    zero_points: bool
    has_g_idx: bool


def _input_major(x: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
    """A weight or scale tensor with the input (K) dimension first.  The
    reference's parameters carry `input_dim` / `output_dim` and are permuted by
    `permute_param_layout_` (marlin.py:120-135): compressed-tensors checkpoints
    hold `weight_packed` as (N, K / pack) and `weight_scale` as (N, groups).
    Here the attributes are honoured when present, else the layout is read off
    the shape, (rows, cols) winning when both fit."""
    input_dim = getattr(x, "input_dim", None)
    output_dim = getattr(x, "output_dim", None)
    if input_dim == 1 or (input_dim is None and output_dim == 0 and x.shape != (rows, cols)):
        x = x.t()
    elif input_dim is None and output_dim is None and x.shape != (rows, cols) and x.shape == (cols, rows):
        x = x.t()
    assert x.shape == (rows, cols), f"expected {(rows, cols)} or its transpose, got {tuple(x.shape)}"
    return x


class MarlinLinearKernel:
    def __init__(self, c: MPLinearLayerConfig, w_q_param_name: str = "qweight",
                 w_s_param_name: str = "scales", w_zp_param_name: str | None = "qzeros",
                 w_gidx_param_name: str | None = "g_idx"):
        ok, why = self.can_implement(c)
        if not ok:
            raise ValueError(why)
        self.config = c
        self.w_q_name = w_q_param_name
        self.w_s_name = w_s_param_name
        self.w_zp_name = w_zp_param_name or "w_zp"
        self.w_gidx_name = w_gidx_param_name or "g_idx"

    @classmethod
    def can_implement(cls, c: MPLinearLayerConfig) -> tuple[bool, str | None]:
        if c.act_type not in (torch.float16, torch.bfloat16, torch.int8, torch.float8_e4m3fn):
            return False, f"activation type {c.act_type} not supported: fp16, bf16, int8 or float8_e4m3fn"
        if c.act_type.itemsize == 1 and c.has_g_idx:
            return False, "act-order is not supported with 8-bit activations"
        quant_types = query_marlin_supported_quant_types(c.zero_points)
        if c.weight_type not in quant_types:
            return False, (f"Quant type ({c.weight_type}) not supported by  Marlin, supported types "
                           f"are: {quant_types}")
        if c.group_size not in MARLIN_SUPPORTED_GROUP_SIZES:
            return False, (f"Group size ({c.group_size}) not supported by Marlin, supported group "
                           f"sizes are: {MARLIN_SUPPORTED_GROUP_SIZES}")
        if c.has_g_idx:
            return check_marlin_supports_shape(c.partition_weight_shape[1], c.partition_weight_shape[0],
                                               c.full_weight_shape[0], c.group_size)
        if (c.group_size != -1 and c.group_size < c.full_weight_shape[0]
                and c.partition_weight_shape[0] % c.group_size != 0):
            return False, (f"in_features per partition {c.partition_weight_shape[0]} is not divisible "
                           f"by group_size = {c.group_size}.")
        return True, None

    def process_weights_after_loading(self, layer) -> None:
        c = self.config
        device = getattr(layer, self.w_q_name).device
        is_a_8bit = c.act_type is not None and c.act_type.itemsize == 1
        if is_a_8bit:   # marlin.py:92-93
            assert c.weight_type == scalar_types.uint4b8, "W8A8 is not supported by marlin kernel."
        row_parallel = c.partition_weight_shape[0] != c.full_weight_shape[0]
        self.is_k_full = marlin_is_k_full(c.has_g_idx, row_parallel)
        size_k, size_n = c.partition_weight_shape
        if c.has_g_idx:
            padded_n, padded_k = size_n, size_k
        else:
            padded_n, padded_k = marlin_padded_nk(size_n, size_k, c.group_size)
        self.workspace = marlin_make_workspace_new(device, existing=getattr(self, "workspace", None))

        if c.has_g_idx:
            g_idx, g_idx_sort_indices = marlin_sort_g_idx(getattr(layer, self.w_gidx_name))
            setattr(layer, self.w_gidx_name, g_idx)
            # A reload keeps the tensor the GEMM (and any recorded graph) reads: new
            # values are copied into it (marlin.py:160-163, replace_parameter with
            # prefer_copy; tests/model_executor/model_loader/test_reload.py:235-258).
            held = getattr(layer, "g_idx_sort_indices", None)
            if (isinstance(held, torch.Tensor) and held.shape == g_idx_sort_indices.shape
                    and held.dtype == g_idx_sort_indices.dtype and held.device == g_idx_sort_indices.device):
                held.data.copy_(g_idx_sort_indices)
            else:
                layer.g_idx_sort_indices = torch.nn.Parameter(g_idx_sort_indices, requires_grad=False)
        else:
            setattr(layer, self.w_gidx_name, marlin_make_empty_g_idx(device))
            layer.g_idx_sort_indices = marlin_make_empty_g_idx(device)

        if c.zero_points:
            grouped_k = size_k // c.group_size if c.group_size != -1 else 1
            padded_grouped_k = padded_k // c.group_size if c.group_size != -1 else 1
            zp = getattr(layer, self.w_zp_name)
            if zp.shape == (size_n // 8, grouped_k) and grouped_k != size_n // 8:
                zp = zp.t().contiguous()      # packed along N and transposed (the converted AWQ form)
            if zp.shape == (grouped_k, size_n // 8):
                zp = unpack_cols(zp, c.weight_type.size_bits, grouped_k, size_n)
            zp = marlin_pad_scales(zp, size_n, size_k, padded_n, padded_k, c.group_size)
            setattr(layer, self.w_zp_name,
                    marlin_zero_points(zp, padded_grouped_k, padded_n, c.weight_type.size_bits,
                                       is_a_8bit=is_a_8bit))
        else:
            setattr(layer, self.w_zp_name, marlin_make_empty_g_idx(device))

        pack = 32 // c.weight_type.size_bits
        w_q = _input_major(getattr(layer, self.w_q_name), size_k // pack, size_n)
        setattr(layer, self.w_q_name, ops.gptq_marlin_repack(
            marlin_pad_qweight(w_q.contiguous(), size_n, size_k, padded_n, padded_k),
            perm=layer.g_idx_sort_indices, size_k=padded_k, size_n=padded_n,
            num_bits=c.weight_type.size_bits, is_a_8bit=is_a_8bit))
        if c.act_type == torch.float8_e4m3fn:   # marlin.py:95-97: sign-and-magnitude codes, scales times 512
            ops.marlin_int4_fp8_preprocess(getattr(layer, self.w_q_name), inplace=True)
        w_s = getattr(layer, self.w_s_name)
        w_s = _input_major(w_s, w_s.numel() // size_n, size_n)
        if c.act_type == torch.float8_e4m3fn:
            w_s = w_s * 512
        w_s = marlin_permute_scales(
            marlin_pad_scales(w_s.contiguous(), size_n, size_k, padded_n, padded_k, c.group_size),
            size_k=padded_k, size_n=padded_n, group_size=c.group_size, is_a_8bit=is_a_8bit)
        num_groups = 1 if c.group_size == -1 else size_k // c.group_size
        layer.input_global_scale = None
        if c.act_type == torch.int8 and num_groups > 1:   # marlin.py:156-163
            w_s, input_global_scale = marlin_act_int8_process_scales(w_s)
            layer.input_global_scale = torch.nn.Parameter(input_global_scale, requires_grad=False)
        setattr(layer, self.w_s_name, w_s)
        if getattr(layer, "bias", None) is not None:
            layer.bias = marlin_permute_bias(marlin_pad_dim(layer.bias, size_n, padded_n))

    def apply_weights(self, layer, x: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
        c = self.config
        return apply_gptq_marlin_linear(
            input=x, weight=getattr(layer, self.w_q_name), weight_scale=getattr(layer, self.w_s_name),
            weight_zp=getattr(layer, self.w_zp_name), g_idx=getattr(layer, self.w_gidx_name),
            g_idx_sort_indices=layer.g_idx_sort_indices, workspace=self.workspace, wtype=c.weight_type,
            input_size_per_partition=c.partition_weight_shape[0],
            output_size_per_partition=c.partition_weight_shape[1], is_k_full=self.is_k_full,
            input_global_scale=getattr(layer, "input_global_scale", None), bias=bias, input_dtype=c.act_type)
