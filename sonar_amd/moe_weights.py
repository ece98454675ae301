"""Checkpoint tensors of a quantised mixture-of-experts layer -> the inputs of
`fused_marlin_moe`.

Mirrors `_process_weights_marlin` (GPTQ-style experts, packed along K) and
`_process_awq_weights_marlin` (AWQ-style experts, packed along N with the AWQ
nibble order) of aphrodite/model_executor/layers/fused_moe/oracle/
int_wna16.py:464-700 and :787-940, for fp16 / bf16 activations (GPTQ-style: 4-
and 8-bit codes with a fixed offset, 4-bit codes with zero points; AWQ-style:
4-bit): pad the intermediate size to what the grouped op takes, sort the
act-order group indices per expert, repack every expert, permute scales, zero
points and biases.  Stacked tensors, expert first:

  GPTQ:  w13_qweight (E, K/8, 2N)   w2_qweight (E, N/8, K)   int32 (K/4, N/4 for 8 bits)
         w13_scales  (E, K/G, 2N)   w2_scales  (E, N/G, K)
         w13_qzeros  (E, K/G, 2N/8) w2_qzeros  (E, N/G, K/8) plain column packing
         w13_g_idx   (E, K)         w2_g_idx   (E, N)
  AWQ:   w13_qweight (E, K, 2N/8)   w2_qweight (E, N, K/8)
         scales as above, qzeros as above but in the AWQ nibble order

with K the hidden size, N the intermediate size, the gate projection in the
first N columns of w13 and the up projection in the last N.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F

from . import ops
from .marlin_utils import (marlin_moe_padded_intermediate, marlin_moe_permute_scales, marlin_permute_bias,
                           moe_awq_to_marlin_zero_points, moe_packed_to_marlin_zero_points)


@dataclass
class MarlinMoEWeights:
    """What `fused_marlin_moe` takes, named as there."""
    w1: torch.Tensor
    w2: torch.Tensor
    w1_scale: torch.Tensor
    w2_scale: torch.Tensor
    g_idx1: torch.Tensor | None
    g_idx2: torch.Tensor | None
    sort_indices1: torch.Tensor
    sort_indices2: torch.Tensor
    w1_zeros: torch.Tensor | None
    w2_zeros: torch.Tensor | None
    bias1: torch.Tensor | None
    bias2: torch.Tensor | None
    intermediate_size: int          # after padding


def _pad_gate_up_cols(x: torch.Tensor, unit: int, padded_unit: int) -> torch.Tensor:
    """(E, rows, 2 * unit) -> (E, rows, 2 * padded_unit): zeros after each of the two halves."""
    if padded_unit == unit:
        return x
    e, rows, _ = x.shape
    return F.pad(x.reshape(e, rows, 2, unit), (0, padded_unit - unit)).reshape(e, rows, 2 * padded_unit).contiguous()


def _pad_rows(x: torch.Tensor, padded_rows: int) -> torch.Tensor:
    if padded_rows == x.size(1):
        return x
    return F.pad(x, (0, 0, 0, padded_rows - x.size(1)))


def _pad_gate_up_bias(bias: torch.Tensor, n: int, padded_n: int) -> torch.Tensor:
    if padded_n == n:
        return bias
    e = bias.size(0)
    return F.pad(bias.reshape(e, 2, n), (0, padded_n - n)).reshape(e, 2 * padded_n).contiguous()


def _empty_index(num_experts: int, device) -> torch.Tensor:
    return torch.empty((num_experts, 0), dtype=torch.int32, device=device)


def process_gptq_moe_weights(intermediate_size: int, num_bits: int, group_size: int, act_order: bool,
                             w13_qweight: torch.Tensor, w2_qweight: torch.Tensor,
                             w13_scales: torch.Tensor, w2_scales: torch.Tensor,
                             w13_g_idx: torch.Tensor | None = None, w2_g_idx: torch.Tensor | None = None,
                             w13_qzeros: torch.Tensor | None = None, w2_qzeros: torch.Tensor | None = None,
                             w13_bias: torch.Tensor | None = None,
                             w2_bias: torch.Tensor | None = None) -> MarlinMoEWeights:
    """int_wna16.py:492-690 for 16-bit activations.  Scales are permuted with the
    K of their own matrix (hidden size for w13, intermediate size for w2); the
    reference passes the intermediate size for both, which selects the same
    permutation unless exactly one of the two sizes is at most group_size."""
    if num_bits not in (4, 8):
        raise NotImplementedError("expert weights of 4 or 8 bits only")
    if num_bits == 8 and (w13_qzeros is not None or w2_qzeros is not None):
        raise NotImplementedError("8-bit expert weights with zero points")
    pack = 32 // num_bits
    n = intermediate_size
    padded_n = marlin_moe_padded_intermediate(n, group_size)
    if padded_n != n:
        assert not act_order, "Marlin MoE thread-tile padding is unsupported with act-order"
        w13_qweight = _pad_gate_up_cols(w13_qweight, n, padded_n)
        w2_qweight = _pad_rows(w2_qweight, padded_n // pack)
        w13_scales = _pad_gate_up_cols(w13_scales, n, padded_n)
        if group_size > 0:
            w2_scales = _pad_rows(w2_scales, padded_n // group_size)
        if w13_qzeros is not None:
            w13_qzeros = _pad_gate_up_cols(w13_qzeros, n // pack, padded_n // pack)
        if w2_qzeros is not None and group_size > 0:
            w2_qzeros = _pad_rows(w2_qzeros, padded_n // group_size)
        if w13_bias is not None:
            w13_bias = _pad_gate_up_bias(w13_bias, n, padded_n)

    e, dev = w13_qweight.shape[0], w13_qweight.device
    if act_order:
        sort13 = torch.argsort(w13_g_idx, dim=1, stable=True).to(torch.int32)
        sort2 = torch.argsort(w2_g_idx, dim=1, stable=True).to(torch.int32)
        g_idx13 = torch.gather(w13_g_idx, 1, sort13.long()).to(torch.int32)
        g_idx2 = torch.gather(w2_g_idx, 1, sort2.long()).to(torch.int32)
    else:
        sort13, sort2 = _empty_index(e, dev), _empty_index(e, dev)
        g_idx13, g_idx2 = _empty_index(e, dev), _empty_index(e, dev)

    hidden = w13_qweight.shape[1] * pack
    w1 = ops.gptq_marlin_moe_repack(w13_qweight.contiguous(), sort13, hidden, w13_qweight.shape[2], num_bits)
    w2 = ops.gptq_marlin_moe_repack(w2_qweight.contiguous(), sort2, w2_qweight.shape[1] * pack,
                                    w2_qweight.shape[2], num_bits)
    s1 = marlin_moe_permute_scales(w13_scales, hidden, w13_scales.shape[2], group_size)
    s2 = marlin_moe_permute_scales(w2_scales, padded_n, w2_scales.shape[2], group_size)
    z1 = z2 = None
    if w13_qzeros is not None and w2_qzeros is not None:
        z1 = moe_packed_to_marlin_zero_points(w13_qzeros, w13_qzeros.shape[1], w13_qzeros.shape[2] * pack, num_bits)
        z2 = moe_packed_to_marlin_zero_points(w2_qzeros, w2_qzeros.shape[1], w2_qzeros.shape[2] * pack, num_bits)
    return MarlinMoEWeights(w1, w2, s1, s2, g_idx13, g_idx2, sort13, sort2, z1, z2,
                            None if w13_bias is None else marlin_permute_bias(w13_bias),
                            None if w2_bias is None else marlin_permute_bias(w2_bias), padded_n)


def process_awq_moe_weights(intermediate_size: int, num_bits: int, group_size: int,
                            w13_qweight: torch.Tensor, w2_qweight: torch.Tensor,
                            w13_scales: torch.Tensor, w2_scales: torch.Tensor,
                            w13_qzeros: torch.Tensor, w2_qzeros: torch.Tensor,
                            w13_bias: torch.Tensor | None = None,
                            w2_bias: torch.Tensor | None = None) -> MarlinMoEWeights:
    """int_wna16.py:787-940 for 16-bit activations."""
    if num_bits != 4:
        raise NotImplementedError("expert weights of 4 bits only")
    pack = 32 // num_bits
    n = intermediate_size
    padded_n = marlin_moe_padded_intermediate(n, group_size)
    if padded_n != n:
        w13_qweight = _pad_gate_up_cols(w13_qweight, n // pack, padded_n // pack)
        w2_qweight = _pad_rows(w2_qweight, padded_n)
        w13_scales = _pad_gate_up_cols(w13_scales, n, padded_n)
        w13_qzeros = _pad_gate_up_cols(w13_qzeros, n // pack, padded_n // pack)
        if group_size > 0:
            w2_scales = _pad_rows(w2_scales, padded_n // group_size)
            w2_qzeros = _pad_rows(w2_qzeros, padded_n // group_size)
        if w13_bias is not None:
            w13_bias = _pad_gate_up_bias(w13_bias, n, padded_n)

    e, dev = w13_qweight.shape[0], w13_qweight.device
    sort13, sort2 = _empty_index(e, dev), _empty_index(e, dev)
    hidden = w13_qweight.shape[1]
    w1 = ops.awq_marlin_moe_repack(w13_qweight.contiguous(), sort13, hidden, w13_qweight.shape[2] * pack, num_bits)
    w2 = ops.awq_marlin_moe_repack(w2_qweight.contiguous(), sort2, w2_qweight.shape[1],
                                   w2_qweight.shape[2] * pack, num_bits)
    s1 = marlin_moe_permute_scales(w13_scales, hidden, w13_scales.shape[2], group_size)
    s2 = marlin_moe_permute_scales(w2_scales, padded_n, w2_scales.shape[2], group_size)
    z1 = moe_awq_to_marlin_zero_points(w13_qzeros, w13_qzeros.shape[1], w13_qzeros.shape[2] * pack, num_bits)
    z2 = moe_awq_to_marlin_zero_points(w2_qzeros, w2_qzeros.shape[1], w2_qzeros.shape[2] * pack, num_bits)
    return MarlinMoEWeights(w1, w2, s1, s2, None, None, sort13, sort2, z1, z2,
                            None if w13_bias is None else marlin_permute_bias(w13_bias),
                            None if w2_bias is None else marlin_permute_bias(w2_bias), padded_n)
