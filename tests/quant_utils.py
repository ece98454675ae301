"""Weight quantisation helpers the reference's Marlin tests build their inputs
with: the counterpart of aphrodite/model_executor/layers/quantization/utils/
quant_utils.py:553-834 (quantize_weights, gptq_quantize_weights, permute_rows,
sort_weights, gptq_pack, awq_pack).  Same names, arguments and results; every
arithmetic step runs in the dtype the reference runs it in, so the same seeded
weights give the same codes, scales and dequantised references."""
from __future__ import annotations

import torch

from sonar_amd.marlin_utils import get_pack_factor, pack_cols
from sonar_amd.scalar_type import ScalarType, scalar_types

SUPPORTED_GPTQ_QUANT_TYPES = [scalar_types.uint4b8, scalar_types.uint8b128]
SUPPORTED_GROUP_SIZES = [-1, 32, 64, 128]
_AWQ_ORDER_4BIT = [0, 2, 4, 6, 1, 3, 5, 7]
_AWQ_ORDER_8BIT = [0, 2, 1, 3]


def quantize_weights(w: torch.Tensor, quant_type: ScalarType, group_size: int | None,
                     zero_points: bool = False, ref_zero_points_after_scales: bool = False):
    """Round-to-nearest quantisation of w (K, N) to `quant_type`, one scale (and
    optionally one zero point) per group of `group_size` rows and column
    (quant_utils.py:588-679).  Returns (w_ref, w_q, scales (groups, N) or None,
    zero points (groups, N) or None); w_q holds the stored codes (the type's
    bias added)."""
    assert quant_type.is_integer(), "Floating point quantization may work but has not been tested"
    assert not zero_points or group_size is not None, (
        "to have group zero points, group_size must be provided (-1 group_size is channelwise)")
    assert w.is_floating_point(), "w must be float"
    size_k, size_n = w.shape
    dtype = w.dtype
    if group_size == -1:
        group_size = size_k
    lo, hi = quant_type.min(), quant_type.max()
    if group_size is None:                       # unscaled
        q = torch.clamp(torch.round(w).int(), lo, hi)
        w_ref = q.to(dtype) * torch.ones((), dtype=torch.float32, device=w.device)
        if quant_type.has_bias():
            q = q + quant_type.bias
        return w_ref, q, None, None

    groups = size_k // group_size
    wg = w.reshape(groups, group_size, size_n)
    max_val = wg.amax(dim=1, keepdim=True)
    min_val = wg.amin(dim=1, keepdim=True)
    zp = None
    if zero_points:
        assert not quant_type.is_signed() and hi > 0
        scale = (max_val - min_val).clamp(min=1e-5) / hi
        zp = torch.round(torch.abs(min_val / scale)).clamp(lo, hi).int()
        q = torch.clamp(torch.round(wg / scale).int() + zp, lo, hi)
        if ref_zero_points_after_scales:
            w_ref = q.to(dtype) * scale - zp.to(dtype) * scale
        else:
            w_ref = (q - zp).to(dtype) * scale
    else:
        # a type without negative (positive) codes takes no part in the choice of scale
        scale = torch.max(torch.abs(max_val / (hi if hi != 0 else float("inf"))),
                          torch.abs(min_val / (lo if lo != 0 else float("inf"))))
        q = torch.clamp(torch.round(wg / scale).int(), lo, hi)
        w_ref = q.to(dtype) * scale
    if quant_type.has_bias():
        q = q + quant_type.bias
    return (w_ref.reshape(size_k, size_n).contiguous(), q.reshape(size_k, size_n).contiguous(),
            scale.reshape(groups, size_n).contiguous(),
            None if zp is None else zp.reshape(groups, size_n).contiguous())


def permute_rows(q_w: torch.Tensor, w_ref: torch.Tensor, group_size: int, test_perm: torch.Tensor | None = None):
    """Act-order as the tests simulate it: a random permutation of the rows, with
    g_idx naming the group every permuted row came from (quant_utils.py:558-585)."""
    assert q_w.shape == w_ref.shape
    size_k = q_w.shape[0]
    rand_perm = test_perm if test_perm is not None else torch.randperm(size_k)
    rand_perm = rand_perm.to(q_w.device)
    g_idx = (rand_perm // group_size).to(torch.int32)
    return w_ref[rand_perm].contiguous(), q_w[rand_perm].contiguous(), g_idx.contiguous(), rand_perm


def gptq_quantize_weights(w: torch.Tensor, quant_type: ScalarType, group_size: int, act_order: bool,
                          test_perm: torch.Tensor | None = None):
    """quant_utils.py:682-707."""
    size_k = w.shape[0]
    assert w.is_floating_point(), "w must be float"
    assert quant_type in SUPPORTED_GPTQ_QUANT_TYPES, f"Unsupported gptq type = {quant_type}"
    assert group_size in SUPPORTED_GROUP_SIZES + [size_k], f"Unsupported groupsize = {group_size}"
    w_ref, w_q, w_s, _ = quantize_weights(w, quant_type, group_size)
    g_idx = torch.empty(0, dtype=torch.int, device=w.device)
    rand_perm = torch.empty(0, dtype=torch.int, device=w.device)
    if act_order:
        assert group_size < size_k, f"For act_order, groupsize = {group_size} must be less than size_k = {size_k}"
        w_ref, w_q, g_idx, rand_perm = permute_rows(w_q, w_ref, group_size, test_perm)
    return w_ref, w_q, w_s, g_idx, rand_perm


def sort_weights(q_w: torch.Tensor, g_idx: torch.Tensor):
    """Rows in increasing group order (quant_utils.py:710-722).  The sort is
    stable here; any order of the rows inside a group serves, as long as the
    same indices go to the repack op and to the GEMM."""
    sort_indices = torch.argsort(g_idx, stable=True).to(torch.int32)
    return q_w[sort_indices.long()].contiguous(), g_idx[sort_indices.long()].contiguous(), sort_indices


def pack_rows(q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    """Codes packed along K: word [k / pack][n] holds rows pack * (k / pack) .. at
    num_bits * (k % pack) (quant_utils.py:725-746)."""
    assert q_w.shape == (size_k, size_n)
    pack = get_pack_factor(num_bits)
    assert size_k % pack == 0
    shifts = (torch.arange(pack, device=q_w.device, dtype=torch.int64) * num_bits).view(1, pack, 1)
    words = (q_w.to(torch.int64).reshape(size_k // pack, pack, size_n) << shifts).sum(dim=1)
    return _to_int32(words)


def _to_int32(words: torch.Tensor) -> torch.Tensor:
    words = words & 0xFFFFFFFF
    return torch.where(words >= 2 ** 31, words - 2 ** 32, words).to(torch.int32)


def gptq_pack(q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    return pack_rows(q_w, num_bits, size_k, size_n)


def awq_pack(q_w: torch.Tensor, num_bits: int, size_k: int, size_n: int) -> torch.Tensor:
    """AWQ packing along N: inside every `pack` columns, slot p holds column
    order[p] (quant_utils.py:815-834)."""
    assert q_w.shape == (size_k, size_n)
    order = _AWQ_ORDER_4BIT if num_bits == 4 else _AWQ_ORDER_8BIT
    q_w = q_w.reshape(-1, len(order))[:, order].reshape(size_k, size_n).contiguous()
    return pack_cols(q_w, num_bits, size_k, size_n)
