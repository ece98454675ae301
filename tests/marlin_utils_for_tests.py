"""Builders of Marlin-format test inputs from real-valued weights: the
counterpart of aphrodite/model_executor/layers/quantization/utils/
marlin_utils_test.py:20-207 (MarlinWorkspace, get_weight_perm,
marlin_permute_weights, marlin_weights, marlin_quantize, awq_marlin_quantize),
for 16-bit and 8-bit activations.  This is the independent statement of the Marlin order
the repack ops are compared against bit for bit, as in the reference's
test_gptq_marlin_repack / test_awq_marlin_repack."""
from __future__ import annotations

import torch

from sonar_amd.marlin_utils import (GPTQ_MARLIN_TILE, get_pack_factor, marlin_permute_scales, marlin_zero_points)
from tests.quant_utils import gptq_quantize_weights, quantize_weights, sort_weights
from sonar_amd import ops
from sonar_amd.scalar_type import ScalarType, scalar_types


class MarlinWorkspace:
    def __init__(self, out_features, min_thread_n, max_parallel):
        assert out_features % min_thread_n == 0, (
            f"out_features = {out_features} is indivisible by min_thread_n = {min_thread_n}")
        self.scratch = torch.zeros((out_features // min_thread_n) * max_parallel, dtype=torch.int, device="cuda")


def get_weight_perm(num_bits: int, is_a_8bit: bool = False) -> torch.Tensor:
    """Where the 1024 codes of four 16 x 16 tiles go inside a row of the Marlin
    matrix (marlin_utils_test.py:69-121).  Entry order: thread slot i = 0..31,
    tile j = 0..3, 8-column half `block`, then the thread's four rows
    2 (i % 4) + {0, 1, 8, 9}; the value is the code's index 16 row + column
    inside its tile, + 256 j.  Codes are then interleaved inside every word."""
    i = torch.arange(32).view(32, 1, 1, 1)
    block = torch.arange(2).view(1, 1, 2, 1)
    if is_a_8bit:
        # two 16-column tiles of 32 rows; the thread's eight rows 4 (i % 4) + {0..3, 16..19}
        j = torch.arange(2).view(1, 2, 1, 1)
        row = 4 * (i % 4) + torch.tensor([0, 1, 2, 3, 16, 17, 18, 19]).view(1, 1, 1, 8)
        perm = (16 * row + i // 4 + 8 * block + 512 * j).reshape(-1)
    else:
        j = torch.arange(4).view(1, 4, 1, 1)
        row = 2 * (i % 4) + torch.tensor([0, 1, 8, 9]).view(1, 1, 1, 4)
        perm = (16 * row + i // 4 + 8 * block + 256 * j).reshape(-1)
    if num_bits == 4:
        interleave = [0, 4, 1, 5, 2, 6, 3, 7] if is_a_8bit else [0, 2, 4, 6, 1, 3, 5, 7]
    elif num_bits == 8:
        interleave = [0, 1, 2, 3] if is_a_8bit else [0, 2, 1, 3]
    else:
        raise Exception(f"num_bits must be 4 or 8, got {num_bits}")
    return perm.reshape(-1, len(interleave))[:, interleave].reshape(-1).contiguous()


def marlin_permute_weights(q_w, size_k, size_n, perm, tile=GPTQ_MARLIN_TILE, is_a_8bit=False):
    """(K, N) codes -> (K / 16, 16 N): 16 x 16 tiles laid side by side, then
    `perm` inside every run of perm.numel() codes (marlin_utils_test.py:31-47)."""
    assert q_w.shape == (size_k, size_n)
    assert size_k % tile == 0, f"size_k = {size_k}, tile = {tile}"
    assert size_n % tile == 0, f"size_k = {size_n}, tile = {tile}"
    rows_per_tile = tile * 2 if is_a_8bit else tile   # 32 x 32 tiles for 8-bit activations
    tiles = q_w.reshape(size_k // rows_per_tile, rows_per_tile, size_n // tile, tile).permute(0, 2, 1, 3)
    rows = tiles.reshape(size_k // tile, size_n * tile)
    return rows.reshape(-1, perm.numel())[:, perm.to(rows.device)].reshape(rows.shape)


def marlin_weights(q_w, size_k, size_n, num_bits, perm, is_a_8bit=False):
    """Permuted codes packed `pack` to a word, code i of a word at bit
    num_bits * i (marlin_utils_test.py:50-66)."""
    q_w = marlin_permute_weights(q_w, size_k, size_n, perm, is_a_8bit=is_a_8bit)
    pack = get_pack_factor(num_bits)
    shifts = torch.arange(pack, device=q_w.device, dtype=torch.int64) * num_bits
    words = (q_w.to(torch.int64).reshape(q_w.shape[0], -1, pack) << shifts).sum(dim=2) & 0xFFFFFFFF
    return torch.where(words >= 2 ** 31, words - 2 ** 32, words).to(torch.int32)


def marlin_quantize(w: torch.Tensor, quant_type: ScalarType, group_size: int, act_order: bool,
                    test_perm: torch.Tensor | None = None, input_dtype: torch.dtype | None = None):
    """w (K, N) -> [w_ref, marlin_q_w, marlin_s, g_idx, sort_indices, rand_perm]
    (marlin_utils_test.py:124-165)."""
    is_a_8bit = input_dtype is not None and input_dtype.itemsize == 1
    size_k, size_n = w.shape
    num_bits = quant_type.size_bits
    if group_size == -1:
        group_size = size_k
    assert group_size <= size_k
    w_ref, q_w, s, g_idx, rand_perm = gptq_quantize_weights(w, quant_type, group_size, act_order, test_perm)
    sort_indices = torch.empty(0, dtype=torch.int, device=w.device)
    if act_order:
        q_w, g_idx, sort_indices = sort_weights(q_w, g_idx)
    marlin_q_w = marlin_weights(q_w, size_k, size_n, num_bits, get_weight_perm(num_bits, is_a_8bit),
                                is_a_8bit=is_a_8bit)
    marlin_s = marlin_permute_scales(s, size_k, size_n, group_size, is_a_8bit=is_a_8bit)
    if input_dtype == torch.float8_e4m3fn and quant_type == scalar_types.uint4b8:   # marlin_utils_test.py:156-158
        ops.marlin_int4_fp8_preprocess(marlin_q_w, inplace=True)
        marlin_s = marlin_s * 512
    return [t.to(w.device) for t in (w_ref, marlin_q_w, marlin_s, g_idx, sort_indices, rand_perm)]


def awq_marlin_quantize(w: torch.Tensor, quant_type: ScalarType, group_size: int,
                        input_dtype: torch.dtype | None = None):
    """w (K, N) -> [w_ref, marlin_q_w, marlin_s, marlin_zp] (marlin_utils_test.py:168-207)."""
    is_a_8bit = input_dtype is not None and input_dtype.itemsize == 1
    size_k, size_n = w.shape
    if group_size == -1:
        group_size = size_k
    assert group_size <= size_k
    assert size_k % group_size == 0
    num_groups = size_k // group_size
    w_ref, q_w, s, zp = quantize_weights(w, quant_type, group_size, zero_points=True)
    if input_dtype == torch.float8_e4m3fn and quant_type == scalar_types.uint4:   # marlin_utils_test.py:190-195
        repeated_zp = zp.repeat_interleave(group_size, 0)
        q_w_old = q_w
        q_w = q_w_old - repeated_zp
        q_w[q_w < 0] = 15 - q_w_old[q_w < 0]
        s = s * 512
    marlin_q_w = marlin_weights(q_w, size_k, size_n, quant_type.size_bits,
                                get_weight_perm(quant_type.size_bits, is_a_8bit), is_a_8bit=is_a_8bit)
    marlin_s = marlin_permute_scales(s, size_k, size_n, group_size, is_a_8bit=is_a_8bit)
    marlin_zp = marlin_zero_points(zp, num_groups, size_n, quant_type.size_bits, is_a_8bit=is_a_8bit)
    return [t.to(w.device) for t in (w_ref, marlin_q_w, marlin_s, marlin_zp)]
