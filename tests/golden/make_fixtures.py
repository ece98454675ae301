#!/usr/bin/env python3
"""Writes the golden fixtures of this directory from the CPU oracle.

The reference's own tests hold no stored vectors for the Marlin path (they
compare against helper code at run time), so these fixtures are this
repository's: seeded inputs and the oracle's outputs, frozen so that a later
change of the oracle or of a kernel shows up as a diff against committed data.
`moe_align_example` is the one literal vector the reference gives
(fused_moe/moe_align_block_size.py:60-73).

Run from the repository root:  python tests/golden/make_fixtures.py
"""
from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import marlin_oracle as mo  # noqa: E402


def layer_fixture(seed, k, n, g, dtype, zero_points, act_order, m):
    layer = mo.make_layer(seed, k, n, g, dtype, zero_points, act_order)
    q = layer["q"]
    out = {"size_k": np.int64(k), "size_n": np.int64(n), "group_size": np.int64(g), "size_m": np.int64(m),
           "q": q.astype(np.uint8), "gptq_packed": mo.gptq_pack(q), "awq_packed": mo.awq_pack(q),
           "scales_bits": mo.to_bits16(layer["scales"], dtype)}
    perm = None
    if act_order:
        g_sorted, perm = mo.stable_sort_g_idx(layer["g_idx"])
        out["g_idx"] = layer["g_idx"].astype(np.int32)
        out["g_idx_sorted"] = g_sorted.astype(np.int32)
        out["perm"] = perm.astype(np.int32)
    marlin = mo.gptq_marlin_repack(mo.gptq_pack(q), perm, k, n)
    out["marlin"] = marlin
    out["gfx950"] = mo.marlin_to_gfx950(marlin, k, n)
    gs = g if g < k else -1
    out["scales_marlin_bits"] = mo.to_bits16(mo.marlin_permute_scales(layer["scales"], k, n, gs), dtype)
    if zero_points:
        out["zeros"] = layer["zeros"].astype(np.uint8)
        out["zeros_marlin"] = mo.marlin_zero_points(layer["zeros"], layer["groups"], n)
    w = mo.dequantize(q, layer["scales"], g, dtype, zeros=layer.get("zeros"), g_idx=layer.get("g_idx"))
    out["dequant_bits"] = mo.to_bits16(w, dtype)
    a = mo.make_activations(seed + 1, m, k, dtype)
    out["a_bits"] = mo.to_bits16(a, dtype)
    out["c_ref"] = mo.gemm_reference(a, w)
    return out


def layer8_fixture(seed, k, n, g, dtype, m):
    """8-bit (uint8b128) weights: codes, the three packings, dequantised bits, GEMM."""
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    scales = mo.round_to_dtype(rng.uniform(1e-4, 1e-3, size=(k // g, n)).astype(np.float32), dtype)
    marlin = mo.gptq_marlin_repack8(mo.pack_rows8(q), None, k, n)
    w = mo.dequantize(q, scales, g, dtype, num_bits=8)
    a = mo.make_activations(seed + 1, m, k, dtype)
    return {"size_k": np.int64(k), "size_n": np.int64(n), "group_size": np.int64(g), "size_m": np.int64(m),
            "q": q.astype(np.uint8), "gptq_packed": mo.pack_rows8(q), "marlin": marlin,
            "gfx950": mo.marlin8_to_gfx950(marlin, k, n), "scales_bits": mo.to_bits16(scales, dtype),
            "scales_marlin_bits": mo.to_bits16(mo.marlin_permute_scales(scales, k, n, g), dtype),
            "dequant_bits": mo.to_bits16(w, dtype), "a_bits": mo.to_bits16(a, dtype),
            "c_ref": mo.gemm_reference(a, w)}


def w4a8_fixture(seed, k, n, g, dtype, m):
    """4-bit weights with int8 activations: the order of 8-bit activations, integer group
    scales, per-token quantised activations and the exact result of the integer GEMM."""
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    zeros = rng.integers(0, 16, size=(k // g, n), dtype=np.int32)
    scales = mo.round_to_dtype(rng.uniform(1e-3, 1e-2, size=(k // g, n)).astype(np.float32), dtype)
    ints, factor = mo.marlin_act_int8_process_scales(scales)
    marlin = mo.gptq_marlin_repack_a8(mo.gptq_pack(q), k, n)
    x = rng.standard_normal((m, k)).astype(np.float32)
    a_q, a_s = mo.per_token_quant_int8(x)
    a_s = (a_s * factor).astype(np.float32)
    return {"size_k": np.int64(k), "size_n": np.int64(n), "group_size": np.int64(g), "size_m": np.int64(m),
            "q": q.astype(np.uint8), "gptq_packed": mo.gptq_pack(q), "awq_packed": mo.awq_pack(q),
            "marlin_a8": marlin, "gfx950": mo.marlin_a8_to_gfx950(marlin, k, n),
            "fp8_preprocessed": mo.int4_fp8_preprocess(q).astype(np.uint8),
            "zeros": zeros.astype(np.uint8), "zeros_marlin_a8": mo.marlin_zero_points_a8(zeros, k // g, n),
            "int_scales": ints, "int_scales_marlin_a8": mo.marlin_permute_scales_a8(ints, k, n, g),
            "x": x, "a_q": a_q, "a_scales": a_s,
            "c_bits": mo.to_bits16(mo.gemm_w4a8_int8(a_q, a_s, q, g, ints, dtype), dtype),
            "c_zp_bits": mo.to_bits16(mo.gemm_w4a8_int8(a_q, a_s, q, g, ints, dtype, zeros), dtype)}


def main():
    np.savez_compressed(os.path.join(HERE, "w4a8_int8_fp16_k256_n128_g64.npz"),
                        **w4a8_fixture(105, 256, 128, 64, "fp16", 9))
    np.savez_compressed(os.path.join(HERE, "gptq8_bf16_k128_n64_g64.npz"),
                        **layer8_fixture(104, 128, 64, 64, "bf16", 6))
    np.savez_compressed(os.path.join(HERE, "gptq_fp16_k128_n128_g64.npz"),
                        **layer_fixture(101, 128, 128, 64, "fp16", False, False, 5))
    np.savez_compressed(os.path.join(HERE, "awq_bf16_k128_n64_g32.npz"),
                        **layer_fixture(102, 128, 64, 32, "bf16", True, False, 3))
    np.savez_compressed(os.path.join(HERE, "actorder_fp16_k256_n64_g128.npz"),
                        **layer_fixture(103, 256, 64, 128, "fp16", False, True, 17))
    ids = np.array([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], dtype=np.int32)
    s, e, p = mo.moe_align_block_size(ids, 4, 5)
    np.savez_compressed(os.path.join(HERE, "moe_align_example.npz"), topk_ids=ids, block_size=np.int64(4),
                        num_experts=np.int64(5), sorted_ids=s, expert_ids=e, num_post_pad=p)
    # every 4-bit code against zero points 0..15 and a spread of scale bit patterns
    rng = np.random.default_rng(7)
    for dtype in ("fp16", "bf16"):
        scales = mo.round_to_dtype(np.concatenate([rng.uniform(1e-3, 1e-2, 24), [0.0, 1.0, 6.1e-5, 3.0e-3]])
                                   .astype(np.float32), dtype)
        codes = np.arange(16, dtype=np.int64)
        table = np.zeros((16, 16, scales.size), dtype=np.uint16)
        for z in range(16):
            table[z] = mo.to_bits16(mo.round_to_dtype(((codes - z)[:, None] * scales[None, :])
                                                      .astype(np.float32), dtype), dtype)
        np.savez_compressed(os.path.join(HERE, f"dequant_table_{dtype}.npz"),
                            scales_bits=mo.to_bits16(scales, dtype), table_bits=table)
    # floating-point weight types: every fp8 code (rows) under 64 channel scales with the exponent bias
    # folded in, and every fp4 code under power-of-two block scales (MXFP4, one exponent byte per 32 rows)
    for dtype in ("fp16", "bf16"):
        scales = mo.round_to_dtype(np.concatenate([rng.uniform(1e-4, 1e-2, 60), [1.0, 0.333, 6.1e-5, 2.0 ** -9]])
                                   .astype(np.float32), dtype)
        fused = mo.fp8_fuse_exponent_bias(scales[None, :], dtype)
        codes = np.arange(256, dtype=np.int32)[:, None].repeat(64, 1)
        np.savez_compressed(os.path.join(HERE, f"fp8_dequant_table_{dtype}.npz"), codes=codes.astype(np.uint8),
                            fused_scales_bits=mo.to_bits16(fused, dtype),
                            dequant_bits=mo.to_bits16(mo.dequantize_fp8(codes, fused, -1, dtype), dtype))
    codes4 = rng.integers(0, 16, size=(128, 64), dtype=np.int32)
    codes4[:16, :] = np.arange(16)[:, None]
    exps = rng.integers(90, 140, size=(4, 64)).astype(np.uint8)
    exps[0, :4] = [0, 1, 127, 250]
    np.savez_compressed(os.path.join(HERE, "mxfp4_dequant_k128_n64.npz"), codes=codes4.astype(np.uint8),
                        exponent_bytes=exps, gptq_packed=mo.gptq_pack(codes4),
                        dequant_bits=mo.to_bits16(mo.dequantize_mxfp4(codes4, exps), "bf16"))
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
