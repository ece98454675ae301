"""Child process of test_gpu_dispatch_paths: the dispatcher reads its
debugging switches once per process, so every switch gets a process of its
own.  Runs a fixed list of dense and grouped cases through the C ABI and
checks each against the oracle; prints one line per case and exits non-zero
on the first failure."""
from __future__ import annotations

import os
import sys

import numpy as np
import torch

from oracle import marlin_oracle as mo
from tests import gpu_util as gu

DENSE = [
    # m, k, n, group, dtype, zp, bias
    (16, 4096, 4096, 128, "bf16", False, False),
    (7, 1024, 4096, 128, "fp16", True, True),
    (48, 1024, 512, 128, "fp16", False, False),
    (64, 2048, 4096, 128, "bf16", True, True),
    (100, 1024, 4224, 128, "fp16", True, False),
    (33, 14336, 1024, 128, "bf16", False, True),
    (200, 512, 4096, 128, "fp16", False, False),
    (300, 1024, 768, 128, "bf16", False, True),
    (300, 1024, 768, 128, "fp16", False, False),
    (600, 1024, 768, 64, "fp16", True, False),
    (1100, 512, 1024, -1, "bf16", False, False),
    (2100, 512, 4096, 128, "bf16", True, True),     # 144 tiles of 256 rows: the wide tile kernel's 256-row form
    (600, 1024, 768, 32, "fp16", True, False),      # groups of 32 rows in either tile kernel
    (128, 1024, 40960, 128, "fp16", False, False),  # 97..128 rows on more than 512 strips: one launch of row blocks
]


def dense() -> None:
    cases = list(DENSE)
    if "SONAR_MARLIN_NO_TWO_TILE_SIZES" in os.environ:
        # 9 x 29 = 261 tiles of 256 rows: a last round of five tiles, which would run as 128-row tiles
        cases.append((2200, 3072, 7360, 128, "fp16", True, True))
    for (m, k, n, g, dtype, zp, bias) in cases:
        layer = gu.DeviceLayer(5 + m, k, n, g, dtype, zero_points=zp, bias=bias)
        a32 = mo.make_activations(m + 1, m, k, dtype, std=0.5)
        c = layer.gemm(gu.dev_bits16(a32, dtype), m)
        torch.cuda.synchronize()
        ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), mo.gemm_reference(a32, layer.w_ref, layer.bias32))
        print("dense", m, k, n, g, dtype, zp, bias, "ok" if ok else f"FAILED max_err={max_err} max_ref={max_ref}",
              flush=True)
        if not ok:
            sys.exit(1)


def dense_mxfp4() -> None:
    """float4_e2m1f weights take the decode, the general and the tile kernel; every
    switch must leave them on a kernel that has the float4 dequantiser."""
    from sonar_amd import _lib
    from tests import test_gpu_parity as tp
    lib = _lib.load()
    for (m, k, n) in [(16, 1024, 4096), (48, 1024, 512), (300, 1024, 768)]:
        L = tp._layer_mxfp4(gu, 9 + m, k, n)
        a32 = mo.make_activations(m + 1, m, k, "bf16", std=0.5)
        a = gu.dev_bits16(a32, "bf16")
        c = torch.empty((m, n), dtype=torch.bfloat16, device=gu.DEV)
        ws = torch.zeros(torch.cuda.get_device_properties(0).multi_processor_count, dtype=torch.int32, device=gu.DEV)
        scratch = torch.empty(max(lib.sonar_marlin_gemm_scratch_bytes(m, n, k), 16), dtype=torch.uint8, device=gu.DEV)
        _lib.check(lib.sonar_marlin_gemm(
            gu.ptr(a), k, gu.ptr(c), gu.ptr(L["native"]), _lib.LAYOUT_GFX950, None, gu.ptr(L["scales"]), None, None,
            None, gu.ptr(ws), ws.numel(), gu.ptr(scratch), scratch.numel(), gu.dtype_code("bf16"),
            _lib.TYPE_FLOAT4_E2M1F, m, n, k, L["groups"], 1, 0, 1, gu.stream()))
        torch.cuda.synchronize()
        ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), mo.gemm_reference(a32, L["w_ref"]))
        print("mxfp4", m, k, n, "ok" if ok else f"FAILED max_err={max_err} max_ref={max_ref}", flush=True)
        if not ok:
            sys.exit(1)


def dense_8bit() -> None:
    """8-bit codes on both tile kernels: one group, groups of 128 and of 32 rows (the test
    functions raise on a mismatch)."""
    from tests import test_gpu_parity as tp
    for (dtype, m, k, n, g) in [("bf16", 1024, 1024, 832, 32), ("fp16", 700, 1280, 4160, 32),
                                ("fp16", 300, 2048, 512, 128), ("bf16", 260, 1024, 4160, -1)]:
        tp.test_fp8_weights_dequant_bit_exact_and_gemm_within_tolerance(gu, dtype, m, k, n, g, True)
        tp.test_w8a16_dequant_bit_exact_and_gemm_within_tolerance(gu, dtype, m, k, n, g, False, False)
        print("8-bit", dtype, m, k, n, g, "ok", flush=True)
    # NVFP4 on both tile kernels
    for (dtype, m, k, n) in [("fp16", 600, 2048, 1536), ("bf16", 2100, 512, 4160)]:
        tp.test_nvfp4_weights_dequant_bit_exact_and_gemm_within_tolerance(gu, m, k, n, True, dtype)
        print("nvfp4", dtype, m, k, n, "ok", flush=True)


def grouped() -> None:
    from tests import test_gpu_moe as tm
    for case in [(300, 4, 2, 256, 256, 128, "fp16", False, False, False, 64, True),
                 (700, 8, 2, 512, 128, 64, "bf16", True, False, True, 64, False),
                 (900, 3, 2, 2048, 256, 128, "bf16", True, False, True, 64, False),   # K split on the device
                 (40, 4, 2, 256, 128, 128, "fp16", False, False, False, 16, True),
                 (3, 8, 2, 512, 256, 128, "bf16", True, False, True, 8, False),
                 (130, 4, 2, 256, 320, -1, "fp16", False, False, True, 32, True),
                 (50, 4, 2, 512, 128, 128, "bf16", False, True, False, 16, True)]:     # act-order
        print("grouped", case, flush=True)
        tm.test_moe_gemm_within_tolerance(case)   # raises on a mismatch
    # NVFP4 experts on 64-slot blocks: the tile kernels, or the general grouped kernel when they are switched off
    from tests import test_gpu_ops as to
    to.test_prepare_nvfp4_moe_layer_and_fused_marlin_moe((1500, 4, 2, 256, 128), "fp16")
    print("grouped nvfp4 ok", flush=True)


def dense_large() -> None:
    """The two large projections of the benchmark's layer at 16 rows: the matrices whose weight copies
    carry the non-temporal bit unless it is switched off (sampled columns against the oracle)."""
    from tests import test_gpu_full_size as tf
    for name in ("gate_up", "down"):
        tf.test_decode_sweep_meets_the_oracle_on_sampled_columns(name, 16)
        print("dense large", name, "ok", flush=True)


if __name__ == "__main__":
    if "SONAR_MARLIN_NO_NT_WEIGHTS" in os.environ:
        dense_large()
    dense()
    dense_mxfp4()
    dense_8bit()
    grouped()
    print("all paths ok", flush=True)
