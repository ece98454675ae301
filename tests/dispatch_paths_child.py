"""Child process of test_gpu_dispatch_paths: the dispatcher reads its
debugging switches once per process, so every switch gets a process of its
own.  Runs a fixed list of dense and grouped cases through the C ABI and
checks each against the oracle; prints one line per case and exits non-zero
on the first failure."""
from __future__ import annotations

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
    (600, 1024, 768, 64, "fp16", True, False),
    (1100, 512, 1024, -1, "bf16", False, False),
]


def dense() -> None:
    for (m, k, n, g, dtype, zp, bias) in DENSE:
        layer = gu.DeviceLayer(5 + m, k, n, g, dtype, zero_points=zp, bias=bias)
        a32 = mo.make_activations(m + 1, m, k, dtype, std=0.5)
        c = layer.gemm(gu.dev_bits16(a32, dtype), m)
        torch.cuda.synchronize()
        ok, max_err, max_ref = mo.gemm_tolerance_ok(gu.host_f32(c), mo.gemm_reference(a32, layer.w_ref, layer.bias32))
        print("dense", m, k, n, g, dtype, zp, bias, "ok" if ok else f"FAILED max_err={max_err} max_ref={max_ref}",
              flush=True)
        if not ok:
            sys.exit(1)


def grouped() -> None:
    from tests import test_gpu_moe as tm
    for case in [(300, 4, 2, 256, 256, 128, "fp16", False, False, False, 64, True),
                 (700, 8, 2, 512, 128, 64, "bf16", True, False, True, 64, False),
                 (40, 4, 2, 256, 128, 128, "fp16", False, False, False, 16, True),
                 (3, 8, 2, 512, 256, 128, "bf16", True, False, True, 8, False),
                 (130, 4, 2, 256, 320, -1, "fp16", False, False, True, 32, True),
                 (50, 4, 2, 512, 128, 128, "bf16", False, True, False, 16, True)]:     # act-order
        print("grouped", case, flush=True)
        tm.test_moe_gemm_within_tolerance(case)   # raises on a mismatch


if __name__ == "__main__":
    dense()
    grouped()
    print("all paths ok", flush=True)
