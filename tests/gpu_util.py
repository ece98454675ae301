"""Helpers for the GPU parity tests: they call the C ABI through ctypes with
torch tensors as device memory, and compare against the CPU oracle."""
from __future__ import annotations

import ctypes

import numpy as np
import torch

from oracle import marlin_oracle as mo
from sonar_amd import _lib

DEV = "cuda:0"


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def dev_i32(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32).copy()).to(DEV)


def dev_bits16(x32: np.ndarray, dtype: str) -> torch.Tensor:
    bits = mo.to_bits16(x32, dtype).view(np.int16).copy()
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    return torch.from_numpy(bits).to(DEV).view(tdt)


def host_f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def dtype_code(dtype: str) -> int:
    return _lib.DTYPE_F16 if dtype == "fp16" else _lib.DTYPE_BF16


def gptq_repack(qw: torch.Tensor, perm, k: int, n: int) -> torch.Tensor:
    lib = _lib.load()
    out = torch.empty((k // 16, 2 * n), dtype=torch.int32, device=DEV)
    _lib.check(lib.sonar_gptq_marlin_repack(ptr(qw), ptr(perm), ptr(out), k, n, 4, stream()))
    return out


def awq_repack(qw: torch.Tensor, k: int, n: int) -> torch.Tensor:
    lib = _lib.load()
    out = torch.empty((k // 16, 2 * n), dtype=torch.int32, device=DEV)
    _lib.check(lib.sonar_awq_marlin_repack(ptr(qw), ptr(out), k, n, 4, stream()))
    return out


def to_gfx950(marlin: torch.Tensor, k: int, n: int) -> torch.Tensor:
    lib = _lib.load()
    out = torch.empty(k * n // 8, dtype=torch.int32, device=DEV)
    _lib.check(lib.sonar_marlin_to_gfx950(ptr(marlin), ptr(out), k, n, stream()))
    return out


def from_gfx950(native: torch.Tensor, k: int, n: int) -> torch.Tensor:
    lib = _lib.load()
    out = torch.empty((k // 16, 2 * n), dtype=torch.int32, device=DEV)
    _lib.check(lib.sonar_gfx950_to_marlin(ptr(native), ptr(out), k, n, stream()))
    return out


class DeviceLayer:
    """A quantised layer prepared the way the reference's callers prepare it
    (repack on the device, scales / zero points / bias permuted on the host by
    the oracle), plus the oracle's dequantised matrix."""

    def __init__(self, seed, k, n, group_size, dtype, zero_points=False, act_order=False,
                 bias=False, awq_source=False):
        self.k, self.n, self.dtype = k, n, dtype
        layer = mo.make_layer(seed, k, n, group_size, dtype, zero_points, act_order)
        self.layer = layer
        q = layer["q"]
        self.groups = layer["groups"]
        gs = group_size if group_size not in (-1, k) else -1
        self.w_ref = mo.dequantize(q, layer["scales"], group_size, dtype,
                                   zeros=layer.get("zeros"), g_idx=layer.get("g_idx"))
        self.perm = None
        self.g_idx = None
        if act_order:
            g_sorted, order = mo.stable_sort_g_idx(layer["g_idx"])
            self.perm = dev_i32(order)
            self.g_idx = dev_i32(g_sorted)
        if awq_source:
            self.marlin = awq_repack(dev_i32(mo.awq_pack(q)), k, n)
        else:
            self.marlin = gptq_repack(dev_i32(mo.gptq_pack(q)), self.perm, k, n)
        self.native = to_gfx950(self.marlin, k, n)
        self.scales = dev_bits16(mo.marlin_permute_scales(layer["scales"], k, n, gs), dtype)
        self.zeros = None
        if zero_points:
            self.zeros = dev_i32(mo.marlin_zero_points(layer["zeros"], self.groups, n))
        self.bias = None
        self.bias32 = None
        if bias:
            rng = np.random.default_rng(seed + 999)
            self.bias32 = mo.round_to_dtype(rng.standard_normal(n).astype(np.float32), dtype)
            self.bias = dev_bits16(mo.marlin_permute_bias(self.bias32), dtype)
        self.b_type = _lib.TYPE_UINT4 if zero_points else _lib.TYPE_UINT4B8
        props = torch.cuda.get_device_properties(0)
        self.workspace = torch.zeros(props.multi_processor_count, dtype=torch.int32, device=DEV)

    def gemm(self, a: torch.Tensor, m: int, is_k_full: bool = True, extra_scratch: int = 0) -> torch.Tensor:
        lib = _lib.load()
        tdt = torch.float16 if self.dtype == "fp16" else torch.bfloat16
        c = torch.empty((m, self.n), dtype=tdt, device=DEV)
        nbytes = lib.sonar_marlin_gemm_scratch_bytes(m, self.n, self.k)
        scratch = torch.empty(max(nbytes, 16) + extra_scratch, dtype=torch.uint8, device=DEV)
        _lib.check(lib.sonar_marlin_gemm(
            ptr(a), a.stride(0) if m > 0 else self.k, ptr(c), ptr(self.native), _lib.LAYOUT_GFX950,
            ptr(self.bias), ptr(self.scales), ptr(self.zeros), ptr(self.g_idx), ptr(self.perm),
            ptr(self.workspace), self.workspace.numel(), ptr(scratch), scratch.numel(),
            dtype_code(self.dtype), self.b_type, m, self.n, self.k, self.groups, int(is_k_full), 0, 1,
            stream()))
        return c

    def dequant(self) -> torch.Tensor:
        lib = _lib.load()
        tdt = torch.float16 if self.dtype == "fp16" else torch.bfloat16
        w = torch.empty((self.k, self.n), dtype=tdt, device=DEV)
        _lib.check(lib.sonar_marlin_dequant(
            ptr(self.native), _lib.LAYOUT_GFX950, ptr(self.scales), ptr(self.zeros), None, ptr(w),
            dtype_code(self.dtype), self.b_type, self.n, self.k, self.groups, 1, stream()))
        return w
