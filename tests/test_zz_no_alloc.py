"""GPU: sonar_marlin_gemm_noalloc (static device scratch, no allocation) against
sonar_marlin_gemm (caller's scratch) on the same inputs, through the C ABI.
The kernels are deterministic, so the two outputs must agree bit for bit wherever
both take the same launches; a call whose partial tiles do not fit the static array
runs without them (another order of summation) and is held to the GEMM tolerance."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import marlin_oracle as mo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gu():
    from tests import gpu_util
    return gpu_util


def _noalloc(gu, layer, a, m, is_k_full=True):
    from sonar_amd import _lib
    lib = _lib.load()
    tdt = torch.float16 if layer.dtype == "fp16" else torch.bfloat16
    c = torch.full((m, layer.n), float("nan"), dtype=tdt, device=gu.DEV)
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]      # the driver's own count: sees a hipMalloc too
    rc = lib.sonar_marlin_gemm_noalloc(
        gu.ptr(a), a.stride(0), gu.ptr(c), gu.ptr(layer.native), _lib.LAYOUT_GFX950, gu.ptr(layer.bias),
        gu.ptr(layer.scales), gu.ptr(layer.zeros), gu.ptr(layer.g_idx), gu.ptr(layer.perm),
        gu.ptr(layer.workspace), layer.workspace.numel(), gu.dtype_code(layer.dtype), layer.b_type, m, layer.n,
        layer.k, layer.groups, int(is_k_full), 0, 1, gu.stream())
    _lib.check(rc)
    assert torch.cuda.memory_allocated() == before
    if getattr(_noalloc, "address_known", False):   # (the first call on a device may load the code object)
        assert torch.cuda.mem_get_info()[0] == free_before
    _noalloc.address_known = True
    return c


# (m, k, n, group, dtype, zero_points, act_order): the first of every pair leaves fp32 partial
# tiles in the scratch array (K split over workgroups), the second is smaller and runs right after
PAIRS = [
    ((16, 4096, 4096, 128, "bf16", False, False), (3, 2048, 1024, 128, "bf16", False, False)),
    ((64, 14336, 4096, 128, "fp16", False, False), (16, 1024, 512, 128, "fp16", True, False)),
    ((512, 4096, 1024, 128, "fp16", False, False), (200, 2048, 512, 64, "fp16", False, False)),
    ((33, 2048, 1024, 128, "bf16", False, True), (5, 1024, 256, 128, "bf16", False, True)),
]


# Calls whose sonar_marlin_gemm_scratch_bytes() exceeds the static array (56 MiB of partial tiles
# each): they run, without the K split
MAKE_DO_PAIRS = [
    ((128, 14336, 4096, 128, "fp16", False, False), (96, 4096, 1024, 128, "fp16", False, False)),
    ((128, 4096, 28672, 128, "bf16", False, False), (16, 1024, 512, 128, "bf16", False, False)),
]


@pytest.mark.parametrize("first,second", MAKE_DO_PAIRS)
def test_noalloc_makes_do_when_the_partial_tiles_do_not_fit(gu, first, second):
    from sonar_amd import _lib
    lib = _lib.load()
    m, k, n = first[:3]
    assert lib.sonar_marlin_gemm_scratch_bytes(m, n, k) > 24 << 20
    for seed, (m, k, n, g, dtype, zp, act) in enumerate((first, second)):
        layer = gu.DeviceLayer(300 + seed, k, n, g, dtype, zero_points=zp, act_order=act)
        a32 = mo.make_activations(seed + 9, m, k, dtype)
        a = gu.dev_bits16(a32, dtype)
        want = layer.gemm(a, m)
        out = _noalloc(gu, layer, a, m)
        torch.cuda.synchronize()
        ref = mo.gemm_reference(a32, layer.w_ref)
        for c in (out, want):
            ok, err, big = mo.gemm_tolerance_ok(gu.host_f32(c), ref)
            assert ok, (err, big)
        if seed == 1:   # the second call fits and takes the same launches as sonar_marlin_gemm
            assert torch.equal(out.view(torch.int16), want.view(torch.int16))
        assert int(layer.workspace.abs().sum().item()) == 0


@pytest.mark.parametrize("first,second", PAIRS)
def test_noalloc_matches_gemm_on_two_calls_in_a_row(gu, first, second):
    outs = []
    wants = []
    layers = []
    for seed, (m, k, n, g, dtype, zp, act) in enumerate((first, second)):
        layer = gu.DeviceLayer(100 + seed, k, n, g, dtype, zero_points=zp, act_order=act)
        a32 = mo.make_activations(seed + 5, m, k, dtype)
        a = gu.dev_bits16(a32, dtype)
        extra = m * k * 2 if act else 0
        wants.append(layer.gemm(a, m, extra_scratch=extra))
        layers.append((layer, a, m, a32))
    torch.cuda.synchronize()
    # the two calls in a row, nothing in between
    for layer, a, m, _ in layers:
        outs.append(_noalloc(gu, layer, a, m))
    torch.cuda.synchronize()
    for out, want, (layer, a, m, a32) in zip(outs, wants, layers):
        assert torch.equal(out.view(torch.int16), want.view(torch.int16))
        ok, err, ref = mo.gemm_tolerance_ok(gu.host_f32(out), mo.gemm_reference(a32, layer.w_ref))
        assert ok, (err, ref)
        assert int(layer.workspace.abs().sum().item()) == 0


def test_noalloc_rejects_what_does_not_fit(gu):
    """Act-order on a shard without whole groups needs the column-permuted copy of A: 32 MiB here,
    more than the static array holds."""
    from sonar_amd import _lib
    lib = _lib.load()
    m, k, n = 4096, 4096, 1024
    dummy = torch.zeros(64, dtype=torch.int32, device=gu.DEV)
    ws = torch.zeros(1024, dtype=torch.int32, device=gu.DEV)
    rc = lib.sonar_marlin_gemm_noalloc(
        gu.ptr(dummy), k, gu.ptr(dummy), gu.ptr(dummy), _lib.LAYOUT_GFX950, None, gu.ptr(dummy), None, gu.ptr(dummy),
        gu.ptr(dummy), gu.ptr(ws), ws.numel(), _lib.DTYPE_F16, _lib.TYPE_UINT4B8, m, n, k, k // 128, 0, 0, 1,
        gu.stream())
    assert rc == _lib.E_INVALID
    assert b"more scratch bytes" in lib.sonar_marlin_last_error()
