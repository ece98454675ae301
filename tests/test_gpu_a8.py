"""W4A8 through the C ABI against the CPU oracle: the weight order for 8-bit
activations and the fp8 preprocess bit for bit, the int8 GEMM bit for bit
(integer sums, one rounding), the fp8 GEMM within the tolerance of the other
floating-point paths (1e-2 of max|ref|)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import marlin_oracle as mo
from sonar_amd import _lib
from tests.gpu_util import DEV, dev_bits16, dev_i32, host_f32, ptr, stream, dtype_code

pytestmark = pytest.mark.gpu


def _repack_a8(words, k, n, awq=False):
    lib = _lib.load()
    out = torch.empty((k // 16, 2 * n), dtype=torch.int32, device=DEV)
    fn = lib.sonar_awq_marlin_repack_a8 if awq else lib.sonar_gptq_marlin_repack_a8
    _lib.check(fn(ptr(words), ptr(out), k, n, 4, stream()))
    return out


def _a8_to_gfx950(marlin, k, n):
    out = torch.empty(k * n // 8, dtype=torch.int32, device=DEV)
    _lib.check(_lib.load().sonar_marlin_a8_to_gfx950(ptr(marlin), ptr(out), k, n, stream()))
    return out


# sizes of the reference's repack test: K = 128 * k_factor, N = 64 / 256 * n_factor
# (tests/kernels/quantization/test_marlin_gemm.py:58-66,196-247)
@pytest.mark.parametrize("k,n", [(128 * 8, 64 * 4), (128 * 5, 256 * 7), (128 * 11, 64 * 13), (32, 64)])
def test_repack_a8_bit_exact(k, n):
    rng = np.random.default_rng(k + n)
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    want = mo.marlin_pack_a8(q)
    got = _repack_a8(dev_i32(mo.gptq_pack(q)), k, n)
    assert np.array_equal(got.cpu().numpy(), want)
    got_awq = _repack_a8(dev_i32(mo.awq_pack(q)), k, n, awq=True)
    assert np.array_equal(got_awq.cpu().numpy(), want)
    native = _a8_to_gfx950(got, k, n)
    assert np.array_equal(native.cpu().numpy(), mo.gfx950_pack(q))
    back = torch.empty_like(got)
    _lib.check(_lib.load().sonar_gfx950_to_marlin_a8(ptr(native), ptr(back), k, n, stream()))
    assert torch.equal(back, got)


@pytest.mark.parametrize("k,n", [(128 * 5, 256 * 7), (32, 64)])
def test_repack8_a8_bit_exact(k, n):
    """8-bit codes in the order of 8-bit activations (produced for parity with the repack op; no GEMM
    takes it)."""
    rng = np.random.default_rng(k * 3 + n)
    q = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    out = torch.empty((k // 16, 4 * n), dtype=torch.int32, device=DEV)
    src = dev_i32(mo.pack_rows8(q))
    _lib.check(_lib.load().sonar_gptq_marlin_repack_a8(ptr(src), ptr(out), k, n, 8, stream()))
    assert np.array_equal(out.cpu().numpy(), mo.marlin_pack8_closed_form_a8(q))


def test_repack_a8_rejections():
    lib = _lib.load()
    w = torch.zeros(64 * 64 // 4, dtype=torch.int32, device=DEV)
    out = torch.zeros(64 * 64 // 4, dtype=torch.int32, device=DEV)
    assert lib.sonar_awq_marlin_repack_a8(ptr(w), ptr(out), 64, 64, 8, stream()) == _lib.E_UNSUPPORTED
    assert lib.sonar_gptq_marlin_repack_a8(ptr(w), ptr(out), 48, 64, 4, stream()) == _lib.E_INVALID
    assert b"32" in lib.sonar_marlin_last_error()
    assert lib.sonar_awq_marlin_repack_a8(ptr(w), ptr(out), 64, 32, 4, stream()) == _lib.E_INVALID


def test_int4_fp8_preprocess_bit_exact():
    lib = _lib.load()
    rng = np.random.default_rng(11)
    k, n, gs = 256, 128, 64
    q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    # without zero points: any packing (here the Marlin order for 8-bit activations)
    packed = mo.marlin_pack_a8(q)
    d = dev_i32(packed)
    out = torch.empty_like(d)
    _lib.check(lib.sonar_marlin_int4_fp8_preprocess(ptr(d), None, ptr(out), d.shape[0], d.shape[1], 0, stream()))
    assert np.array_equal(out.cpu().numpy(), mo.marlin_pack_a8(mo.int4_fp8_preprocess(q)))
    _lib.check(lib.sonar_marlin_int4_fp8_preprocess(ptr(d), None, ptr(d), d.shape[0], d.shape[1], 0, stream()))
    assert torch.equal(d, out)                      # in place
    # AWQ: qweight (K, N/8) and qzeros (K/group, N/8) in the checkpoint's packing
    z = rng.integers(0, 16, size=(k // gs, n), dtype=np.int32)
    dq, dz = dev_i32(mo.awq_pack(q)), dev_i32(mo.awq_pack(z))
    out = torch.empty_like(dq)
    _lib.check(lib.sonar_marlin_int4_fp8_preprocess(ptr(dq), ptr(dz), ptr(out), k, n // 8, gs, stream()))
    assert np.array_equal(out.cpu().numpy(), mo.awq_pack(mo.int4_fp8_preprocess(q, z, gs)))


class A8Layer:
    def __init__(self, seed, k, n, group_size, dtype, zero_points, act, bias=False):
        rng = np.random.default_rng(seed)
        self.k, self.n, self.dtype, self.act, self.group_size = k, n, dtype, act, group_size
        self.q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
        self.groups = 1 if group_size == -1 else k // group_size
        self.zeros = rng.integers(0, 16, size=(self.groups, n), dtype=np.int32) if zero_points else None
        s = mo.round_to_dtype(rng.uniform(1e-3, 1e-2, size=(self.groups, n)).astype(np.float32), dtype)
        self.factor = np.float32(1.0)
        if act == "int8" and self.groups > 1:
            ints, self.factor = mo.marlin_act_int8_process_scales(s)
            self.scales = ints
            dev_s = torch.from_numpy(mo.marlin_permute_scales_a8(ints, k, n, group_size).copy()).to(DEV)
        else:
            if act == "fp8":
                s = mo.round_to_dtype(s * np.float32(512.0), dtype)   # the factor of the fp8 weights
            self.scales = s
            dev_s = dev_bits16(mo.marlin_permute_scales_a8(s, k, n, group_size), dtype)
        self.dev_scales = dev_s
        codes = self.q
        if act == "fp8":
            codes = mo.int4_fp8_preprocess(self.q, self.zeros, k // self.groups)
        self.native = _a8_to_gfx950(_repack_a8(dev_i32(mo.gptq_pack(codes)), k, n), k, n)
        self.dev_zeros = dev_i32(mo.marlin_zero_points_a8(self.zeros, self.groups, n)) if zero_points else None
        self.bias32, self.dev_bias = None, None
        if bias:
            self.bias32 = mo.round_to_dtype(rng.standard_normal(n).astype(np.float32), dtype)
            self.dev_bias = dev_bits16(mo.marlin_permute_bias(self.bias32), dtype)
        self.b_type = _lib.TYPE_UINT4 if zero_points else _lib.TYPE_UINT4B8

    def gemm(self, a_dev, a_scales_dev, m):
        lib = _lib.load()
        tdt = torch.float16 if self.dtype == "fp16" else torch.bfloat16
        c = torch.full((m, self.n), float("nan"), dtype=tdt, device=DEV)
        nbytes = lib.sonar_marlin_gemm_a8_scratch_bytes(m, self.n, self.k, self.groups)
        scratch = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=DEV)
        _lib.check(lib.sonar_marlin_gemm_a8(
            ptr(a_dev), a_dev.stride(0) if m else self.k, _lib.ADTYPE_INT8 if self.act == "int8" else _lib.ADTYPE_FP8,
            ptr(c), ptr(self.native), _lib.LAYOUT_GFX950, ptr(self.dev_bias), ptr(self.dev_scales),
            ptr(a_scales_dev), ptr(self.dev_zeros), ptr(scratch), scratch.numel(), dtype_code(self.dtype),
            self.b_type, m, self.n, self.k, self.groups, stream()))
        return c


INT8_CASES = [
    # k, n, group, zp, dtype, bias, M list
    (256, 128, -1, False, "fp16", False, [1, 16, 33]),
    (256, 128, 32, False, "bf16", True, [7, 64]),
    (1024, 256, 64, False, "fp16", False, [1, 100]),
    (1024, 256, 128, False, "bf16", False, [5, 257]),
    (512, 192, -1, True, "bf16", True, [3, 48]),
    (512, 192, 32, True, "fp16", False, [17, 65]),
    (1024, 64, 64, True, "bf16", False, [2]),
    (8192, 64, 128, False, "fp16", True, [1, 20]),     # K split over workgroups
    (4096, 128, -1, False, "bf16", False, [9]),         # channelwise, a long K in one range
    (1056, 128, -1, False, "fp16", False, [4]),         # K a multiple of 32 only
    # the tiled kernel (more than 64 rows, N a multiple of 128, K of 128, groups of 64 rows or more)
    (1024, 256, -1, False, "fp16", True, [65, 200]),
    (1024, 256, 64, False, "bf16", False, [128, 300]),
    (512, 384, 128, False, "fp16", True, [129]),
    (1024, 128, -1, True, "bf16", False, [100]),
    (512, 256, 64, True, "fp16", True, [257]),
    (1024, 256, 128, True, "fp16", False, [96]),
    (8192, 128, 128, False, "fp16", False, [128]),      # K split over workgroups
    (8192, 128, -1, False, "bf16", True, [70]),
    (1024, 256, 32, False, "fp16", False, [100]),       # groups of 32: the slab kernel
    # 33..48 rows on a matrix the tiled kernel does not take (N = 192): three blocks of 16 rows
    (512, 192, -1, False, "fp16", False, [40]),
    (512, 192, 64, False, "fp16", True, [40]),
    (512, 192, -1, True, "fp16", False, [40]),
    (512, 192, 32, True, "fp16", True, [40]),
    (8192, 128, -1, False, "fp16", True, [9]),          # channelwise, K split
]


@pytest.mark.parametrize("k,n,group,zp,dtype,bias,ms", INT8_CASES)
def test_w4a8_int8_gemm_bit_exact(k, n, group, zp, dtype, bias, ms):
    layer = A8Layer(100 + k + n + group, k, n, group, dtype, zp, "int8", bias)
    for m in ms:
        rng = np.random.default_rng(m)
        x = rng.standard_normal((m, k)).astype(np.float32)
        a_q, a_s = mo.per_token_quant_int8(x)
        a_s = (a_s * layer.factor).astype(np.float32)
        got = layer.gemm(torch.from_numpy(a_q).to(DEV), torch.from_numpy(a_s.reshape(-1)).to(DEV), m)
        want = mo.gemm_w4a8_int8(a_q, a_s, layer.q, group, layer.scales, dtype, layer.zeros, layer.bias32)
        assert np.array_equal(host_f32(got), want), (m, np.abs(host_f32(got) - want).max())


FP8_CASES = [
    (256, 128, -1, False, "fp16", False, [1, 16]),
    (512, 128, 32, False, "bf16", True, [7, 64]),
    (1024, 256, 64, False, "fp16", False, [33]),
    (1024, 256, 128, False, "bf16", False, [100]),
    (512, 192, 64, True, "fp16", False, [5, 40]),
    (512, 64, -1, True, "bf16", True, [2]),
    (8192, 64, 128, False, "bf16", False, [3]),
    # the tiled kernel
    (1024, 256, -1, False, "fp16", True, [65, 200]),
    (1024, 256, 128, False, "bf16", False, [128, 300]),
    (1024, 256, 64, False, "fp16", False, [100]),
    (512, 384, 128, True, "fp16", True, [129]),
    (1024, 128, -1, True, "bf16", False, [100]),
    (512, 256, 64, True, "bf16", False, [257]),
    (8192, 128, 128, False, "fp16", False, [128]),
    # 33..48 rows on a matrix the tiled kernel does not take (N = 192): three blocks of 16 rows
    (512, 192, -1, False, "fp16", False, [40]),
    (512, 192, 64, False, "fp16", True, [40]),
    (512, 192, -1, True, "fp16", False, [40]),
    # channelwise, K split over workgroups
    (8192, 128, -1, False, "fp16", True, [9]),
    (8192, 128, -1, False, "bf16", False, [9]),
]


@pytest.mark.parametrize("k,n,group,zp,dtype,bias,ms", FP8_CASES)
def test_w4a8_fp8_gemm_within_tolerance(k, n, group, zp, dtype, bias, ms):
    layer = A8Layer(200 + k + n + group, k, n, group, dtype, zp, "fp8", bias)
    for m in ms:
        g = torch.Generator().manual_seed(m)
        x = torch.randn((m, k), generator=g)
        a_s = (x.abs().amax(dim=1, keepdim=True) / 448.0).clamp_min(1e-10)
        a_fp8 = (x / a_s).to(torch.float8_e4m3fn)
        got = layer.gemm(a_fp8.view(torch.uint8).to(DEV), a_s.reshape(-1).to(DEV), m)
        # the scales as the kernel holds them (times 512), the weights as (q - z) * 2^-9
        want = mo.gemm_w4a8_fp8(a_fp8.float().numpy(), a_s.numpy(), layer.q, group,
                                layer.scales / np.float32(512.0), layer.zeros, layer.bias32)
        ok, max_err, max_ref = mo.gemm_tolerance_ok(host_f32(got), want)
        assert ok, (m, max_err, max_ref)


FP4_CASES = [
    # k, n, dtype, bias, M list   (bfloat16 outputs only: generate_kernels.py:152-161)
    (256, 128, "bf16", False, [1, 16]),
    (512, 192, "bf16", True, [7, 20, 33]),
    (1024, 256, "bf16", True, [64, 100]),
    (8192, 64, "bf16", False, [3]),
    (1024, 256, "bf16", False, [257]),
]


@pytest.mark.parametrize("k,n,dtype,bias,ms", FP4_CASES)
def test_w4a8_fp4_gemm_within_tolerance(k, n, dtype, bias, ms):
    """MXFP4 weights (float4_e2m1f codes, an exponent byte per column and 32 rows) with
    float8_e4m3fn activations."""
    lib = _lib.load()
    rng = np.random.default_rng(k + n)
    codes = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    e8 = rng.integers(110, 125, size=(k // 32, n)).astype(np.uint8)
    native = _a8_to_gfx950(_repack_a8(dev_i32(mo.gptq_pack(codes)), k, n), k, n)
    dev_s = torch.from_numpy(mo.mxfp4_process_scales_a8(mo.marlin_permute_scales_a8(e8, k, n, 32))).to(DEV)
    bias32 = dev_bias = None
    if bias:
        bias32 = mo.round_to_dtype((rng.standard_normal(n) * 1e-3).astype(np.float32), dtype)
        dev_bias = dev_bits16(mo.marlin_permute_bias(bias32), dtype)
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    for m in ms:
        g = torch.Generator().manual_seed(m)
        x = torch.randn((m, k), generator=g)
        a_s = (x.abs().amax(dim=1, keepdim=True) / 448.0).clamp_min(1e-10)
        a_fp8 = (x / a_s).to(torch.float8_e4m3fn)
        a_dev, s_dev = a_fp8.view(torch.uint8).to(DEV), a_s.reshape(-1).to(DEV)
        c = torch.full((m, n), float("nan"), dtype=tdt, device=DEV)
        nbytes = lib.sonar_marlin_gemm_a8_scratch_bytes(m, n, k, k // 32)
        scratch = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=DEV)
        _lib.check(lib.sonar_marlin_gemm_a8(
            ptr(a_dev), k, _lib.ADTYPE_FP8, ptr(c), ptr(native), _lib.LAYOUT_GFX950, ptr(dev_bias), ptr(dev_s),
            ptr(s_dev), None, ptr(scratch), scratch.numel(), dtype_code(dtype), _lib.TYPE_FLOAT4_E2M1F, m, n, k,
            k // 32, stream()))
        want = mo.gemm_w4a8_fp4(a_fp8.float().numpy(), a_s.numpy(), codes, e8, bias32)
        ok, max_err, max_ref = mo.gemm_tolerance_ok(host_f32(c), want)
        assert ok, (m, max_err, max_ref)
    # int8 activations, zero points and groups other than 32 rows are refused
    a = torch.zeros((4, k), dtype=torch.int8, device=DEV)
    c = torch.empty((4, n), dtype=tdt, device=DEV)

    def call(adt=_lib.ADTYPE_FP8, zeros=None, groups=k // 32, out=dtype_code(dtype)):
        return lib.sonar_marlin_gemm_a8(ptr(a), k, adt, ptr(c), ptr(native), _lib.LAYOUT_GFX950, None, ptr(dev_s),
                                        ptr(s_dev), ptr(zeros), None, 0, out, _lib.TYPE_FLOAT4_E2M1F,
                                        4, n, k, groups, stream())

    assert call(adt=_lib.ADTYPE_INT8) == _lib.E_UNSUPPORTED
    assert call(zeros=dev_s) == _lib.E_INVALID
    assert call(groups=k // 64) == _lib.E_INVALID
    assert call(out=_lib.DTYPE_F16) == _lib.E_UNSUPPORTED      # no float16 outputs


def test_w4a8_rejections():
    lib = _lib.load()
    layer = A8Layer(1, 256, 64, 64, "fp16", False, "int8")
    a = torch.zeros((4, 256), dtype=torch.int8, device=DEV)
    s = torch.ones(4, device=DEV)
    c = torch.empty((4, 64), dtype=torch.float16, device=DEV)

    def call(**kw):
        args = dict(a=a, stride=256, adt=_lib.ADTYPE_INT8, b_type=_lib.TYPE_UINT4B8, zeros=None, groups=4, k=256)
        args.update(kw)
        return lib.sonar_marlin_gemm_a8(ptr(args["a"]), args["stride"], args["adt"], ptr(c), ptr(layer.native),
                                        _lib.LAYOUT_GFX950, None, ptr(layer.dev_scales), ptr(s), ptr(args["zeros"]),
                                        None, 0, _lib.DTYPE_F16, args["b_type"], 4, 64, args["k"], args["groups"],
                                        stream())

    assert call() == _lib.OK
    assert call(b_type=_lib.TYPE_UINT8B128) == _lib.E_UNSUPPORTED      # W8A8 is not a Marlin mode
    assert call(adt=7) == _lib.E_INVALID
    assert call(groups=16) == _lib.E_INVALID                           # group size 16
    assert call(b_type=_lib.TYPE_UINT4) == _lib.E_INVALID              # zero points missing
    assert call(stride=260) == _lib.E_INVALID
    assert call(a=None) == _lib.E_INVALID


# ---------------------------------------------------------------- grouped (mixture of experts)
MOE_A8_CASES = [
    # m, k, n, experts, top_k, block, group, zp, dtype, bias, mul_topk
    (1, 256, 128, 4, 2, 16, 64, False, "fp16", False, False),
    (33, 512, 192, 5, 2, 16, 128, False, "bf16", True, True),
    (70, 256, 128, 3, 3, 32, -1, False, "fp16", False, True),
    (19, 512, 64, 6, 2, 8, 32, True, "bf16", False, False),
    (100, 1024, 128, 4, 1, 64, 128, True, "fp16", True, False),
    (47, 256, 256, 7, 4, 48, 64, False, "bf16", False, True),
    # blocks of more than 32 slots, N a multiple of 256: the tiled kernel's grouped form
    (300, 1024, 512, 4, 2, 64, 128, False, "fp16", True, True),
    (150, 512, 256, 3, 2, 64, -1, False, "bf16", False, False),
    (90, 512, 256, 5, 3, 48, 64, True, "fp16", False, True),
    (200, 256, 512, 6, 1, 64, 128, True, "bf16", True, False),
    (200, 512, 256, 4, 2, 64, -1, True, "bf16", False, True),      # ... channelwise with zero points
    (200, 512, 256, 4, 2, 64, 64, True, "bf16", True, False),      # ... groups of 64 rows
    (200, 512, 256, 4, 2, 64, 128, False, "bf16", False, True),    # ... groups of 128 rows
] + [
    # one scale per column on a matrix the tiled kernel does not take (N = 128): the general grouped kernel
    # with one to four blocks of 16 rows, either output type, with and without zero points
    (2 * block, 256, 128, 3, 2, block, -1, zp, dtype, block == 32, block != 48)
    for dtype in ("fp16", "bf16") for block in (16, 32, 48, 64) for zp in (False, True)
]


@pytest.mark.parametrize("m,k,n,e,top_k,block,group,zp,dtype,bias,mul_topk", MOE_A8_CASES)
@pytest.mark.parametrize("act", ["int8", "fp8"])
def test_moe_w4a8_gemm(act, m, k, n, e, top_k, block, group, zp, dtype, bias, mul_topk):
    """The grouped entry point: int8 bit for bit against the oracle, fp8 within tolerance.  One
    expert id is set to -1 (held elsewhere): its rows must stay untouched."""
    lib = _lib.load()
    rng = np.random.default_rng(m * 7 + k + e)
    layers = [A8Layer(300 + i + k + n, k, n, group, dtype, zp, act, bias) for i in range(e)]
    # the integer group scales of all experts share one factor (the layer-wide maximum) in the
    # reference; the per-expert factors of these test layers go into per-row scales instead
    topk_ids = np.stack([rng.permutation(e)[:top_k] for _ in range(m)]).astype(np.int32)
    sorted_ids, expert_ids, post_pad = mo.moe_align_block_size(topk_ids, block, e)
    post_pad = int(post_pad[0])
    expert_ids = expert_ids.copy()
    skipped = int(expert_ids[0])
    expert_ids[expert_ids == skipped] = -1 if e > 1 and m > 1 else skipped
    topk_w = rng.uniform(0.1, 1.0, size=(m, top_k)).astype(np.float32)
    x = rng.standard_normal((m, k)).astype(np.float32)
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    if act == "int8":
        a_q, a_s = mo.per_token_quant_int8(x)
        a_s = (a_s * layers[0].factor).astype(np.float32)      # one factor: the experts below share scales' scale
        a_dev = torch.from_numpy(a_q).to(DEV)
    else:
        xt = torch.from_numpy(x)
        a_s_t = (xt.abs().amax(dim=1, keepdim=True) / 448.0).clamp_min(1e-10)
        a_fp8 = (xt / a_s_t).to(torch.float8_e4m3fn)
        a_s = a_s_t.numpy()
        a_dev = a_fp8.view(torch.uint8).to(DEV)
    w_all = torch.stack([l.native for l in layers]).contiguous()
    s_all = torch.stack([l.dev_scales for l in layers]).contiguous()
    z_all = torch.stack([l.dev_zeros for l in layers]).contiguous() if zp else None
    b_all = torch.stack([l.dev_bias for l in layers]).contiguous() if bias else None
    c = torch.full((m * top_k, n), 7.0, dtype=tdt, device=DEV)
    # device copies held in names: a temporary would hand its memory to the next allocation
    d_as = torch.from_numpy(a_s.reshape(-1).copy()).to(DEV)
    d_sorted, d_experts = dev_i32(sorted_ids), dev_i32(expert_ids)
    d_past = dev_i32(np.array([post_pad], dtype=np.int32))
    d_tw = torch.from_numpy(topk_w.reshape(-1).copy()).to(DEV)
    _lib.check(lib.sonar_moe_wna16_marlin_gemm_a8(
        ptr(a_dev), _lib.ADTYPE_INT8 if act == "int8" else _lib.ADTYPE_FP8, ptr(c), ptr(w_all), _lib.LAYOUT_GFX950,
        ptr(b_all), ptr(s_all), ptr(d_as), ptr(z_all), ptr(d_sorted), sorted_ids.size, ptr(d_experts), ptr(d_past),
        ptr(d_tw), block, top_k, int(mul_topk), e, dtype_code(dtype), layers[0].b_type, m, n, k, layers[0].groups,
        stream()))
    torch.cuda.synchronize()
    got = host_f32(c)
    written = np.zeros(m * top_k, dtype=bool)
    for b in range(post_pad // block):
        if expert_ids[b] >= 0:
            ids = sorted_ids[b * block:(b + 1) * block]
            written[ids[ids < m * top_k]] = True
    assert np.all(got[~written] == 7.0)
    if act == "int8":
        experts = [dict(q=l.q, group_size=group, scales=l.scales, zeros=l.zeros, bias32=l.bias32) for l in layers]
        want = mo.moe_gemm_w4a8_int8(a_q, a_s, experts, sorted_ids, expert_ids, post_pad, block, top_k,
                                     topk_w if mul_topk else None, dtype)
        assert np.array_equal(got[written], want[written]), np.abs(got[written] - want[written]).max()
    else:
        want = np.zeros_like(got)
        for b in range(post_pad // block):
            ex = int(expert_ids[b])
            if ex < 0:
                continue
            ids = sorted_ids[b * block:(b + 1) * block]
            ids = ids[ids < m * top_k]
            l = layers[ex]
            r = mo.gemm_w4a8_fp8(a_fp8.float().numpy()[ids // top_k], a_s.reshape(-1)[ids // top_k], l.q, group,
                                 l.scales / np.float32(512.0), l.zeros, l.bias32)
            if mul_topk:
                r = r * topk_w.reshape(-1)[ids][:, None]
            want[ids] = r
        ok, max_err, max_ref = mo.gemm_tolerance_ok(got[written], want[written])
        assert ok, (max_err, max_ref)
