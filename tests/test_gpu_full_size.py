"""GPU parity at the full sizes of the benchmark configurations, through the C ABI.

The matrices are too large for the oracle to dequantise whole in seconds, so the
weights are drawn on the device (GPTQ words, repacked by the library) and the
oracle is applied to sampled output columns only: the GPTQ words of those columns
are unpacked and dequantised on the CPU (oracle.unpack_rows / oracle.dequantize)
and multiplied with the activations in fp32.  Every real launch shape of the
decode sweep (M = 1 .. 64 on the four Llama-3-8B projections), of the prefill
sweep (M = 256, 1024, 4096, 8192 on the same four), of the Mixtral-sized grouped
GEMMs at 16 and 4096 tokens and of the W4A8 shapes the benchmark times (K = 4096,
N = 11008 dense; Mixtral-sized experts grouped) meets the oracle this way.
Tolerance: max|err| <= 1e-2 max|ref| and |err| <= 1e-2 max|ref| + 1e-2 |ref|
(oracle.gemm_tolerance_ok); int8 activations: bit for bit."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import marlin_oracle as mo
from sonar_amd import _lib
from tests import gpu_util as gu

pytestmark = pytest.mark.gpu

GROUP = 128
LLAMA = {"qkv": (4096, 6144), "o": (4096, 4096), "gate_up": (4096, 28672), "down": (14336, 4096)}


class BigLayer:
    """uint4b8 weights drawn on the device, prepared like the reference's callers do."""

    def __init__(self, seed, k, n, dtype):
        from sonar_amd import marlin_utils
        self.k, self.n, self.dtype = k, n, dtype
        self.tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
        gen = torch.Generator(device=gu.DEV).manual_seed(seed)
        self.qweight = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 8, n), dtype=torch.int32, device=gu.DEV,
                                     generator=gen)
        self.native = gu.to_gfx950(gu.gptq_repack(self.qweight, None, k, n), k, n)
        self.scales_plain = (torch.rand((k // GROUP, n), device=gu.DEV, generator=gen) * 9e-3 + 1e-3).to(self.tdt)
        self.scales = marlin_utils.marlin_permute_scales(self.scales_plain, k, n, GROUP).contiguous()
        props = torch.cuda.get_device_properties(0)
        self.workspace = torch.zeros(props.multi_processor_count, dtype=torch.int32, device=gu.DEV)

    def w_ref_columns(self, cols):
        """The oracle's dequantised values of the given columns, (K, len(cols)) fp32."""
        idx = torch.as_tensor(cols, device=gu.DEV)
        words = self.qweight[:, idx].cpu().numpy()
        q = mo.unpack_rows(words)
        s32 = self.scales_plain[:, idx].float().cpu().numpy()
        return mo.dequantize(q, s32, GROUP, self.dtype)

    def gemm(self, a, m):
        lib = _lib.load()
        c = torch.full((m, self.n), float("nan"), dtype=self.tdt, device=gu.DEV)
        nbytes = lib.sonar_marlin_gemm_scratch_bytes(m, self.n, self.k)
        scratch = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=gu.DEV)
        _lib.check(lib.sonar_marlin_gemm(
            gu.ptr(a), a.stride(0), gu.ptr(c), gu.ptr(self.native), _lib.LAYOUT_GFX950, None, gu.ptr(self.scales),
            None, None, None, gu.ptr(self.workspace), self.workspace.numel(), gu.ptr(scratch), scratch.numel(),
            gu.dtype_code(self.dtype), _lib.TYPE_UINT4B8, m, self.n, self.k, self.k // GROUP, 1, 0, 1, gu.stream()))
        return c


_layers = {}


def big_layer(name, dtype):
    key = (name, dtype)
    if key not in _layers:
        if len(_layers) >= 3:   # keep device memory bounded
            _layers.pop(next(iter(_layers)))
        k, n = LLAMA[name]
        _layers[key] = BigLayer(sum(map(ord, name + dtype)), k, n, dtype)
    return _layers[key]


def sampled_columns(n, count, seed):
    rng = np.random.default_rng(seed)
    cols = set(int(x) for x in rng.integers(0, n, count))
    cols.update((0, n - 1, 63, 64 if n > 64 else 0))   # strip edges
    return sorted(cols)


def check_columns(layer, a, c, m, cols, rows=None):
    a32 = a.float().cpu().numpy()
    w = layer.w_ref_columns(cols)
    ref = a32 @ w
    got = c[:, torch.as_tensor(cols, device=gu.DEV)].float().cpu().numpy()
    ok, err, big = mo.gemm_tolerance_ok(got, ref)
    assert ok, (err, big)


@pytest.mark.parametrize("m", [1, 2, 4, 8, 16, 32, 48, 64])
@pytest.mark.parametrize("name", list(LLAMA))
def test_decode_sweep_meets_the_oracle_on_sampled_columns(name, m):
    """Benchmark configuration 2: bf16, every M of the sweep on every projection shape."""
    layer = big_layer(name, "bf16")
    gen = torch.Generator(device=gu.DEV).manual_seed(m)
    a = torch.randn((m, layer.k), device=gu.DEV, generator=gen).to(torch.bfloat16)
    c = layer.gemm(a, m)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(c.float()).all())
    assert int(layer.workspace.abs().sum().item()) == 0
    check_columns(layer, a, c, m, sampled_columns(layer.n, 8, m))
    c2 = layer.gemm(a, m)   # fixed order of summation: the same bits again
    assert torch.equal(c.view(torch.int16), c2.view(torch.int16))


@pytest.mark.parametrize("m", [256, 1024, 4096, 8192])
@pytest.mark.parametrize("name", list(LLAMA))
def test_prefill_sweep_meets_the_oracle_on_sampled_columns(name, m):
    """Benchmark configuration 3: fp16 activations ~ N(0, 0.5), every M of the sweep on every
    projection shape (the launches the benchmark's MFMA figure is made of among them)."""
    layer = big_layer(name, "fp16")
    gen = torch.Generator(device=gu.DEV).manual_seed(m)
    a = (torch.randn((m, layer.k), device=gu.DEV, generator=gen) * 0.5).to(torch.float16)
    c = layer.gemm(a, m)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(c.float()).all())
    check_columns(layer, a, c, m, sampled_columns(layer.n, 6, m))


@pytest.mark.parametrize("name,m,dtype", [
    ("o", 16, "bf16"),        # decode kernel, four pieces per strip summed through tickets in the workspace
    ("down", 16, "bf16"),     # ... with non-temporal weight copies
    ("gate_up", 48, "bf16"),  # ... blocks of rows, more workgroups than compute units
    ("o", 256, "fp16"),       # tile kernel, 128-row tiles cut along K, partial tiles summed by a second kernel
    ("qkv", 4096, "fp16"),    # tile kernel, two launches (256-row tiles, then the short last round as 128-row tiles)
])
def test_gemm_replayed_from_a_hip_graph_gives_the_eager_bits(name, m, dtype):
    """The launches of one call captured into a HIP graph and replayed three times, with an eager
    call of another size on the same workspace between the replays: every replay gives the bits of
    the eager call and leaves the workspace zero (nothing in the library's launches depends on
    state the host set up for one launch only)."""
    layer = big_layer(name, dtype)
    gen = torch.Generator(device=gu.DEV).manual_seed(m + 7)
    a = (torch.randn((m, layer.k), device=gu.DEV, generator=gen) * 0.5).to(layer.tdt)
    want = layer.gemm(a, m)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            got = layer.gemm(a, m)
        for _ in range(3):
            other_m = max(1, m // 2 - 1)
            other = layer.gemm(a[:other_m], other_m)      # eager work between the replays
            graph.replay()
            stream.synchronize()
            assert torch.equal(got.view(torch.int16), want.view(torch.int16))
            assert bool(torch.isfinite(other.float()).all())
            assert int(layer.workspace.abs().sum().item()) == 0
            got.zero_()
    torch.cuda.synchronize()


@pytest.mark.parametrize("m", [16, 300])
def test_calls_on_two_streams_with_their_own_workspace_do_not_interfere(m):
    """Two matrices, each with its own workspace and scratch, called ten times side by side on
    two streams: every call gives the bits of the call made alone (the library keeps no device
    state of its own between or across calls; tickets and partial tiles live in the caller's
    buffers)."""
    one, two = big_layer("o", "bf16"), big_layer("down", "bf16")
    gen = torch.Generator(device=gu.DEV).manual_seed(m)
    a1 = torch.randn((m, one.k), device=gu.DEV, generator=gen).to(torch.bfloat16)
    a2 = torch.randn((m, two.k), device=gu.DEV, generator=gen).to(torch.bfloat16)
    want1, want2 = one.gemm(a1, m), two.gemm(a2, m)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs = []
    for _ in range(10):
        with torch.cuda.stream(s1):
            c1 = one.gemm(a1, m)
        with torch.cuda.stream(s2):
            c2 = two.gemm(a2, m)
        outs.append((c1, c2))
    torch.cuda.synchronize()
    for c1, c2 in outs:
        assert torch.equal(c1.view(torch.int16), want1.view(torch.int16))
        assert torch.equal(c2.view(torch.int16), want2.view(torch.int16))
    assert int(one.workspace.abs().sum().item()) == 0 and int(two.workspace.abs().sum().item()) == 0


_experts = {}


def mixtral_experts(k, n):
    """Eight experts of one Mixtral-sized matrix, kept for the cases that share them."""
    if (k, n) not in _experts:
        _experts.clear()                      # one set at a time: 0.5 GB of device memory each
        _layers.clear()
        _experts[(k, n)] = [BigLayer(50 + i, k, n, "bf16") for i in range(8)]
    return _experts[(k, n)]


def test_prefill_short_last_round_with_split_k_meets_the_oracle():
    """M = 3900 on the qkv shape: 384 tiles of 256 rows whose last round is 128 tiles, the last row
    of tiles less than half full: that round's tiles are cut along K and summed by
    tile_reduce_kernel (at M = 4096 the round runs as 128-row tiles instead)."""
    layer = big_layer("qkv", "fp16")
    m = 3900
    gen = torch.Generator(device=gu.DEV).manual_seed(m)
    a = (torch.randn((m, layer.k), device=gu.DEV, generator=gen) * 0.5).to(torch.float16)
    c = layer.gemm(a, m)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(c.float()).all())
    check_columns(layer, a, c, m, sampled_columns(layer.n, 6, m))


@pytest.mark.parametrize("tokens", [16, 4096])
@pytest.mark.parametrize("k,n,top_k,mul", [(4096, 28672, 2, False), (14336, 4096, 1, True)])
def test_mixtral_sized_grouped_gemm(k, n, top_k, mul, tokens):
    """Benchmark configuration 5 at T = 16 and T = 4096 on the real expert shapes (w13: K = 4096,
    N = 28672 with top-2 routing; w2: K = 14336, N = 4096 on the routed rows with the routing
    weights multiplied in): 8-slot blocks in the grouped decode kernel, 64-slot blocks in the
    tiled grouped kernel.  Every routed row is checked on sampled columns against the oracle,
    and sampled rows against the dense GEMM of that row with its expert."""
    from sonar_amd import fused_moe, marlin_utils
    e = 8
    experts = mixtral_experts(k, n)
    native = torch.stack([x.native for x in experts]).contiguous()
    scales = torch.stack([x.scales for x in experts]).contiguous()
    gen = torch.Generator(device=gu.DEV).manual_seed(9)
    logits = torch.randn((tokens, e), device=gu.DEV, generator=gen)
    tw2, ti2 = torch.topk(torch.softmax(logits, dim=1), 2, dim=1)
    ti2 = ti2.to(torch.int32)
    bs = fused_moe.moe_block_size(tokens, 2, e)
    assert bs == (64 if tokens == 4096 else 8)
    sorted_ids, expert_ids, past = fused_moe.moe_align_block_size(ti2, bs, e)
    rows_a = tokens if top_k == 2 else tokens * 2     # the second GEMM of a layer takes one row per routed slot
    a = (torch.randn((rows_a, k), device=gu.DEV, generator=gen) * 0.5).to(torch.bfloat16)
    c = torch.full((tokens * 2, n), float("nan"), dtype=torch.bfloat16, device=gu.DEV)
    lib = _lib.load()
    ws = torch.zeros(1024, dtype=torch.int32, device=gu.DEV)
    nbytes = lib.sonar_moe_marlin_gemm_scratch_bytes(sorted_ids.numel(), bs, n, k)
    scr = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=gu.DEV)
    tw = tw2.reshape(-1).contiguous().float()
    _lib.check(lib.sonar_moe_wna16_marlin_gemm(
        gu.ptr(a), gu.ptr(c), gu.ptr(native), _lib.LAYOUT_GFX950, None, gu.ptr(scales), None, None, None,
        gu.ptr(ws), ws.numel(), gu.ptr(scr), nbytes, gu.ptr(sorted_ids), sorted_ids.numel(), gu.ptr(expert_ids),
        gu.ptr(past), gu.ptr(tw), bs, top_k, int(mul), e, _lib.DTYPE_BF16, _lib.TYPE_UINT4B8, rows_a, n, k,
        k // GROUP, 1, 0, 1, gu.stream()))
    torch.cuda.synchronize()
    assert bool(torch.isfinite(c.float()).all()), "a routed row was not written"
    assert int(ws.abs().sum().item()) == 0

    # every routed row on sampled columns against the oracle
    cols = sampled_columns(n, 6, k)
    idx = torch.as_tensor(cols, device=gu.DEV)
    ids = ti2.reshape(-1).cpu().numpy()                 # expert of routed row r = token * 2 + j
    a32 = a.float().cpu().numpy()
    got = c[:, idx].float().cpu().numpy()
    want = np.zeros_like(got)
    wt = mo.round_to_dtype(tw.cpu().numpy(), "bf16")
    for ex in range(e):
        rows = np.nonzero(ids == ex)[0]
        src = rows // 2 if top_k == 2 else rows
        r = mo.round_to_dtype(a32[src] @ experts[ex].w_ref_columns(cols), "bf16")
        if mul:
            r = mo.round_to_dtype(r * wt[rows, None], "bf16")
        want[rows] = r
    ok, err, big = mo.gemm_tolerance_ok(got, want)
    assert ok, (err, big)

    # sampled rows, all columns, against the dense GEMM of that row with its expert
    scale = float(c.float().abs().max())
    rng = np.random.default_rng(1)
    for r in rng.integers(0, tokens * 2, 4):
        ex = int(ids[r])
        src = int(r) // 2 if top_k == 2 else int(r)
        dense = experts[ex].gemm(a[src:src + 1].contiguous(), 1).float()
        if mul:
            dense = (dense.to(torch.bfloat16) * tw[r].to(torch.bfloat16)).float()
        err = float((dense - c[r].float()).abs().max())
        assert err <= 1e-2 * scale, (int(r), err, scale)


# ---------------------------------------------------------------------------
# W4A8 at the sizes the benchmark times
class BigA8Layer:
    """uint4b8 weights drawn on the device in the order of 8-bit activations, groups of 128 rows."""

    def __init__(self, seed, k, n, dtype, act):
        from tests.test_gpu_a8 import _a8_to_gfx950, _repack_a8
        self.k, self.n, self.dtype, self.act = k, n, dtype, act
        self.tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
        gen = torch.Generator(device=gu.DEV).manual_seed(seed)
        self.qweight = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 8, n), dtype=torch.int32, device=gu.DEV,
                                     generator=gen)
        words = self.qweight
        if act == "fp8":     # sign-and-magnitude nibbles, as marlin_int4_fp8_preprocess leaves them
            words = torch.empty_like(self.qweight)
            _lib.check(_lib.load().sonar_marlin_int4_fp8_preprocess(gu.ptr(self.qweight), None, gu.ptr(words),
                                                                     k // 8, n, 0, gu.stream()))
        self.native = _a8_to_gfx950(_repack_a8(words, k, n), k, n)
        rng = np.random.default_rng(seed)
        s = mo.round_to_dtype(rng.uniform(1e-3, 1e-2, size=(k // GROUP, n)).astype(np.float32), dtype)
        self.factor = np.float32(1.0)
        if act == "int8":
            self.scales, self.factor = mo.marlin_act_int8_process_scales(s)      # 16-bit integers
            self.dev_scales = torch.from_numpy(mo.marlin_permute_scales_a8(self.scales, k, n, GROUP).copy()).to(gu.DEV)
        else:
            self.scales = mo.round_to_dtype(s * np.float32(512.0), dtype)
            self.dev_scales = gu.dev_bits16(mo.marlin_permute_scales_a8(self.scales, k, n, GROUP), dtype)

    def q_columns(self, cols):
        idx = torch.as_tensor(cols, device=gu.DEV)
        return mo.unpack_rows(self.qweight[:, idx].cpu().numpy())

    def gemm(self, a_dev, a_scales_dev, m):
        lib = _lib.load()
        c = torch.full((m, self.n), float("nan"), dtype=self.tdt, device=gu.DEV)
        nbytes = lib.sonar_marlin_gemm_a8_scratch_bytes(m, self.n, self.k, self.k // GROUP)
        scratch = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=gu.DEV)
        _lib.check(lib.sonar_marlin_gemm_a8(
            gu.ptr(a_dev), self.k, _lib.ADTYPE_INT8 if self.act == "int8" else _lib.ADTYPE_FP8, gu.ptr(c),
            gu.ptr(self.native), _lib.LAYOUT_GFX950, None, gu.ptr(self.dev_scales), gu.ptr(a_scales_dev), None,
            gu.ptr(scratch), scratch.numel(), gu.dtype_code(self.dtype), _lib.TYPE_UINT4B8, m, self.n, self.k,
            self.k // GROUP, gu.stream()))
        return c


@pytest.mark.parametrize("m", [1, 64, 512, 4096])
def test_w4a8_int8_at_benchmark_size_bit_exact_on_sampled_columns(m):
    """K = 4096, N = 11008 (the shape bench.py times W4A8 on): the slab kernel and the tiled
    kernel with many tiles and no K split, bit for bit against the oracle."""
    k, n = 4096, 11008
    layer = BigA8Layer(700, k, n, "fp16", "int8")
    rng = np.random.default_rng(m)
    a_q, a_s = mo.per_token_quant_int8(rng.standard_normal((m, k)).astype(np.float32))
    a_s = (a_s * layer.factor).astype(np.float32)
    got = layer.gemm(torch.from_numpy(a_q).to(gu.DEV), torch.from_numpy(a_s.reshape(-1)).to(gu.DEV), m)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(got.float()).all())
    cols = sampled_columns(n, 8, m)
    want = mo.gemm_w4a8_int8(a_q, a_s, layer.q_columns(cols), GROUP, layer.scales[:, cols], "fp16")
    have = got[:, torch.as_tensor(cols, device=gu.DEV)].float().cpu().numpy()
    assert np.array_equal(have, want), np.abs(have - want).max()


@pytest.mark.parametrize("m", [64, 4096])
def test_w4a8_fp8_at_benchmark_size_on_sampled_columns(m):
    k, n = 4096, 11008
    layer = BigA8Layer(701, k, n, "bf16", "fp8")
    g = torch.Generator().manual_seed(m)
    x = torch.randn((m, k), generator=g)
    a_s = (x.abs().amax(dim=1, keepdim=True) / 448.0).clamp_min(1e-10)
    a_fp8 = (x / a_s).to(torch.float8_e4m3fn)
    got = layer.gemm(a_fp8.view(torch.uint8).to(gu.DEV), a_s.reshape(-1).to(gu.DEV), m)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(got.float()).all())
    cols = sampled_columns(n, 8, m)
    want = mo.gemm_w4a8_fp8(a_fp8.float().numpy(), a_s.numpy(), layer.q_columns(cols), GROUP,
                            layer.scales[:, cols] / np.float32(512.0))
    have = got[:, torch.as_tensor(cols, device=gu.DEV)].float().cpu().numpy()
    ok, err, big = mo.gemm_tolerance_ok(have, want)
    assert ok, (err, big)


def test_w4a8_int8_grouped_at_mixtral_size_bit_exact_on_sampled_columns():
    """The grouped W4A8 entry point on 64-slot blocks at the size bench.py times (8 experts of
    K = 4096, N = 28672, 4096 tokens, top 2): every routed row on sampled columns, bit for bit."""
    from sonar_amd import fused_moe
    _layers.clear()
    _experts.clear()
    tokens, e, k, n, top_k = 4096, 8, 4096, 28672, 2
    experts = [BigA8Layer(720 + i, k, n, "bf16", "int8") for i in range(e)]
    # one factor for all experts, as the reference's layer-wide maximum gives
    factor = experts[0].factor
    native = torch.stack([x.native for x in experts]).contiguous()
    scales = torch.stack([x.dev_scales for x in experts]).contiguous()
    gen = torch.Generator(device=gu.DEV).manual_seed(11)
    logits = torch.randn((tokens, e), device=gu.DEV, generator=gen)
    tw2, ti2 = torch.topk(torch.softmax(logits, dim=1), top_k, dim=1)
    ti2 = ti2.to(torch.int32)
    bs = 64
    sorted_ids, expert_ids, past = fused_moe.moe_align_block_size(ti2, bs, e)
    rng = np.random.default_rng(5)
    a_q, a_s = mo.per_token_quant_int8(rng.standard_normal((tokens, k)).astype(np.float32))
    a_s = (a_s * factor).astype(np.float32)
    d_a, d_as = torch.from_numpy(a_q).to(gu.DEV), torch.from_numpy(a_s.reshape(-1).copy()).to(gu.DEV)
    c = torch.full((tokens * top_k, n), float("nan"), dtype=torch.bfloat16, device=gu.DEV)
    tw = tw2.reshape(-1).contiguous().float()
    lib = _lib.load()
    _lib.check(lib.sonar_moe_wna16_marlin_gemm_a8(
        gu.ptr(d_a), _lib.ADTYPE_INT8, gu.ptr(c), gu.ptr(native), _lib.LAYOUT_GFX950, None, gu.ptr(scales),
        gu.ptr(d_as), None, gu.ptr(sorted_ids), sorted_ids.numel(), gu.ptr(expert_ids), gu.ptr(past), gu.ptr(tw),
        bs, top_k, 0, e, _lib.DTYPE_BF16, _lib.TYPE_UINT4B8, tokens, n, k, k // GROUP, gu.stream()))
    torch.cuda.synchronize()
    assert bool(torch.isfinite(c.float()).all()), "a routed row was not written"
    cols = sampled_columns(n, 6, 3)
    have = c[:, torch.as_tensor(cols, device=gu.DEV)].float().cpu().numpy()
    ids = ti2.reshape(-1).cpu().numpy()
    want = np.zeros_like(have)
    for ex in range(e):
        rows = np.nonzero(ids == ex)[0]
        want[rows] = mo.gemm_w4a8_int8(a_q[rows // top_k], a_s.reshape(-1)[rows // top_k], experts[ex].q_columns(cols),
                                       GROUP, experts[ex].scales[:, cols], "bf16")
    assert np.array_equal(have, want), np.abs(have - want).max()
