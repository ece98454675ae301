"""GPU tests of the torch-op layer and the host mirror above it: the ops are
called the way the reference's callers call them (apply_gptq_marlin_linear,
MarlinLinearKernel, fused_marlin_moe) and compared with the oracle."""
from __future__ import annotations

import types

import numpy as np
import pytest
import torch

from oracle import marlin_oracle as mo
from tests import gpu_util as gu

pytestmark = pytest.mark.gpu


def U32(x):
    return np.ascontiguousarray(x).view(np.uint32)


def _tdt(dtype):
    return torch.float16 if dtype == "fp16" else torch.bfloat16


def test_repack_ops_bit_exact_and_fresh_output():
    from sonar_amd import ops
    k, n = 256, 192
    layer = mo.make_layer(3, k, n, 128, "fp16", zero_points=True, act_order=True)
    q = layer["q"]
    g_sorted, order = mo.stable_sort_g_idx(layer["g_idx"])
    got = ops.gptq_marlin_repack(gu.dev_i32(mo.gptq_pack(q)), gu.dev_i32(order), k, n, 4)
    want = mo.gptq_marlin_repack(mo.gptq_pack(q), order, k, n)
    assert got.shape == (k // 16, 2 * n) and got.dtype == torch.int32
    assert np.array_equal(got.cpu().numpy().view(np.uint32), U32(want))
    empty = torch.empty(0, dtype=torch.int32, device=gu.DEV)
    got = ops.gptq_marlin_repack(gu.dev_i32(mo.gptq_pack(q)), empty, k, n, 4)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), U32(mo.gptq_marlin_repack(mo.gptq_pack(q), None, k, n)))
    got = ops.awq_marlin_repack(gu.dev_i32(mo.awq_pack(q)), k, n, 4)
    assert np.array_equal(got.cpu().numpy().view(np.uint32), U32(mo.awq_marlin_repack(mo.awq_pack(q), k, n)))
    with pytest.raises(RuntimeError):
        ops.gptq_marlin_repack(gu.dev_i32(mo.gptq_pack(q)), empty, k, n, 8)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("m", [1, 16, 48, 300])
def test_marlin_gemm_op_and_weight_cache(dtype, m):
    from sonar_amd import ops
    from sonar_amd.scalar_type import scalar_types
    k, n = 512, 256
    dl = gu.DeviceLayer(21, k, n, 128, dtype)
    a32 = mo.make_activations(m, m, k, dtype)
    a = gu.dev_bits16(a32, dtype)
    empty = torch.empty(0, dtype=torch.int32, device=gu.DEV)
    ops.marlin_weight_cache_clear()
    outs = []
    for _ in range(2):   # second call takes the cached streaming-order copy
        outs.append(ops.marlin_gemm(a, None, dl.marlin, None, dl.scales, None, None, empty, empty, empty,
                                    dl.workspace, scalar_types.uint4b8, m, n, k, True, False, True, False))
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(outs[0]), mo.gemm_reference(a32, dl.w_ref))
    assert ok, worst
    assert int(dl.workspace.abs().sum()) == 0
    # writing into a caller's tensor returns that tensor
    c = torch.empty((m, n), dtype=_tdt(dtype), device=gu.DEV)
    r = ops.marlin_gemm(a, c, dl.marlin, None, dl.scales, None, None, empty, empty, empty, dl.workspace,
                        scalar_types.uint4b8, m, n, k, True, False, True, False)
    assert r.data_ptr() == c.data_ptr() and torch.equal(r, outs[0])
    # the cache notices an in-place change of the weight
    dl.marlin.copy_(gu.DeviceLayer(22, k, n, 128, dtype).marlin)
    other = ops.marlin_gemm(a, None, dl.marlin, None, dl.scales, None, None, empty, empty, empty,
                            dl.workspace, scalar_types.uint4b8, m, n, k, True, False, True, False)
    assert not torch.equal(other, outs[0])
    assert ops.marlin_weight_cache_clear() >= 1


def test_weight_cache_lets_go_of_dropped_weights():
    """The streaming-order copy of a weight whose Marlin tensor the caller has
    dropped (a reloaded layer) leaves the cache at the next conversion."""
    from sonar_amd import ops
    from sonar_amd.scalar_type import scalar_types
    k, n, m = 256, 128, 4
    a = gu.dev_bits16(mo.make_activations(1, m, k, "fp16"), "fp16")
    empty = torch.empty(0, dtype=torch.int32, device=gu.DEV)

    def run(dl):
        ops.marlin_gemm(a, None, dl.marlin, None, dl.scales, None, None, empty, empty, empty, dl.workspace,
                        scalar_types.uint4b8, m, n, k, True, False, True, False)

    ops.marlin_weight_cache_clear()
    first, second = gu.DeviceLayer(1, k, n, 128, "fp16"), gu.DeviceLayer(2, k, n, 128, "fp16")
    run(first)
    run(second)
    assert ops.marlin_weight_cache_clear() == 2
    run(first)
    del first                      # the only holder of its Marlin tensor
    run(second)
    torch.cuda.synchronize()
    assert ops.marlin_weight_cache_clear() == 1


def _gemm_through_op(a, marlin, scales, ws, m, n, k):
    from sonar_amd import ops
    from sonar_amd.scalar_type import scalar_types
    empty = torch.empty(0, dtype=torch.int32, device=gu.DEV)
    return ops.marlin_gemm(a, None, marlin, None, scales, None, None, empty, empty, empty, ws,
                           scalar_types.uint4b8, m, n, k, True, False, True, False)


def test_weight_cache_follows_the_reference_reload_idioms():
    """The ways a caller replaces a weight after its first GEMM: `x.data = repack(...)`
    (the reference's own idiom, marlin.py transform_w_q), also when the allocator
    hands the old address back; `x.data.copy_(...)` followed by
    marlin_weight_cache_invalidate; an inference-mode tensor refilled in place."""
    from sonar_amd import ops
    k, n, m = 512, 256, 8
    a32 = mo.make_activations(3, m, k, "fp16")
    a = gu.dev_bits16(a32, "fp16")
    first, second = gu.DeviceLayer(31, k, n, 128, "fp16"), gu.DeviceLayer(32, k, n, 128, "fp16")

    def check(out, layer):
        ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(out), mo.gemm_reference(a32, layer.w_ref))
        assert ok, worst

    ops.marlin_weight_cache_clear()
    # 1. x.data = new tensor from the repack op
    param = torch.nn.Parameter(first.marlin.clone(), requires_grad=False)
    check(_gemm_through_op(a, param, first.scales, first.workspace, m, n, k), first)
    param.data = gu.gptq_repack(gu.dev_i32(mo.gptq_pack(second.layer["q"])), None, k, n)
    check(_gemm_through_op(a, param, second.scales, first.workspace, m, n, k), second)
    assert ops.marlin_weight_cache_clear() == 1      # the entry of the old address is gone

    # 2. the same when the new weight lands on the old address: the repack op itself forgets that memory
    qw_first, qw_second = gu.dev_i32(mo.gptq_pack(first.layer["q"])), gu.dev_i32(mo.gptq_pack(second.layer["q"]))
    empty = torch.empty(0, dtype=torch.int32, device=gu.DEV)
    holder = ops.gptq_marlin_repack(qw_first, empty, k, n, 4)
    param = torch.nn.Parameter(holder, requires_grad=False)
    check(_gemm_through_op(a, param, first.scales, first.workspace, m, n, k), first)
    address = param.data_ptr()
    del holder
    param.data = torch.empty(0, dtype=torch.int32, device=gu.DEV)     # frees the block; the allocator reuses it
    param.data = ops.gptq_marlin_repack(qw_second, empty, k, n, 4)
    if param.data_ptr() != address:
        pytest.skip("the allocator did not hand the old block back")
    check(_gemm_through_op(a, param, second.scales, first.workspace, m, n, k), second)

    # 3. bytes rewritten through .data (no version bump): the caller invalidates
    param = torch.nn.Parameter(first.marlin.clone(), requires_grad=False)
    check(_gemm_through_op(a, param, first.scales, first.workspace, m, n, k), first)
    version = param._version
    param.data.copy_(second.marlin)
    assert param._version == version
    assert ops.marlin_weight_cache_invalidate(param) == 1
    check(_gemm_through_op(a, param, second.scales, first.workspace, m, n, k), second)

    # 4. an inference-mode tensor refilled in place
    with torch.inference_mode():
        w = first.marlin.clone()
        check(_gemm_through_op(a, w, first.scales, first.workspace, m, n, k), first)
        w.copy_(second.marlin)
        assert ops.marlin_weight_cache_invalidate(w) == 1
        check(_gemm_through_op(a, w, second.scales, first.workspace, m, n, k), second)
    ops.marlin_weight_cache_clear()


def test_first_use_of_a_weight_inside_graph_capture_is_refused():
    from sonar_amd import ops
    k, n, m = 256, 128, 4
    dl = gu.DeviceLayer(41, k, n, 128, "fp16")
    a = gu.dev_bits16(mo.make_activations(1, m, k, "fp16"), "fp16")
    ops.marlin_weight_cache_clear()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with pytest.raises(RuntimeError, match="warm-up"):
            with torch.cuda.graph(graph, stream=stream):
                _gemm_through_op(a, dl.marlin, dl.scales, dl.workspace, m, n, k)
    torch.cuda.synchronize()
    # after a warm-up call the capture goes through and replays give the eager result
    want = _gemm_through_op(a, dl.marlin, dl.scales, dl.workspace, m, n, k)
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            got = _gemm_through_op(a, dl.marlin, dl.scales, dl.workspace, m, n, k)
        for _ in range(3):
            got.zero_()
            graph.replay()
            stream.synchronize()
            assert torch.equal(got, want)


def test_capture_on_the_stream_that_converted_the_weight():
    """One warm-up call on a side stream, then a capture on that same stream: the hit
    inside the capture must not touch the conversion's event (an event query there
    invalidates the capture)."""
    from sonar_amd import ops
    k, n, m = 256, 128, 4
    dl = gu.DeviceLayer(42, k, n, 128, "fp16")
    a = gu.dev_bits16(mo.make_activations(2, m, k, "fp16"), "fp16")
    ops.marlin_weight_cache_clear()
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        want = _gemm_through_op(a, dl.marlin, dl.scales, dl.workspace, m, n, k)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            got = _gemm_through_op(a, dl.marlin, dl.scales, dl.workspace, m, n, k)
        for _ in range(3):
            got.zero_()
            graph.replay()
            stream.synchronize()
            assert torch.equal(got, want)
        again = _gemm_through_op(a, dl.marlin, dl.scales, dl.workspace, m, n, k)   # eager hit drops the event
        stream.synchronize()
        assert torch.equal(again, want)
    ops.marlin_weight_cache_clear()


def test_weight_converted_on_one_stream_is_safe_on_another():
    from sonar_amd import ops
    k, n, m = 4096, 4096, 4
    dl = gu.DeviceLayer(43, 512, 256, 128, "fp16")          # oracle-sized reference
    big = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 16, 2 * n), dtype=torch.int32, device=gu.DEV)
    scales = torch.full((k // 128, n), 0.01, dtype=torch.float16, device=gu.DEV)
    a = torch.randn((m, k), device=gu.DEV, dtype=torch.float16)
    ws = dl.workspace
    ops.marlin_weight_cache_clear()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(s1):
        first = _gemm_through_op(a, big, scales, ws, m, n, k)      # converts on s1
    with torch.cuda.stream(s2):
        second = _gemm_through_op(a, big, scales, torch.zeros_like(ws), m, n, k)   # hits the cache from s2
    torch.cuda.synchronize()
    assert torch.equal(first, second)
    ops.marlin_weight_cache_clear()


def test_marlin_gemm_op_rejects_like_the_reference():
    from sonar_amd import ops
    from sonar_amd.scalar_type import scalar_types
    k, n, m = 256, 128, 4
    dl = gu.DeviceLayer(5, k, n, 128, "fp16")
    a = gu.dev_bits16(mo.make_activations(1, m, k, "fp16"), "fp16")
    empty = torch.empty(0, dtype=torch.int32, device=gu.DEV)

    def call(**kw):
        args = dict(a=a, c=None, b=dl.marlin, s=dl.scales, z=empty, ws=dl.workspace, t=scalar_types.uint4b8,
                    m=m, n=n, k=k)
        args.update(kw)
        return ops.marlin_gemm(args["a"], args["c"], args["b"], None, args["s"], None, None, args["z"], empty,
                               empty, args["ws"], args["t"], args["m"], args["n"], args["k"], True, False, True,
                               False)

    call()
    with pytest.raises(RuntimeError, match="size_m"):
        call(m=m + 1)
    with pytest.raises(RuntimeError):
        call(t=scalar_types.uint4)            # uint4 needs zero points
    with pytest.raises(RuntimeError):
        call(t=scalar_types.uint8b128)        # 4-bit packing under the 8-bit type: wrong size_n
    with pytest.raises(RuntimeError, match="workspace"):
        call(ws=dl.workspace[:8])
    with pytest.raises(RuntimeError):
        call(s=dl.scales.to(torch.bfloat16))  # scales must have the activation type
    assert call(a=a[:0], m=0).shape == (0, n)


@pytest.mark.parametrize("cfg", [
    # (k, n, group, dtype, zero_points, act_order, bias, batch shape)
    (256, 128, 128, "fp16", False, False, False, (5,)),
    (512, 192, 64, "bf16", False, False, True, (2, 3)),
    (256, 128, -1, "fp16", False, False, False, (1,)),
    (256, 128, 128, "bf16", True, False, False, (7,)),
    (512, 128, 128, "fp16", False, True, True, (9,)),
    (136, 72, 8 * 17, "fp16", False, False, False, (4,)),     # padded N and K (one group)
    # compressed-tensors layout: weight_packed (N, K/8), weight_scale (N, groups), zero points (N/8, groups)
    (512, 192, 128, "bf16", False, False, False, (6,), "ct"),
    (256, 128, 64, "fp16", True, False, True, (3,), "ct"),
    (512, 128, 128, "fp16", False, True, False, (20,), "ct"),
], ids=str)
def test_marlin_linear_kernel_round_trip(cfg):
    """Checkpoint-format tensors -> process_weights_after_loading -> apply_weights
    (kernels/linear/mixed_precision/marlin.py:88-235)."""
    from sonar_amd.marlin_linear import MarlinLinearKernel, MPLinearLayerConfig
    from sonar_amd.marlin_utils import pack_cols
    from sonar_amd.scalar_type import scalar_types
    k, n, g, dtype, zp, act, bias, batch = cfg[:8]
    ct = len(cfg) > 8
    gs = k if g == -1 or g >= k else g
    layer_np = mo.make_layer(11, k, n, gs, dtype, zero_points=zp, act_order=act)
    w_ref = mo.dequantize(layer_np["q"], layer_np["scales"], gs, dtype, zeros=layer_np.get("zeros"),
                          g_idx=layer_np.get("g_idx"))
    layer = types.SimpleNamespace()
    layer.qweight = gu.dev_i32(mo.gptq_pack(layer_np["q"]))
    layer.scales = gu.dev_bits16(layer_np["scales"], dtype)
    layer.bias = None
    if zp:
        layer.qzeros = pack_cols(torch.from_numpy(layer_np["zeros"].astype(np.int32)).to(gu.DEV), 4,
                                 layer_np["groups"], n)
    if act:
        layer.g_idx = gu.dev_i32(layer_np["g_idx"])
    if ct:
        layer.qweight = layer.qweight.t().contiguous()
        layer.scales = layer.scales.t().contiguous()
        if zp:
            layer.qzeros = layer.qzeros.t().contiguous()
    bias32 = None
    if bias:
        bias32 = mo.round_to_dtype(np.random.default_rng(4).standard_normal(n).astype(np.float32), dtype)
        layer.bias = gu.dev_bits16(bias32, dtype)
    cfgobj = MPLinearLayerConfig((k, n), (k, n), scalar_types.uint4 if zp else scalar_types.uint4b8,
                                 _tdt(dtype), g if g != 8 * 17 else -1, zp, act)
    kern = MarlinLinearKernel(cfgobj, w_zp_param_name="qzeros" if zp else None,
                              w_gidx_param_name="g_idx" if act else None)
    kern.process_weights_after_loading(layer)
    rows = int(np.prod(batch))
    x32 = mo.make_activations(8, rows, k, dtype)
    x = gu.dev_bits16(x32, dtype).reshape(*batch, k)
    y = kern.apply_weights(layer, x, layer.bias)
    assert y.shape == (*batch, n)
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(y).reshape(rows, n), mo.gemm_reference(x32, w_ref, bias32))
    assert ok, worst


@pytest.mark.parametrize("k,n,g,dtype,rows", [(512, 256, 128, "fp16", 5), (1024, 4096, 128, "bf16", 40)])
def test_awq_checkpoint_through_the_linear_kernel(k, n, g, dtype, rows):
    """AutoAWQ tensors -> convert_awq_to_standard_format -> MarlinLinearKernel
    (auto_awq.py:93-153 feeding kernels/linear/mixed_precision/marlin.py)."""
    from sonar_amd.marlin_linear import (MarlinLinearKernel, MPLinearLayerConfig,
                                         convert_awq_to_standard_format)
    from sonar_amd.scalar_type import scalar_types
    layer_np = mo.make_layer(19, k, n, g, dtype, zero_points=True)
    w_ref = mo.dequantize(layer_np["q"], layer_np["scales"], g, dtype, zeros=layer_np["zeros"])
    layer = types.SimpleNamespace(bias=None)
    layer.qweight = gu.dev_i32(mo.awq_pack(layer_np["q"]))
    layer.qzeros = gu.dev_i32(mo.awq_pack(layer_np["zeros"].astype(np.int32)))
    layer.scales = gu.dev_bits16(layer_np["scales"], dtype)
    convert_awq_to_standard_format(layer)
    kern = MarlinLinearKernel(MPLinearLayerConfig((k, n), (k, n), scalar_types.uint4, _tdt(dtype), g, True, False),
                              w_gidx_param_name=None)
    kern.process_weights_after_loading(layer)
    x32 = mo.make_activations(3, rows, k, dtype)
    y = kern.apply_weights(layer, gu.dev_bits16(x32, dtype), None)
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(y), mo.gemm_reference(x32, w_ref))
    assert ok, worst


@pytest.mark.parametrize("dtype,rows", [("fp16", 3), ("bf16", 70)])
def test_linear_kernel_row_parallel_act_order_shard(dtype, rows):
    """A row-parallel rank's slice of an act-order layer: is_k_full = False, the
    scales of every group on every rank (marlin_utils.py: marlin_is_k_full,
    marlin_repeat_scales_on_all_ranks; marlin.py:88-235)."""
    from sonar_amd.marlin_linear import MarlinLinearKernel, MPLinearLayerConfig
    from sonar_amd.scalar_type import scalar_types
    k_full, n, g = 1024, 256, 128
    full = mo.make_layer(23, k_full, n, g, dtype, act_order=True)
    lo, hi = 512, 1024                       # rank 1 of 2
    k = hi - lo
    w_ref = mo.dequantize(full["q"][lo:hi], full["scales"], g, dtype, g_idx=full["g_idx"][lo:hi])
    layer = types.SimpleNamespace(bias=None)
    layer.qweight = gu.dev_i32(mo.gptq_pack(full["q"][lo:hi]))
    layer.scales = gu.dev_bits16(full["scales"], dtype)
    layer.g_idx = gu.dev_i32(full["g_idx"][lo:hi])
    kern = MarlinLinearKernel(MPLinearLayerConfig((k_full, n), (k, n), scalar_types.uint4b8, _tdt(dtype), g, False,
                                                  True), w_zp_param_name=None)
    kern.process_weights_after_loading(layer)
    assert kern.is_k_full is False
    x32 = mo.make_activations(6, rows, k, dtype)
    y = kern.apply_weights(layer, gu.dev_bits16(x32, dtype), None)
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(y), mo.gemm_reference(x32, w_ref))
    assert ok, worst


@pytest.mark.parametrize("k,n,g,dtype,rows", [(512, 256, 128, "fp16", 3), (1024, 4096, 128, "bf16", 70),
                                              (4000, 192, -1, "fp16", 9)])
def test_w8a16_through_the_ops_and_the_linear_kernel(k, n, g, dtype, rows):
    """uint8b128 checkpoint tensors (qweight (K/4, N), scales) -> gptq_marlin_repack
    with num_bits = 8 -> marlin_gemm, through MarlinLinearKernel (with tile
    padding of K for the third case)."""
    from sonar_amd.marlin_linear import MarlinLinearKernel, MPLinearLayerConfig
    from sonar_amd.scalar_type import scalar_types
    rng = np.random.default_rng(k + n)
    q = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    groups = 1 if g == -1 else k // g
    scales = mo.round_to_dtype(rng.uniform(1e-4, 1e-3, size=(groups, n)).astype(np.float32), dtype)
    w_ref = mo.dequantize(q, scales, g, dtype, num_bits=8)
    layer = types.SimpleNamespace(bias=None)
    layer.qweight = gu.dev_i32(mo.pack_rows8(q))
    layer.scales = gu.dev_bits16(scales, dtype)
    kern = MarlinLinearKernel(MPLinearLayerConfig((k, n), (k, n), scalar_types.uint8b128, _tdt(dtype), g, False,
                                                  False), w_zp_param_name=None, w_gidx_param_name=None)
    kern.process_weights_after_loading(layer)
    x32 = mo.make_activations(2, rows, k, dtype, std=0.5)
    y = kern.apply_weights(layer, gu.dev_bits16(x32, dtype), None)
    assert y.shape == (rows, n)
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(y), mo.gemm_reference(x32, w_ref))
    assert ok, worst


def _moe_layer(seed, e, hidden, inter, g, dtype, zp):
    """Expert weights in the layouts fused_marlin_moe takes, plus dequantised references."""
    from sonar_amd import marlin_utils as mu
    from sonar_amd import ops
    w13, w2 = [], []
    for i in range(e):
        w13.append(mo.make_layer(seed + i, hidden, 2 * inter, g, dtype, zero_points=zp))
        w2.append(mo.make_layer(seed + 100 + i, inter, hidden, g, dtype, zero_points=zp))

    def pack(layers, k, n):
        q = torch.stack([gu.dev_i32(mo.gptq_pack(l["q"])) for l in layers])
        empty = torch.empty((e, 0), dtype=torch.int32, device=gu.DEV)
        marlin = ops.gptq_marlin_moe_repack(q, empty, k, n, 4)
        s = torch.stack([gu.dev_bits16(l["scales"], dtype) for l in layers])
        s = mu.marlin_moe_permute_scales(s, k, n, g)
        z = None
        if zp:
            z = torch.stack([mu.marlin_zero_points(torch.from_numpy(l["zeros"].astype(np.int32)).to(gu.DEV),
                                                   l["groups"], n, 4) for l in layers])
        ref = [mo.dequantize(l["q"], l["scales"], g, dtype, zeros=l.get("zeros")) for l in layers]
        return marlin, s, z, ref

    return pack(w13, hidden, 2 * inter), pack(w2, inter, hidden)


def _moe_reference(x32, ref13, ref2, topk_ids, topk_w, dtype, bias13=None, bias2=None):
    """torch_experts restated (tests/kernels/utils.py:817-931): per routed
    slot silu(x W_gate) * (x W_up) -> W_down, weighted sum over the slots."""
    m, hidden = x32.shape
    inter = ref2[0].shape[0]
    out = np.zeros((m, hidden), dtype=np.float32)
    for t in range(m):
        for j in range(topk_ids.shape[1]):
            ex = int(topk_ids[t, j])
            h = x32[t:t + 1] @ ref13[ex]
            h = mo.round_to_dtype(h if bias13 is None else h + bias13[ex][None, :], dtype)
            gate, up = h[:, :inter], h[:, inter:]
            act = mo.round_to_dtype(mo.round_to_dtype(gate / (1.0 + np.exp(-gate)), dtype) * up, dtype)
            y = act @ ref2[ex]
            y = mo.round_to_dtype(y if bias2 is None else y + bias2[ex][None, :], dtype)
            out[t] += topk_w[t, j] * y[0]
    return out


@pytest.mark.parametrize("cfg", [
    (4, 8, 2, 256, 128, 128, "bf16", False),
    (40, 4, 2, 256, 256, 64, "fp16", False),
    (200, 4, 2, 128, 128, 128, "bf16", True),
    (3, 16, 4, 256, 128, 128, "fp16", False),
], ids=str)
def test_fused_marlin_moe_against_per_token_reference(cfg):
    from sonar_amd.fused_moe import fused_marlin_moe
    from sonar_amd.scalar_type import scalar_types
    m, e, topk, hidden, inter, g, dtype, zp = cfg
    (w1, s1, z1, ref13), (w2, s2, z2, ref2) = _moe_layer(40, e, hidden, inter, g, dtype, zp)
    rng = np.random.default_rng(m)
    logits = rng.standard_normal((m, e)).astype(np.float32)
    prob = np.exp(logits - logits.max(1, keepdims=True))
    prob /= prob.sum(1, keepdims=True)
    topk_ids = np.argsort(-prob, axis=1, kind="stable")[:, :topk].astype(np.int32)
    topk_w = np.take_along_axis(prob, topk_ids, axis=1).astype(np.float32)
    x32 = mo.round_to_dtype(0.5 * mo.make_activations(m, m, hidden, dtype), dtype)
    x = gu.dev_bits16(x32, dtype)
    qtype = scalar_types.uint4 if zp else scalar_types.uint4b8
    y = fused_marlin_moe(x, w1, w2, None, None, s1, s2, torch.from_numpy(topk_w).to(gu.DEV),
                         torch.from_numpy(topk_ids).to(gu.DEV), qtype.id, w1_zeros=z1, w2_zeros=z2)
    torch.cuda.synchronize()
    want = _moe_reference(x32, ref13, ref2, topk_ids, topk_w, dtype)
    got = gu.host_f32(y)
    max_ref = np.abs(want).max()
    # two chained GEMMs and three roundings per slot: 2x the single-GEMM bound
    assert np.abs(got - want).max() <= 2e-2 * max_ref, (np.abs(got - want).max(), max_ref)


def _route(m, e, topk, seed):
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((m, e)).astype(np.float32)
    prob = np.exp(logits - logits.max(1, keepdims=True))
    prob /= prob.sum(1, keepdims=True)
    ids = np.argsort(-prob, axis=1, kind="stable")[:, :topk].astype(np.int32)
    return ids, np.take_along_axis(prob, ids, axis=1).astype(np.float32)


@pytest.mark.parametrize("cfg", [
    # m, experts, topk, hidden, intermediate, group, dtype, format, act_order, bias
    (5, 4, 2, 256, 128, 128, "fp16", "gptq", False, False),
    (70, 4, 2, 256, 256, 64, "bf16", "gptq", True, True),
    (33, 8, 2, 128, 128, 128, "bf16", "gptq_zp", False, False),
    (40, 4, 2, 256, 128, 128, "fp16", "awq", False, True),
    (9, 4, 2, 256, 96, 32, "fp16", "gptq", False, True),      # intermediate size padded 96 -> 128
    (9, 4, 2, 128, 160, 32, "bf16", "awq", False, False),     # 160 -> 192
    (21, 4, 2, 256, 128, 128, "fp16", "gptq8", False, True),  # 8-bit codes
    (70, 4, 2, 256, 256, 64, "bf16", "gptq8", True, False),
    (9, 4, 2, 256, 96, 32, "fp16", "gptq8", False, False),    # 8-bit codes, 96 -> 128
], ids=str)
def test_moe_checkpoint_tensors_through_weight_processing(cfg):
    """Stacked expert tensors as a GPTQ / AWQ checkpoint holds them ->
    process_*_moe_weights -> fused_marlin_moe, against the per-token reference
    on the weights dequantised from the same checkpoint tensors."""
    from sonar_amd import moe_weights as mw
    from sonar_amd.fused_moe import fused_marlin_moe
    from sonar_amd.scalar_type import scalar_types
    m, e, topk, hidden, inter, g, dtype, fmt, act, bias = cfg
    zp = fmt in ("gptq_zp", "awq")
    bits = 8 if fmt == "gptq8" else 4
    rng = np.random.default_rng(hidden + inter)

    def expert_set(seed, k, n):
        layers = [mo.make_layer(seed + i, k, n, g, dtype, zero_points=zp, act_order=act) for i in range(e)]
        if bits == 8:
            for i, l in enumerate(layers):   # codes over all of 0..255, scales a sixteenth
                l["q"] = np.random.default_rng(seed + 50 + i).integers(0, 256, size=(k, n), dtype=np.int32)
                l["scales"] = mo.round_to_dtype(l["scales"] / 16, dtype)
        ref = [mo.dequantize(l["q"], l["scales"], g, dtype, zeros=l.get("zeros"), g_idx=l.get("g_idx"),
                             num_bits=bits) for l in layers]
        if bits == 8:
            qw = torch.stack([gu.dev_i32(mo.pack_rows8(l["q"])) for l in layers])
            qz = None
        elif fmt == "awq":
            qw = torch.stack([gu.dev_i32(mo.awq_pack(l["q"])) for l in layers])
            qz = torch.stack([gu.dev_i32(mo.awq_pack(l["zeros"])) for l in layers])
        else:
            qw = torch.stack([gu.dev_i32(mo.gptq_pack(l["q"])) for l in layers])
            qz = torch.stack([gu.dev_i32(mo.pack_cols(l["zeros"])) for l in layers]) if zp else None
        sc = torch.stack([gu.dev_bits16(l["scales"], dtype) for l in layers])
        gi = torch.stack([gu.dev_i32(l["g_idx"]) for l in layers]) if act else None
        b32 = mo.round_to_dtype(rng.standard_normal((e, n)).astype(np.float32), dtype) if bias else None
        return qw, qz, sc, gi, ref, b32

    qw13, qz13, s13, gi13, ref13, b13 = expert_set(300, hidden, 2 * inter)
    qw2, qz2, s2, gi2, ref2, b2 = expert_set(400, inter, hidden)
    dev_bias = lambda b: None if b is None else gu.dev_bits16(b, dtype)
    if fmt == "awq":
        w = mw.process_awq_moe_weights(inter, 4, g, qw13, qw2, s13, s2, qz13, qz2, dev_bias(b13), dev_bias(b2))
    else:
        w = mw.process_gptq_moe_weights(inter, bits, g, act, qw13, qw2, s13, s2, gi13, gi2, qz13, qz2,
                                        dev_bias(b13), dev_bias(b2))
    assert w.intermediate_size == mw.marlin_moe_padded_intermediate(inter, g)
    topk_ids, topk_w = _route(m, e, topk, m)
    x32 = mo.round_to_dtype(0.5 * mo.make_activations(m, m, hidden, dtype), dtype)
    qtype = scalar_types.uint8b128 if bits == 8 else scalar_types.uint4 if zp else scalar_types.uint4b8
    y = fused_marlin_moe(gu.dev_bits16(x32, dtype), w.w1, w.w2, w.bias1, w.bias2, w.w1_scale, w.w2_scale,
                         torch.from_numpy(topk_w).to(gu.DEV), torch.from_numpy(topk_ids).to(gu.DEV), qtype.id,
                         g_idx1=w.g_idx1, g_idx2=w.g_idx2, sort_indices1=w.sort_indices1,
                         sort_indices2=w.sort_indices2, w1_zeros=w.w1_zeros, w2_zeros=w.w2_zeros)
    torch.cuda.synchronize()
    want = _moe_reference(x32, ref13, ref2, topk_ids, topk_w, dtype, b13, b2)
    got = gu.host_f32(y)
    max_ref = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-2 * max_ref, (np.abs(got - want).max(), max_ref)


@pytest.mark.parametrize("cfg", [
    # experts, max tokens per expert, hidden, intermediate, group, dtype, zero points
    (4, 5, 256, 128, 128, "fp16", False),
    (8, 20, 256, 256, 64, "bf16", False),
    (4, 70, 128, 128, 128, "bf16", True),
], ids=str)
def test_batched_fused_marlin_moe_against_per_token_reference(cfg):
    """Tokens already batched by expert (marlin_moe.py:395-560): the valid rows of
    batch e go through expert e; rows past expert_num_tokens[e] are left alone."""
    from sonar_amd.fused_moe import batched_fused_marlin_moe
    from sonar_amd.scalar_type import scalar_types
    e, max_tokens, hidden, inter, g, dtype, zp = cfg
    (w1, s1, z1, ref13), (w2, s2, z2, ref2) = _moe_layer(60, e, hidden, inter, g, dtype, zp)
    rng = np.random.default_rng(max_tokens)
    counts = rng.integers(0, max_tokens + 1, size=e).astype(np.int32)
    counts[0] = max_tokens                  # one full batch, and
    counts[-1] = 0                          # one empty
    x32 = mo.round_to_dtype(0.5 * mo.make_activations(7, e * max_tokens, hidden, dtype), dtype)
    x = gu.dev_bits16(x32, dtype).view(e, max_tokens, hidden)
    qtype = scalar_types.uint4 if zp else scalar_types.uint4b8
    marker = torch.full((e, max_tokens, hidden), 7.0, dtype=x.dtype, device=gu.DEV)
    y = batched_fused_marlin_moe(x, torch.from_numpy(counts).to(gu.DEV), w1, w2, None, None, s1, s2, qtype.id,
                                 w1_zeros=z1, w2_zeros=z2, output=marker)
    torch.cuda.synchronize()
    got = gu.host_f32(y)
    for b in range(e):
        rows = x32[b * max_tokens:b * max_tokens + counts[b]]
        if counts[b]:
            ids = np.full((counts[b], 1), b, dtype=np.int32)
            want = _moe_reference(rows, ref13, ref2, ids, np.ones((counts[b], 1), np.float32), dtype)
            max_ref = np.abs(want).max()
            assert np.abs(got[b, :counts[b]] - want).max() <= 2e-2 * max_ref, (b, counts[b])
        assert np.all(got[b, counts[b]:] == 7.0), "rows of invalid tokens must not be written"


@pytest.mark.parametrize("zp", [False, True])
def test_marlin_experts_classes_run_the_layer(zp):
    """MarlinExperts / BatchedMarlinExperts (marlin_moe.py:707-1096) called the way the reference's
    modular kernel calls them (workspaces of workspace_shapes(), output buffer given): the same
    bits as fused_marlin_moe / batched_fused_marlin_moe on the same inputs."""
    from sonar_amd import marlin_experts as me
    from sonar_amd.fused_moe import batched_fused_marlin_moe, fused_marlin_moe
    from sonar_amd.scalar_type import scalar_types
    m, e, topk, hidden, inter, dtype = 37, 4, 2, 256, 128, "bf16"
    (w1, s1, z1, _), (w2, s2, z2, _) = _moe_layer(61, e, hidden, inter, 128, dtype, zp)
    quant = me.ExpertsQuantConfig(use_int4_w4a16=True, w1_scale=s1, w2_scale=s2, w1_zp=z1, w2_zp=z2)
    experts = me.MarlinExperts(me.ExpertsMoeConfig(), quant)
    assert experts.quant_type_id == (scalar_types.uint4.id if zp else scalar_types.uint4b8.id)
    topk_ids, topk_w = _route(m, e, topk, m)
    tw, ti = torch.from_numpy(topk_w).to(gu.DEV), torch.from_numpy(topk_ids).to(gu.DEV)
    x = gu.dev_bits16(mo.round_to_dtype(0.5 * mo.make_activations(3, m, hidden, dtype), dtype), dtype)
    E, M, N, K, k = experts.moe_problem_size(x, w1, w2, ti)
    assert (E, M, N, K, k) == (e, m, inter, hidden, topk)
    ws13, ws2, out_shape = experts.workspace_shapes(M, N, K, k, e, e, None, "silu")
    buf13 = torch.empty(ws13, dtype=x.dtype, device=gu.DEV)
    buf2 = torch.empty(ws2, dtype=x.dtype, device=gu.DEV)
    out = torch.full(out_shape, 9.0, dtype=x.dtype, device=gu.DEV)
    experts.apply(out, x, w1, w2, tw, ti, "silu", e, None, None, None, buf13, buf2, None, False)
    want = fused_marlin_moe(x, w1, w2, None, None, s1, s2, tw, ti, experts.quant_type_id, w1_zeros=z1, w2_zeros=z2)
    torch.cuda.synchronize()
    assert torch.equal(out, want)

    max_tokens, dispatchers = 20, 1
    batched = me.BatchedMarlinExperts(me.ExpertsMoeConfig(), quant, max_tokens, dispatchers)
    counts = torch.tensor([max_tokens, 3, 0, 11], dtype=torch.int32, device=gu.DEV)
    xb = gu.dev_bits16(mo.round_to_dtype(0.5 * mo.make_activations(4, e * max_tokens, hidden, dtype), dtype),
                       dtype).view(e, max_tokens, hidden)
    ws13, ws2, out_shape = batched.workspace_shapes(max_tokens, inter, hidden, 1, e, e, None, "silu")
    assert out_shape == (e, max_tokens, hidden)
    buf13 = torch.empty(ws13, dtype=x.dtype, device=gu.DEV)
    buf2 = torch.empty(ws2, dtype=x.dtype, device=gu.DEV)
    outb = torch.full(out_shape, 9.0, dtype=x.dtype, device=gu.DEV)

    class Meta:
        expert_num_tokens = counts

    batched.apply(outb, xb, w1, w2, None, None, "silu", e, None, None, None, buf13, buf2, Meta, False)
    wantb = batched_fused_marlin_moe(xb, counts, w1, w2, None, None, s1, s2, batched.quant_type_id, w1_zeros=z1,
                                     w2_zeros=z2, output=torch.full(out_shape, 9.0, dtype=x.dtype, device=gu.DEV))
    torch.cuda.synchronize()
    assert torch.equal(outb, wantb)


def test_fused_marlin_moe_replays_in_a_hip_graph():
    """The layer reads no device value on the host, so it can be recorded; every
    replay must reproduce the eager result, also after the routing changed."""
    from sonar_amd.fused_moe import fused_marlin_moe
    from sonar_amd.scalar_type import scalar_types
    m, e, topk, hidden, inter = 6, 8, 2, 256, 128
    (w1, s1, _, _), (w2, s2, _, _) = _moe_layer(60, e, hidden, inter, 128, "bf16", False)
    x = gu.dev_bits16(mo.make_activations(1, m, hidden, "bf16"), "bf16")
    gen = torch.Generator(device="cpu").manual_seed(0)

    def routing():
        w = torch.softmax(torch.randn((m, e), generator=gen), dim=1)
        tw, ti = torch.topk(w, topk, dim=1)
        return tw.to(gu.DEV), ti.to(torch.int32).to(gu.DEV)

    tw, ti = routing()
    run = lambda: fused_marlin_moe(x, w1, w2, None, None, s1, s2, tw, ti, scalar_types.uint4b8.id)
    eager = run().clone()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        run()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            out = run()
    for rep in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
        tw2, ti2 = routing()
        tw.copy_(tw2)
        ti.copy_(ti2)
        eager = run().clone()
        torch.cuda.synchronize()


# ---------------------------------------------------------------- fp8 weights (float8_e4m3fn)
@pytest.mark.parametrize("m,k,n,g,dtype", [(1, 512, 256, -1, "fp16"), (33, 1024, 320, 128, "bf16"),
                                           (16, 4096, 4096, 128, "fp16"), (200, 256, 512, -1, "bf16")])
def test_fp8_quantise_helper_and_marlin_gemm(m, k, n, g, dtype):
    """The reference's fp8 case of its Marlin GEMM test (tests/kernels/quantization/
    test_marlin_gemm.py with marlin_quant_fp8_torch): quantise a random weight,
    run the op, compare with the matmul on the dequantised weight."""
    from sonar_amd import marlin_utils_fp8 as f8
    from sonar_amd import ops
    from sonar_amd.marlin_utils import marlin_make_workspace_new
    from sonar_amd.scalar_type import scalar_types
    gen = torch.Generator(device="cpu").manual_seed(m + k)
    weight = torch.randn((n, k), generator=gen).to(_tdt(dtype)).to(gu.DEV)
    a = (0.5 * torch.randn((m, k), generator=gen)).to(_tdt(dtype)).to(gu.DEV)
    w_ref, qweight, scales = f8.marlin_quant_fp8_torch(weight, g)
    assert qweight.shape == (k // 16, 4 * n) and scales.shape == (1 if g == -1 else k // g, n)
    out = ops.marlin_gemm(a, None, qweight, None, scales, None, None, None, None, None,
                          marlin_make_workspace_new(a.device), scalar_types.float8_e4m3fn, m, n, k)
    torch.cuda.synchronize()
    want = (a.float() @ w_ref.float()).cpu().numpy()
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(out), want)
    assert ok, worst


@pytest.mark.parametrize("mode,dtype", [("block", "bf16"), ("tensor", "fp16"), ("shards", "bf16"),
                                        ("channel", "fp16"), ("block_padded", "fp16")])
def test_prepare_fp8_layer_and_apply(mode, dtype):
    """An fp8 checkpoint layer (weight (N, K) fp8, scales per tensor / per fused
    shard / per channel / per 128 x 128 block) -> prepare_fp8_layer_for_marlin ->
    apply_fp8_marlin_linear, against the oracle on the same bytes and scales."""
    from sonar_amd import marlin_utils_fp8 as f8
    k, n = (512, 384) if mode != "block_padded" else (384, 320)   # 320 columns: padded to 384 inside
    rng = np.random.default_rng(len(mode))
    codes = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    codes[(codes & 0x7F) == 0x7F] = 0x30
    layer = types.SimpleNamespace(output_size_per_partition=n, input_size_per_partition=k, orig_dtype=_tdt(dtype))
    layer.weight = torch.from_numpy(codes.T.astype(np.uint8)).contiguous().to(gu.DEV).view(torch.float8_e4m3fn)
    g = -1
    if mode.startswith("block"):
        layer.weight_block_size = [128, 128]
        g = 128
        blocks = rng.uniform(2e-4, 2e-3, size=((n + 127) // 128, k // 128)).astype(np.float32)
        layer.weight_scale_inv = torch.from_numpy(blocks).to(gu.DEV)
        s_full = np.repeat(blocks.T, 128, axis=1)[:, :n]
    elif mode == "tensor":
        layer.weight_scale = torch.tensor(7e-4, device=gu.DEV)
        s_full = np.full((1, n), 7e-4, dtype=np.float32)
    elif mode == "shards":
        layer.logical_widths = [128, 64, 192]
        per = np.array([3e-4, 9e-4, 5e-4], dtype=np.float32)
        layer.weight_scale = torch.from_numpy(per).to(gu.DEV)
        s_full = np.repeat(per, layer.logical_widths)[None, :]
    else:
        per = rng.uniform(2e-4, 2e-3, size=n).astype(np.float32)
        layer.weight_scale = torch.from_numpy(per).to(gu.DEV)
        s_full = per[None, :]
    bias32 = mo.round_to_dtype(rng.standard_normal(n).astype(np.float32), dtype)
    layer.bias = gu.dev_bits16(bias32, dtype)
    s_full = mo.round_to_dtype(s_full, dtype)
    w_ref = mo.dequantize_fp8(codes, mo.fp8_fuse_exponent_bias(s_full, dtype), g, dtype)

    f8.prepare_fp8_layer_for_marlin(layer, size_k_first=False)
    scales = layer.weight_scale_inv if mode.startswith("block") else layer.weight_scale
    x32 = mo.make_activations(3, 5, k, dtype, std=0.5)
    y = f8.apply_fp8_marlin_linear(gu.dev_bits16(x32, dtype).view(1, 5, k), layer.weight, scales, layer.workspace,
                                   n, k, layer.bias)
    torch.cuda.synchronize()
    assert y.shape == (1, 5, n)
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(y.view(5, n)), mo.gemm_reference(x32, w_ref, bias32))
    assert ok, worst


@pytest.mark.parametrize("cfg", [
    # m, experts, topk, hidden, intermediate, dtype, scales
    (5, 4, 2, 256, 128, "fp16", "tensor"),
    (70, 4, 2, 256, 256, "bf16", "block"),
    (33, 8, 2, 128, 128, "bf16", "channel"),
    (9, 4, 2, 256, 96, "fp16", "channel"),      # intermediate size padded 96 -> 128
], ids=str)
def test_prepare_fp8_moe_layer_and_fused_marlin_moe(cfg):
    """fp8 expert weights (w13 (E, 2N, K), w2 (E, K, N)) -> prepare_fp8_moe_layer_for_marlin
    -> fused_marlin_moe, against the per-token reference on the same bytes."""
    from sonar_amd import marlin_utils_fp8 as f8
    from sonar_amd.fused_moe import fused_marlin_moe
    from sonar_amd.scalar_type import scalar_types
    m, e, topk, hidden, inter, dtype, mode = cfg
    rng = np.random.default_rng(hidden + inter + m)
    layer = types.SimpleNamespace(num_experts=e, hidden_size=hidden, intermediate_size_per_partition=inter,
                                  orig_dtype=_tdt(dtype))
    if mode == "block":
        layer.weight_block_size = [128, 128]

    def expert_set(rows, cols):   # checkpoint shape (E, rows = N of the GEMM, cols = K of the GEMM)
        codes = rng.integers(0, 256, size=(e, rows, cols), dtype=np.int32)
        codes[(codes & 0x7F) == 0x7F] = 0x30
        weight = torch.from_numpy(codes.astype(np.uint8)).to(gu.DEV).view(torch.float8_e4m3fn)
        if mode == "tensor":
            raw = rng.uniform(2e-4, 2e-3, size=e).astype(np.float32)
            full = np.broadcast_to(raw[:, None, None], (e, 1, rows))
        elif mode == "channel":
            raw = rng.uniform(2e-4, 2e-3, size=(e, rows)).astype(np.float32)
            full = raw[:, None, :]
        else:
            raw = rng.uniform(2e-4, 2e-3, size=(e, (rows + 127) // 128, cols // 128)).astype(np.float32)
            full = np.repeat(raw.transpose(0, 2, 1), 128, axis=2)[..., :rows]
        full = mo.round_to_dtype(np.ascontiguousarray(full), dtype)
        g = 128 if mode == "block" else -1
        ref = [mo.dequantize_fp8(codes[i].T, mo.fp8_fuse_exponent_bias(full[i], dtype), g, dtype) for i in range(e)]
        return weight, torch.from_numpy(raw).to(gu.DEV), ref

    w13, s13, ref13 = expert_set(2 * inter, hidden)
    w2, s2, ref2 = expert_set(hidden, inter)
    layer.w13_weight = w13
    mw13, mw2, ms13, ms2 = f8.prepare_fp8_moe_layer_for_marlin(layer, w13, w2, s13, s2)
    topk_ids, topk_w = _route(m, e, topk, m)
    x32 = mo.round_to_dtype(0.5 * mo.make_activations(m, m, hidden, dtype), dtype)
    y = fused_marlin_moe(gu.dev_bits16(x32, dtype), mw13, mw2, None, None, ms13, ms2,
                         torch.from_numpy(topk_w).to(gu.DEV), torch.from_numpy(topk_ids).to(gu.DEV),
                         scalar_types.float8_e4m3fn.id)
    torch.cuda.synchronize()
    want = _moe_reference(x32, ref13, ref2, topk_ids, topk_w, dtype)
    got = gu.host_f32(y)
    max_ref = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-2 * max_ref, (np.abs(got - want).max(), max_ref)


# ---------------------------------------------------------------- MXFP4 weights (float4_e2m1f, e8m0 block scales)
@pytest.mark.parametrize("m,k,n", [(1, 512, 256), (33, 1024, 320), (16, 2880, 5760), (200, 256, 512)])
def test_mxfp4_random_weight_helper_and_marlin_gemm(m, k, n):
    """The reference's MXFP4 case of its Marlin GEMM test (test_marlin_gemm.py with
    rand_marlin_weight_mxfp4_like): the op takes the float8_e8m0fnu scales in the
    reference's order; compared with the matmul on the dequantised weight."""
    from sonar_amd import marlin_utils_fp4 as f4
    from sonar_amd import ops
    from sonar_amd.marlin_utils import marlin_make_workspace_new
    from sonar_amd.scalar_type import scalar_types
    torch.manual_seed(m + k)
    weight = torch.empty((n, k), dtype=torch.bfloat16, device=gu.DEV)
    a = (0.5 * torch.randn((m, k), device=gu.DEV)).to(torch.bfloat16)
    w_ref, qweight, scales = f4.rand_marlin_weight_mxfp4_like(weight, 32)
    assert qweight.shape == (k // 16, 2 * n) and scales.shape == (k // 32, n)
    assert scales.dtype == torch.float8_e8m0fnu
    workspace = marlin_make_workspace_new(a.device)
    out = ops.marlin_gemm(a, None, qweight, None, scales, None, None, None, None, None, workspace,
                          scalar_types.float4_e2m1f, m, n, k)
    again = ops.marlin_gemm(a, None, qweight, None, scales, None, None, None, None, None, workspace,
                            scalar_types.float4_e2m1f, m, n, k)     # converted scales come from the cache
    torch.cuda.synchronize()
    assert torch.equal(out, again)
    want = (a.float() @ w_ref.float()).cpu().numpy()
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(out), want)
    assert ok, worst
    with pytest.raises(RuntimeError, match="bfloat16"):
        ops.marlin_gemm(a.half(), None, qweight, None, scales, None, None, None, None, None, workspace,
                        scalar_types.float4_e2m1f, m, n, k)
    with pytest.raises(RuntimeError, match="global_scale parameter must be passed for nvfp4"):
        ops.marlin_gemm(a, None, qweight, None, scales.view(torch.float8_e4m3fn), None, None, None, None, None,
                        workspace, scalar_types.float4_e2m1f, m, n, k)


@pytest.mark.parametrize("k,n", [(512, 384), (384, 320)])   # 320 columns: padded to 384 inside
def test_prepare_mxfp4_layer_and_apply(k, n):
    """An MXFP4 checkpoint layer (weight (N, K/2) bytes, low nibble first; scales
    (N, K/32) exponent bytes) -> prepare_fp4_layer_for_marlin ->
    apply_fp4_marlin_linear, against the oracle on the same bytes."""
    from sonar_amd import marlin_utils_fp4 as f4
    rng = np.random.default_rng(k + n)
    codes = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    e = rng.integers(108, 122, size=(k // 32, n)).astype(np.uint8)
    w_ref = mo.dequantize_mxfp4(codes, e)
    by_n = codes.T                                            # (N, K)
    packed = np.ascontiguousarray((by_n[:, 0::2] | (by_n[:, 1::2] << 4)).astype(np.uint8))
    layer = types.SimpleNamespace(output_size_per_partition=n, input_size_per_partition=k,
                                  params_dtype=torch.bfloat16)
    layer.weight = torch.from_numpy(packed).to(gu.DEV)
    layer.weight_scale = torch.from_numpy(np.ascontiguousarray(e.T)).to(gu.DEV)
    bias32 = mo.round_to_dtype(1e-2 * rng.standard_normal(n).astype(np.float32), "bf16")
    layer.bias = gu.dev_bits16(bias32, "bf16")
    f4.prepare_fp4_layer_for_marlin(layer)
    assert layer.weight_scale.dtype == torch.float8_e8m0fnu
    x32 = mo.make_activations(4, 6, k, "bf16", std=0.5)
    y = f4.apply_fp4_marlin_linear(gu.dev_bits16(x32, "bf16").view(2, 3, k), layer.weight, layer.weight_scale, None,
                                   layer.workspace, n, k, layer.bias)
    torch.cuda.synchronize()
    assert y.shape == (2, 3, n)
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(y.view(6, n)), mo.gemm_reference(x32, w_ref, bias32))
    assert ok, worst


@pytest.mark.parametrize("k,n", [(512, 384), (384, 320)])
def test_prepare_mxfp4_layer_and_apply_with_fp8_activations(k, n):
    """The same checkpoint layer prepared for float8_e4m3fn activations (the weight order and the scale
    order of 8-bit activations, exponent bytes plus 6): apply_fp4_marlin_linear quantises the input
    per row; against the oracle's product on the quantised-then-dequantised input."""
    from sonar_amd import marlin_utils as mu
    from sonar_amd import marlin_utils_fp4 as f4
    rng = np.random.default_rng(k + n)
    codes = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    e = rng.integers(108, 122, size=(k // 32, n)).astype(np.uint8)
    by_n = codes.T
    packed = np.ascontiguousarray((by_n[:, 0::2] | (by_n[:, 1::2] << 4)).astype(np.uint8))
    layer = types.SimpleNamespace(output_size_per_partition=n, input_size_per_partition=k,
                                  params_dtype=torch.bfloat16)
    layer.weight = torch.from_numpy(packed).to(gu.DEV)
    layer.weight_scale = torch.from_numpy(np.ascontiguousarray(e.T)).to(gu.DEV)
    bias32 = mo.round_to_dtype(1e-2 * rng.standard_normal(n).astype(np.float32), "bf16")
    layer.bias = gu.dev_bits16(bias32, "bf16")
    with pytest.raises(RuntimeError, match="MXFP4 weight \\+ INT8 activation is not supported."):
        f4.prepare_fp4_layer_for_marlin(layer, input_dtype=torch.int8)
    f4.prepare_fp4_layer_for_marlin(layer, input_dtype=torch.float8_e4m3fn)
    assert layer.weight_scale.dtype == torch.float8_e8m0fnu
    x32 = mo.make_activations(4, 6, k, "bf16", std=0.5)
    x = gu.dev_bits16(x32, "bf16")
    y = f4.apply_fp4_marlin_linear(x.view(2, 3, k), layer.weight, layer.weight_scale, None, layer.workspace, n, k,
                                   layer.bias, input_dtype=torch.float8_e4m3fn)
    torch.cuda.synchronize()
    assert y.shape == (2, 3, n) and y.dtype == torch.bfloat16
    a_q, a_s = mu.per_token_quant_fp8(x)
    want = mo.gemm_w4a8_fp4(a_q.float().cpu().numpy(), a_s.cpu().numpy(), codes, e, bias32)
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(y.view(6, n)), want)
    assert ok, worst
    with pytest.raises(RuntimeError, match="MXFP4 weight \\+ INT8 activation is not supported."):
        f4.apply_fp4_marlin_linear(x, layer.weight, layer.weight_scale, None, layer.workspace, n, k,
                                   input_dtype=torch.int8)
    with pytest.raises(RuntimeError, match="NVFP4 weight \\+ INT8/FP8 activation is not supported."):
        f4.apply_fp4_marlin_linear(x, layer.weight, layer.weight_scale, torch.ones(1, device=gu.DEV),
                                   layer.workspace, n, k, input_dtype=torch.float8_e4m3fn)
    # the op itself: c names the output type in this mode
    from sonar_amd import ops
    from sonar_amd.scalar_type import scalar_types as st
    with pytest.raises(RuntimeError, match="c must be passed for W4A8-FP4"):
        ops.marlin_gemm(a_q, None, layer.weight, None, layer.weight_scale, a_s, None, None, None, None,
                        layer.workspace, st.float4_e2m1f, 6, layer.weight.size(1) // 2, k)


# ---------------------------------------------------------------- NVFP4 weights (float4_e2m1f, e4m3 block scales, global scale)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,k,n", [(1, 512, 256), (33, 1024, 320), (16, 2880, 5760), (200, 256, 512), (700, 1024, 768)])
def test_nvfp4_random_weight_helper_and_marlin_gemm(m, k, n, dtype):
    """The reference's NVFP4 case of its Marlin GEMM test (test_marlin_gemm.py with
    rand_marlin_weight_nvfp4_like): the op takes the scale bytes and the processed
    global scale as the reference's callers hold them; compared with the matmul on
    the dequantised weight."""
    from sonar_amd import marlin_utils_fp4 as f4
    from sonar_amd import ops
    from sonar_amd.marlin_utils import marlin_make_workspace_new
    from sonar_amd.scalar_type import scalar_types
    torch.manual_seed(m + k)
    weight = torch.randn((n, k), dtype=dtype, device=gu.DEV)
    a = (0.5 * torch.randn((m, k), device=gu.DEV)).to(dtype)
    w_ref, qweight, scales, global_scale = f4.rand_marlin_weight_nvfp4_like(weight, 16)
    assert qweight.shape == (k // 16, 2 * n) and scales.shape == (k // 16, n)
    assert scales.dtype == torch.float8_e4m3fn and global_scale.dtype == torch.float32
    workspace = marlin_make_workspace_new(a.device)
    out = ops.marlin_gemm(a, None, qweight, None, scales, None, global_scale.reshape(1), None, None, None, workspace,
                          scalar_types.float4_e2m1f, m, n, k)
    again = ops.marlin_gemm(a, None, qweight, None, scales, None, global_scale.reshape(1), None, None, None,
                            workspace, scalar_types.float4_e2m1f, m, n, k)     # converted scales come from the cache
    torch.cuda.synchronize()
    assert torch.equal(out, again)
    want = (a.float() @ w_ref.float()).cpu().numpy()
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(out), want)
    assert ok, worst
    with pytest.raises(RuntimeError, match="global_scale can only be used for nvfp4"):
        ops.marlin_gemm(a, None, qweight, None, scales.view(torch.float8_e8m0fnu), None, global_scale.reshape(1),
                        None, None, None, workspace, scalar_types.float4_e2m1f, m, n, k)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("k,n", [(512, 384), (384, 320)])   # 320 columns: padded to 384 inside
def test_prepare_nvfp4_layer_and_apply(k, n, dtype):
    """An NVFP4 checkpoint layer (weight (N, K/2) bytes, low nibble first; scales
    (N, K/16) float8_e4m3fn; a global scale) -> prepare_fp4_layer_for_marlin ->
    apply_fp4_marlin_linear, against value * scale * global scale on the same bytes."""
    from sonar_amd import marlin_utils_fp4 as f4
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    rng = np.random.default_rng(k + n)
    codes = rng.integers(0, 16, size=(k, n), dtype=np.int32)
    sbytes = torch.from_numpy(rng.integers(0x28, 0x70, size=(k // 16, n)).astype(np.uint8))
    scales = sbytes.view(torch.float8_e4m3fn).float().numpy()
    g = 0.0021
    w_ref = mo.fp4_e2m1_values()[codes] * np.repeat(scales, 16, axis=0) * np.float32(g)
    by_n = codes.T                                            # (N, K)
    packed = np.ascontiguousarray((by_n[:, 0::2] | (by_n[:, 1::2] << 4)).astype(np.uint8))
    layer = types.SimpleNamespace(output_size_per_partition=n, input_size_per_partition=k, params_dtype=tdt)
    layer.weight = torch.from_numpy(packed).to(gu.DEV)
    layer.weight_scale = sbytes.T.contiguous().view(torch.float8_e4m3fn).to(gu.DEV)
    layer.weight_global_scale = torch.tensor(g, dtype=torch.float32, device=gu.DEV)
    bias32 = mo.round_to_dtype(1e-2 * rng.standard_normal(n).astype(np.float32), dtype)
    layer.bias = gu.dev_bits16(bias32, dtype)
    f4.prepare_fp4_layer_for_marlin(layer)
    assert layer.weight_scale.dtype == torch.float8_e4m3fn and layer.weight_global_scale.dtype == torch.float32
    x32 = mo.make_activations(4, 6, k, dtype, std=0.5)
    y = f4.apply_fp4_marlin_linear(gu.dev_bits16(x32, dtype).view(2, 3, k), layer.weight, layer.weight_scale,
                                   layer.weight_global_scale.reshape(1), layer.workspace, n, k, layer.bias)
    torch.cuda.synchronize()
    assert y.shape == (2, 3, n)
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(y.view(6, n)), mo.gemm_reference(x32, w_ref, bias32))
    assert ok, worst


@pytest.mark.parametrize("cfg", [
    # m, experts, topk, hidden, intermediate, bias
    (5, 4, 2, 256, 128, False),
    (70, 4, 2, 256, 256, True),
    (200, 8, 2, 128, 128, False),
    (700, 4, 2, 512, 256, True),     # 64-slot blocks, K a multiple of 256: the wide tile kernel's grouped MXFP4 form
], ids=str)
def test_prepare_moe_mxfp4_layer_and_fused_marlin_moe(cfg):
    """MXFP4 expert weights (w13 (E, 2N, K/2), w2 (E, K, N/2) bytes, exponent-byte
    scales) -> prepare_moe_mxfp4_layer_for_marlin -> fused_marlin_moe, against the
    per-token reference on the same bytes."""
    from sonar_amd import marlin_utils_fp4 as f4
    from sonar_amd.fused_moe import fused_marlin_moe
    from sonar_amd.scalar_type import scalar_types
    m, e, topk, hidden, inter, bias = cfg
    rng = np.random.default_rng(hidden + inter + m)
    layer = types.SimpleNamespace(params_dtype=torch.bfloat16)

    def expert_set(rows, cols):   # checkpoint shape (E, rows = N of the GEMM, cols = K of the GEMM)
        codes = rng.integers(0, 16, size=(e, rows, cols), dtype=np.int32)
        ex = rng.integers(116, 124, size=(e, rows, cols // 32)).astype(np.uint8)
        packed = np.ascontiguousarray((codes[:, :, 0::2] | (codes[:, :, 1::2] << 4)).astype(np.uint8))
        ref = [mo.dequantize_mxfp4(codes[i].T, np.ascontiguousarray(ex[i].T)) for i in range(e)]
        b32 = mo.round_to_dtype(0.1 * rng.standard_normal((e, rows)).astype(np.float32), "bf16") if bias else None
        return torch.from_numpy(packed).to(gu.DEV), torch.from_numpy(ex).to(gu.DEV), ref, b32

    w13, s13, ref13, b13 = expert_set(2 * inter, hidden)
    w2, s2, ref2, b2 = expert_set(hidden, inter)
    dev_bias = lambda b: None if b is None else gu.dev_bits16(b, "bf16")
    mw13, mw2, ms13, ms2, mb13, mb2 = f4.prepare_moe_mxfp4_layer_for_marlin(layer, w13, w2, s13, s2, dev_bias(b13),
                                                                            dev_bias(b2))
    topk_ids, topk_w = _route(m, e, topk, m)
    x32 = mo.round_to_dtype(0.5 * mo.make_activations(m, m, hidden, "bf16"), "bf16")
    y = fused_marlin_moe(gu.dev_bits16(x32, "bf16"), mw13, mw2, mb13, mb2, ms13, ms2,
                         torch.from_numpy(topk_w).to(gu.DEV), torch.from_numpy(topk_ids).to(gu.DEV),
                         scalar_types.float4_e2m1f.id)
    torch.cuda.synchronize()
    want = _moe_reference(x32, ref13, ref2, topk_ids, topk_w, "bf16", b13, b2)
    got = gu.host_f32(y)
    max_ref = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-2 * max_ref, (np.abs(got - want).max(), max_ref)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("cfg", [
    # m, experts, topk, hidden, intermediate
    (5, 4, 2, 256, 128),
    (70, 4, 2, 256, 256),
    (200, 8, 2, 128, 96),      # intermediate size padded to 128 inside
    (1500, 4, 2, 256, 128),    # 64-slot blocks: the tiled grouped kernel
    (40, 4, 2, 256, 128),      # 32-slot blocks: two blocks of rows per workgroup of the general grouped kernel
], ids=str)
def test_prepare_nvfp4_moe_layer_and_fused_marlin_moe(cfg, dtype):
    """NVFP4 expert weights (w13 (E, 2N, K/2), w2 (E, K, N/2) bytes, float8_e4m3fn block
    scales per 16, a global scale per expert) -> prepare_nvfp4_moe_layer_for_marlin ->
    fused_marlin_moe, against the per-token reference on value * scale * global scale."""
    from sonar_amd import marlin_utils_fp4 as f4
    from sonar_amd.fused_moe import fused_marlin_moe
    from sonar_amd.scalar_type import scalar_types
    m, e, topk, hidden, inter = cfg
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    rng = np.random.default_rng(hidden + inter + m)
    layer = types.SimpleNamespace(params_dtype=tdt, num_experts=e, hidden_size=hidden,
                                  intermediate_size_per_partition=inter)

    def expert_set(rows, cols):   # checkpoint shape (E, rows = N of the GEMM, cols = K of the GEMM)
        codes = rng.integers(0, 16, size=(e, rows, cols), dtype=np.int32)
        sb = torch.from_numpy(rng.integers(0x30, 0x60, size=(e, rows, cols // 16)).astype(np.uint8))
        sc = sb.view(torch.float8_e4m3fn).float().numpy()
        g = (0.02 + 0.01 * rng.random(e)).astype(np.float32)
        packed = np.ascontiguousarray((codes[:, :, 0::2] | (codes[:, :, 1::2] << 4)).astype(np.uint8))
        ref = [(mo.fp4_e2m1_values()[codes[i]] * np.repeat(sc[i], 16, axis=1) * g[i]).T.astype(np.float32)
               for i in range(e)]
        return (torch.from_numpy(packed).to(gu.DEV), sb.view(torch.float8_e4m3fn).to(gu.DEV),
                torch.from_numpy(g).to(gu.DEV), ref)

    w13, s13, g13, ref13 = expert_set(2 * inter, hidden)
    w2, s2, g2, ref2 = expert_set(hidden, inter)
    mw13, ms13, mg13, mw2, ms2, mg2 = f4.prepare_nvfp4_moe_layer_for_marlin(layer, w13, s13, g13, w2, s2, g2)
    assert ms13.dtype == torch.float8_e4m3fn and mg13.dtype == torch.float32 and mg13.shape == (e,)
    topk_ids, topk_w = _route(m, e, topk, m)
    x32 = mo.round_to_dtype(0.5 * mo.make_activations(m, m, hidden, dtype), dtype)
    y = fused_marlin_moe(gu.dev_bits16(x32, dtype), mw13, mw2, None, None, ms13, ms2,
                         torch.from_numpy(topk_w).to(gu.DEV), torch.from_numpy(topk_ids).to(gu.DEV),
                         scalar_types.float4_e2m1f.id, global_scale1=mg13, global_scale2=mg2)
    torch.cuda.synchronize()
    want = _moe_reference(x32, ref13, ref2, topk_ids, topk_w, dtype, None, None)
    got = gu.host_f32(y)
    max_ref = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-2 * max_ref, (np.abs(got - want).max(), max_ref)


# ---------------------------------------------------------------- MXFP8 weights (float8_e4m3fn, e8m0 block scales)
def _mxfp8_reference(codes_kn, exps_gn):
    """Oracle matrix for fp8 codes (K, N) and exponent bytes (K/32, N), bf16."""
    fused = mo.fp8_fuse_exponent_bias(mo.mx_scale_values(exps_gn), "bf16")
    return mo.dequantize_fp8(codes_kn, fused, 32, "bf16")


@pytest.mark.parametrize("m,k,n", [(3, 512, 384), (40, 384, 320), (16, 4096, 1024)])   # 320 columns: padded inside
def test_prepare_mxfp8_layer_and_apply(m, k, n):
    """An MXFP8 checkpoint layer (weight (N, K) fp8, scales (N, K/32) exponent
    bytes) -> prepare_mxfp8_layer_for_marlin -> apply_mxfp8_marlin_linear (the op
    takes the float8_e8m0fnu scales), against the oracle on the same bytes."""
    from sonar_amd import marlin_utils_fp8 as f8
    rng = np.random.default_rng(k + n + m)
    codes = rng.integers(0, 256, size=(k, n), dtype=np.int32)
    codes[(codes & 0x7F) == 0x7F] = 0x30
    e = rng.integers(112, 122, size=(k // 32, n)).astype(np.uint8)
    w_ref = _mxfp8_reference(codes, e)
    layer = types.SimpleNamespace(output_size_per_partition=n, input_size_per_partition=k)
    layer.weight = torch.from_numpy(np.ascontiguousarray(codes.T.astype(np.uint8))).to(gu.DEV).view(torch.float8_e4m3fn)
    layer.weight_scale = torch.from_numpy(np.ascontiguousarray(e.T)).to(gu.DEV)
    bias32 = mo.round_to_dtype(rng.standard_normal(n).astype(np.float32), "bf16")
    layer.bias = gu.dev_bits16(bias32, "bf16")
    f8.prepare_mxfp8_layer_for_marlin(layer)
    assert layer.weight_scale.dtype == torch.float8_e8m0fnu
    x32 = mo.make_activations(4, m, k, "bf16", std=0.5)
    y = f8.apply_mxfp8_marlin_linear(gu.dev_bits16(x32, "bf16"), layer.weight, layer.weight_scale, layer.workspace,
                                     n, k, layer.bias)
    torch.cuda.synchronize()
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(y), mo.gemm_reference(x32, w_ref, bias32))
    assert ok, worst
    with pytest.raises(RuntimeError, match="bfloat16"):
        f8.apply_mxfp8_marlin_linear(gu.dev_bits16(x32, "bf16").half(), layer.weight, layer.weight_scale,
                                     layer.workspace, n, k, None)


@pytest.mark.parametrize("cfg", [(5, 4, 2, 256, 128), (70, 4, 2, 256, 256), (9, 4, 2, 256, 96),
                                 (700, 4, 2, 512, 256)], ids=str)
def test_prepare_mxfp8_moe_layer_and_fused_marlin_moe(cfg):
    """MXFP8 expert weights -> prepare_mxfp8_moe_layer_for_marlin -> fused_marlin_moe,
    against the per-token reference on the same bytes (the third case pads the
    intermediate size 96 -> 128; the fourth runs on 64-slot blocks: the tile kernels'
    grouped form)."""
    from sonar_amd import marlin_utils_fp8 as f8
    from sonar_amd.fused_moe import fused_marlin_moe
    from sonar_amd.scalar_type import scalar_types
    m, e, topk, hidden, inter = cfg
    rng = np.random.default_rng(hidden + inter + m)
    layer = types.SimpleNamespace()

    def expert_set(rows, cols):   # checkpoint shape (E, rows = N of the GEMM, cols = K of the GEMM)
        codes = rng.integers(0, 256, size=(e, rows, cols), dtype=np.int32)
        codes[(codes & 0x7F) == 0x7F] = 0x30
        ex = rng.integers(114, 120, size=(e, rows, cols // 32)).astype(np.uint8)
        ref = [_mxfp8_reference(codes[i].T, np.ascontiguousarray(ex[i].T)) for i in range(e)]
        weight = torch.from_numpy(codes.astype(np.uint8)).to(gu.DEV).view(torch.float8_e4m3fn)
        return weight, torch.from_numpy(ex).to(gu.DEV), ref

    w13, s13, ref13 = expert_set(2 * inter, hidden)
    w2, s2, ref2 = expert_set(hidden, inter)
    mw13, mw2, ms13, ms2 = f8.prepare_mxfp8_moe_layer_for_marlin(layer, w13, w2, s13, s2)
    topk_ids, topk_w = _route(m, e, topk, m)
    x32 = mo.round_to_dtype(0.5 * mo.make_activations(m, m, hidden, "bf16"), "bf16")
    y = fused_marlin_moe(gu.dev_bits16(x32, "bf16"), mw13, mw2, None, None, ms13, ms2,
                         torch.from_numpy(topk_w).to(gu.DEV), torch.from_numpy(topk_ids).to(gu.DEV),
                         scalar_types.float8_e4m3fn.id)
    torch.cuda.synchronize()
    want = _moe_reference(x32, ref13, ref2, topk_ids, topk_w, "bf16")
    got = gu.host_f32(y)
    max_ref = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-2 * max_ref, (np.abs(got - want).max(), max_ref)


# ---------------------------------------------------------------- 8-bit activations (W4A8)
def test_marlin_int4_fp8_preprocess_reference_formulas():
    """The reference's own two tests of the op (tests/kernels/quantization/test_marlin_gemm.py:148-188)."""
    from sonar_amd import ops
    qweight_unpacked = torch.randint(0, 16, size=(2048, 2048), dtype=torch.int32, device="cuda")
    qweight_packed = (qweight_unpacked[:, ::2] * 16 + qweight_unpacked[:, 1::2]).to(torch.int8).view(torch.int32)
    res = ops.marlin_int4_fp8_preprocess(qweight_packed)
    want = torch.where(qweight_unpacked >= 8, qweight_unpacked - 8, 15 - qweight_unpacked)
    want = (want[:, ::2] * 16 + want[:, 1::2]).to(torch.int8).view(torch.int32)
    assert (res == want).all()
    assert res.data_ptr() != qweight_packed.data_ptr()
    same = ops.marlin_int4_fp8_preprocess(qweight_packed, inplace=True)
    assert same.data_ptr() == qweight_packed.data_ptr() and (qweight_packed == want).all()

    group_size = 128
    qzeros_unpacked = torch.randint(0, 16, size=(2048 // group_size, 2048), dtype=torch.int32, device="cuda")
    qweight_packed = (qweight_unpacked[:, ::2] * 16 + qweight_unpacked[:, 1::2]).to(torch.int8).view(torch.int32)
    qzeros_packed = (qzeros_unpacked[:, ::2] * 16 + qzeros_unpacked[:, 1::2]).to(torch.int8).view(torch.int32)
    res = ops.marlin_int4_fp8_preprocess(qweight_packed, qzeros_packed)
    want = qweight_unpacked - qzeros_unpacked.repeat_interleave(group_size, 0)
    want[want < 0] = 15 - qweight_unpacked[want < 0]
    want = (want[:, ::2] * 16 + want[:, 1::2]).to(torch.int8).view(torch.int32)
    assert (res == want).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_per_token_quant_ops_bit_exact(dtype):
    """int8 against the oracle, fp8 against the same formula in torch's fp32 arithmetic on the
    CPU (IEEE division and multiplication, round-to-nearest-even conversion)."""
    from oracle import marlin_oracle as mo
    from sonar_amd.marlin_utils import marlin_quant_input, per_token_quant_fp8, per_token_quant_int8
    x = torch.randn((3, 11, 520), device="cuda", dtype=dtype) * 3
    x[0, 0] = 0                                           # a row of zeros: the floors of the scales
    q, s = per_token_quant_int8(x)
    want_q, want_s = mo.per_token_quant_int8(x.float().cpu().numpy().reshape(33, 520))
    assert q.dtype == torch.int8 and s.dtype == torch.float32 and q.shape == x.shape and s.shape == (3, 11, 1)
    assert np.array_equal(q.cpu().numpy().reshape(33, 520), want_q)
    assert np.array_equal(s.cpu().numpy().reshape(33, 1), want_s)
    f, fs = per_token_quant_fp8(x)
    xc = x.float().cpu()
    want_fs = (xc.abs().amax(dim=-1, keepdim=True) / 448.0).clamp(min=1.0 / (448.0 * 512.0))
    want_f = (xc * want_fs.reciprocal()).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    assert f.dtype == torch.float8_e4m3fn and fs.shape == (3, 11, 1)
    assert torch.equal(fs.cpu(), want_fs)
    assert torch.equal(f.cpu().view(torch.uint8), want_f.view(torch.uint8))
    # a view with a row stride, and the reference's dispatcher
    wide = torch.randn((8, 1024), device="cuda", dtype=dtype)
    q2, s2 = marlin_quant_input(wide[:, :512], torch.int8)
    q3, s3 = per_token_quant_int8(wide[:, :512].contiguous())
    assert torch.equal(q2, q3) and torch.equal(s2, s3)
    with pytest.raises(ValueError, match="unsupported quant_dtype"):
        marlin_quant_input(wide, torch.float16)


@pytest.mark.parametrize("act_type", [torch.int8, torch.float8_e4m3fn])
@pytest.mark.parametrize("group_size", [-1, 128])
def test_linear_kernel_with_8bit_activations(act_type, group_size):
    """MarlinLinearKernel with act_type int8 / fp8 (marlin.py:88-163,214-235): repack with
    is_a_8bit, fp8 preprocess and scales times 512, integer group scales and
    input_global_scale; the output follows the 16-bit kernel's within the quantisation error
    of the activations."""
    from sonar_amd.marlin_linear import MarlinLinearKernel, MPLinearLayerConfig
    from sonar_amd.scalar_type import scalar_types
    from tests.quant_utils import gptq_pack, gptq_quantize_weights
    k, n, m = 512, 256, 24
    w = torch.randn((k, n), device="cuda", dtype=torch.float16)
    w_ref, q_w, s, _, _ = gptq_quantize_weights(w, scalar_types.uint4b8, k if group_size == -1 else group_size, False)
    outs = {}
    for act in (torch.float16, act_type):
        cfg = MPLinearLayerConfig(full_weight_shape=(k, n), partition_weight_shape=(k, n),
                                  weight_type=scalar_types.uint4b8, act_type=act, group_size=group_size,
                                  zero_points=False, has_g_idx=False)
        layer = types.SimpleNamespace(qweight=gptq_pack(q_w, 4, k, n), scales=s.clone(), bias=None)
        kernel = MarlinLinearKernel(cfg, w_zp_param_name=None, w_gidx_param_name=None)
        kernel.process_weights_after_loading(layer)
        if act == torch.int8:
            assert (layer.input_global_scale is not None) == (group_size != -1)
        torch.manual_seed(0)
        x = torch.randn((m, k), device="cuda", dtype=torch.float16)
        outs[act] = kernel.apply_weights(layer, x)
        assert outs[act].dtype == torch.float16 and outs[act].shape == (m, n)
    ref = torch.matmul(x, w_ref)
    rel = lambda o: (torch.mean(torch.abs(o - ref)) / torch.mean(torch.abs(ref))).item()
    assert rel(outs[torch.float16]) < 0.01
    assert rel(outs[act_type]) < 0.04


def test_w4a8_op_rejections():
    from sonar_amd import ops
    from sonar_amd.marlin_utils import marlin_make_workspace_new, per_token_quant_int8
    from sonar_amd.scalar_type import scalar_types
    from tests.marlin_utils_for_tests import marlin_quantize
    k, n, m = 256, 128, 4
    w = torch.randn((k, n), device="cuda", dtype=torch.float16)
    w_ref, q_w, s, g_idx, sort_idx, _ = marlin_quantize(w, scalar_types.uint4b8, 128, False, input_dtype=torch.int8)
    ws = marlin_make_workspace_new(w.device)
    a, a_s = per_token_quant_int8(torch.randn((m, k), device="cuda", dtype=torch.float16))

    def call(a=a, a_s=a_s, b_type=scalar_types.uint4b8, scales=s, gs=None, g=None, p=None):
        return ops.marlin_gemm(a, None, q_w, None, scales, a_s, gs, None, g, p, ws, b_type, m, n, k)

    assert call().shape == (m, n)
    with pytest.raises(RuntimeError, match="a_scales parameter must be passed for 8bit activation"):
        call(a_s=None)
    with pytest.raises(RuntimeError, match="W8A8-INT8 is not supported"):
        call(b_type=scalar_types.uint8b128)
    with pytest.raises(RuntimeError, match="global_scale can only be used for nvfp4"):
        call(gs=torch.ones(1, device="cuda"))
    with pytest.raises(RuntimeError, match="act-order is not supported with 8-bit activations"):
        perm = torch.randperm(k, device="cuda").int()
        call(g=torch.zeros(k, dtype=torch.int32, device="cuda"), p=perm)
    with pytest.raises(RuntimeError, match="a_scales can only be used for 8bit activation"):
        ops.marlin_gemm(torch.randn((m, k), device="cuda", dtype=torch.float16), None, q_w, None, s, a_s, None, None,
                        None, None, ws, scalar_types.uint4b8, m, n, k)
    with pytest.raises(RuntimeError, match="Unsupported repack config"):
        ops.gptq_marlin_repack(torch.zeros((k // 8, n), dtype=torch.int32, device="cuda"),
                               torch.randperm(k, device="cuda").int(), k, n, 4, True)
