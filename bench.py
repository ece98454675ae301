#!/usr/bin/env python3
"""Benchmark of the W4A16 Marlin-family GEMM on one MI355X.

A step is one pass over the four W4A16 projection GEMMs of a Llama-3-8B decoder
layer (qkv 4096x6144, o 4096x4096, gate_up 4096x28672, down 14336x4096;
int4 weights, group size 128) at M = 16 bf16 activation rows, through the same
torch ops the reference's callers use.  Weights of `--copies` distinct layers
are visited round-robin so that every step streams its weights from HBM: 24 by
default, because the two large matrices are copied with the non-temporal bit
and leave the 256 MB last-level cache to the two small ones, whose 24 copies
(519 MB) are what it would have to hold between two uses (with 6 copies the
step measures 4 % faster than with 12, 24 or 48, which agree).  The K timed steps are recorded in one HIP
graph; the graph is replayed `REPLAYS` times, each replay between two events on
the launching stream, and the line reports the median replay (with the 10th
and 90th percentile beside it).

The same line carries the MFMA half of the metric: the four GEMMs at M = 4096
with fp16 activations (`roofline_mfma`), timed the same way.

Prints one JSON line; `--sweep` adds the M sweep of the decode and prefill
shapes under "sweep".
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E
# HBM bytes per GEMM launch of the default workload (M = 16, 24 weight copies), from one
# `rocprofv3 --pmc FETCH_SIZE` and one `--pmc WRITE_SIZE` run of
# `bench.py --no-prefill --eager --calibrate`
# (profiles/marlin_stream_fast_kernel_llama3-8b-layer_m16_hbm-traffic.txt): FETCH_SIZE scaled
# by 2.000 and WRITE_SIZE by 1.000, the factors that make the `--calibrate` pass (256 MiB
# read, 256 MiB written) come out right.  Average over the four GEMMs of the layer.  Counters
# cannot be read from inside a run: the figure belongs to the launches of that profile
# (PROFILED_LAUNCHES: workgroups, threads per workgroup, pieces per strip, non-temporal weight
# copies, as sonar_marlin_last_decode_launch reports them) and is reported only while the run's
# own launches are the same, for M = 16 with the default number of weight copies; otherwise `traffic` is null.
MEASURED_TRAFFIC_M16 = 32_400_000
PROFILED_LAUNCHES = {"qkv": [192, 512, 2, 1], "o": [256, 512, 4, 0], "gate_up": [448, 256, 1, 1],
                     "down": [256, 512, 4, 1]}
REPLAYS = 21                # graph replays per timing; the median is reported
DEFAULT_COPIES = 24          # distinct layers visited round-robin (see the module docstring)
MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense fp16 / bf16
MFMA_PEAK_8BIT_TFLOPS = 5000.0   # MI355X dense int8 / fp8
GROUP = 128
LAYER_SHAPES = [("qkv", 4096, 6144), ("o", 4096, 4096), ("gate_up", 4096, 28672), ("down", 14336, 4096)]


def algorithmic_bytes(m: int, k: int, n: int, zeros: bool = False, act_order: bool = False) -> int:
    b = k * n // 2 + (k // GROUP) * n * 2 + m * k * 2 + m * n * 2
    if zeros:
        b += (k // GROUP) * n // 2
    if act_order:
        b += 8 * k
    return b


class Layer:
    """One quantised projection with random codes and scales, already on the
    device in the layouts the ops take."""

    def __init__(self, torch, k, n, dtype, gen):
        from sonar_amd import marlin_utils
        self.k, self.n = k, n
        dev = "cuda:0"
        self.qweight = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 16, 2 * n), dtype=torch.int32,
                                     device=dev, generator=gen)
        self.scales = (torch.rand((k // GROUP, n), device=dev, generator=gen) * 9e-3 + 1e-3).to(dtype)
        self.empty = torch.empty(0, dtype=torch.int32, device=dev)
        self.workspace = marlin_utils.marlin_make_workspace_new(torch.device(dev))

    def run(self, ops, a, wtype):
        return ops.marlin_gemm(a, None, self.qweight, None, self.scales, None, None, self.empty,
                               self.empty, self.empty, self.workspace, wtype, a.shape[0], self.n, self.k,
                               True, False, True, False)


def time_graph(torch, fn, reps, replays=REPLAYS, spread=False):
    """Records `reps` calls of fn() in a HIP graph, replays it once untimed and
    `replays` times between two events each; returns the median seconds per
    call (with `spread`: median, 10th and 90th percentile)."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        # every weight copy fn cycles through gets its one-time layout conversion here,
        # outside the graph (fn(i) uses copy i modulo the number of copies, at most 32)
        for i in range(min(reps, 32)):
            fn(i)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(reps):
                fn(i)
        graph.replay()
        stream.synchronize()
        times = []
        for _ in range(replays):
            t0 = torch.cuda.Event(enable_timing=True)
            t1 = torch.cuda.Event(enable_timing=True)
            t0.record(stream)
            graph.replay()
            t1.record(stream)
            stream.synchronize()
            times.append(t0.elapsed_time(t1) * 1e-3 / reps)
    times.sort()
    median = times[len(times) // 2]
    if spread:
        return median, times[len(times) // 10], times[(len(times) * 9) // 10]
    return median


def memory_yardsticks(torch):
    """What the box sustains on plain streaming passes over 1 GiB, with the
    framework's own kernels (not part of the product path): a reduction (reads
    1 GiB) and a copy (reads and writes 1 GiB each).  Puts the GEMM's GB/s next
    to a measured ceiling instead of the 8 TB/s headline alone."""
    x = torch.empty(256 * 1024 * 1024, dtype=torch.float32, device="cuda:0").normal_()
    y = torch.empty_like(x)
    out = {}
    for name, fn, nbytes in (("read_1GiB_GBps", lambda: x.sum(), x.numel() * 4),
                             ("copy_1GiB_GBps", lambda: y.copy_(x), 2 * x.numel() * 4)):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = torch.cuda.Event(enable_timing=True)
        t1 = torch.cuda.Event(enable_timing=True)
        t0.record()
        for _ in range(10):
            fn()
        t1.record()
        torch.cuda.synchronize()
        out[name] = round(nbytes * 10 / (t0.elapsed_time(t1) * 1e-3) / 1e9, 1)
    del x, y
    return out


def launch_floors(torch, time_graph):
    """What one launch costs and how long the chip takes to stream the weights of
    each GEMM of the layer when nothing is computed, with the yardstick kernels of
    sonar_amd/csrc/bench_floor.hip (not part of the product path): an empty kernel
    as a node of a HIP graph, and kernels that only fetch a matrix's bytes on all
    compute units, over six regions of 1 GiB / 6 in turn so that nothing comes from
    a cache, in four load styles: the decode kernel's own asynchronous copies into
    LDS without and with the non-temporal bit (`stream`, `stream_nt`: the decode kernel
    copies its weights with it), plain 16-byte loads into registers at eight wavefronts
    per SIMD (`stream_reg`), and the same with the non-temporal bit (`stream_reg_nt`)."""
    import ctypes
    from sonar_amd import build
    if not os.path.exists(build.BENCH_PATH):
        return None
    lib = ctypes.CDLL(build.BENCH_PATH)
    lib.sonar_bench_empty.argtypes = [ctypes.c_int, ctypes.c_void_p]
    lib.sonar_bench_stream.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.sonar_bench_stream_reg.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                                           ctypes.c_void_p, ctypes.c_void_p]
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    buf = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").random_(0, 256)
    sink = torch.zeros(16, dtype=torch.uint8, device="cuda:0")
    region = (1 << 30) // 6 // 4096 * 4096

    def raw_stream():
        return torch.cuda.current_stream().cuda_stream

    def check(rc):
        if rc != 0:
            raise RuntimeError("bench_floor launch failed: %d" % rc)

    out = {"empty_kernel_us": round(time_graph(torch, lambda i=0: check(lib.sonar_bench_empty(cus, raw_stream())),
                                               24) * 1e6, 2)}
    styles = {
        "stream": lambda src, nbytes: lib.sonar_bench_stream(src, nbytes, cus, 0, raw_stream()),
        "stream_nt": lambda src, nbytes: lib.sonar_bench_stream(src, nbytes, cus, 1, raw_stream()),
        "stream_reg": lambda src, nbytes: lib.sonar_bench_stream_reg(src, nbytes, 2 * cus, 0, sink.data_ptr(),
                                                                     raw_stream()),
        "stream_reg_nt": lambda src, nbytes: lib.sonar_bench_stream_reg(src, nbytes, 2 * cus, 1, sink.data_ptr(),
                                                                        raw_stream()),
    }
    for style, launch in styles.items():
        out[style] = []
        total = 0.0
        for name, k, n in LAYER_SHAPES:
            nbytes = k * n // 2 + (k // GROUP) * n * 2          # packed weights and scales
            assert nbytes <= region

            def one(i=0, nbytes=nbytes, launch=launch):
                check(launch(buf.data_ptr() + (i % 6) * region, nbytes))
            s = time_graph(torch, one, 24)
            total += s
            out[style].append({"gemm": name, "bytes": nbytes, "us": round(s * 1e6, 2),
                               "GBps": round(nbytes / s / 1e9, 1)})
        out[style + "_step_us"] = round(total * 1e6, 2)
    del buf
    return out


def cpu_baseline(threads: int):
    """The layer's CPU path (int4 dequantise + fp32 torch.matmul) from the
    oracle at M = 16: `value` on the o_proj shape (BASELINE configuration 1), and
    the same on the other three projection shapes under `layer` (a bounded sample:
    one layer's four GEMMs, 2 + 5 runs each, 20 to 30 s of CPU work)."""
    import numpy as np

    from oracle import marlin_oracle as mo
    m = 16
    rows = []
    for name, k, n in LAYER_SHAPES:
        rng = np.random.default_rng(k + n)
        q = rng.integers(0, 16, size=(k, n), dtype=np.int32)
        scales = mo.round_to_dtype(rng.uniform(1e-3, 1e-2, size=(k // GROUP, n)).astype(np.float32), "fp16")
        a = mo.make_activations(1, m, k, "fp16")
        t_full, t_mm, _ = mo.cpu_layer_baseline(mo.gptq_pack(q), scales, a, GROUP, threads, repeats=5, warmup=2)
        nbytes = algorithmic_bytes(m, k, n)
        rows.append({"gemm": name, "k": k, "n": n, "m": m, "ms": round(t_full * 1e3, 2),
                     "matmul_alone_ms": round(t_mm * 1e3, 2), "GBps": round(nbytes / t_full / 1e9, 3),
                     "gflops": round(2 * m * n * k / t_full / 1e9, 2)})
        del q, scales
    o = next(r for r in rows if r["gemm"] == "o")
    return {"value": o["GBps"], "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "o_proj 4096x4096, M=16, fp16: dequantise+matmul fp32, median of 5 "
                      f"({o['ms']:.1f} ms; matmul alone {o['matmul_alone_ms']:.1f} ms); `layer`: the same on "
                      "all four projection shapes",
            "gflops": o["gflops"], "layer": rows,
            "layer_ms": round(sum(r["ms"] for r in rows), 2)}


def variants_sweep(torch, ops, gen, time_graph):
    """K = 4096, N = 11008 at M = 1 and 512 (W4A8 also at 4096): act-order (perm gathers the columns
    of A, weights repacked in sorted-group order), AWQ (per-group zero points),
    8-bit weights (uint8b128), fp8 weights (float8_e4m3fn, scales with the
    exponent bias folded in), MXFP8 and MXFP4 weights (float8_e4m3fn /
    float4_e2m1f, exponent-byte scales per 32 rows, bf16 activations), NVFP4
    weights (float4_e2m1f, float8_e4m3fn scales per 16 rows, a global scale),
    W4A8 (uint4b8 weights in the order of 8-bit activations; int8 activations with
    16-bit integer group scales, float8_e4m3fn activations with the weights as
    marlin_int4_fp8_preprocess leaves them; one fp32 scale per activation row;
    frac_mfma is then against the 8-bit peak)."""
    from sonar_amd import marlin_utils
    from sonar_amd.scalar_type import scalar_types
    dev = "cuda:0"
    k, n = 4096, 11008
    out = []
    for name in ("act_order", "awq", "w8a16", "fp8", "mxfp8", "mxfp4", "nvfp4", "w4a8_int8", "w4a8_fp8"):
        layers = []
        words = 4 * n if name in ("w8a16", "fp8", "mxfp8") else 2 * n     # 8-bit codes: four per word
        act_dtype = torch.bfloat16 if name in ("mxfp4", "mxfp8") else torch.float16
        for _ in range(16):   # 16 x 22.5 MB of 4-bit codes: more than the 256 MB last-level cache holds
            qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 16, words), dtype=torch.int32, device=dev, generator=gen)
            sc = (torch.rand((k // GROUP, n), device=dev, generator=gen) * 9e-3 + 1e-3).to(torch.float16)
            ws = marlin_utils.marlin_make_workspace_new(torch.device(dev))
            empty = torch.empty(0, dtype=torch.int32, device=dev)
            if name == "act_order":
                g_idx = (torch.arange(k, device=dev) // GROUP).to(torch.int32)
                perm = torch.randperm(k, device=dev, generator=gen).to(torch.int32)
                layers.append((qw, sc, empty, g_idx, perm, ws, scalar_types.uint4b8))
            elif name == "w8a16":
                layers.append((qw, sc * 0.0625, empty, empty, empty, ws, scalar_types.uint8b128))
            elif name == "w4a8_int8":
                ints = torch.randint(1, 4097, (k // GROUP, n), dtype=torch.int16, device=dev, generator=gen)
                layers.append((qw, ints.view(torch.float16), empty, empty, empty, ws, scalar_types.uint4b8))
            elif name == "w4a8_fp8":
                layers.append((qw, sc * 512, empty, empty, empty, ws, scalar_types.uint4b8))
            elif name == "fp8":
                layers.append((qw, sc * 0.0625 * 256, empty, empty, empty, ws, scalar_types.float8_e4m3fn))
            elif name == "nvfp4":
                # scale bytes of the kernel-side format: top bit set, as nvfp4_marlin_process_scales leaves them
                sb = torch.randint(0x90, 0xC0, (k // 16, n), dtype=torch.uint8, device=dev, generator=gen)
                gs = torch.full((1,), 2.0 ** -3, dtype=torch.float32, device=dev)
                layers.append((qw, sb.view(torch.float8_e4m3fn), gs, empty, empty, ws, scalar_types.float4_e2m1f))
            elif name in ("mxfp4", "mxfp8"):
                e8 = torch.randint(110, 120, (k // 32, n), dtype=torch.uint8, device=dev, generator=gen)
                wt = scalar_types.float4_e2m1f if name == "mxfp4" else scalar_types.float8_e4m3fn
                layers.append((qw, e8.view(torch.float8_e8m0fnu), empty, empty, empty, ws, wt))
            else:
                zp = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // GROUP, n // 8), dtype=torch.int32, device=dev,
                                   generator=gen)
                layers.append((qw, sc, zp, empty, empty, ws, scalar_types.uint4))
        for m in (1, 512) + ((4096,) if name.startswith("w4a8") else ()):
            a = torch.randn((m, k), device=dev, generator=gen).to(act_dtype)
            a_scales = None
            if name.startswith("w4a8"):
                a, a_scales = (ops.per_token_quant_int8 if name == "w4a8_int8" else ops.per_token_quant_fp8)(a)
                a_scales = a_scales * (2.0 ** -12 if name == "w4a8_int8" else 1.0)

            def one(i=0, a=a, m=m, name=name, a_scales=a_scales):
                qw, sc, zp, g_idx, perm, ws, wt = layers[i % len(layers)]
                if a_scales is not None:
                    ops.marlin_gemm(a, None, qw, None, sc, a_scales, None, None, None, None, ws, wt, m, n, k, True,
                                    False, True, False)
                    return
                if name == "nvfp4":   # the third entry is the global scale
                    ops.marlin_gemm(a, None, qw, None, sc, None, zp, None, g_idx, perm, ws, wt, m, n, k, True,
                                    False, True, False)
                    return
                ops.marlin_gemm(a, None, qw, None, sc, None, None, zp, g_idx, perm, ws, wt, m, n, k, True,
                                False, True, False)
            s = time_graph(torch, one, 24 if m == 1 else 6)
            nb = algorithmic_bytes(m, k, n, zeros=name == "awq", act_order=name == "act_order")
            if name in ("w8a16", "fp8", "mxfp8"):
                nb += k * n // 2                        # a byte per weight instead of half
            if name in ("mxfp4", "mxfp8"):
                nb += (k // 32 - 2 * (k // GROUP)) * n  # a byte per 32 rows instead of two per 128
            if name == "nvfp4":
                nb += (k // 16 - 2 * (k // GROUP)) * n  # a byte per 16 rows
            if a_scales is not None:
                nb += 4 * m - m * k                     # a byte per activation instead of two, a scale per row
            fl = 2 * m * k * n
            peak = MFMA_PEAK_8BIT_TFLOPS if a_scales is not None else MFMA_PEAK_TFLOPS
            out.append({"variant": name, "m": m, "k": k, "n": n, "us": round(s * 1e6, 2),
                        "GBps": round(nb / s / 1e9, 1), "TFLOPs": round(fl / s / 1e12, 2),
                        "frac_hbm": round(nb / s / 1e9 / HBM_PEAK_GBPS, 4),
                        "frac_mfma": round(fl / s / 1e12 / peak, 4)})
            print("variant", json.dumps(out[-1]), file=sys.stderr, flush=True)
    return out


def moe_sweep(torch, gen, time_graph):
    """Mixtral-8x7B-shaped grouped GEMMs (8 experts, hidden 4096, intermediate
    14336, top-2, bf16) at T = 16 and 4096 tokens: gate/up GEMM, down GEMM and
    the whole layer (routing + both GEMMs + activation + sum)."""
    from sonar_amd import fused_moe, ops
    from sonar_amd.scalar_type import scalar_types
    dev = "cuda:0"
    e, hidden, inter, topk = 8, 4096, 14336, 2
    dt = torch.bfloat16
    w1 = torch.randint(-2 ** 31, 2 ** 31 - 1, (e, hidden // 16, 2 * 2 * inter), dtype=torch.int32, device=dev,
                       generator=gen)
    w2 = torch.randint(-2 ** 31, 2 ** 31 - 1, (e, inter // 16, 2 * hidden), dtype=torch.int32, device=dev,
                       generator=gen)
    s1 = (torch.rand((e, hidden // GROUP, 2 * inter), device=dev, generator=gen) * 9e-3 + 1e-3).to(dt)
    s2 = (torch.rand((e, inter // GROUP, hidden), device=dev, generator=gen) * 9e-3 + 1e-3).to(dt)
    # a second set of expert weights: the timed GEMMs alternate between the two, so that the 235 MB of the
    # down experts cannot stay in the 256 MB last-level cache from one launch to the next
    w1s = [w1, torch.randint(-2 ** 31, 2 ** 31 - 1, w1.shape, dtype=torch.int32, device=dev, generator=gen)]
    w2s = [w2, torch.randint(-2 ** 31, 2 ** 31 - 1, w2.shape, dtype=torch.int32, device=dev, generator=gen)]
    out = []
    for t in (16, 4096):
        x = torch.randn((t, hidden), device=dev, generator=gen).to(dt)
        logits = torch.randn((t, e), device=dev, generator=gen)
        tw, ti = torch.topk(torch.softmax(logits, dim=1), topk, dim=1)
        ti = ti.to(torch.int32)
        bs = fused_moe.moe_block_size(t, topk, e)
        sorted_ids, expert_ids, past = fused_moe.moe_align_block_size(ti, bs, e)
        ws = torch.zeros(1024, dtype=torch.int32, device=dev)
        h1 = torch.empty((t * topk, 2 * inter), dtype=dt, device=dev)
        h2 = torch.randn((t * topk, inter), device=dev, generator=gen).to(dt)
        y = torch.empty((t * topk, hidden), dtype=dt, device=dev)
        routed = int(torch.unique(ti).numel())

        def gemm1(i=0):
            ops.moe_wna16_marlin_gemm(x, h1, w1s[i % 2], None, s1, None, None, None, None, None, ws, sorted_ids,
                                      expert_ids, past, tw, bs, topk, False, scalar_types.uint4b8, t, 2 * inter,
                                      hidden, True, False, True, False)

        def gemm2(i=0):
            ops.moe_wna16_marlin_gemm(h2, y, w2s[i % 2], None, s2, None, None, None, None, None, ws, sorted_ids,
                                      expert_ids, past, tw, bs, 1, True, scalar_types.uint4b8, t * topk, hidden,
                                      inter, True, False, True, False)

        def layer(i=0):
            fused_moe.fused_marlin_moe(x, w1, w2, None, None, s1, s2, tw, ti, scalar_types.uint4b8.id)

        # the same codes read as MXFP4 (float4_e2m1f, an exponent byte per 32 rows)
        e1 = torch.randint(110, 120, (e, hidden // 32, 2 * inter), dtype=torch.uint8, device=dev, generator=gen)
        e2 = torch.randint(110, 120, (e, inter // 32, hidden), dtype=torch.uint8, device=dev, generator=gen)
        e1, e2 = e1.view(torch.float8_e8m0fnu), e2.view(torch.float8_e8m0fnu)

        def gemm1_mx(i=0):
            ops.moe_wna16_marlin_gemm(x, h1, w1s[i % 2], None, e1, None, None, None, None, None, ws, sorted_ids,
                                      expert_ids, past, tw, bs, topk, False, scalar_types.float4_e2m1f, t, 2 * inter,
                                      hidden, True, False, True, False)

        def gemm2_mx(i=0):
            ops.moe_wna16_marlin_gemm(h2, y, w2s[i % 2], None, e2, None, None, None, None, None, ws, sorted_ids,
                                      expert_ids, past, tw, bs, 1, True, scalar_types.float4_e2m1f, t * topk, hidden,
                                      inter, True, False, True, False)

        # the same codes in the order of 8-bit activations, int8 tokens with a scale a row, 16-bit integer
        # group scales; blocks of at least 16 slots (marlin_moe.py:328-329)
        bs8 = max(bs, 16)
        sorted8, experts8, past8 = (sorted_ids, expert_ids, past) if bs8 == bs else \
            fused_moe.moe_align_block_size(ti, bs8, e)
        i1 = torch.randint(1, 4097, (e, hidden // GROUP, 2 * inter), dtype=torch.int16, device=dev,
                           generator=gen).view(dt)
        i2 = torch.randint(1, 4097, (e, inter // GROUP, hidden), dtype=torch.int16, device=dev, generator=gen).view(dt)
        xq, xs = ops.per_token_quant_int8(x)
        h2q, h2s = ops.per_token_quant_int8(h2)
        xs, h2s = xs * 2.0 ** -12, h2s * 2.0 ** -12

        def gemm1_a8(i=0):
            ops.moe_wna16_marlin_gemm(xq, h1, w1s[i % 2], None, i1, xs, None, None, None, None, ws, sorted8, experts8, past8,
                                      tw, bs8, topk, False, scalar_types.uint4b8, t, 2 * inter, hidden, True, False,
                                      True, False)

        def gemm2_a8(i=0):
            ops.moe_wna16_marlin_gemm(h2q, y, w2s[i % 2], None, i2, h2s, None, None, None, None, ws, sorted8, experts8, past8,
                                      tw, bs8, 1, True, scalar_types.uint4b8, t * topk, hidden, inter, True, False,
                                      True, False)

        reps = 8 if t == 16 else 2
        cases = [("gate_up", gemm1, hidden, 2 * inter, t, GROUP, 2), ("down", gemm2, inter, hidden, t * topk, GROUP, 2),
                 ("gate_up (mxfp4)", gemm1_mx, hidden, 2 * inter, t, 32, 1),
                 ("down (mxfp4)", gemm2_mx, inter, hidden, t * topk, 32, 1),
                 ("gate_up (w4a8 int8)", gemm1_a8, hidden, 2 * inter, t, GROUP, 2),
                 ("down (w4a8 int8)", gemm2_a8, inter, hidden, t * topk, GROUP, 2)]
        for name, fn, k, n, rows, group, scale_bytes in cases:
            s = time_graph(torch, fn, reps)
            weights = routed * (k * n // 2 + (k // group) * n * scale_bytes)
            a8 = "w4a8" in name
            nb = weights + rows * k * (1 if a8 else 2) + t * topk * n * 2 + sorted_ids.numel() * 4 + \
                expert_ids.numel() * 4
            fl = 2 * t * topk * n * k
            out.append({"tokens": t, "gemm": name, "block_size": bs, "experts_routed": routed,
                        "us": round(s * 1e6, 1), "GBps": round(nb / s / 1e9, 1), "TFLOPs": round(fl / s / 1e12, 2),
                        "frac_hbm": round(nb / s / 1e9 / HBM_PEAK_GBPS, 4),
                        "frac_mfma": round(fl / s / 1e12 / (MFMA_PEAK_8BIT_TFLOPS if a8 else MFMA_PEAK_TFLOPS), 4)})
            print("moe", json.dumps(out[-1]), file=sys.stderr, flush=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            layer()
        torch.cuda.synchronize()
        out.append({"tokens": t, "gemm": "whole layer (eager)", "us": round((time.perf_counter() - t0) / reps * 1e6, 1)})
        print("moe", json.dumps(out[-1]), file=sys.stderr, flush=True)
        # routing, both GEMMs, activation and sum recorded in one HIP graph
        out.append({"tokens": t, "gemm": "whole layer (graph)", "us": round(time_graph(torch, layer, reps) * 1e6, 1)})
        print("moe", json.dumps(out[-1]), file=sys.stderr, flush=True)
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--m", type=int, default=16, help="activation rows of the decode step (1..64)")
    ap.add_argument("--copies", type=int, default=DEFAULT_COPIES)
    ap.add_argument("--sweep", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-prefill", action="store_true", help="skip the M = 4096 half of the metric")
    ap.add_argument("--eager", action="store_true",
                    help="time the K steps launched one by one instead of in a HIP graph (for counter runs)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run three elementwise passes over 256 MiB (read 256 MiB, write 256 MiB each) so "
                         "a counter run has a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the GEMM is rank-local; no multi-GPU path "
              "exists); run with --gpus 1", file=sys.stderr)
        return 2
    if not 1 <= args.m <= 64:
        print("bench.py: --m is the row count of the decode step, 1..64 (the M = 4096 half of the metric is "
              "always timed beside it; --sweep covers every other M)", file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py: needs a GPU", file=sys.stderr)
        return 2
    from sonar_amd import ops
    from sonar_amd.scalar_type import scalar_types
    torch.cuda.set_device(0)
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(1234)
    dtype = torch.bfloat16
    wtype = scalar_types.uint4b8
    m = args.m

    copies = [[Layer(torch, k, n, dtype, gen) for (_, k, n) in LAYER_SHAPES] for _ in range(args.copies)]
    acts = {k: torch.randn((m, k), device="cuda:0", generator=gen).to(dtype) for k in (4096, 14336)}

    def step(i=0):
        for layer in copies[i % args.copies]:
            layer.run(ops, acts[layer.k], wtype)

    # warm-up (also converts every weight to the streaming order, once)
    for i in range(max(args.warmup, args.copies)):
        step(i)
    torch.cuda.synchronize()

    # the launch every GEMM of the step makes (read back from the library, one eager call each)
    import ctypes
    from sonar_amd import _lib
    lib = _lib.load()
    launch_shapes = {}
    for idx, (name, k, n) in enumerate(LAYER_SHAPES):
        copies[0][idx].run(ops, acts[k], wtype)
        shape = (ctypes.c_int32 * 4)()
        lib.sonar_marlin_last_decode_launch(shape, 4)
        launch_shapes[name] = list(shape)
    torch.cuda.synchronize()

    if args.calibrate:
        x = torch.zeros(64 * 1024 * 1024, dtype=torch.int32, device="cuda:0")
        for _ in range(3):
            y = x + 1
        torch.cuda.synchronize()
        del x, y

    # eager timing: K steps launched one by one
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    eager_s = (time.perf_counter() - t0) / args.steps

    # timed region: exactly K steps in one graph, events on the launching stream; median of REPLAYS replays
    torch.cuda.synchronize()
    if args.eager:
        step_s = p10 = p90 = eager_s
    else:
        step_s, p10, p90 = time_graph(torch, step, args.steps, spread=True)

    step_bytes = sum(algorithmic_bytes(m, k, n) for (_, k, n) in LAYER_SHAPES)
    step_flops = sum(2 * m * k * n for (_, k, n) in LAYER_SHAPES)
    launches = len(LAYER_SHAPES)
    gbps = step_bytes / step_s / 1e9

    per_gemm = []
    for idx, (name, k, n) in enumerate(LAYER_SHAPES):
        def one(i=0, idx=idx, k=k):
            copies[i % args.copies][idx].run(ops, acts[k], wtype)
        if args.eager:
            s = lo = hi = eager_s
        else:
            s, lo, hi = time_graph(torch, one, max(24, args.copies * 4), spread=True)
        nb = algorithmic_bytes(m, k, n)
        per_gemm.append({"gemm": name, "k": k, "n": n, "m": m, "us": round(s * 1e6, 2),
                         "us_p10": round(lo * 1e6, 2), "us_p90": round(hi * 1e6, 2),
                         "GBps": round(nb / s / 1e9, 1), "frac_hbm": round(nb / s / 1e9 / HBM_PEAK_GBPS, 4)})

    kernel = "marlin_stream_fast_kernel<bf16>"
    if m > 16:
        kernel += " (blocks of 16 or 32 rows per workgroup)"
    out = {
        "metric": "W4A16 GEMM TFLOP/s + HBM GB/s (% roofline), Llama-3-8B shapes, M=1..8192",
        "value": round(gbps, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 5),
        "ms_per_step_p10": round(p10 * 1e3, 5),
        "ms_per_step_p90": round(p90 * 1e3, 5),
        "replays": 1 if args.eager else REPLAYS,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"llama3-8b decoder layer W4A16 GEMMs (qkv+o+gate_up+down), M={m}, "
                               f"bf16 activations, uint4b8 weights, group_size 128, {args.copies} "
                               f"weight copies round-robin, K steps in one HIP graph, median of {REPLAYS} replays",
                   "global_batch": m},
        "tflops": round(step_flops / step_s / 1e12, 2),
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC_M16 if (m == 16 and args.copies == DEFAULT_COPIES and
                                                         launch_shapes == PROFILED_LAUNCHES) else None,
                     "launches": launch_shapes,
                     "kernel": kernel,
                     "bytes_per_launch": step_bytes // launches,
                     "us_per_launch": round(step_s / launches * 1e6, 3)},
        "eager_ms_per_step": round(eager_s * 1e3, 5),
        "per_gemm": per_gemm,
    }

    if not args.no_prefill:
        # the MFMA half of the metric: the same four GEMMs at M = 4096, fp16 activations ~ N(0, 0.5)
        pm = 4096
        fl_layers = [[Layer(torch, k, n, torch.float16, gen) for (_, k, n) in LAYER_SHAPES] for _ in range(2)]
        pa = {k: (torch.randn((pm, k), device="cuda:0", generator=gen) * 0.5).to(torch.float16) for k in (4096, 14336)}

        def prefill_step(i=0):
            for layer in fl_layers[i % 2]:
                layer.run(ops, pa[layer.k], wtype)

        def timed(fn, reps):
            """(median, p10, p90) seconds per call of fn: graph replays, or with --eager `reps` plain launches."""
            if not args.eager:
                return time_graph(torch, fn, reps, spread=True)
            for i in range(2):
                fn(i)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(reps):
                fn(i)
            torch.cuda.synchronize()
            dt = (time.perf_counter() - t0) / reps
            return dt, dt, dt

        ps, plo, phi = timed(prefill_step, 4)
        pflops = sum(2 * pm * k * n for (_, k, n) in LAYER_SHAPES)
        per_prefill = []
        for idx, (name, k, n) in enumerate(LAYER_SHAPES):
            def one(i=0, idx=idx, k=k):
                fl_layers[i % 2][idx].run(ops, pa[k], wtype)
            s, lo, hi = timed(one, 4)
            fl = 2 * pm * k * n
            per_prefill.append({"gemm": name, "k": k, "n": n, "m": pm, "us": round(s * 1e6, 1),
                                "us_p10": round(lo * 1e6, 1), "us_p90": round(hi * 1e6, 1),
                                "TFLOPs": round(fl / s / 1e12, 1),
                                "frac_mfma": round(fl / s / 1e12 / MFMA_PEAK_TFLOPS, 4)})
        out["roofline_mfma"] = {"bound": "mfma", "achieved": round(pflops / ps / 1e12, 1), "peak": MFMA_PEAK_TFLOPS,
                                "unit": "TFLOP/s", "frac": round(pflops / ps / 1e12 / MFMA_PEAK_TFLOPS, 4),
                                "kernel": "marlin_tile_wide_kernel<f16> (+ tile_reduce_kernel where K is split)",
                                "workload": "the four GEMMs of the layer at M=4096, fp16 activations ~ N(0,0.5), "
                                            + ("4 plain launches of the step" if args.eager else
                                               f"4 steps per graph, median of {REPLAYS} replays"),
                                "flops_per_launch": pflops // launches,
                                "us_per_launch": round(ps / launches * 1e6, 2),
                                "ms_per_step": round(ps * 1e3, 4), "ms_per_step_p10": round(plo * 1e3, 4),
                                "ms_per_step_p90": round(phi * 1e3, 4), "per_gemm": per_prefill}
        del fl_layers, pa

    if args.sweep:
        sweep = []
        for (regime, ms, dt) in (("decode", (1, 2, 4, 8, 16, 32, 64), torch.bfloat16),
                                 ("prefill", (256, 1024, 4096, 8192), torch.float16)):
            layers = copies if dt == dtype else [[Layer(torch, k, n, dt, gen) for (_, k, n) in LAYER_SHAPES]
                                                 for _ in range(2)]
            for mm in ms:
                for idx, (name, k, n) in enumerate(LAYER_SHAPES):
                    a = torch.randn((mm, k), device="cuda:0", generator=gen).to(dt)
                    if regime == "prefill":
                        a = a * 0.5

                    def one(i=0, idx=idx, a=a, layers=layers):
                        layers[i % len(layers)][idx].run(ops, a, wtype)
                    reps = 24 if regime == "decode" else 4
                    s = time_graph(torch, one, reps)
                    nb = algorithmic_bytes(mm, k, n)
                    fl = 2 * mm * k * n
                    sweep.append({"regime": regime, "gemm": name, "m": mm, "k": k, "n": n,
                                  "us": round(s * 1e6, 2), "GBps": round(nb / s / 1e9, 1),
                                  "TFLOPs": round(fl / s / 1e12, 2),
                                  "frac_hbm": round(nb / s / 1e9 / HBM_PEAK_GBPS, 4),
                                  "frac_mfma": round(fl / s / 1e12 / MFMA_PEAK_TFLOPS, 4)})
                    if regime == "prefill" and mm >= 4096:
                        # yardstick: the vendor library's dense 16-bit GEMM on the same activations
                        # and a dense matrix of the same shape (what the box sustains on this much
                        # matrix work with real data; not part of the product path)
                        w_dense = torch.randn((k, n), device="cuda:0", generator=gen).to(dt) * 0.05

                        def dense(i=0, a=a, w_dense=w_dense):
                            torch.matmul(a, w_dense)
                        sd = time_graph(torch, dense, reps)
                        sweep[-1]["dense_matmul_TFLOPs"] = round(fl / sd / 1e12, 2)
                        del w_dense
                    print("sweep", json.dumps(sweep[-1]), file=sys.stderr, flush=True)
        out["sweep"] = sweep
        out["variants"] = variants_sweep(torch, ops, gen, time_graph)
        out["moe"] = moe_sweep(torch, gen, time_graph)

    out["yardsticks"] = memory_yardsticks(torch)
    floors = launch_floors(torch, time_graph)
    if floors is not None:
        out["floors"] = floors
        # how far the step is from a kernel that only streams the same weights (the faster of the copy styles)
        floor_us = min(floors[k] for k in floors if k.endswith("_step_us"))
        out["roofline"]["stream_floor_us"] = floor_us
        out["roofline"]["step_over_stream_floor"] = round(step_s * 1e6 / floor_us, 3)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(min(os.cpu_count() or 1, 16))
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
