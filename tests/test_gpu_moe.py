"""GPU parity of the grouped (mixture-of-experts) W4A16 GEMM, through the C ABI,
against the oracle's restatement of moe_wna16_marlin_gemm
(csrc/libtorch_stable/moe/marlin_moe_wna16/ops.cu:544-897).  The routing
(moe_align_block_size) is the oracle's; the cases follow
tests/kernels/moe/test_moe.py:560-700 (experts, top-k, group sizes, act-order,
zero points) at sizes the oracle finishes in seconds."""
from __future__ import annotations

import os

import numpy as np
import pytest
import torch

from oracle import marlin_oracle as mo
from sonar_amd import _lib
from tests import gpu_util as gu

pytestmark = pytest.mark.gpu


class Experts:
    def __init__(self, seed, e, k, n, group_size, dtype, zero_points=False, act_order=False, bias=False):
        self.layers = [gu.DeviceLayer(seed + 17 * i, k, n, group_size, dtype, zero_points, act_order, bias)
                       for i in range(e)]
        first = self.layers[0]
        self.e, self.k, self.n, self.dtype = e, k, n, dtype
        self.groups, self.b_type = first.groups, first.b_type
        cat = lambda name: (torch.stack([getattr(l, name) for l in self.layers]).contiguous()
                            if getattr(first, name) is not None else None)
        self.native = cat("native")
        self.scales = cat("scales")
        self.zeros = cat("zeros")
        self.bias = cat("bias")
        self.g_idx = cat("g_idx")
        self.perm = cat("perm")
        self.workspace = first.workspace

    def reference(self, a32, sorted_ids, expert_ids, past, bs, top_k, m, weights):
        w = [l.w_ref for l in self.layers]
        if self.bias is None:
            return mo.moe_gemm_reference(a32, w, sorted_ids, expert_ids, past, bs, top_k, m, weights, self.dtype)
        # bias is added before the routing weight is applied
        out = np.zeros((m * top_k, self.n), dtype=np.float32)
        for b in range(past // bs):
            ex = int(expert_ids[b])
            if ex < 0:
                continue
            ids = sorted_ids[b * bs:(b + 1) * bs]
            ids = ids[ids < m * top_k]
            c = mo.round_to_dtype(a32[ids // top_k] @ w[ex] + self.layers[ex].bias32[None, :], self.dtype)
            if weights is not None:
                wt = mo.round_to_dtype(weights.reshape(-1)[ids].astype(np.float32), self.dtype)
                c = mo.round_to_dtype(c * wt[:, None], self.dtype)
            out[ids] = c
        return out

    def gemm(self, a, sorted_ids, expert_ids, past, weights, bs, top_k, m, mul, scratch=True, permuted_copy=False):
        lib = _lib.load()
        tdt = torch.float16 if self.dtype == "fp16" else torch.bfloat16
        c = torch.zeros((m * top_k, self.n), dtype=tdt, device=gu.DEV)
        sid = gu.dev_i32(sorted_ids)
        eid = gu.dev_i32(expert_ids)
        npp = gu.dev_i32(np.array([past], dtype=np.int32))
        tw = torch.from_numpy(weights.astype(np.float32).reshape(-1)).to(gu.DEV) if weights is not None else None
        nbytes = lib.sonar_moe_marlin_gemm_scratch_bytes(sid.numel(), bs, self.n, self.k) if scratch else 0
        if permuted_copy:   # act-order: room for a column-permuted copy of A per slot
            nbytes = (nbytes + 255) // 256 * 256 + sid.numel() * self.k * 2
        scr = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=gu.DEV) if scratch else None
        _lib.check(lib.sonar_moe_wna16_marlin_gemm(
            gu.ptr(a), gu.ptr(c), gu.ptr(self.native), _lib.LAYOUT_GFX950, gu.ptr(self.bias),
            gu.ptr(self.scales), gu.ptr(self.zeros), gu.ptr(self.g_idx), gu.ptr(self.perm),
            gu.ptr(self.workspace), self.workspace.numel(), gu.ptr(scr), nbytes, gu.ptr(sid), sid.numel(),
            gu.ptr(eid), gu.ptr(npp), gu.ptr(tw), bs, top_k, int(mul), self.e,
            gu.dtype_code(self.dtype), self.b_type, m, self.n, self.k, self.groups, 1, 0, 1, gu.stream()))
        torch.cuda.synchronize()
        return c


def route(seed, m, e, top_k):
    rng = np.random.default_rng(seed)
    ids = np.stack([rng.permutation(e)[:top_k] for _ in range(m)]).astype(np.int32)
    w = rng.random((m, top_k)).astype(np.float32)
    w /= w.sum(axis=1, keepdims=True)
    return ids, w


# (m, e, top_k, k, n, group, dtype, zero_points, act_order, bias, block_size or None, mul)
MOE_CASES = [
    (1, 8, 2, 256, 128, 128, "fp16", False, False, False, None, False),
    (7, 8, 2, 512, 256, 128, "bf16", False, False, False, None, True),
    (33, 4, 2, 512, 192, 64, "fp16", True, False, False, None, True),
    (64, 8, 3, 384, 128, 32, "bf16", False, False, True, None, True),
    (20, 4, 1, 256, 128, -1, "fp16", False, False, False, None, False),
    (40, 6, 2, 512, 128, 128, "fp16", False, True, False, None, True),
    (16, 8, 2, 256, 128, 128, "bf16", True, False, False, 8, False),
    (150, 4, 2, 256, 256, 128, "fp16", False, False, False, 48, True),
    (222, 3, 2, 288, 128, 32, "bf16", False, False, False, 64, True),
    (5, 64, 6, 256, 128, 128, "fp16", False, False, False, 16, True),
    # 64-slot blocks with groups of at least 64 rows: the MFMA-tiled grouped kernel
    (300, 4, 2, 512, 256, 128, "fp16", False, False, False, 64, True),
    (513, 3, 2, 256, 320, 64, "bf16", True, False, True, 64, True),
    (90, 8, 2, 384, 128, -1, "fp16", False, False, False, 64, False),
    (1100, 2, 1, 128, 512, 128, "bf16", False, False, True, 64, False),
    (900, 2, 2, 256, 512, 32, "fp16", True, False, True, 64, True),      # groups of 32 rows in the tile kernel
    # K of 16 steps or more in whole passes of four: the wide kernel cuts its few tiles along K on the device
    # (fp32 partial tiles through scratch, moe_tile_reduce_kernel); act-order through the permuted copy
    (700, 4, 2, 1024, 320, 128, "fp16", False, False, False, 64, True),
    (900, 3, 2, 2048, 256, 128, "bf16", True, False, True, 64, False),
    (640, 5, 2, 1280, 192, 64, "bf16", False, False, True, 64, True),
    (650, 2, 2, 1024, 256, 128, "fp16", False, True, False, 64, True),
    # groups of 32 rows in the grouped tile kernel: the other activation type, with and without zero points
    (700, 2, 2, 256, 512, 32, "bf16", False, False, False, 64, True),
    (700, 2, 2, 256, 512, 32, "fp16", False, False, True, 64, False),
    (700, 2, 2, 512, 256, 32, "bf16", True, False, False, 64, True),
    # fp16 with zero points on 64-slot blocks: 256- and 128-row tiles, without and with the K split
    (600, 4, 2, 512, 256, 128, "fp16", True, False, True, 64, True),
    (500, 3, 2, 1024, 320, 64, "fp16", True, False, False, 64, False),
    # more tiles than compute units with a short last round (9 row tiles x 33 = 297) and K of 48 steps
    (1100, 3, 2, 3072, 8448, 128, "bf16", False, False, True, 64, True),
    # blocks of 16 slots on more (block, strip) pairs than compute units: the decode kernel's workgroups of
    # four wavefronts, with one, two and four groups per 128 rows, both activation types, with and without
    # zero points
    (200, 4, 2, 256, 1024, 128, "fp16", False, False, False, 16, True),
    (200, 4, 2, 256, 1024, 128, "fp16", True, False, True, 16, False),
    (200, 4, 2, 256, 1024, 128, "bf16", True, False, False, 16, True),
    (200, 4, 2, 256, 1024, 64, "fp16", False, False, True, 16, True),
    (200, 4, 2, 256, 1024, 64, "fp16", True, False, False, 16, True),
    (200, 4, 2, 256, 1024, 64, "bf16", False, False, False, 16, False),
    (200, 4, 2, 256, 1024, 64, "bf16", True, False, True, 16, True),
    (200, 4, 2, 256, 1024, 32, "fp16", False, False, False, 16, True),
    (200, 4, 2, 256, 1024, 32, "fp16", True, False, True, 16, True),
    (200, 4, 2, 256, 1024, 32, "bf16", False, False, True, 16, False),
    (200, 4, 2, 256, 1024, 32, "bf16", True, False, False, 16, True),
    # ... blocks of 32 slots (two blocks of rows per workgroup) with zero points, and eight wavefronts on two groups
    (200, 4, 2, 256, 1024, 128, "bf16", True, False, False, 32, True),
    (10, 4, 2, 256, 256, 64, "bf16", True, False, True, 16, True),
    # 64-slot blocks, more slots than the decode kernel takes, K of 10 steps (not a whole number of the wide
    # kernel's passes of four): the eight-wavefront grouped tile kernel, with groups of 128, 64 and 32 rows
    (700, 2, 2, 640, 256, 128, "fp16", False, False, True, 64, True),
    (700, 2, 2, 640, 256, 64, "fp16", True, False, False, 64, False),
    (700, 2, 2, 640, 256, 32, "bf16", False, False, False, 64, True),
    (700, 2, 2, 640, 256, 32, "bf16", True, False, True, 64, True),
    (700, 2, 2, 640, 256, 32, "fp16", False, False, True, 64, False),
    (700, 2, 2, 640, 256, 32, "fp16", True, False, False, 64, True),
    # K = 192 is not a whole number of the decode kernel's 128-row units: the general grouped kernel
    (9, 4, 2, 192, 128, 64, "fp16", True, False, False, 16, True),
    # act-order on blocks of 48 slots: the gathering kernel with three blocks of rows, then the permuted copy
    (100, 3, 2, 512, 128, 128, "fp16", False, True, False, 48, True),
]


@pytest.mark.parametrize("case", MOE_CASES, ids=lambda c: "-".join(str(x) for x in c))
def test_moe_gemm_within_tolerance(case):
    m, e, top_k, k, n, g, dtype, zp, act, bias, bs, mul = case
    print("moe case", case, flush=True)
    ex = Experts(500 + m, e, k, n, g, dtype, zp, act, bias)
    topk_ids, topk_w = route(m, m, e, top_k)
    if bs is None:
        bs = mo.moe_block_size_rule(m, top_k, e)
    sorted_ids, expert_ids, past = mo.moe_align_block_size(topk_ids, bs, e)
    a32 = mo.make_activations(m + 3, m, k, dtype)
    a = gu.dev_bits16(a32, dtype)
    got = gu.host_f32(ex.gemm(a, sorted_ids, expert_ids, int(past[0]), topk_w, bs, top_k, m, mul))
    want = ex.reference(a32, sorted_ids, expert_ids, int(past[0]), bs, top_k, m, topk_w if mul else None)
    # every row of C is produced by exactly one slot
    assert np.all(np.isfinite(got))
    ok, *worst = mo.gemm_tolerance_ok(got, want)
    assert ok, worst
    if act:   # with room for the permuted copy of A the kernels without a gather run
        got = gu.host_f32(ex.gemm(a, sorted_ids, expert_ids, int(past[0]), topk_w, bs, top_k, m, mul,
                                  permuted_copy=True))
        ok, *worst = mo.gemm_tolerance_ok(got, want)
        assert ok, worst


def _random_moe_cases(count=int(os.environ.get("SONAR_RANDOM_CASES", "32"))):
    """Seeded draws over tokens, experts, top_k, shapes, group sizes, block sizes
    (8, 16, 32, 48, 64 or the reference's rule), zero points, act-order, bias."""
    rng = np.random.default_rng(77)
    cases = []
    while len(cases) < count:
        m = int(rng.choice([1, 3, 16, 17, 40, 64, 130, 300, 700]))
        e = int(rng.choice([2, 4, 8, 16]))
        top_k = int(rng.choice([1, 2, 4]))
        if top_k > e:
            continue
        k = int(rng.choice([128, 256, 384, 512]))
        n = int(rng.choice([64, 128, 256, 320]))
        g = int(rng.choice([32, 64, 128, -1]))
        if g != -1 and k % g != 0:
            continue
        zp = bool(rng.integers(0, 2))
        act = (not zp) and g != -1 and k // g > 1 and bool(rng.integers(0, 4) == 0)
        bs = rng.choice([None, 8, 16, 32, 48, 64])
        cases.append((m, e, top_k, k, n, g, "fp16" if rng.integers(0, 2) else "bf16", zp, act,
                      bool(rng.integers(0, 2)), None if bs is None else int(bs), bool(rng.integers(0, 2))))
    return cases


@pytest.mark.parametrize("case", _random_moe_cases(), ids=lambda c: "-".join(str(x) for x in c))
def test_random_moe_cases_against_oracle(case):
    test_moe_gemm_within_tolerance(case)


@pytest.mark.parametrize("copy", [False, True], ids=["gather", "permuted_copy"])
@pytest.mark.parametrize("cfg", [(9, 4, 2, 16, "fp16", True), (70, 3, 2, 32, "bf16", False), (200, 2, 1, 64, "fp16", True),
                                 (9, 4, 2, 16, "bf16", False), (70, 3, 2, 32, "fp16", True), (100, 2, 2, 48, "fp16", True),
                                 (100, 2, 2, 48, "bf16", True), (200, 2, 1, 64, "bf16", False)],
                         ids=str)
def test_moe_act_order_shard_without_whole_groups(cfg, copy):
    """Row-parallel shards of act-order experts (is_k_full = False; the
    reference's scenario (133, 256, 256, 5, 2, 1, act_order, k_full = False),
    tests/kernels/moe/test_moe.py:688-710): the shard's rows lie in all groups
    and every row finds its scale through g_idx.  `copy`: with room for a
    column-permuted copy of A per slot the kernels run without the gather."""
    m, e, top_k, bs, dtype, mul = cfg
    k_full, n, g = 1024, 192, 128
    lo, hi = 384, 768
    k = hi - lo
    native, scales, perms, g_sorted_all, w_ref = [], [], [], [], []
    for i in range(e):
        full = mo.make_layer(700 + i, k_full, n, g, dtype, act_order=True)
        q, g_idx = full["q"][lo:hi], full["g_idx"][lo:hi]
        assert np.bincount(g_idx, minlength=k_full // g).max() < g     # no whole group in the shard
        w_ref.append(mo.dequantize(q, full["scales"], g, dtype, g_idx=g_idx))
        g_sorted, order = mo.stable_sort_g_idx(g_idx)
        perm = gu.dev_i32(order)
        native.append(gu.to_gfx950(gu.gptq_repack(gu.dev_i32(mo.gptq_pack(q)), perm, k, n), k, n))
        scales.append(gu.dev_bits16(mo.marlin_permute_scales(full["scales"], k_full, n, g), dtype))
        perms.append(perm)
        g_sorted_all.append(gu.dev_i32(g_sorted))
    native, scales = torch.stack(native).contiguous(), torch.stack(scales).contiguous()
    perm, g_dev = torch.stack(perms).contiguous(), torch.stack(g_sorted_all).contiguous()
    topk_ids, topk_w = route(m + 1, m, e, top_k)
    sorted_ids, expert_ids, past = mo.moe_align_block_size(topk_ids, bs, e)
    a32 = mo.make_activations(m + 9, m, k, dtype, std=0.5)
    a = gu.dev_bits16(a32, dtype)
    lib = _lib.load()
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    c = torch.zeros((m * top_k, n), dtype=tdt, device=gu.DEV)
    sid, eid = gu.dev_i32(sorted_ids), gu.dev_i32(expert_ids)
    npp = gu.dev_i32(np.array([int(past[0])], dtype=np.int32))
    tw = torch.from_numpy(topk_w.astype(np.float32).reshape(-1)).to(gu.DEV)
    workspace = torch.zeros(1024, dtype=torch.int32, device=gu.DEV)
    scr, nbytes = None, 0
    if copy:
        nbytes = (lib.sonar_moe_marlin_gemm_scratch_bytes(sid.numel(), bs, n, k) + 255) // 256 * 256 + sid.numel() * k * 2
        scr = torch.empty(nbytes, dtype=torch.uint8, device=gu.DEV)
    _lib.check(lib.sonar_moe_wna16_marlin_gemm(
        gu.ptr(a), gu.ptr(c), gu.ptr(native), _lib.LAYOUT_GFX950, None, gu.ptr(scales), None, gu.ptr(g_dev),
        gu.ptr(perm), gu.ptr(workspace), workspace.numel(), gu.ptr(scr), nbytes, gu.ptr(sid), sid.numel(), gu.ptr(eid),
        gu.ptr(npp), gu.ptr(tw), bs, top_k, int(mul), e, gu.dtype_code(dtype), _lib.TYPE_UINT4B8, m, n, k,
        k_full // g, 0, 0, 1, gu.stream()))
    torch.cuda.synchronize()
    want = mo.moe_gemm_reference(a32, w_ref, sorted_ids, expert_ids, int(past[0]), bs, top_k, m,
                                 topk_w if mul else None, dtype)
    ok, *worst = mo.gemm_tolerance_ok(gu.host_f32(c), want)
    assert ok, worst


def test_moe_skips_invalid_blocks_and_rows():
    """Blocks with expert id -1, blocks past num_tokens_past_padded and padding
    slots leave C untouched (marlin_template.h(moe):471-570)."""
    m, e, top_k, k, n, bs = 12, 4, 2, 256, 128, 16
    ex = Experts(77, e, k, n, 128, "fp16")
    topk_ids, topk_w = route(5, m, e, top_k)
    sorted_ids, expert_ids, past = mo.moe_align_block_size(topk_ids, bs, e)
    expert_ids = expert_ids.copy()
    expert_ids[1] = -1
    past_cut = int(past[0]) - bs      # the last block is declared padding
    a32 = mo.make_activations(9, m, k, "fp16")
    a = gu.dev_bits16(a32, "fp16")
    got = gu.host_f32(ex.gemm(a, sorted_ids, expert_ids, past_cut, topk_w, bs, top_k, m, False))
    want = ex.reference(a32, sorted_ids, expert_ids, past_cut, bs, top_k, m, None)
    ok, *worst = mo.gemm_tolerance_ok(got, want)
    assert ok, worst
    untouched = np.ones(m * top_k, dtype=bool)
    for b in range(past_cut // bs):
        if expert_ids[b] >= 0:
            ids = sorted_ids[b * bs:(b + 1) * bs]
            untouched[ids[ids < m * top_k]] = False
    assert untouched.any()
    assert np.all(got[untouched] == 0.0)


def test_moe_matches_dense_gemm_per_expert():
    """With top_k = 1 and all tokens routed to one expert the grouped GEMM is
    the dense GEMM of that expert, bit for bit up to the summation order: both
    must satisfy the tolerance against the same reference and each other."""
    m, e, k, n, bs = 16, 3, 512, 128, 16
    ex = Experts(31, e, k, n, 128, "bf16")
    topk_ids = np.full((m, 1), 2, dtype=np.int32)
    sorted_ids, expert_ids, past = mo.moe_align_block_size(topk_ids, bs, e)
    a32 = mo.make_activations(2, m, k, "bf16")
    a = gu.dev_bits16(a32, "bf16")
    got = gu.host_f32(ex.gemm(a, sorted_ids, expert_ids, int(past[0]), None, bs, 1, m, False))
    dense = gu.host_f32(ex.layers[2].gemm(a, m))
    ok, *worst = mo.gemm_tolerance_ok(got, dense)
    assert ok, worst


@pytest.mark.parametrize("tokens,k,n,wtype", [
    (16, 4096, 28672, "uint4b8"), (64, 14336, 4096, "uint4b8"), (256, 4096, 28672, "uint4b8"),
    (600, 14336, 4096, "uint4b8"),
    # 8-bit codes: blocks of 64 slots run the tile kernel's 8-bit form, smaller ones the general grouped kernel
    (700, 4096, 2048, "uint8b128"), (2048, 2048, 1024, "fp8"), (64, 2048, 1024, "uint8b128"),
    # MXFP4 in the tile kernel with few tiles, and with a short last round of them (384 = 256 + 128): both cut along K
    (700, 4096, 2048, "mxfp4"), (2100, 14336, 4096, "mxfp4"),
    # ... and in the decode kernel on more (block, strip) pairs than compute units (workgroups of four wavefronts)
    (16, 4096, 4096, "mxfp4"),
    # the fp16 instantiations of the grouped tile kernel's 8-bit and 4-bit forms (256- and 128-row tiles)
    (700, 2048, 1024, "uint8b128/fp16"), (700, 2048, 1024, "fp8/fp16"), (700, 2048, 1024, "uint4b8/fp16"),
    # 8-bit codes with a scale per 32 rows (the layout of MXFP8), either activation type
    (700, 2048, 1024, "uint8b128g32"), (700, 2048, 1024, "uint8b128g32/fp16"), (700, 2048, 1024, "fp8g32/fp16"),
    # K of 10 steps, not a whole number of the wide kernel's passes: the eight-wavefront grouped tile kernel's 8-bit forms
    (700, 640, 512, "uint8b128"), (700, 640, 512, "fp8"), (700, 640, 512, "uint8b128/fp16"), (700, 640, 512, "fp8/fp16"),
    (700, 640, 512, "uint8b128g32"), (700, 640, 512, "fp8g32"), (700, 640, 512, "uint8b128g32/fp16"),
    (700, 640, 512, "fp8g32/fp16"),
    # blocks of 8, 32 and 48 slots of 8-bit codes: the general grouped kernel with one, two and three blocks of rows
    (8, 512, 256, "uint8b128"), (8, 512, 256, "uint8b128g32"), (100, 512, 256, "uint8b128g32"),
    (150, 512, 256, "uint8b128g32"), (8, 512, 256, "fp8g32/fp16"), (100, 512, 256, "fp8g32/fp16"),
    (150, 512, 256, "fp8g32/fp16"),
    # MXFP4 on a K that is not a whole number of the decode kernel's units (the gpt-oss expert shape): the general kernel
    (8, 2880, 5760, "mxfp4"),
    # 64-slot blocks without the scratch the tile kernel needs: the general grouped kernel with four blocks of rows
    (300, 512, 256, "uint8b128!"), (300, 512, 256, "uint8b128g32!"), (300, 512, 256, "uint8b128/fp16!"),
    (300, 512, 256, "uint8b128g32/fp16!"), (300, 512, 256, "fp8/fp16!"), (300, 512, 256, "fp8g32/fp16!"),
    (300, 512, 256, "mxfp4!")])
def test_full_size_grouped_gemm_agrees_with_dense_rows(tokens, k, n, wtype):
    """Mixtral-8x7B expert shapes (8 experts, top 2, the block size of the
    reference's rule), where the CPU oracle is too slow: every routed slot must
    equal, within the GEMM tolerance, the dense op on the same token row and
    the same expert's weights (the dense decode kernel is checked against the
    oracle elsewhere).  Random device weights; the grouped call covers blocks
    of 8, 32 and 64 slots, i.e. the grouped decode kernel with one and two
    blocks of rows, its two-halves form and the tile kernel."""
    e, top_k, dtype = 8, 2, torch.bfloat16
    with_scratch = not wtype.endswith("!")
    wtype = wtype.rstrip("!")
    if wtype.endswith("/fp16"):
        wtype, dtype = wtype[:-5], torch.float16
    dtype_code = _lib.DTYPE_BF16 if dtype == torch.bfloat16 else _lib.DTYPE_F16
    group = 128
    if wtype.endswith("g32"):
        wtype, group = wtype[:-3], 32
    gen = torch.Generator(device=gu.DEV).manual_seed(tokens + n)
    lib = _lib.load()
    b_type = {"uint4b8": _lib.TYPE_UINT4B8, "uint8b128": _lib.TYPE_UINT8B128, "fp8": _lib.TYPE_FLOAT8_E4M3FN,
              "mxfp4": _lib.TYPE_FLOAT4_E2M1F}[wtype]
    words = k * n // (8 if wtype in ("uint4b8", "mxfp4") else 4)
    groups = k // (32 if wtype == "mxfp4" else group)
    native = torch.randint(-2 ** 31, 2 ** 31 - 1, (e, words), dtype=torch.int32, device=gu.DEV, generator=gen)
    scales = torch.rand((e, groups, n), device=gu.DEV, generator=gen) * 9e-3 + 1e-3
    if wtype == "mxfp4":   # powers of two
        scales = torch.exp2(torch.randint(-9, -5, (e, groups, n), device=gu.DEV, generator=gen).float())
    if wtype == "uint8b128":
        scales = scales / 16
    if wtype == "fp8":   # the exponent bias of the codes is folded into the scales: 2^120 for bf16, 2^8 for fp16
        scales = scales * (2.0 ** 120 if dtype == torch.bfloat16 else 2.0 ** 8)
    scales = scales.to(dtype)
    a = torch.randn((tokens, k), device=gu.DEV, generator=gen).to(dtype)
    topk_ids, topk_w = route(tokens, tokens, e, top_k)
    bs = mo.moe_block_size_rule(tokens, top_k, e)
    sorted_ids, expert_ids, past = mo.moe_align_block_size(topk_ids, bs, e)
    sid, eid = gu.dev_i32(sorted_ids), gu.dev_i32(expert_ids)
    npp = gu.dev_i32(np.array([int(past[0])], dtype=np.int32))
    c = torch.zeros((tokens * top_k, n), dtype=dtype, device=gu.DEV)
    workspace = torch.zeros(1024, dtype=torch.int32, device=gu.DEV)
    nbytes = lib.sonar_moe_marlin_gemm_scratch_bytes(sid.numel(), bs, n, k) if with_scratch else 0
    scr = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=gu.DEV) if with_scratch else None
    _lib.check(lib.sonar_moe_wna16_marlin_gemm(
        gu.ptr(a), gu.ptr(c), gu.ptr(native), _lib.LAYOUT_GFX950, None, gu.ptr(scales), None, None, None,
        gu.ptr(workspace), workspace.numel(), gu.ptr(scr), nbytes, gu.ptr(sid), sid.numel(), gu.ptr(eid),
        gu.ptr(npp), None, bs, top_k, 0, e, dtype_code, b_type, tokens, n, k, groups, 1, 0, 1,
        gu.stream()))
    torch.cuda.synchronize()
    assert bool(torch.isfinite(c.float()).all())
    scale = float(c.float().abs().max())
    checked = 0
    for ex in range(e):
        slots = np.nonzero(topk_ids.reshape(-1) == ex)[0][:16]      # up to 16 slots of this expert
        if len(slots) == 0:
            continue
        rows = a[torch.from_numpy(slots // top_k).to(gu.DEV)].contiguous()
        m = rows.shape[0]
        dense = torch.empty((m, n), dtype=dtype, device=gu.DEV)
        dscr = torch.empty(max(lib.sonar_marlin_gemm_scratch_bytes(m, n, k), 16), dtype=torch.uint8, device=gu.DEV)
        _lib.check(lib.sonar_marlin_gemm(
            gu.ptr(rows), k, gu.ptr(dense), gu.ptr(native[ex]), _lib.LAYOUT_GFX950, None, gu.ptr(scales[ex]), None,
            None, None, gu.ptr(workspace), workspace.numel(), gu.ptr(dscr), dscr.numel(), dtype_code,
            b_type, m, n, k, groups, 1, 0, 1, gu.stream()))
        got = c[torch.from_numpy(slots).to(gu.DEV)].float()
        err = float((got - dense.float()).abs().max())
        assert err <= 1e-2 * scale, (ex, err, scale)
        checked += m
    assert checked >= min(16, tokens)


def test_moe_error_paths():
    lib = _lib.load()
    ex = Experts(3, 2, 256, 128, 128, "fp16")
    a = torch.zeros((4, 256), dtype=torch.float16, device=gu.DEV)
    c = torch.zeros((8, 128), dtype=torch.float16, device=gu.DEV)
    sid = torch.zeros(32, dtype=torch.int32, device=gu.DEV)
    eid = torch.zeros(2, dtype=torch.int32, device=gu.DEV)
    npp = torch.zeros(1, dtype=torch.int32, device=gu.DEV)

    def call(bs=16, b_type=_lib.TYPE_UINT4B8, k=256):
        return lib.sonar_moe_wna16_marlin_gemm(
            gu.ptr(a), gu.ptr(c), gu.ptr(ex.native), _lib.LAYOUT_GFX950, None, gu.ptr(ex.scales), None, None,
            None, gu.ptr(ex.workspace), ex.workspace.numel(), None, 0, gu.ptr(sid), sid.numel(), gu.ptr(eid),
            gu.ptr(npp), None, bs, 2, 0, 2, _lib.DTYPE_F16, b_type, 4, 128, k, 2, 1, 0, 1, gu.stream())

    assert call() == _lib.OK
    assert call(bs=24) == _lib.E_INVALID
    assert b"moe_block_size" in lib.sonar_marlin_last_error()
    assert call(b_type=_lib.TYPE_UINT4) == _lib.E_INVALID
    assert call(k=250) == _lib.E_INVALID
    torch.cuda.synchronize()


# ---------------------------------------------------------------- helper kernels around the GEMMs
@pytest.mark.parametrize("m,topk,e,bs", [(4, 3, 5, 4), (1, 2, 8, 8), (33, 2, 8, 16), (257, 2, 4, 64),
                                         (5, 6, 64, 16), (100, 1, 3, 48), (4096, 2, 8, 64), (700, 8, 256, 16)])
def test_moe_align_kernel_matches_oracle(m, topk, e, bs):
    lib = _lib.load()
    rng = np.random.default_rng(m * 31 + e)
    ids = np.stack([rng.permutation(e)[:topk] for _ in range(m)]).astype(np.int32)
    want_sorted, want_experts, want_past = mo.moe_align_block_size(ids, bs, e)
    d_ids = gu.dev_i32(ids.reshape(-1))
    sorted_ids = torch.empty(want_sorted.size, dtype=torch.int32, device=gu.DEV)
    expert_ids = torch.empty(want_experts.size, dtype=torch.int32, device=gu.DEV)
    past = torch.empty(1, dtype=torch.int32, device=gu.DEV)
    offsets = torch.empty(e, dtype=torch.int32, device=gu.DEV)
    _lib.check(lib.sonar_moe_align_block_size(gu.ptr(d_ids), ids.size, e, bs, gu.ptr(sorted_ids), sorted_ids.numel(),
                                              gu.ptr(expert_ids), expert_ids.numel(), gu.ptr(past), None,
                                              gu.ptr(offsets), gu.stream()))
    torch.cuda.synchronize()
    assert int(past[0]) == int(want_past[0])
    assert np.array_equal(sorted_ids.cpu().numpy(), want_sorted)        # bit-exact, padding included
    assert np.array_equal(expert_ids.cpu().numpy(), want_experts)


def test_moe_align_op_with_expert_map_matches_torch_expressions():
    from sonar_amd import fused_moe
    rng = np.random.default_rng(3)
    m, topk, e, bs = 50, 2, 8, 16
    ids = torch.from_numpy(np.stack([rng.permutation(e)[:topk] for _ in range(m)]).astype(np.int32))
    emap = torch.tensor([-1, 2, -1, 0, 1, -1, 3, -1], dtype=torch.int32)
    for ignore in (True, False):
        want = fused_moe.moe_align_block_size(ids, bs, e, emap, ignore_invalid_experts=ignore)        # CPU: torch
        got = fused_moe.moe_align_block_size(ids.to(gu.DEV), bs, e, emap.to(gu.DEV), ignore_invalid_experts=ignore)
        torch.cuda.synchronize()
        past = int(want[2][0])
        assert int(got[2][0]) == past
        assert torch.equal(got[0].cpu()[:past], want[0][:past]) and bool((got[0].cpu()[past:] == ids.numel()).all())
        assert torch.equal(got[1].cpu(), want[1])


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_silu_and_mul_and_moe_sum_kernels(dtype):
    lib = _lib.load()
    rng = np.random.default_rng(11)
    rows, d, topk = 37, 264, 3
    x32 = mo.round_to_dtype((rng.standard_normal((rows, 2 * d)) * 3).astype(np.float32), dtype)
    x = gu.dev_bits16(x32, dtype)
    out = torch.empty((rows, d), dtype=x.dtype, device=gu.DEV)
    _lib.check(lib.sonar_silu_and_mul(gu.ptr(out), gu.ptr(x), rows, d, gu.dtype_code(dtype), gu.stream()))
    g, u = x32[:, :d].astype(np.float64), x32[:, d:]
    silu = mo.round_to_dtype((g / (1.0 + np.exp(-g))).astype(np.float32), dtype)
    want = mo.round_to_dtype(silu * u, dtype)
    got = gu.host_f32(out)
    # expf in the kernel vs exp here: allow one unit in the last place of the activation
    ulp = 2.0 ** (-10 if dtype == "fp16" else -7)
    assert np.all(np.abs(got - want) <= ulp * np.abs(want) * 2 + 1e-6)
    assert np.mean(got == want) > 0.98

    y32 = mo.round_to_dtype(rng.standard_normal((rows, topk, d)).astype(np.float32), dtype)
    y = gu.dev_bits16(y32.reshape(rows * topk, d), dtype).reshape(rows, topk, d)
    s = torch.empty((rows, d), dtype=y.dtype, device=gu.DEV)
    _lib.check(lib.sonar_moe_sum(gu.ptr(s), gu.ptr(y), rows, topk, d, gu.dtype_code(dtype), gu.stream()))
    want = mo.round_to_dtype(((y32[:, 0] + y32[:, 1]) + y32[:, 2]).astype(np.float32), dtype)
    assert np.array_equal(gu.host_f32(s), want)        # fp32 sum in k order, one rounding


ACTIVATIONS = [
    # name, kind, limit, alpha, beta, oracle keywords
    ("silu", 1, 3.0, 1.0, 0.0, dict(clamp_limit=3.0)),
    ("swigluoai_uninterleave", 1, 7.0, 1.702, 1.0, dict(clamp_limit=7.0, alpha=1.702, beta=1.0)),
    ("gelu", 2, 0.0, 1.0, 0.0, {}),
    ("gelu_tanh", 3, 0.0, 1.0, 0.0, {}),
    ("swigluoai", 4, 7.0, 1.702, 0.0, {}),
    ("situ", 5, 0.0, 4.0, 3.0, dict(situ_beta=4.0, situ_linear_beta=3.0)),
    ("situ", 5, 0.0, 2.5, -1.0, dict(situ_beta=2.5, situ_linear_beta=None)),
    ("swiglustep", 6, 7.0, 1.0, 0.0, {}),
]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("name,kind,limit,alpha,beta,kw", ACTIVATIONS, ids=lambda v: str(v) if isinstance(v, str) else None)
def test_gated_activation_kernels(name, kind, limit, alpha, beta, kw, dtype):
    """sonar_moe_activation against oracle.moe_activation: values beyond the clamp limits on
    both sides included.  The kernel's float32 exp / tanh / erf against float64 there: at most
    one unit in the last place of an intermediate rounding, and nearly every value equal."""
    lib = _lib.load()
    rng = np.random.default_rng(kind * 7 + len(name))
    rows, d = 29, 136
    x32 = mo.round_to_dtype((rng.standard_normal((rows, 2 * d)) * 4).astype(np.float32), dtype)
    x = gu.dev_bits16(x32, dtype)
    out = torch.empty((rows, d), dtype=x.dtype, device=gu.DEV)
    _lib.check(lib.sonar_moe_activation(gu.ptr(out), gu.ptr(x), rows, d, kind, limit, alpha, beta,
                                        gu.dtype_code(dtype), gu.stream()))
    want = mo.moe_activation(name, x32, dtype, **kw)
    got = gu.host_f32(out)
    ulp = 2.0 ** (-10 if dtype == "fp16" else -7)
    assert np.all(np.isfinite(got))
    tol = 2 * ulp * np.abs(want) + 1e-6
    if name.startswith("gelu"):   # 1 + erf / 1 + tanh in float32: the last place of that sum, times gate * up
        tol = tol + 2.0 ** -20 * np.abs(x32[:, :d] * x32[:, d:])
    assert np.all(np.abs(got - want) <= tol), np.abs(got - want).max()
    assert np.mean(got == want) > 0.95
    # the torch op and the dispatcher of the fused layer give the same bits
    from sonar_amd import fused_moe
    out2 = torch.empty_like(out)
    fused_moe.apply_moe_activation(name, out2, x, clamp_limit=kw.get("clamp_limit"), alpha=kw.get("alpha", 1.0),
                                   beta=kw.get("beta", 0.0), activation_situ_beta=kw.get("situ_beta"),
                                   activation_situ_linear_beta=kw.get("situ_linear_beta"))
    assert torch.equal(out2.view(torch.int16), out.view(torch.int16))
    # ... and its torch expressions for CPU tensors agree to the same bar
    cpu = torch.empty((rows, d), dtype=x.dtype)
    fused_moe.apply_moe_activation(name, cpu, x.cpu(), clamp_limit=kw.get("clamp_limit"), alpha=kw.get("alpha", 1.0),
                                   beta=kw.get("beta", 0.0), activation_situ_beta=kw.get("situ_beta"),
                                   activation_situ_linear_beta=kw.get("situ_linear_beta"))
    assert np.all(np.abs(cpu.float().numpy() - want) <= tol)


def test_gated_activation_rejections():
    lib = _lib.load()
    x = torch.zeros((4, 32), dtype=torch.float16, device=gu.DEV)
    out = torch.zeros((4, 16), dtype=torch.float16, device=gu.DEV)
    assert lib.sonar_moe_activation(gu.ptr(out), gu.ptr(x), 4, 16, 9, 1.0, 1.0, 0.0, 0, gu.stream()) == _lib.E_INVALID
    assert lib.sonar_moe_activation(gu.ptr(out), gu.ptr(x), 4, 16, 1, 0.0, 1.0, 0.0, 0, gu.stream()) == _lib.E_INVALID
    assert b"limit" in lib.sonar_marlin_last_error()
    assert lib.sonar_moe_activation(gu.ptr(out), gu.ptr(x), 4, 12, 2, 0.0, 1.0, 0.0, 0, gu.stream()) == _lib.E_INVALID


@pytest.mark.parametrize("dtype,zp", [("bf16", False), ("fp16", False), ("fp16", True), ("bf16", True)])
def test_moe_tiled_and_streaming_kernels_agree(dtype, zp):
    """The same 64-slot-block call (more slots than the decode kernel takes) with
    and without the scratch the tiled kernel needs for its table takes two
    different kernels; both meet the tolerance against the reference and each
    other."""
    m, e, top_k, k, n, bs = 700, 4, 2, 512, 256, 64
    ex = Experts(91, e, k, n, 128, dtype, zero_points=zp)
    topk_ids, topk_w = route(7, m, e, top_k)
    sorted_ids, expert_ids, past = mo.moe_align_block_size(topk_ids, bs, e)
    a32 = mo.make_activations(4, m, k, dtype)
    a = gu.dev_bits16(a32, dtype)
    tiled = gu.host_f32(ex.gemm(a, sorted_ids, expert_ids, int(past[0]), topk_w, bs, top_k, m, True, scratch=True))
    streamed = gu.host_f32(ex.gemm(a, sorted_ids, expert_ids, int(past[0]), topk_w, bs, top_k, m, True, scratch=False))
    want = ex.reference(a32, sorted_ids, expert_ids, int(past[0]), bs, top_k, m, topk_w)
    for got in (tiled, streamed):
        ok, *worst = mo.gemm_tolerance_ok(got, want)
        assert ok, worst
    ok, *worst = mo.gemm_tolerance_ok(tiled, streamed)
    assert ok, worst


def test_full_size_grouped_tile_gemm_agrees_with_dense_rows():
    """Mixtral-sized grouped GEMM at 4096 tokens (64-slot blocks, tiled kernel):
    every routed slot must equal the dense GEMM of its token with its expert."""
    from sonar_amd import fused_moe
    m, e, top_k, k, n = 4096, 8, 2, 4096, 2048
    ex = Experts(13, e, k, n, 128, "bf16")
    gen = torch.Generator(device=gu.DEV).manual_seed(2)
    a = (torch.randn((m, k), device=gu.DEV, generator=gen) * 0.5).to(torch.bfloat16)
    logits = torch.randn((m, e), device=gu.DEV, generator=gen)
    tw, ti = torch.topk(torch.softmax(logits, dim=1), top_k, dim=1)
    ti = ti.to(torch.int32)
    bs = fused_moe.moe_block_size(m, top_k, e)
    assert bs == 64
    sorted_ids, expert_ids, past = fused_moe.moe_align_block_size(ti, bs, e)
    got = ex.gemm(a, sorted_ids.cpu().numpy(), expert_ids.cpu().numpy(), int(past[0]), tw.cpu().numpy(), bs, top_k, m,
                  False)
    assert bool(torch.isfinite(got.float()).all())
    scale = float(got.float().abs().max())
    ti_host = ti.cpu().numpy()
    rng = np.random.default_rng(0)
    for t in rng.integers(0, m, 6):
        for j in range(top_k):
            dense = ex.layers[int(ti_host[t, j])].gemm(a[t:t + 1].contiguous(), 1)
            err = float((dense.float() - got[t * top_k + j].float()).abs().max())
            assert err <= 1e-2 * scale, (t, j, err, scale)


def test_tile_kernel_with_expert_ids_that_are_not_grouped_by_expert():
    """64-slot blocks whose experts alternate, with blocks of absent experts (-1) in
    between: every block is a run of its own, more runs than experts.  The table of
    row tiles has an entry per block, so no block may be dropped."""
    m, e, top_k, k, n, bs = 64 * 14, 3, 1, 256, 256, 64
    ex = Experts(301, e, k, n, 128, "bf16")
    blocks = m // bs
    pattern = [0, 1, -1, 2, 0, -1, 1, 2, 0, 1, 2, -1, 0, 2]
    assert len(pattern) == blocks
    expert_ids = np.array(pattern, dtype=np.int32)
    rng = np.random.default_rng(5)
    sorted_ids = rng.permutation(m).astype(np.int32)          # every block full, ids in any order
    weights = rng.random((m, top_k)).astype(np.float32)
    a32 = mo.make_activations(9, m, k, "bf16")
    a = gu.dev_bits16(a32, "bf16")
    got = gu.host_f32(ex.gemm(a, sorted_ids, expert_ids, m, weights, bs, top_k, m, True))
    want = ex.reference(a32, sorted_ids, expert_ids, m, bs, top_k, m, weights)
    written = np.concatenate([sorted_ids[b * bs:(b + 1) * bs] for b in range(blocks) if pattern[b] >= 0])
    ok, *worst = mo.gemm_tolerance_ok(got[written], want[written])
    assert ok, worst
    skipped = np.concatenate([sorted_ids[b * bs:(b + 1) * bs] for b in range(blocks) if pattern[b] < 0])
    assert np.all(got[skipped] == 0)          # Experts.gemm hands the op a zeroed output
