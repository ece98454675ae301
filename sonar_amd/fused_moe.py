"""Host side of the Marlin mixture-of-experts layer: token routing into blocks
and the two grouped W4A16 GEMMs around the gated activation.

Mirrors aphrodite/model_executor/layers/fused_moe/moe_align_block_size.py:11-101
(`moe_align_block_size`) and .../fused_moe/experts/marlin_moe.py:57-392
(`fused_marlin_moe`) for 4- and 8-bit integer, fp8 and MXFP4 weights with fp16 / bf16
activations.
On the GPU the routing, the activation and the final sum are the HIP kernels
behind `torch.ops.sonar_amd.{moe_align_block_size, silu_and_mul, moe_sum}`; the
torch expressions kept here serve CPU tensors (and the tests of those kernels).
Neither reads a device value on the host, so the whole layer can be recorded
in a HIP graph; the two GEMMs are the `_moe_C::moe_wna16_marlin_gemm` op.
"""
from __future__ import annotations

import math

import torch

from . import ops
from .marlin_utils import marlin_make_workspace_new, marlin_quant_input
from .scalar_type import ScalarType, scalar_types

_SUPPORTED = {t.id: t for t in (scalar_types.uint4, scalar_types.uint4b8, scalar_types.uint8b128,
                                scalar_types.float8_e4m3fn, scalar_types.float4_e2m1f)}


def moe_block_size(num_tokens: int, top_k: int, num_experts: int) -> int:
    """Smallest block size whose expected fill is below 0.9 (marlin_moe.py:322-329)."""
    for block_size_m in (8, 16, 32, 48, 64):
        if num_tokens * top_k / num_experts / block_size_m < 0.9:
            break
    return block_size_m


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int,
                         expert_map: torch.Tensor | None = None, pad_sorted_ids: bool = False,
                         ignore_invalid_experts: bool = False
                         ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Sorts the flattened (token, k) slots by expert, pads every expert's run
    to a multiple of `block_size` with the sentinel `topk_ids.numel()`, and
    names the expert of each block.  Returns (sorted_token_ids int32
    [max_num_tokens_padded], expert_ids int32 [blocks], num_tokens_post_padded
    int32 [1]).  Slots of one expert keep ascending order.  Blocks past
    num_tokens_post_padded carry expert id -1.

    With `expert_map` (global -> local id, -1 = not on this rank): when
    `ignore_invalid_experts` the slots of absent experts are dropped before
    counting and expert_ids holds local ids; otherwise every expert is counted
    and expert_ids of absent experts become -1."""
    numel = topk_ids.numel()
    dev = topk_ids.device
    max_num_tokens_padded = numel + num_experts * (block_size - 1)
    if pad_sorted_ids:
        max_num_tokens_padded = -(-max_num_tokens_padded // block_size) * block_size
    if numel < num_experts:
        max_num_tokens_padded = min(numel * block_size, max_num_tokens_padded)
    max_blocks = -(-max_num_tokens_padded // block_size)

    if topk_ids.is_cuda:
        sorted_ids = torch.empty((max_num_tokens_padded,), dtype=torch.int32, device=dev)
        expert_ids = torch.empty((max_blocks,), dtype=torch.int32, device=dev)
        num_tokens_post_pad = torch.empty((1,), dtype=torch.int32, device=dev)
        ids = topk_ids if topk_ids.dtype == torch.int32 else topk_ids.to(torch.int32)
        emap = None
        if expert_map is not None and ignore_invalid_experts:
            emap = expert_map if expert_map.dtype == torch.int32 else expert_map.to(torch.int32)
        torch.ops.sonar_amd.moe_align_block_size(ids.contiguous(), num_experts, block_size, sorted_ids,
                                                 expert_ids, num_tokens_post_pad, emap)
        if expert_map is not None and not ignore_invalid_experts:
            mapped = expert_map.to(torch.int32)[expert_ids.clamp(min=0).to(torch.int64)]
            expert_ids = torch.where(expert_ids >= 0, mapped, expert_ids)
        return sorted_ids, expert_ids, num_tokens_post_pad
    return _moe_align_block_size_torch(topk_ids, block_size, num_experts, expert_map, ignore_invalid_experts,
                                       max_num_tokens_padded, max_blocks)


def _moe_align_block_size_torch(topk_ids, block_size, num_experts, expert_map, ignore_invalid_experts,
                                max_num_tokens_padded, max_blocks):
    """The same routing as torch expressions (any device)."""
    numel = topk_ids.numel()
    dev = topk_ids.device
    flat = topk_ids.reshape(-1).to(torch.int64)
    valid = (flat >= 0) & (flat < num_experts)
    key = flat
    if expert_map is not None and ignore_invalid_experts:
        # experts are numbered and ordered by their mapped (local) ids
        key = expert_map.to(torch.int64)[flat.clamp(0, num_experts - 1)]
        valid &= (key >= 0) & (key < num_experts)
    # invalid slots sort behind every expert and are never placed
    key = torch.where(valid, key, torch.full_like(flat, num_experts))
    counts = torch.zeros(num_experts + 1, dtype=torch.int64, device=dev).scatter_add_(
        0, key, torch.ones_like(key))[:num_experts]
    padded = (counts + block_size - 1) // block_size * block_size
    pad_end = torch.cumsum(padded, 0)
    pad_begin = pad_end - padded
    run_begin = torch.cumsum(counts, 0) - counts

    order = torch.sort(key, stable=True).indices          # slot ids, expert-major, ascending inside
    sorted_key = key[order]
    placed = sorted_key < num_experts
    e_of = sorted_key.clamp(max=num_experts - 1)
    rank = torch.arange(numel, device=dev) - run_begin[e_of]
    dest = torch.where(placed, pad_begin[e_of] + rank, torch.full_like(rank, max_num_tokens_padded))
    sorted_ids = torch.full((max_num_tokens_padded + 1,), numel, dtype=torch.int32, device=dev)
    sorted_ids.scatter_(0, dest, order.to(torch.int32))
    sorted_ids = sorted_ids[:max_num_tokens_padded]

    block_start = torch.arange(max_blocks, device=dev) * block_size
    expert_of_block = torch.searchsorted(pad_end, block_start, right=True)
    total = pad_end[-1]
    in_range = block_start < total
    expert_ids = torch.where(in_range, expert_of_block, torch.full_like(expert_of_block, -1))
    if expert_map is not None and not ignore_invalid_experts:
        mapped = expert_map.to(torch.int64)[expert_ids.clamp(0, num_experts - 1)]
        expert_ids = torch.where(in_range, mapped, expert_ids)
    return sorted_ids, expert_ids.to(torch.int32), total.to(torch.int32).reshape(1)


def batched_moe_align_block_size(max_tokens_per_batch: int, block_size: int,
                                 expert_num_tokens: torch.Tensor):
    """Routing tables for tokens that are already batched by expert: batch b holds
    the tokens of expert b in rows b * max_tokens_per_batch .., the first
    expert_num_tokens[b] of them valid (moe_align_block_size.py:100-186; the
    arithmetic follows batched_moe_align_block_size_kernel,
    csrc/libtorch_stable/moe/moe_align_sum_kernels.cu:26-82).  Every batch is
    padded to whole blocks; padding slots hold B * max_tokens_per_batch, unused
    blocks expert -1.  Index arithmetic only: nothing is read back to the host."""
    B = expert_num_tokens.size(0)
    dev = expert_num_tokens.device
    total = B * ((max_tokens_per_batch + block_size - 1) // block_size * block_size)
    sentinel = B * max_tokens_per_batch
    n = expert_num_tokens.to(torch.int64)
    padded = (n + block_size - 1) // block_size * block_size
    ends = torch.cumsum(padded, 0)
    starts = ends - padded

    def owner(pos):                      # batch whose padded range holds slot pos, B past the last one
        return torch.searchsorted(ends, pos, right=True)

    pos = torch.arange(total, device=dev)
    b = owner(pos)
    bc = b.clamp(max=B - 1)
    off = pos - starts[bc]
    valid = (b < B) & (off < n[bc])
    sorted_ids = torch.where(valid, bc * max_tokens_per_batch + off,
                             torch.full_like(pos, sentinel)).to(torch.int32)
    bb = owner(torch.arange(total // block_size, device=dev) * block_size)
    expert_ids = torch.where(bb < B, bb, torch.full_like(bb, -1)).to(torch.int32)
    return sorted_ids, expert_ids, ends[-1:].to(torch.int32)


def silu_and_mul(out: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """out = silu(x[:, :d]) * x[:, d:] in the tensor's own dtype."""
    d = x.shape[-1] // 2
    if x.is_cuda and x.is_contiguous() and out.is_contiguous() and d % 8 == 0:
        torch.ops.sonar_amd.silu_and_mul(out, x)
        return out
    torch.mul(torch.nn.functional.silu(x[..., :d]), x[..., d:], out=out)
    return out


def moe_sum(moe_output: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = sum over k of moe_output[t, k], accumulated in fp32."""
    if moe_output.is_cuda and moe_output.is_contiguous() and out.is_contiguous() and out.shape[-1] % 8 == 0:
        torch.ops.sonar_amd.moe_sum(moe_output, out)
        return out
    return torch.sum(moe_output, dim=1, out=out)


def _activation_name(activation) -> str:
    """`activation` as the reference passes it (a MoEActivation enum member, whose value is
    the name) or as a plain string."""
    name = str(getattr(activation, "value", activation)).lower()
    return {"gelu_pytorch_tanh": "gelu_tanh"}.get(name, name)


# the reference's MoEActivation values (fused_moe/activation.py:11-38)
_GATED = ("silu", "gelu", "gelu_tanh", "swigluoai", "situ", "swigluoai_uninterleave", "swiglustep")
_NOT_GATED = ("silu_no_mul", "gelu_no_mul", "gelu_tanh_no_mul", "relu2_no_mul")


def activation_is_gated(activation) -> bool:
    """MoEActivation.is_gated: a gated activation takes [.., 2 d] and gives [.., d]."""
    return not _activation_name(activation).endswith("_no_mul")


def _gated_on_gpu(op, output, input, *args) -> bool:
    d = output.shape[-1]
    if input.is_cuda and input.is_contiguous() and output.is_contiguous() and d % 8 == 0:
        op(output, input, *args)
        return True
    return False


def apply_moe_activation(activation, output: torch.Tensor, input: torch.Tensor, *, clamp_limit=None,
                         alpha: float = 1.0, beta: float = 0.0, topk_ids=None, expert_map=None,
                         activation_situ_beta=None, activation_situ_linear_beta=None) -> torch.Tensor:
    """The reference's dispatcher between the two grouped GEMMs
    (fused_moe/activation.py:128-205): `output` [rows, d] from `input` [rows, 2 d] (gated) or
    [rows, d].  `clamp_limit` / `alpha` / `beta` drive the clamped SwiGLU: SILU with a
    clamp_limit and SWIGLUOAI_UNINTERLEAVE are both silu_and_mul_with_clamp.  The gated forms
    run as HIP kernels on GPU tensors (torch expressions of the same arithmetic serve CPU
    tensors); the forms without a gate are torch functions in the reference as well.
    `topk_ids` / `expert_map` are accepted as in the reference: its pad-aware variant skips
    slots that nobody reads, the values of the others are the same."""
    name = _activation_name(activation)
    assert input.dim() == 2 and output.dim() == 2, "input and output must be 2D"
    d = output.shape[-1]
    if activation_is_gated(name):
        assert d * 2 == input.shape[-1], f"{name} expects 2x ratio: {d * 2} vs {input.shape[-1]}"
    else:
        assert d == input.shape[-1], f"{name} expects equal sizes: {d} vs {input.shape[-1]}"
    f32 = torch.float32
    dt = output.dtype

    def halves():   # gate and up in fp32, for the torch expressions only (a pass over the tensor each)
        return input[..., :d].to(f32), input[..., d:].to(f32)

    if name == "silu" and clamp_limit is None:
        silu_and_mul(output, input)
    elif name in ("silu", "swigluoai_uninterleave"):
        assert clamp_limit is not None, "SWIGLUOAI_UNINTERLEAVE requires clamp_limit"
        a, b = (1.0, 0.0) if name == "silu" else (float(alpha), float(beta))
        if not _gated_on_gpu(torch.ops.sonar_amd.silu_and_mul_with_clamp, output, input, float(clamp_limit), a, b):
            g, u = halves()
            gc = g.clamp(max=clamp_limit).to(dt).to(f32)
            act = (gc / (1.0 + torch.exp(-gc * a))).to(dt).to(f32)
            output.copy_((act * (u.clamp(-clamp_limit, clamp_limit) + b)).to(dt))
    elif name == "gelu":
        if not _gated_on_gpu(torch.ops.sonar_amd.gelu_and_mul, output, input):
            g, u = halves()
            output.copy_((torch.nn.functional.gelu(g).to(dt).to(f32) * u).to(dt))
    elif name == "gelu_tanh":
        if not _gated_on_gpu(torch.ops.sonar_amd.gelu_tanh_and_mul, output, input):
            g, u = halves()
            output.copy_((torch.nn.functional.gelu(g, approximate="tanh").to(dt).to(f32) * u).to(dt))
    elif name == "swigluoai":      # gate and up alternate (gpt-oss checkpoints); alpha 1.702, limit 7.0
        if not _gated_on_gpu(torch.ops.sonar_amd.swigluoai_and_mul, output, input, 1.702, 7.0):
            gi = input[..., 0::2].to(f32).clamp(max=7.0)
            ui = input[..., 1::2].to(f32).clamp(-7.0, 7.0)
            output.copy_(((ui + 1.0) * gi / (1.0 + torch.exp(-gi * 1.702))).to(dt))
    elif name == "situ":
        assert activation_situ_beta is not None, "SITU requires activation_situ_beta"
        lb = -1.0 if activation_situ_linear_beta is None else float(activation_situ_linear_beta)
        if not _gated_on_gpu(torch.ops.sonar_amd.situ_and_mul, output, input, float(activation_situ_beta), lb):
            g, u = halves()
            bt = float(activation_situ_beta)
            up = lb * torch.tanh(u / lb) if lb > 0 else u
            output.copy_((bt * torch.tanh(g / bt) / (1.0 + torch.exp(-g)) * up).to(dt))
    elif name == "swiglustep":
        if not _gated_on_gpu(torch.ops.sonar_amd.swiglustep_and_mul, output, input, 7.0):
            g, u = halves()
            output.copy_(((g * torch.sigmoid(g)).clamp(max=7.0) * u.clamp(-7.0, 7.0)).to(dt))
    elif name == "silu_no_mul":
        output.copy_(torch.nn.functional.silu(input))
    elif name == "gelu_no_mul":
        output.copy_(torch.nn.functional.gelu(input))
    elif name == "gelu_tanh_no_mul":
        output.copy_(torch.nn.functional.gelu(input, approximate="tanh"))
    elif name == "relu2_no_mul":
        torch.nn.functional.relu(input, inplace=True)
        torch.square(input, out=output)
    else:
        raise ValueError(f"Unsupported FusedMoe activation: {activation}")
    return output


def _check_arguments(activation, input_dtype, global_scales) -> None:
    name = _activation_name(activation)
    if name not in _GATED + _NOT_GATED:
        raise ValueError(f"Unknown MoE activation: {activation!r}. Valid activations: {list(_GATED + _NOT_GATED)}")
    if input_dtype is not None and input_dtype not in (torch.int8, torch.float8_e4m3fn, torch.float16,
                                                       torch.bfloat16):
        raise ValueError(f"unsupported input_dtype {input_dtype}")
    if input_dtype != torch.int8 and any(g is not None for g in global_scales[:2]):
        raise ValueError("input_global_scale1 / input_global_scale2 go with int8 activations (input_dtype = "
                         "torch.int8) only")


def _fused_marlin_moe(hidden_states, w1, w2, bias1, bias2, w1_scale, w2_scale, topk_weights, num_topk,
                      quant_type: ScalarType, apply_router_weight_on_input, expert_map, block_size_m,
                      sorted_token_ids, expert_ids, num_tokens_post_padded, activation="silu",
                      activation_func=None, topk_ids=None, input_global_scale1=None, input_global_scale2=None,
                      global_scale1=None, global_scale2=None, g_idx1=None, g_idx2=None, sort_indices1=None,
                      sort_indices2=None, w1_zeros=None, w2_zeros=None, workspace=None,
                      intermediate_cache13=None, intermediate_cache2=None, output=None, input_dtype=None,
                      is_k_full=True, clamp_limit=None, gemm1_alpha=1.0, gemm1_beta=0.0,
                      activation_situ_beta=None, activation_situ_linear_beta=None):
    """Gate/up GEMM -> activation -> down GEMM over already routed slots
    (marlin_moe.py:57-223; same parameters in the same order).  `activation_func`, when
    given, is called like the reference's apply_moe_activation: activation_func(activation,
    out [M * top_k, N], in [M * top_k, shards * N], clamp_limit=, alpha=, beta=, topk_ids=,
    expert_map=, activation_situ_beta=, activation_situ_linear_beta=); the default is
    apply_moe_activation above.  A gated activation takes the gate and up projections from the
    first GEMM (shards = 2), one without a gate takes one projection.  `expert_map` is otherwise
    accepted for signature parity (the routing passed in already reflects it).  Returns the
    [M * top_k, K] per-slot outputs."""
    _check_arguments(activation, input_dtype, (input_global_scale1, input_global_scale2, global_scale1,
                                               global_scale2))
    assert hidden_states.ndim == 2
    M, K = hidden_states.shape
    N = w2.shape[1] * 16                       # intermediate size: w2 is (E, N/16, 2K)
    shards = 2 if activation_is_gated(activation) else 1
    dev, dt = hidden_states.device, hidden_states.dtype
    if workspace is None:
        workspace = marlin_make_workspace_new(dev, 4)
    if intermediate_cache13 is None:
        intermediate_cache13 = torch.empty((M * num_topk * max(shards * N, K),), device=dev, dtype=dt)
    if intermediate_cache2 is None:
        intermediate_cache2 = torch.empty((M * num_topk, N), device=dev, dtype=dt)
    cache1 = intermediate_cache13[:M * num_topk * shards * N].view(M * num_topk, shards * N)
    cache3 = intermediate_cache13[:M * num_topk * K].view(M * num_topk, K)
    cache2 = intermediate_cache2.view(-1)[:M * num_topk * N].view(M * num_topk, N)

    # 8-bit activations: one scale per token row, times the factor of the integer group scales
    # (marlin_moe.py:126-133,181-187)
    a_scales1 = a_scales2 = None
    gate_up_input = hidden_states
    if input_dtype in (torch.int8, torch.float8_e4m3fn):
        gate_up_input, a_scales1 = marlin_quant_input(hidden_states, input_dtype)
        if input_dtype == torch.int8 and input_global_scale1 is not None:
            a_scales1 = a_scales1 * input_global_scale1
    cache1 = ops.moe_wna16_marlin_gemm(
        gate_up_input, cache1, w1, bias1, w1_scale, a_scales1, global_scale1, w1_zeros, g_idx1, sort_indices1,
        workspace,
        sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights, moe_block_size=block_size_m,
        top_k=num_topk, mul_topk_weights=apply_router_weight_on_input, b_q_type=quant_type, size_m=M,
        size_n=shards * N, size_k=K, is_k_full=is_k_full, use_atomic_add=False, use_fp32_reduce=True,
        is_zp_float=False)
    # (SILU with a clamp_limit and SWIGLUOAI_UNINTERLEAVE both come out as silu_and_mul_with_clamp)
    (activation_func or apply_moe_activation)(
        activation, cache2, cache1.view(-1, shards * N), clamp_limit=clamp_limit, alpha=gemm1_alpha,
        beta=gemm1_beta, topk_ids=topk_ids, expert_map=expert_map, activation_situ_beta=activation_situ_beta,
        activation_situ_linear_beta=activation_situ_linear_beta)
    if output is None:
        output = cache3
    if input_dtype in (torch.int8, torch.float8_e4m3fn):
        cache2, a_scales2 = marlin_quant_input(cache2, input_dtype)
        if input_dtype == torch.int8 and input_global_scale2 is not None:
            a_scales2 = a_scales2 * input_global_scale2
    return ops.moe_wna16_marlin_gemm(
        cache2, output, w2, bias2, w2_scale, a_scales2, global_scale2, w2_zeros, g_idx2, sort_indices2, workspace,
        sorted_token_ids, expert_ids, num_tokens_post_padded, topk_weights, moe_block_size=block_size_m,
        top_k=1, mul_topk_weights=not apply_router_weight_on_input, b_q_type=quant_type,
        size_m=M * num_topk, size_n=K, size_k=N, is_k_full=is_k_full, use_atomic_add=False,
        use_fp32_reduce=True, is_zp_float=False)


def fused_marlin_moe(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                     bias1: torch.Tensor | None, bias2: torch.Tensor | None, w1_scale: torch.Tensor,
                     w2_scale: torch.Tensor, topk_weights: torch.Tensor, topk_ids: torch.Tensor,
                     quant_type_id: int, apply_router_weight_on_input: bool = False,
                     global_num_experts: int = -1, activation="silu", activation_func=None,
                     moe_sum=None, expert_map: torch.Tensor | None = None,
                     input_global_scale1: torch.Tensor | None = None,
                     input_global_scale2: torch.Tensor | None = None,
                     global_scale1: torch.Tensor | None = None, global_scale2: torch.Tensor | None = None,
                     g_idx1: torch.Tensor | None = None, g_idx2: torch.Tensor | None = None,
                     sort_indices1: torch.Tensor | None = None, sort_indices2: torch.Tensor | None = None,
                     w1_zeros: torch.Tensor | None = None, w2_zeros: torch.Tensor | None = None,
                     workspace: torch.Tensor | None = None,
                     intermediate_cache13: torch.Tensor | None = None,
                     intermediate_cache2: torch.Tensor | None = None, is_k_full: bool = True,
                     output: torch.Tensor | None = None, input_dtype: torch.dtype | None = None,
                     clamp_limit: float | None = None, gemm1_alpha: float = 1.0, gemm1_beta: float = 0.0,
                     activation_situ_beta: float | None = None,
                     activation_situ_linear_beta: float | None = None) -> torch.Tensor:
    """Mixture-of-experts layer with Marlin int4 expert weights and top-k gating
    (marlin_moe.py:226-392).  w1: (E, K/16, 2 * 2N) gate and up projections,
    w2: (E, N/16, 2K); scales (E, groups, 2N) / (E, groups, K); topk_weights
    fp32 [M, top_k]; topk_ids [M, top_k].  Returns [M, K].  Parameters and their order are
    the reference's: `activation` any of its MoEActivation values (a gated one takes w1 with the
    gate and up projections, (E, K/16, 2 * 2N); one without a gate takes (E, K/16, 2N)), with
    clamp_limit / gemm1_alpha / gemm1_beta for the clamped SwiGLU forms (SILU with a clamp_limit,
    SWIGLUOAI_UNINTERLEAVE: the experts of gpt-oss) and activation_situ_beta /
    activation_situ_linear_beta for SITU; global_scale1 / global_scale2 are the per-expert global
    scales of NVFP4 experts.  input_dtype torch.int8 / torch.float8_e4m3fn:
    the tokens and the activation's output are quantised per row and both GEMMs run on the 8-bit
    matrix cores (4-bit expert weights repacked with is_a_8bit; input_global_scale1 / 2 are the
    factors marlin_act_int8_process_scales returns for the integer group scales).
    `activation_func(activation, out, in, **parameters)` and `moe_sum(moe_output [M, top_k, K],
    output, topk_ids, expert_map)` replace the built-in HIP kernels when given, as in the reference."""
    _check_arguments(activation, input_dtype, (input_global_scale1, input_global_scale2, global_scale1,
                                               global_scale2))
    if quant_type_id not in _SUPPORTED:
        raise NotImplementedError(f"quant type id {quant_type_id}: only uint4, uint4b8, uint8b128, "
                                  "float8_e4m3fn and float4_e2m1f (MXFP4, NVFP4) expert weights are built")
    quant_type = _SUPPORTED[quant_type_id]
    M, K = hidden_states.shape
    E = w1.shape[0]
    topk = topk_ids.shape[1]
    assert w1.shape[1] * 16 == K, "Hidden size mismatch w1"
    assert w2.shape[2] // (_SUPPORTED[quant_type_id].size_bits // 2) == K, "Hidden size mismatch w2"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.is_contiguous(), "Expert weights1 must be contiguous"
    assert w2.is_contiguous(), "Expert weights2 must be contiguous"
    assert hidden_states.dtype in (torch.float16, torch.bfloat16)
    assert topk_weights.dtype == torch.float32

    m_est = M
    if global_num_experts == -1:
        global_num_experts = E
    else:
        m_est = math.ceil(M * E / global_num_experts)   # expected tokens for the local experts
    block_size_m = moe_block_size(m_est, topk, E)
    if input_dtype is not None and input_dtype.itemsize == 1:
        block_size_m = max(block_size_m, 16)             # marlin_moe.py:328-329
    sorted_token_ids, expert_ids, num_tokens_post_padded = moe_align_block_size(
        topk_ids, block_size_m, global_num_experts, expert_map, ignore_invalid_experts=True)

    sum_rows = moe_sum
    moe_output = _fused_marlin_moe(
        hidden_states, w1, w2, bias1, bias2, w1_scale, w2_scale, topk_weights, topk, quant_type,
        apply_router_weight_on_input, expert_map, block_size_m, sorted_token_ids, expert_ids,
        num_tokens_post_padded, activation=activation, activation_func=activation_func, topk_ids=topk_ids,
        input_global_scale1=input_global_scale1, input_global_scale2=input_global_scale2,
        global_scale1=global_scale1, global_scale2=global_scale2, g_idx1=g_idx1, g_idx2=g_idx2,
        sort_indices1=sort_indices1, sort_indices2=sort_indices2,
        w1_zeros=w1_zeros, w2_zeros=w2_zeros, workspace=workspace,
        intermediate_cache13=intermediate_cache13, intermediate_cache2=intermediate_cache2, output=None,
        input_dtype=input_dtype, is_k_full=is_k_full, clamp_limit=clamp_limit, gemm1_alpha=gemm1_alpha,
        gemm1_beta=gemm1_beta, activation_situ_beta=activation_situ_beta,
        activation_situ_linear_beta=activation_situ_linear_beta).view(-1, topk, K)
    if output is None:
        output = torch.empty_like(hidden_states)
    if expert_map is not None:
        # slots of experts held elsewhere (or with an id outside the table) were never written
        ids = topk_ids.to(torch.int64)
        inside = (ids >= 0) & (ids < global_num_experts)
        local = inside & (expert_map.to(torch.int64)[ids.clamp(0, global_num_experts - 1)] >= 0)
        moe_output = torch.where(local.unsqueeze(-1), moe_output, torch.zeros_like(moe_output))
    if sum_rows is not None:   # called as the reference calls it (marlin_moe.py:391)
        sum_rows(moe_output.contiguous(), output, topk_ids, expert_map)
        return output
    return globals()["moe_sum"](moe_output.contiguous(), output)


def batched_fused_marlin_moe(hidden_states: torch.Tensor, expert_num_tokens: torch.Tensor, w1: torch.Tensor,
                             w2: torch.Tensor, bias1: torch.Tensor | None, bias2: torch.Tensor | None,
                             w1_scale: torch.Tensor, w2_scale: torch.Tensor, quant_type_id: int,
                             apply_router_weight_on_input: bool = False, global_num_experts: int = -1,
                             activation="silu", expert_map: torch.Tensor | None = None,
                             input_global_scale1: torch.Tensor | None = None,
                             input_global_scale2: torch.Tensor | None = None,
                             global_scale1: torch.Tensor | None = None, global_scale2: torch.Tensor | None = None,
                             g_idx1: torch.Tensor | None = None, g_idx2: torch.Tensor | None = None,
                             sort_indices1: torch.Tensor | None = None, sort_indices2: torch.Tensor | None = None,
                             w1_zeros: torch.Tensor | None = None, w2_zeros: torch.Tensor | None = None,
                             workspace: torch.Tensor | None = None,
                             intermediate_cache13: torch.Tensor | None = None,
                             intermediate_cache2: torch.Tensor | None = None, is_k_full: bool = True,
                             output: torch.Tensor | None = None, input_dtype: torch.dtype | None = None,
                             clamp_limit: float | None = None, gemm1_alpha: float = 1.0, gemm1_beta: float = 0.0,
                             activation_func=None, activation_situ_beta: float | None = None,
                             activation_situ_linear_beta: float | None = None) -> torch.Tensor:
    """The layer on tokens already batched by expert (marlin_moe.py:395-560; same
    parameters in the same order): hidden_states [E, max_tokens, K], of which the first
    expert_num_tokens[e] rows of batch e are valid.  Every row belongs to one expert, so
    top_k = 1 and the routing weights are ones.  Returns [E, max_tokens, K]; rows of invalid
    tokens are not written.  global_num_experts and expert_map are accepted for signature
    parity (the batches are the local experts already)."""
    if quant_type_id not in _SUPPORTED:
        raise NotImplementedError(f"quant type id {quant_type_id}: only uint4, uint4b8, uint8b128, "
                                  "float8_e4m3fn and float4_e2m1f (MXFP4, NVFP4) expert weights are built")
    assert hidden_states.ndim == 3, f"hidden states must be batched. e.g. [B, MAX_TOKENS, K].But got {hidden_states.size()}"
    B, max_tokens, K = hidden_states.shape
    E = w1.shape[0]
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert hidden_states.dtype in (torch.float16, torch.bfloat16)
    assert expert_num_tokens.size(0) == E
    assert B == E, "Batch must be as big as number of experts as the tokens are sorted into the batch/expert they belong to"
    assert w1.shape[1] * 16 == K, "Hidden size mismatch w1"
    assert w2.shape[2] // (_SUPPORTED[quant_type_id].size_bits // 2) == K, "Hidden size mismatch w2"
    assert w1.is_contiguous() and w2.is_contiguous(), "Expert weights must be contiguous"
    block_size_m = 64
    for b_m in (8, 16, 32, 48, 64):
        if max_tokens / b_m < 0.9:
            block_size_m = b_m
            break
    if input_dtype is not None and input_dtype.itemsize == 1:
        block_size_m = max(block_size_m, 16)             # marlin_moe.py:507-508
    sorted_token_ids, expert_ids, num_tokens_post_padded = batched_moe_align_block_size(
        max_tokens, block_size_m, expert_num_tokens)
    M = B * max_tokens
    topk_weights = torch.ones((M, 1), device=hidden_states.device, dtype=torch.float32)
    out = _fused_marlin_moe(
        hidden_states.view(-1, K), w1, w2, bias1, bias2, w1_scale, w2_scale, topk_weights, 1,
        _SUPPORTED[quant_type_id], apply_router_weight_on_input, None, block_size_m, sorted_token_ids,
        expert_ids, num_tokens_post_padded, activation=activation, activation_func=activation_func,
        input_global_scale1=input_global_scale1, input_global_scale2=input_global_scale2,
        global_scale1=global_scale1, global_scale2=global_scale2, g_idx1=g_idx1, g_idx2=g_idx2,
        sort_indices1=sort_indices1, sort_indices2=sort_indices2, w1_zeros=w1_zeros, w2_zeros=w2_zeros,
        workspace=workspace, intermediate_cache13=intermediate_cache13, intermediate_cache2=intermediate_cache2,
        output=output.view(-1, K) if output is not None else None, input_dtype=input_dtype, is_k_full=is_k_full,
        clamp_limit=clamp_limit, gemm1_alpha=gemm1_alpha, gemm1_beta=gemm1_beta,
        activation_situ_beta=activation_situ_beta, activation_situ_linear_beta=activation_situ_linear_beta)
    return out.view(B, max_tokens, K)
