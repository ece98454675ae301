"""The reference's expert classes for the Marlin mixture-of-experts layer
(aphrodite/model_executor/layers/fused_moe/experts/marlin_moe.py:568-1096: MarlinExpertsBase,
MarlinExperts, BatchedMarlinExperts), with the same constructor arguments, properties and
`workspace_shapes` / `apply` / `moe_sum` signatures, on top of this package's
fused_marlin_moe / batched_fused_marlin_moe.

The reference derives them from its modular-kernel framework (FusedMoEExpertsModular) and
takes FusedMoEConfig / FusedMoEQuantConfig objects from it.  That framework is not part of
this package, so the classes here stand alone and read the configuration objects by
attribute: anything with the reference's attribute names serves (`ExpertsQuantConfig` below
is a plain holder of them).  The LoRA injection of the reference's MarlinExperts.apply
(its `_lora_context` branch) belongs to that framework too and is not here."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .fused_moe import (_NOT_GATED, _GATED, _activation_name, apply_moe_activation, batched_fused_marlin_moe,
                        fused_marlin_moe)
from .fused_moe import moe_sum as _moe_sum
from .marlin_utils import get_marlin_input_dtype, marlin_moe_intermediate_size
from .scalar_type import scalar_types


@dataclass
class ExpertsQuantConfig:
    """The fields of the reference's FusedMoEQuantConfig that the Marlin expert classes read
    (fused_moe/config.py; marlin_moe.py:583-603, 665-677, 768-803)."""
    use_int4_w4a16: bool = False
    use_int8_w8a16: bool = False
    use_fp8_w8a16: bool = False
    use_mxfp4_w4a16: bool = False
    use_nvfp4_w4a16: bool = False
    w1_scale: torch.Tensor | None = None
    w2_scale: torch.Tensor | None = None
    w1_zp: torch.Tensor | None = None
    w2_zp: torch.Tensor | None = None
    w1_bias: torch.Tensor | None = None
    w2_bias: torch.Tensor | None = None
    g1_alphas: torch.Tensor | None = None      # NVFP4: the experts' global scales
    g2_alphas: torch.Tensor | None = None
    a1_gscale: torch.Tensor | None = None      # int8 activations: factors of the integer group scales
    a2_gscale: torch.Tensor | None = None
    gemm1_clamp_limit: float | None = None
    gemm1_alpha: float | None = None
    gemm1_beta: float | None = None


@dataclass
class ExpertsMoeConfig:
    """The fields of the reference's FusedMoEConfig read here (marlin_moe.py:793-794)."""
    activation_situ_beta: float | None = None
    activation_situ_linear_beta: float | None = None


class MarlinExpertsBase:
    """marlin_moe.py:568-704."""

    def __init__(self, moe_config, quant_config, max_num_tokens: int | None = None,
                 num_dispatchers: int | None = None, w13_g_idx: torch.Tensor | None = None,
                 w2_g_idx: torch.Tensor | None = None, w13_g_idx_sort_indices: torch.Tensor | None = None,
                 w2_g_idx_sort_indices: torch.Tensor | None = None, is_k_full: bool = True):
        assert (quant_config.use_mxfp4_w4a16 or quant_config.use_nvfp4_w4a16 or quant_config.use_int4_w4a16
                or quant_config.use_int8_w8a16 or quant_config.use_fp8_w8a16), \
            "Supports only {mxfp,nvfp,int}4_w4a16, int8_w8a16 or fp8_w8a16"
        self.moe_config = moe_config
        self.quant_config = quant_config
        self.max_num_tokens = max_num_tokens
        self.num_dispatchers = num_dispatchers
        self.w13_g_idx = w13_g_idx
        self.w2_g_idx = w2_g_idx
        self.w13_g_idx_sort_indices = w13_g_idx_sort_indices
        self.w2_g_idx_sort_indices = w2_g_idx_sort_indices
        self.is_k_full = is_k_full
        self.input_dtype = get_marlin_input_dtype()
        self.gemm1_clamp_limit = quant_config.gemm1_clamp_limit
        # silu is swigluoai with alpha = 1, beta = 0: configurations that set neither get that
        self.gemm1_alpha = quant_config.gemm1_alpha if quant_config.gemm1_alpha is not None else 1.0
        self.gemm1_beta = quant_config.gemm1_beta if quant_config.gemm1_beta is not None else 0.0

    # what the modular-kernel base class forwards from the quantisation configuration
    w1_scale = property(lambda self: self.quant_config.w1_scale)
    w2_scale = property(lambda self: self.quant_config.w2_scale)
    w1_zp = property(lambda self: self.quant_config.w1_zp)
    w2_zp = property(lambda self: self.quant_config.w2_zp)
    w1_bias = property(lambda self: self.quant_config.w1_bias)
    w2_bias = property(lambda self: self.quant_config.w2_bias)
    g1_alphas = property(lambda self: self.quant_config.g1_alphas)
    g2_alphas = property(lambda self: self.quant_config.g2_alphas)
    a1_gscale = property(lambda self: self.quant_config.a1_gscale)
    a2_gscale = property(lambda self: self.quant_config.a2_gscale)

    @staticmethod
    def _supports_current_device() -> bool:
        """The reference asks for CUDA with capability 7.5; here: a gfx950 device."""
        if not torch.cuda.is_available():
            return False
        return "gfx950" in getattr(torch.cuda.get_device_properties(0), "gcnArchName", "")

    @staticmethod
    def _supports_no_act_and_mul() -> bool:
        return True

    @staticmethod
    def _supports_activation(activation) -> bool:
        """Every activation apply_moe_activation dispatches (marlin_moe.py:636-652)."""
        return _activation_name(activation) in _GATED + _NOT_GATED

    def activation(self, activation, output: torch.Tensor, input: torch.Tensor, **parameters) -> None:
        apply_moe_activation(activation, output, input, **parameters)

    @property
    def quant_type_id(self) -> int:
        if self.quant_config.use_int4_w4a16:
            if self.w1_zp is not None or self.w2_zp is not None:
                return scalar_types.uint4.id
            return scalar_types.uint4b8.id
        if self.quant_config.use_int8_w8a16:
            return scalar_types.uint8b128.id
        if self.quant_config.use_mxfp4_w4a16 or self.quant_config.use_nvfp4_w4a16:
            return scalar_types.float4_e2m1f.id
        if self.quant_config.use_fp8_w8a16:
            return scalar_types.float8_e4m3fn.id
        raise NotImplementedError("Unsupported quantization type.")

    def moe_problem_size(self, a1: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                         topk_ids: torch.Tensor) -> tuple[int, int, int, int, int]:
        """(E, M, N, K, topk); a1 [M, K], or [E, max_num_tokens, K] in the batched format."""
        assert w1.dim() == 3 and w2.dim() == 3
        E = w1.size(0)
        K = a1.size(-1)
        N = marlin_moe_intermediate_size(w1, w2)
        if a1.dim() == 2:
            assert topk_ids.size(0) == a1.size(0), f"{topk_ids.size(0)} != {a1.size(0)}"
            M = a1.size(0)
        else:
            assert a1.dim() == 3
            assert a1.size(0) == E, f"{a1.size(0)} == {E}"
            M = a1.size(1)
        assert topk_ids.dim() == 2
        return E, M, N, K, topk_ids.size(1)


class MarlinExperts(MarlinExpertsBase):
    """marlin_moe.py:707-952 without the LoRA branch: tokens in the standard format."""

    @staticmethod
    def activation_format() -> str:
        return "standard"

    def workspace_shapes(self, M: int, N: int, K: int, topk: int, global_num_experts: int,
                         local_num_experts: int, expert_tokens_meta, activation):
        """(workspace13, workspace2, output).  As in the reference the two workspaces are swapped
        against fused_marlin_moe's intermediate caches, so that the output buffer (provisioned
        from workspace13 by the caller) never overlaps the input of the final sum."""
        workspace1 = (M * topk, max(N, K))
        workspace2 = (M * topk * max(2 * N, K),)
        output = (M, K)
        return workspace1, workspace2, output

    def apply(self, output: torch.Tensor, hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
              topk_weights: torch.Tensor, topk_ids: torch.Tensor, activation, global_num_experts: int,
              expert_map: torch.Tensor | None, a1q_scale: torch.Tensor | None, a2_scale: torch.Tensor | None,
              workspace13: torch.Tensor, workspace2: torch.Tensor, expert_tokens_meta,
              apply_router_weight_on_input: bool):
        assert self.w1_scale is not None
        assert self.w2_scale is not None
        fused_marlin_moe(
            hidden_states=hidden_states, w1=w1, w2=w2, bias1=self.w1_bias, bias2=self.w2_bias,
            w1_scale=self.w1_scale, w2_scale=self.w2_scale, topk_weights=topk_weights, topk_ids=topk_ids,
            global_scale1=self.g1_alphas, global_scale2=self.g2_alphas, input_global_scale1=self.a1_gscale,
            input_global_scale2=self.a2_gscale, w1_zeros=self.w1_zp, w2_zeros=self.w2_zp,
            quant_type_id=self.quant_type_id, apply_router_weight_on_input=apply_router_weight_on_input,
            global_num_experts=global_num_experts, activation=activation, activation_func=self.activation,
            activation_situ_beta=self.moe_config.activation_situ_beta,
            activation_situ_linear_beta=self.moe_config.activation_situ_linear_beta,
            moe_sum=self.moe_sum, expert_map=expert_map, output=output,
            intermediate_cache13=workspace2, intermediate_cache2=workspace13,      # swapped: see workspace_shapes
            g_idx1=self.w13_g_idx, g_idx2=self.w2_g_idx, sort_indices1=self.w13_g_idx_sort_indices,
            sort_indices2=self.w2_g_idx_sort_indices, is_k_full=self.is_k_full, input_dtype=self.input_dtype,
            clamp_limit=self.gemm1_clamp_limit, gemm1_alpha=self.gemm1_alpha, gemm1_beta=self.gemm1_beta)

    def moe_sum(self, input: torch.Tensor, output: torch.Tensor, topk_ids: torch.Tensor,
                expert_map: torch.Tensor | None) -> None:
        """output[t] = sum over the top-k slots of input[t] (slots of experts held elsewhere arrive
        as zeros from fused_marlin_moe, so the map needs no second look)."""
        _moe_sum(input, output)


class BatchedMarlinExperts(MarlinExpertsBase):
    """marlin_moe.py:955-1096: tokens already batched by expert, [E, max_num_tokens, K]."""

    def __init__(self, moe_config, quant_config, max_num_tokens: int, num_dispatchers: int,
                 w13_g_idx: torch.Tensor | None = None, w2_g_idx: torch.Tensor | None = None,
                 w13_g_idx_sort_indices: torch.Tensor | None = None,
                 w2_g_idx_sort_indices: torch.Tensor | None = None, is_k_full: bool = True):
        super().__init__(moe_config=moe_config, quant_config=quant_config, max_num_tokens=max_num_tokens,
                         num_dispatchers=num_dispatchers, w13_g_idx=w13_g_idx, w2_g_idx=w2_g_idx,
                         w13_g_idx_sort_indices=w13_g_idx_sort_indices,
                         w2_g_idx_sort_indices=w2_g_idx_sort_indices, is_k_full=is_k_full)

    @staticmethod
    def activation_format() -> str:
        return "batched_experts"

    def workspace_shapes(self, M: int, N: int, K: int, topk: int, global_num_experts: int,
                         local_num_experts: int, expert_tokens_meta, activation):
        assert self.num_dispatchers is not None
        assert self.max_num_tokens is not None
        rows = local_num_experts * self.max_num_tokens * self.num_dispatchers
        workspace13 = (rows, max(K, N * 2))
        workspace2 = (rows, N)
        output = (local_num_experts, self.max_num_tokens * self.num_dispatchers, K)
        return workspace13, workspace2, output

    def apply(self, output: torch.Tensor, hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
              topk_weights: torch.Tensor, topk_ids: torch.Tensor, activation, global_num_experts: int,
              expert_map: torch.Tensor | None, a1q_scale: torch.Tensor | None, a2_scale: torch.Tensor | None,
              workspace13: torch.Tensor, workspace2: torch.Tensor, expert_tokens_meta,
              apply_router_weight_on_input: bool):
        """`expert_tokens_meta.expert_num_tokens`: the valid rows of every batch.  (The reference
        runs SITU through a kernel that skips the invalid rows; here the plain kernel runs over all
        of them: rows of invalid tokens are never read back.)"""
        assert expert_tokens_meta is not None, "Num valid tokens per batch is required"
        return batched_fused_marlin_moe(
            hidden_states=hidden_states, expert_num_tokens=expert_tokens_meta.expert_num_tokens, w1=w1, w2=w2,
            bias1=self.w1_bias, bias2=self.w2_bias, w1_scale=self.w1_scale, w2_scale=self.w2_scale,
            quant_type_id=self.quant_type_id, apply_router_weight_on_input=apply_router_weight_on_input,
            global_num_experts=global_num_experts, activation=activation, expert_map=expert_map,
            input_global_scale1=self.a1_gscale, input_global_scale2=self.a2_gscale, output=output,
            intermediate_cache13=workspace13, intermediate_cache2=workspace2, g_idx1=self.w13_g_idx,
            g_idx2=self.w2_g_idx, sort_indices1=self.w13_g_idx_sort_indices,
            sort_indices2=self.w2_g_idx_sort_indices, w1_zeros=self.w1_zp, w2_zeros=self.w2_zp,
            input_dtype=self.input_dtype, is_k_full=self.is_k_full, clamp_limit=self.gemm1_clamp_limit,
            gemm1_alpha=self.gemm1_alpha, gemm1_beta=self.gemm1_beta, activation_func=self.activation,
            activation_situ_beta=self.moe_config.activation_situ_beta,
            activation_situ_linear_beta=self.moe_config.activation_situ_linear_beta)
