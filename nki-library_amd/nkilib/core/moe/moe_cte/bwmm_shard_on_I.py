"""Intermediate-sharded variants of the reference: same math as ``bwmm_shard_on_block``
(one golden serves all, test_moe_cte_common.py:267-447); only the return shape differs
(``[T+1, H]``, src/nkilib_src/nkilib/core/moe/moe_cte/bwmm_shard_on_I.py:293).  The
Trainium-specific split of I over two cores has no GPU counterpart.  Signatures:
bwmm_shard_on_I.py:86-114, :326-355, :2013-2036."""

from typing import Optional

import torch

from ...._entry import KernelEntry
from ...utils.common_types import ActFnType, ExpertAffinityScaleMode
from ...utils.kernel_assert import kernel_assert
from .bwmm_shard_on_block import run_dense_variant
from .moe_cte_utils import SkipMode


def _blockwise_mm_baseline_shard_intermediate(
    hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight, block_size, token_position_to_id,
    block_to_expert, gate_and_up_proj_bias=None, down_proj_bias=None, gate_up_proj_scale=None, down_proj_scale=None,
    activation_function: ActFnType = ActFnType.SiLU, skip_dma: SkipMode = SkipMode(), compute_dtype=torch.bfloat16,
    is_tensor_update_accumulating=True, expert_affinities_scaling_mode=ExpertAffinityScaleMode.PRE_SCALE,
    gate_clamp_upper_limit: Optional[float] = None, gate_clamp_lower_limit: Optional[float] = None,
    up_clamp_lower_limit: Optional[float] = None, up_clamp_upper_limit: Optional[float] = None,
    checkpoint_activation=False, expert_affinity_multiply_on_I=False,
):
    """``checkpoint_activation``: also returns ``gate_up_activations_T`` ``[N, 2, I, B]`` (gate / up projections
    after scale, bias and clamp, before the activation: the golden's in-place views,
    test_moe_cte_common.py:383-405) and, unless ``expert_affinity_multiply_on_I``, ``down_activations``
    ``[N, B, H]`` (before the affinity, :410-421), as bwmm_shard_on_I.py:314-323 does.
    ``expert_affinity_multiply_on_I`` itself only moves a multiplication inside the reference kernel; the one
    golden serves both settings and so does this kernel."""
    return run_dense_variant(
        hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight, block_size,
        token_position_to_id, block_to_expert, "TH", gate_and_up_proj_bias=gate_and_up_proj_bias,
        down_proj_bias=down_proj_bias, gate_up_proj_scale=gate_up_proj_scale, down_proj_scale=down_proj_scale,
        activation_function=activation_function, skip_dma=skip_dma,
        expert_affinities_scaling_mode=expert_affinities_scaling_mode,
        gate_clamp_upper_limit=gate_clamp_upper_limit, gate_clamp_lower_limit=gate_clamp_lower_limit,
        up_clamp_upper_limit=up_clamp_upper_limit, up_clamp_lower_limit=up_clamp_lower_limit,
        checkpoint_gate_up=bool(checkpoint_activation),
        checkpoint_down=bool(checkpoint_activation) and not expert_affinity_multiply_on_I,
    )


def _blockwise_mm_baseline_shard_intermediate_hybrid(
    conditions, hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight, block_size: int,
    token_position_to_id, block_to_expert, num_static_block: Optional[int] = None, gate_and_up_proj_bias=None,
    down_proj_bias=None, gate_up_proj_scale=None, down_proj_scale=None, gate_up_activations_T=None,
    down_activations=None, activation_function: ActFnType = ActFnType.SiLU, skip_dma: SkipMode = SkipMode(),
    compute_dtype=torch.bfloat16, is_tensor_update_accumulating=True,
    expert_affinities_scaling_mode=ExpertAffinityScaleMode.POST_SCALE, gate_clamp_upper_limit: Optional[float] = None,
    gate_clamp_lower_limit: Optional[float] = None, up_clamp_lower_limit: Optional[float] = None,
    up_clamp_upper_limit: Optional[float] = None,
):
    """``conditions`` stops the block loop at its first zero (test_moe_cte_common.py:331-333);
    ``num_static_block`` only tunes the reference's static/dynamic loop split and is ignored."""
    kernel_assert(gate_up_activations_T is None and down_activations is None,
                  "activation checkpoint outputs are not supported on gfx950")
    return run_dense_variant(
        hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight, block_size,
        token_position_to_id, block_to_expert, "TH", conditions=conditions,
        gate_and_up_proj_bias=gate_and_up_proj_bias, down_proj_bias=down_proj_bias,
        gate_up_proj_scale=gate_up_proj_scale, down_proj_scale=down_proj_scale,
        activation_function=activation_function, skip_dma=skip_dma,
        expert_affinities_scaling_mode=expert_affinities_scaling_mode,
        gate_clamp_upper_limit=gate_clamp_upper_limit, gate_clamp_lower_limit=gate_clamp_lower_limit,
        up_clamp_upper_limit=up_clamp_upper_limit, up_clamp_lower_limit=up_clamp_lower_limit,
    )


def _blockwise_mm_shard_intermediate_dropping(
    hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight, block_size, token_position_to_id,
    block_to_expert, gate_and_up_proj_bias=None, down_proj_bias=None, gate_up_proj_scale=None, down_proj_scale=None,
    activation_function: ActFnType = ActFnType.SiLU, skip_dma: SkipMode = SkipMode(), compute_dtype=torch.bfloat16,
    is_tensor_update_accumulating=True, expert_affinities_scaling_mode=ExpertAffinityScaleMode.PRE_SCALE,
    expert_affinity_multiply_on_I: bool = False, gate_clamp_upper_limit: Optional[float] = None,
    gate_clamp_lower_limit: Optional[float] = None, up_clamp_lower_limit: Optional[float] = None,
    up_clamp_upper_limit: Optional[float] = None,
):
    """Token-dropping layer (bwmm_shard_on_I.py:2014-2159): N == E blocks, block b belongs to expert b
    (``block_to_expert`` is not read), tokens beyond an expert's block were dropped by the caller.  Always returns
    the checkpoints: ``(output, gate_up_activations_T)`` with ``expert_affinity_multiply_on_I``, else
    ``(output, gate_up_activations_T, down_activations)``."""
    if expert_affinities_scaling_mode == ExpertAffinityScaleMode.PRE_SCALE_DELAYED:
        expert_affinities_scaling_mode = ExpertAffinityScaleMode.PRE_SCALE  # bwmm_shard_on_I.py:2084-2085
    E = gate_up_proj_weight.shape[0]
    N = token_position_to_id.numel() // int(block_size)
    kernel_assert(N == E, f"the dropping layer has one block per expert: N ({N}) must equal E ({E})")
    own_expert = torch.arange(N, dtype=torch.int32, device=hidden_states.device)
    return run_dense_variant(
        hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight, block_size,
        token_position_to_id, own_expert, "TH", gate_and_up_proj_bias=gate_and_up_proj_bias,
        down_proj_bias=down_proj_bias, gate_up_proj_scale=gate_up_proj_scale, down_proj_scale=down_proj_scale,
        activation_function=activation_function, skip_dma=skip_dma,
        expert_affinities_scaling_mode=expert_affinities_scaling_mode,
        gate_clamp_upper_limit=gate_clamp_upper_limit, gate_clamp_lower_limit=gate_clamp_lower_limit,
        up_clamp_upper_limit=up_clamp_upper_limit, up_clamp_lower_limit=up_clamp_lower_limit,
        checkpoint_gate_up=True, checkpoint_down=not expert_affinity_multiply_on_I,
    )


blockwise_mm_baseline_shard_intermediate = KernelEntry(_blockwise_mm_baseline_shard_intermediate)
blockwise_mm_baseline_shard_intermediate_hybrid = KernelEntry(_blockwise_mm_baseline_shard_intermediate_hybrid)
blockwise_mm_shard_intermediate_dropping = KernelEntry(_blockwise_mm_shard_intermediate_dropping)
