"""MX blockwise MoE, the reference's intermediate-sharded entry points.

``blockwise_mm_shard_intermediate_mx`` and ``blockwise_mm_shard_intermediate_mx_hybrid``
(src/nkilib_src/nkilib/core/moe/moe_cte/bwmm_shard_on_I_mx.py:95-117, :400-426) compute what
``bwmm_shard_on_block_mx`` computes (one golden serves both, test/integration/nkilib/core/moe/moe_cte/
test_utils.py:474-735); they differ in the Trainium core sharding (I split over two cores, no GPU counterpart),
in the return shape -- the output has the shape of ``hidden_states``, ``[T+1, H]`` (:298, :609) -- and in the
form of ``conditions`` (one entry per block plus one, test_moe_cte_common.py:251-254).  Both run on the same
gfx950 kernels as the shard-on-block variant.
"""

from typing import Any, Optional

import torch

from ...._entry import KernelEntry
from ...utils.common_types import ActFnType, ExpertAffinityScaleMode
from ...utils.kernel_assert import kernel_assert
from .bwmm_shard_on_block_mx import _bwmm_shard_on_block_mx
from .moe_cte_utils import SkipMode


def _run(conditions, hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight,
         token_position_to_id, block_to_expert, gate_and_up_proj_bias, down_proj_bias, gate_up_proj_scale,
         down_proj_scale, block_size, activation_function, skip_dma, compute_dtype, weight_dtype,
         is_tensor_update_accumulating, expert_affinities_scaling_mode, gate_clamp_upper_limit,
         gate_clamp_lower_limit, up_clamp_lower_limit, up_clamp_upper_limit, hidden_states_scale):
    # PRE_SCALE_DELAYED is folded into PRE_SCALE (bwmm_shard_on_I_mx.py:222-223), which the kernel then refuses
    # (:914-915)
    kernel_assert(expert_affinities_scaling_mode not in (ExpertAffinityScaleMode.PRE_SCALE,
                                                         ExpertAffinityScaleMode.PRE_SCALE_DELAYED),
                  "PRE_SCALE mode not implemented")
    kernel_assert(not (skip_dma or SkipMode()).skip_weight, "DMA weight skipping not supported for MXFP4/MXFP8 kernel")
    if conditions is not None:
        N = token_position_to_id.numel() // block_size
        kernel_assert(conditions.numel() >= N, f"conditions must hold one entry per block ({N}), got {conditions.numel()}")
    return _bwmm_shard_on_block_mx(
        hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight, token_position_to_id,
        block_to_expert, conditions=conditions, gate_and_up_proj_bias=gate_and_up_proj_bias,
        down_proj_bias=down_proj_bias, gate_up_proj_scale=gate_up_proj_scale, down_proj_scale=down_proj_scale,
        block_size=block_size, activation_function=activation_function, skip_dma=skip_dma or SkipMode(),
        compute_dtype=compute_dtype, weight_dtype=weight_dtype,
        is_tensor_update_accumulating=is_tensor_update_accumulating,
        expert_affinities_scaling_mode=expert_affinities_scaling_mode, gate_clamp_upper_limit=gate_clamp_upper_limit,
        gate_clamp_lower_limit=gate_clamp_lower_limit, up_clamp_lower_limit=up_clamp_lower_limit,
        up_clamp_upper_limit=up_clamp_upper_limit, hidden_states_scale=hidden_states_scale, _out_shape_kind="TH")


def _blockwise_mm_shard_intermediate_mx(
    hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight, token_position_to_id,
    block_to_expert, gate_and_up_proj_bias=None, down_proj_bias=None, gate_up_proj_scale=None, down_proj_scale=None,
    block_size: int = None, activation_function: ActFnType = ActFnType.SiLU, skip_dma: SkipMode = SkipMode(),
    compute_dtype=torch.bfloat16, weight_dtype: Any = None, is_tensor_update_accumulating: bool = True,
    expert_affinities_scaling_mode: ExpertAffinityScaleMode = ExpertAffinityScaleMode.PRE_SCALE,
    gate_clamp_upper_limit: Optional[float] = None, gate_clamp_lower_limit: Optional[float] = None,
    up_clamp_lower_limit: Optional[float] = None, up_clamp_upper_limit: Optional[float] = None,
    hidden_states_scale: Optional[torch.Tensor] = None,
):
    """Returns bf16 ``[T+1, H]``.  The default scaling mode is the reference's (PRE_SCALE), which the reference
    kernel itself refuses: callers pass POST_SCALE, as its tests do."""
    return _run(None, hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight,
                token_position_to_id, block_to_expert, gate_and_up_proj_bias, down_proj_bias, gate_up_proj_scale,
                down_proj_scale, block_size, activation_function, skip_dma, compute_dtype, weight_dtype,
                is_tensor_update_accumulating, expert_affinities_scaling_mode, gate_clamp_upper_limit,
                gate_clamp_lower_limit, up_clamp_lower_limit, up_clamp_upper_limit, hidden_states_scale)


def _blockwise_mm_shard_intermediate_mx_hybrid(
    conditions, hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight, token_position_to_id,
    block_to_expert, gate_and_up_proj_bias=None, down_proj_bias=None, gate_up_proj_scale=None, down_proj_scale=None,
    block_size: int = None, num_static_block: Optional[int] = None, activation_function: ActFnType = ActFnType.SiLU,
    skip_dma: SkipMode = SkipMode(), compute_dtype=torch.bfloat16, weight_dtype: Any = None,
    is_tensor_update_accumulating: bool = True,
    expert_affinities_scaling_mode: ExpertAffinityScaleMode = ExpertAffinityScaleMode.POST_SCALE,
    gate_clamp_upper_limit: Optional[float] = None, gate_clamp_lower_limit: Optional[float] = None,
    up_clamp_lower_limit: Optional[float] = None, up_clamp_upper_limit: Optional[float] = None,
    hidden_states_scale: Optional[torch.Tensor] = None,
):
    """Returns bf16 ``[T+1, H]``.  Blocks from the first ``conditions[b] == 0`` on are skipped;
    ``num_static_block`` only tunes the reference's static / dynamic loop split and is ignored."""
    kernel_assert(conditions is not None, "conditions is required by the hybrid variant")
    return _run(conditions, hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight,
                token_position_to_id, block_to_expert, gate_and_up_proj_bias, down_proj_bias, gate_up_proj_scale,
                down_proj_scale, block_size, activation_function, skip_dma, compute_dtype, weight_dtype,
                is_tensor_update_accumulating, expert_affinities_scaling_mode, gate_clamp_upper_limit,
                gate_clamp_lower_limit, up_clamp_lower_limit, up_clamp_upper_limit, hidden_states_scale)


blockwise_mm_shard_intermediate_mx = KernelEntry(_blockwise_mm_shard_intermediate_mx)
blockwise_mm_shard_intermediate_mx_hybrid = KernelEntry(_blockwise_mm_shard_intermediate_mx_hybrid)
