"""bf16 / fp8 blockwise MoE (block-sharded variant of the reference): host side.

Signature of ``bwmm_shard_on_block``
(src/nkilib_src/nkilib/core/moe/moe_cte/bwmm_shard_on_block.py:71-96).  On one GPU the
"two shards" of the reference do not exist; the return shape ``[T+1, 2, H]`` (result in
slot 0, slot 1 zero, :237-242 and :1041-1065) is kept so that callers index the same way.
"""

from typing import Any, Optional

import torch

from .... import _native as nv
from ...._entry import KernelEntry
from ...utils.common_types import ActFnType, ExpertAffinityScaleMode
from ...utils.kernel_assert import kernel_assert
from ._launch import run_blockwise
from .moe_cte_utils import BlockShardStrategy, SkipMode


def _expand_scale(scale, E, width, what):
    """fp32 weight scales to per-output-channel form [E or 1, width].

    Accepts the reference's quantize strategies (test_moe_cte_common.py:154-170):
    per tensor [1,1,2] / [E,1,2] (gate, up) or [.,1,1], and per channel [.,1,2I] / [.,1,H].
    """
    s = scale.to(torch.float32)
    kernel_assert(s.dim() == 3 and s.shape[1] == 1, f"{what} must be [E or 1, 1, n] but got {tuple(s.shape)}")
    kernel_assert(s.shape[0] in (1, E), f"{what} first dimension must be 1 or E={E} but got {s.shape[0]}")
    n = s.shape[2]
    if n == width:
        return s.reshape(s.shape[0], width).contiguous()
    if n == 1:
        return s.reshape(s.shape[0], 1).expand(s.shape[0], width).contiguous()
    kernel_assert(n == 2 and width % 2 == 0, f"{what} last dimension must be 1, 2 or {width} but got {n}")
    return s.reshape(s.shape[0], 2, 1).expand(s.shape[0], 2, width // 2).reshape(s.shape[0], width).contiguous()


def run_dense_variant(
    hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight, block_size, token_position_to_id,
    block_to_expert, out_shape_kind, conditions=None, gate_and_up_proj_bias=None, down_proj_bias=None,
    gate_up_proj_scale=None, down_proj_scale=None, activation_function=ActFnType.SiLU, skip_dma=None,
    expert_affinities_scaling_mode=ExpertAffinityScaleMode.POST_SCALE, gate_clamp_upper_limit=None,
    gate_clamp_lower_limit=None, up_clamp_upper_limit=None, up_clamp_lower_limit=None, checkpoint_gate_up=False,
    checkpoint_down=False,
):
    """Common body of the non-MX variants (they share one golden, test_moe_cte_common.py:267-447)."""
    hidden_states = nv.require_device_tensor(hidden_states, "hidden_states")
    guw = nv.require_device_tensor(gate_up_proj_weight, "gate_up_proj_weight")
    dw = nv.require_device_tensor(down_proj_weight, "down_proj_weight")
    kernel_assert(hidden_states.dim() == 2, f"hidden_states must be [T+1, H] but got {tuple(hidden_states.shape)}")
    kernel_assert(guw.dim() == 4 and guw.shape[2] == 2,
                  f"gate_up_proj_weight must be [E, H, 2, I] but got {tuple(guw.shape)}")
    E, H, _, I = guw.shape
    kernel_assert(dw.dim() == 3 and dw.shape[0] == E and dw.shape[2] == H and dw.shape[1] >= I,
                  f"down_proj_weight must be [E, I_padded, H] = [{E}, >={I}, {H}] but got {tuple(dw.shape)}")
    kernel_assert(expert_affinities_scaling_mode != ExpertAffinityScaleMode.PRE_SCALE_DELAYED,
                  "Currently ExpertAffinityScaleMode PRE_SCALE_DELAYED is not support ")
    T1 = hidden_states.shape[0]
    dims = {"T1": T1, "H": H, "I": I, "E": E, "I_pad": dw.shape[1]}
    fp8_w = guw.dtype in (torch.float8_e4m3fn, torch.uint8, torch.int8)
    kernel_assert(fp8_w == (dw.dtype in (torch.float8_e4m3fn, torch.uint8, torch.int8)),
                  "gate_up_proj_weight and down_proj_weight must have the same element type")
    gus = ds = None
    scale_experts = 0
    if gate_up_proj_scale is not None or down_proj_scale is not None:
        kernel_assert(gate_up_proj_scale is not None and down_proj_scale is not None,
                      "gate_up_proj_scale and down_proj_scale must be given together")
        gus = _expand_scale(nv.require_device_tensor(gate_up_proj_scale, "gate_up_proj_scale"), E, 2 * I,
                            "gate_up_proj_scale")
        ds = _expand_scale(nv.require_device_tensor(down_proj_scale, "down_proj_scale"), E, H, "down_proj_scale")
        kernel_assert(gus.shape[0] == ds.shape[0], "weight scales must agree on their expert dimension")
        scale_experts = gus.shape[0]
    if gate_and_up_proj_bias is not None:
        kernel_assert(tuple(gate_and_up_proj_bias.shape) == (E, 2, I),
                      f"gate_and_up_proj_bias must be [E, 2, I] but got {tuple(gate_and_up_proj_bias.shape)}")

    fp8_act = hidden_states.dtype in (torch.float8_e4m3fn, torch.uint8)
    if fp8_act:
        # RMSNorm-Quant ROW records: [T+1, H+4] (rmsnorm_quant.py:149-156)
        kernel_assert(hidden_states.shape[1] == H + 4,
                      f"fp8 hidden_states must be rmsnorm_quant ROW records [T+1, H+4={H + 4}] but got "
                      f"{tuple(hidden_states.shape)}")
        kernel_assert(fp8_w and gus is not None, "fp8 activations need fp8 weights with per-channel scales")
        kind, wdt = nv.KIND_FP8_ROW, nv.DT_FP8
    else:
        kernel_assert(hidden_states.dtype == torch.bfloat16,
                      f"hidden_states must be bfloat16 (or fp8 ROW records) but got {hidden_states.dtype}")
        kernel_assert(hidden_states.shape[1] == H, f"hidden_states must be [T+1, {H}] but got {tuple(hidden_states.shape)}")
        if fp8_w:
            kernel_assert(gus is not None, "fp8 weights need gate_up_proj_scale / down_proj_scale")
            kind, wdt = nv.KIND_BF16, nv.DT_FP8
        else:
            kernel_assert(guw.dtype == torch.bfloat16, f"weights must be bfloat16 or fp8 but got {guw.dtype}")
            kind, wdt = nv.KIND_BF16, nv.DT_BF16
    return run_blockwise(
        kind, hidden_states, expert_affinities_masked, guw, dw, token_position_to_id, block_to_expert, block_size,
        out_shape_kind, dims, conditions=conditions, gate_and_up_proj_bias=gate_and_up_proj_bias,
        down_proj_bias=down_proj_bias, gate_up_proj_scale=gus, down_proj_scale=ds,
        activation_function=activation_function, skip_dma=skip_dma,
        expert_affinities_scaling_mode=expert_affinities_scaling_mode,
        gate_clamp_upper_limit=gate_clamp_upper_limit, gate_clamp_lower_limit=gate_clamp_lower_limit,
        up_clamp_upper_limit=up_clamp_upper_limit, up_clamp_lower_limit=up_clamp_lower_limit, weight_dtype=wdt,
        scale_experts=scale_experts, checkpoint_gate_up=checkpoint_gate_up, checkpoint_down=checkpoint_down,
    )


def _bwmm_shard_on_block(
    hidden_states: torch.Tensor,
    expert_affinities_masked: torch.Tensor,
    gate_up_proj_weight: torch.Tensor,
    down_proj_weight: torch.Tensor,
    block_size: int,
    token_position_to_id: torch.Tensor,
    block_to_expert: torch.Tensor,
    gate_and_up_proj_bias: Optional[torch.Tensor] = None,
    down_proj_bias: Optional[torch.Tensor] = None,
    gate_up_proj_scale: Optional[torch.Tensor] = None,
    down_proj_scale: Optional[torch.Tensor] = None,
    down_activations: Optional[torch.Tensor] = None,
    activation_function: ActFnType = ActFnType.SiLU,
    skip_dma: SkipMode = SkipMode(False, False),
    compute_dtype: Any = torch.bfloat16,
    is_tensor_update_accumulating: bool = True,
    expert_affinities_scaling_mode: ExpertAffinityScaleMode = ExpertAffinityScaleMode.POST_SCALE,
    n_block_per_iter: int = 1,
    gate_clamp_upper_limit: Optional[float] = None,
    gate_clamp_lower_limit: Optional[float] = None,
    up_clamp_upper_limit: Optional[float] = None,
    up_clamp_lower_limit: Optional[float] = None,
    block_sharding_strategy: BlockShardStrategy = BlockShardStrategy.PING_PONG,
):
    """Returns bf16 ``[T+1, 2, H]`` (accumulating; result in ``[:, 0, :]``) or ``[T+1, H]``."""
    kernel_assert(down_activations is None, "down_activations (activation checkpointing) is not supported on gfx950")
    return run_dense_variant(
        hidden_states, expert_affinities_masked, gate_up_proj_weight, down_proj_weight, block_size,
        token_position_to_id, block_to_expert, "T2H" if is_tensor_update_accumulating else "TH",
        gate_and_up_proj_bias=gate_and_up_proj_bias, down_proj_bias=down_proj_bias,
        gate_up_proj_scale=gate_up_proj_scale, down_proj_scale=down_proj_scale,
        activation_function=activation_function, skip_dma=skip_dma,
        expert_affinities_scaling_mode=expert_affinities_scaling_mode,
        gate_clamp_upper_limit=gate_clamp_upper_limit, gate_clamp_lower_limit=gate_clamp_lower_limit,
        up_clamp_upper_limit=up_clamp_upper_limit, up_clamp_lower_limit=up_clamp_lower_limit,
    )


bwmm_shard_on_block = KernelEntry(_bwmm_shard_on_block)
