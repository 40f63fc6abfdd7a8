"""MXFP8 blockwise MoE: host side.

Signature of ``bwmm_shard_on_block_mx``
(src/nkilib_src/nkilib/core/moe/moe_cte/bwmm_shard_on_block_mx.py:70-102) plus one additive
keyword, ``hidden_states_scale``: when given, ``hidden_states`` holds activations that were
already quantised to MXFP8 by the RMSNorm front end (uint8 / float8 codes ``[T+1, H]`` in k'
order with uint8 E8M0 scales ``[T+1, H/32]``) and the online quantisation pass is skipped.
The reference has the same convention on its decode kernel (``moe_tkg(..., hidden_input_scale)``,
src/nkilib_src/nkilib/core/moe/moe_tkg/moe_tkg.py:55).
"""

from typing import Any, Optional

import torch

from .... import _native as nv
from ...._entry import KernelEntry
from ...utils.common_types import ActFnType, ExpertAffinityScaleMode
from ...utils.kernel_assert import kernel_assert
from ._launch import run_blockwise
from .moe_cte_utils import SkipMode


def _as_bytes(t, what):
    """View an x4-packed tensor (uint32/int32/float32 containers, or 1-byte dtypes) as uint8."""
    t = nv.require_device_tensor(t, what)
    return t.view(torch.uint8)


def _bwmm_shard_on_block_mx(
    hidden_states,
    expert_affinities_masked,
    gate_up_proj_weight,
    down_proj_weight,
    token_position_to_id,
    block_to_expert,
    conditions=None,
    gate_and_up_proj_bias=None,
    down_proj_bias=None,
    gate_up_proj_scale=None,
    down_proj_scale=None,
    block_size=None,
    n_static_blocks: int = -1,
    n_dynamic_blocks: int = 55,
    gate_up_activations_T=None,
    down_activations=None,
    activation_function: ActFnType = ActFnType.SiLU,
    skip_dma: SkipMode = SkipMode(False, False),
    compute_dtype=torch.bfloat16,
    weight_dtype: Any = None,
    is_tensor_update_accumulating=True,
    expert_affinities_scaling_mode=ExpertAffinityScaleMode.POST_SCALE,
    gate_clamp_upper_limit: Optional[float] = None,
    gate_clamp_lower_limit: Optional[float] = None,
    up_clamp_lower_limit: Optional[float] = None,
    up_clamp_upper_limit: Optional[float] = None,
    hidden_states_scale: Optional[torch.Tensor] = None,
    _out_shape_kind: str = "2TH",
):
    """Returns bf16 ``[2, T+1, H]`` with the result in ``[0]`` (``[1]`` is zero).

    gate_up_proj_weight: MXFP8 (e4m3 or e5m2) x4 ``[E, 128, 2, H/512, I]`` (4-byte elements, or uint8 with a
    trailing axis of 4) or MXFP4 x4 (2-byte elements: four 4-bit values each); gate_up_proj_scale uint8 ``[E, 16, 2, H/512, I]``; down_proj_weight x4
    ``[E, p_I, ceil(I/512), H]``; down_proj_scale uint8 ``[E, ceil(p_I/8), ceil(I/512), H]``;
    biases ``[E, p_I, 2, ceil(I/512), 4]`` and ``[E, H]``.  ``n_static_blocks`` /
    ``n_dynamic_blocks`` tune the reference's loop structure and are ignored; ``conditions``
    keeps its meaning (blocks from the first zero on are skipped).
    """
    kernel_assert(gate_up_activations_T is None and down_activations is None,
                  "gate_up_activations_T / down_activations are not supported, please set to None")
    kernel_assert(block_size is not None, "block_size must be given")
    kernel_assert(gate_up_proj_scale is not None and down_proj_scale is not None,
                  "gate_up_proj_scale and down_proj_scale are required for MX weights")
    # the element format of the x4 weights: the reference reads it off the tensor's nl dtype or takes
    # it from ``weight_dtype`` for uint containers; here it is ``weight_dtype`` (a name containing
    # "float4" or "e5m2", or a torch float8 dtype), else the weight tensor's own dtype (2-byte elements
    # are MXFP4, torch.float8_e5m2 is e5m2), else e4m3
    if weight_dtype is not None:
        wd = str(weight_dtype)
    else:
        wd = str(getattr(gate_up_proj_weight, "dtype", ""))
        if getattr(gate_up_proj_weight, "element_size", lambda: 0)() == 2:
            wd = "float4_e2m1fn_x4"
    wdt = nv.DT_FP4_E2M1 if "float4" in wd else (nv.DT_FP8_E5M2 if "e5m2" in wd else nv.DT_FP8)
    wbytes = 2 if wdt == nv.DT_FP4_E2M1 else 4  # bytes of an x4 element
    hidden_states = nv.require_device_tensor(hidden_states, "hidden_states")
    kernel_assert(hidden_states.dim() == 2, f"hidden_states must be [T+1, H] but got {tuple(hidden_states.shape)}")
    T1, H = hidden_states.shape
    kernel_assert(block_size % 128 == 0, "Blocksize must be a multiple of 128")
    kernel_assert(H % 512 == 0, f"Hidden dim size must be multiples of 512, found {H} ")
    kernel_assert(512 <= H <= 16384, f"Hidden dims must be between 512 and 16384, found {H}")
    guw = _as_bytes(gate_up_proj_weight, "gate_up_proj_weight")
    dw = _as_bytes(down_proj_weight, "down_proj_weight")
    gus = nv.require_device_tensor(gate_up_proj_scale, "gate_up_proj_scale")
    ds = nv.require_device_tensor(down_proj_scale, "down_proj_scale")
    kernel_assert(gus.dtype == torch.uint8 and ds.dtype == torch.uint8, "MX scales must be uint8 (E8M0)")
    kernel_assert(gus.dim() == 5 and gus.shape[1] == 16 and gus.shape[2] == 2 and gus.shape[3] == H // 512,
                  f"gate_up_proj_scale must be [E, 16, 2, H/512, I] but got {tuple(gus.shape)}")
    E, I = gus.shape[0], gus.shape[4]
    nI = (I + 511) // 512
    pI = 128 if I > 512 else I // 4
    kernel_assert(I % 16 == 0, f"down_proj_weight I must be divisible by 16, found {I} . Please pad it")
    kernel_assert(I % 512 == 0 or (I % 512) % 32 == 0, f"I tail must be a multiple of 32, found {I}")
    kernel_assert(guw.numel() == E * 128 * 2 * (H // 512) * I * wbytes,
                  f"gate_up_proj_weight must be x4 [E={E}, 128, 2, {H // 512}, {I}] of {wbytes}-byte elements "
                  f"but holds {guw.numel()} bytes")
    kernel_assert(dw.numel() == E * pI * nI * H * wbytes,
                  f"down_proj_weight must be x4 [E={E}, {pI}, {nI}, {H}] of {wbytes}-byte elements but holds {dw.numel()} bytes")
    kernel_assert(tuple(ds.shape) == (E, (pI + 7) // 8, nI, H),
                  f"down_proj_scale must be [{E}, {(pI + 7) // 8}, {nI}, {H}] but got {tuple(ds.shape)}")
    if gate_and_up_proj_bias is not None:
        kernel_assert(tuple(gate_and_up_proj_bias.shape) == (E, pI, 2, nI, 4),
                      f"gate_and_up_proj_bias must be [{E}, {pI}, 2, {nI}, 4] but got {tuple(gate_and_up_proj_bias.shape)}")
    kernel_assert(is_tensor_update_accumulating, "Only support topK > 1 at the moment.")
    kernel_assert(expert_affinities_scaling_mode in (ExpertAffinityScaleMode.POST_SCALE, ExpertAffinityScaleMode.NO_SCALE),
                  "MX blockwise MoE supports POST_SCALE / NO_SCALE only")
    xs = None
    if hidden_states_scale is not None:
        xs = nv.require_device_tensor(hidden_states_scale, "hidden_states_scale")
        kernel_assert(hidden_states.dtype in (torch.uint8, torch.float8_e4m3fn),
                      "pre-quantised hidden_states must be uint8 / float8_e4m3fn codes")
        kernel_assert(xs.dtype == torch.uint8 and tuple(xs.shape) == (T1, H // 32),
                      f"hidden_states_scale must be uint8 [{T1}, {H // 32}] but got {tuple(xs.shape)}")
    else:
        kernel_assert(hidden_states.dtype == torch.bfloat16,
                      f"hidden_states must be bfloat16 (or MXFP8 codes with hidden_states_scale) but got {hidden_states.dtype}")
    if conditions is not None and _out_shape_kind == "2TH":
        N = token_position_to_id.numel() // block_size
        kernel_assert(conditions.numel() == N + 2,
                      f"condition vector must have exactly N+2 elements, got {conditions.numel()} != N + 2 ({N} + 2)")
    dims = {"T1": T1, "H": H, "I": I, "E": E}
    return run_blockwise(
        nv.KIND_MXFP8, hidden_states, expert_affinities_masked, guw, dw, token_position_to_id, block_to_expert,
        block_size, _out_shape_kind, dims, conditions=conditions, gate_and_up_proj_bias=gate_and_up_proj_bias,
        down_proj_bias=down_proj_bias, gate_up_proj_scale=gus, down_proj_scale=ds, hidden_states_scale=xs,
        activation_function=activation_function, skip_dma=skip_dma,
        expert_affinities_scaling_mode=expert_affinities_scaling_mode,
        gate_clamp_upper_limit=gate_clamp_upper_limit, gate_clamp_lower_limit=gate_clamp_lower_limit,
        up_clamp_upper_limit=up_clamp_upper_limit, up_clamp_lower_limit=up_clamp_lower_limit, weight_dtype=wdt,
        weight_objects=(gate_up_proj_weight, down_proj_weight),
    )


bwmm_shard_on_block_mx = KernelEntry(_bwmm_shard_on_block_mx)
