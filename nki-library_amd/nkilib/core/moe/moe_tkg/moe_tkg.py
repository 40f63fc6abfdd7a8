"""Token-generation MoE on the MI355X: the reference's ``moe_tkg`` operator
(src/nkilib_src/nkilib/core/moe/moe_tkg/moe_tkg.py:45-72) on the blockwise kernels of the context-encoding path.

Semantics are those of ``moe_tkg_torch_ref`` (src/nkilib_src/nkilib/core/moe/moe_tkg/moe_tkg_torch.py:35-226 dense,
:320-442 MX): every token goes through its top-k experts (selective mode) or through every local expert
(all-expert mode), the expert outputs are summed, weighted by the affinities with ``POST_SCALE``.  Here the
(token, expert) pairs are sorted into blocks on the device (``moe_build_blocks``; for the all-expert mode the
blocks are every token under every expert) and run through the gate/up and down GEMM kernels that ``moe_cte``
uses: at decode sizes almost every expert holds one nearly empty block, so the two GEMMs stream the expert
weights once, which is what bounds this regime.
"""

from typing import Optional

import torch

from .... import _native as nv
from ...._entry import KernelEntry
from ...utils.common_types import ActFnType, ExpertAffinityScaleMode
from ...utils.kernel_assert import kernel_assert
from ..moe_cte.block_index import build_token_blocks, get_n_blocks
from ..moe_cte.bwmm_shard_on_block import run_dense_variant
from ..moe_cte.bwmm_shard_on_block_mx import _bwmm_shard_on_block_mx
from ..moe_cte.moe_cte_utils import SkipMode

_PREFIX = "[MoE TKG Kernel]"
_BLOCK = 128  # tokens per block of the internal block structure


def _is_mx(w, scale) -> bool:
    """x4-packed MX weights: 5-D gate/up weights ``[E_L, 128, 2, H/512, I]`` (the dense form is 4-D)."""
    return w.dim() >= 5 and scale is not None and scale.dtype == torch.uint8


def _moe_tkg(
    hidden_input, expert_gate_up_weights, expert_down_weights, expert_affinities, expert_index, is_all_expert: bool,
    rank_id=None, expert_gate_up_bias=None, expert_down_bias=None, expert_gate_up_weights_scale=None,
    expert_down_weights_scale=None, hidden_input_scale=None, gate_up_input_scale=None, down_input_scale=None,
    mask_unselected_experts: bool = False, expert_affinities_eager=None,
    expert_affinities_scaling_mode: ExpertAffinityScaleMode = ExpertAffinityScaleMode.NO_SCALE,
    activation_fn: ActFnType = ActFnType.SiLU, output_dtype=None, gate_clamp_upper_limit: Optional[float] = None,
    gate_clamp_lower_limit: Optional[float] = None, up_clamp_upper_limit: Optional[float] = None,
    up_clamp_lower_limit: Optional[float] = None, output_in_sbuf: bool = False, is_all_expert_dynamic: bool = False,
    block_size: int = None, weight_dtype=None,
):
    """Same arguments as the reference kernel (+ ``weight_dtype`` for MX weights in uint containers, as
    ``bwmm_shard_on_block_mx`` takes it).  ``hidden_input`` bf16 ``[T, H]``; weights bf16 (or fp8 with row scales
    ``[E_L, 2, I]`` / ``[E_L, H]``) ``[E_L, H, 2, I]`` / ``[E_L, I, H]``, or MX x4 ``[E_L, 128, 2, H/512, I]`` /
    ``[E_L, I_p, ceil(I/512), H]`` with uint8 scales; ``expert_affinities`` ``[T, E]``; ``expert_index`` ``[T, K]``.
    All-expert mode with affinity scaling: ``rank_id`` ``[1, 1]`` selects the columns ``[E_L * rank, E_L * (rank +
    1))`` of the affinities (read on the device), ``mask_unselected_experts`` zeroes the affinities of experts
    that ``expert_index`` does not list for a token.  Returns ``[T, H]`` in ``output_dtype`` (default: the input's).
    The token limit of the reference's selective mode (T <= 128) does not apply; ``output_in_sbuf``,
    ``is_all_expert_dynamic`` and ``block_size`` describe Trainium scheduling and only their consistency is checked.
    """
    x = nv.require_device_tensor(hidden_input, "hidden_input")
    guw = nv.require_device_tensor(expert_gate_up_weights, "expert_gate_up_weights")
    dw = nv.require_device_tensor(expert_down_weights, "expert_down_weights")
    kernel_assert(x.dim() == 2, f"{_PREFIX} hidden_input must be [T, H] but got {tuple(x.shape)}")
    T, H = x.shape
    E_L = guw.shape[0]
    mode = ExpertAffinityScaleMode(expert_affinities_scaling_mode)
    act = ActFnType(activation_fn)
    is_mx = _is_mx(guw, expert_gate_up_weights_scale)
    # moe_tkg.py:316-402
    if is_mx:
        kernel_assert(expert_gate_up_weights_scale is not None and expert_down_weights_scale is not None,
                      f"{_PREFIX} Scales must be set when using MX weights")
    if is_all_expert_dynamic:
        kernel_assert(is_all_expert, f"{_PREFIX} is_all_expert_dynamic=True requires is_all_expert=True, but got "
                                     f"{is_all_expert=}")
        kernel_assert(block_size is not None, f"{_PREFIX} is_all_expert_dynamic=True requires block_size != None, "
                                              f"but got {block_size=}")
    kernel_assert(hidden_input_scale is None,
                  f"{_PREFIX} hidden_input_scale describes a pre-quantised input in SBUF, which has no counterpart on "
                  "gfx950; pass bfloat16 hidden_input")
    kernel_assert(mode != ExpertAffinityScaleMode.PRE_SCALE_DELAYED,
                  f"{_PREFIX} PRE_SCALE_DELAYED option is only applicable in CTE expert_mlp case")
    kernel_assert(mode != ExpertAffinityScaleMode.PRE_SCALE, f"{_PREFIX} Kernel does not support pre-scale mode")
    kernel_assert(gate_up_input_scale is None and down_input_scale is None,
                  f"{_PREFIX} Static quantization is not supported in MoE TKG kernel")
    if is_all_expert:
        kernel_assert(expert_affinities_eager is None,
                      f"{_PREFIX} expert_affinities eager mode not supported with is_all_expert=True")
    dev = x.device
    B = _BLOCK
    scaled = mode != ExpertAffinityScaleMode.NO_SCALE

    if is_all_expert:
        # every token under every local expert: ceil(T / B) blocks per expert
        nb = (T + B - 1) // B
        slot = torch.arange(nb * B, dtype=torch.int32, device=dev)
        tp2id = torch.where(slot < T, slot, torch.full_like(slot, -1)).repeat(E_L)
        b2e = torch.arange(E_L, dtype=torch.int32, device=dev).repeat_interleave(nb)
        table = None
        if scaled:
            kernel_assert(rank_id is not None,
                          f"{_PREFIX} rank_id is required for all-expert mode with affinity scaling")
            aff = nv.require_device_tensor(expert_affinities, "expert_affinities")
            kernel_assert(aff.dim() == 2 and aff.shape[0] == T, f"{_PREFIX} expert_affinities must be [T, E]")
            rank = nv.require_device_tensor(rank_id, "rank_id").reshape(-1)[:1].to(torch.int64)
            cols = rank * E_L + torch.arange(E_L, dtype=torch.int64, device=dev)  # moe_tkg_affinity_masking.py:81-89
            table = aff.index_select(1, cols)
            if mask_unselected_experts:
                idx = nv.require_device_tensor(expert_index, "expert_index").to(torch.int64)
                chosen = torch.zeros(aff.shape, dtype=torch.bool, device=dev)
                chosen.scatter_(1, idx, True)
                table = torch.where(chosen.index_select(1, cols), table, torch.zeros_like(table))
            table = table.contiguous()
    else:
        idx = nv.require_device_tensor(expert_index, "expert_index")
        kernel_assert(idx.dim() == 2 and idx.shape[0] == T, f"{_PREFIX} expert_index must be [T, K]")
        K = idx.shape[1]
        ids = idx.to(torch.int32).contiguous()
        N = get_n_blocks(T, K, E_L, B)
        tp2id, b2e, _ = build_token_blocks(ids, E_L, B, N, skip_token=True)
        table = None
        if scaled:
            if expert_affinities_eager is not None:
                eager = nv.require_device_tensor(expert_affinities_eager, "expert_affinities_eager")
                kernel_assert(tuple(eager.shape) == (T, K), f"{_PREFIX} expert_affinities_eager must be [T, K]")
                table = torch.zeros((T, E_L), dtype=eager.dtype, device=dev)
                table.scatter_(1, idx.to(torch.int64), eager)
            else:
                table = nv.require_device_tensor(expert_affinities, "expert_affinities")
                kernel_assert(tuple(table.shape) == (T, E_L),
                              f"{_PREFIX} expert_affinities must be [T, E] = [{T}, {E_L}] but got {tuple(table.shape)}")
    if table is not None and table.dtype not in (torch.bfloat16, torch.float32):
        table = table.to(torch.float32)

    common = dict(
        activation_function=act, skip_dma=SkipMode(True, False), expert_affinities_scaling_mode=mode,
        gate_clamp_upper_limit=gate_clamp_upper_limit, gate_clamp_lower_limit=gate_clamp_lower_limit,
        up_clamp_upper_limit=up_clamp_upper_limit, up_clamp_lower_limit=up_clamp_lower_limit,
    )
    if is_mx:
        out = _bwmm_shard_on_block_mx(
            x, table, guw, dw, tp2id, b2e, gate_and_up_proj_bias=expert_gate_up_bias, down_proj_bias=expert_down_bias,
            gate_up_proj_scale=expert_gate_up_weights_scale, down_proj_scale=expert_down_weights_scale, block_size=B,
            weight_dtype=weight_dtype, _out_shape_kind="TH", **common)
    else:
        gus = ds = None
        if expert_gate_up_weights_scale is not None or expert_down_weights_scale is not None:
            kernel_assert(expert_gate_up_weights_scale is not None and expert_down_weights_scale is not None,
                          f"{_PREFIX} gate/up and down weight scales must be given together")
            I = guw.shape[-1]
            gus = nv.require_device_tensor(expert_gate_up_weights_scale, "expert_gate_up_weights_scale")
            ds = nv.require_device_tensor(expert_down_weights_scale, "expert_down_weights_scale")
            kernel_assert(tuple(gus.shape) == (E_L, 2, I) and tuple(ds.shape) == (E_L, H),
                          f"{_PREFIX} row scales must be [E_L, 2, I] and [E_L, H] but got {tuple(gus.shape)}, "
                          f"{tuple(ds.shape)}")
            gus, ds = gus.reshape(E_L, 1, 2 * I), ds.reshape(E_L, 1, H)
        out = run_dense_variant(
            x, table, guw, dw, B, tp2id, b2e, "TH", gate_and_up_proj_bias=expert_gate_up_bias,
            down_proj_bias=expert_down_bias, gate_up_proj_scale=gus, down_proj_scale=ds, **common)
    if output_dtype is not None and output_dtype != out.dtype:
        out = out.to(output_dtype)
    return out


moe_tkg = KernelEntry(_moe_tkg)
