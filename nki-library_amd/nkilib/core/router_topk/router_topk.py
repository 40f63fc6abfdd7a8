"""Router top-k front end on the MI355X: the reference's ``router_topk`` operator
(src/nkilib_src/nkilib/core/router_topk/router_topk.py:55-75) over ``moe_router_topk`` of the C ABI.

Semantics are those of ``router_topk_torch_ref``
(src/nkilib_src/nkilib/core/router_topk/router_topk_torch.py:23-135).  Logits are kept in fp32 for the
selection (the reference's bf16 logits tie often and leave the choice among tied experts to ``argsort``);
ties go to the lower expert index.
"""

import torch

from ... import _native as nv
from ..._entry import KernelEntry
from ..utils.common_types import RouterActFnType
from ..utils.kernel_assert import kernel_assert


def _router_topk(x, w, w_bias, router_logits, expert_affinities, expert_index, act_fn, k, x_hbm_layout=0,
                 x_sb_layout=0, router_pre_norm=True, norm_topk_prob=False, use_column_tiling=False,
                 use_indirect_dma_scatter=False, return_eager_affi=False, use_PE_broadcast_w_bias=False,
                 shard_on_tokens=False, skip_store_expert_index=False, skip_store_router_logits=False,
                 _mask_to_topk=False, _pad_row=False):
    """Same arguments as the reference kernel.  ``x`` is ``[H, T]`` (``x_hbm_layout == 0``) or ``[T, H]`` (1);
    ``router_logits`` / ``expert_affinities`` / ``expert_index`` are caller-provided outputs (``None`` allocates
    them); the Trainium scheduling switches (``x_sb_layout``, ``use_column_tiling``, ``use_indirect_dma_scatter``,
    ``use_PE_broadcast_w_bias``, ``shard_on_tokens``) are accepted and have no effect here.  Returns
    ``[router_logits, expert_index, expert_affinities]`` (+ the ``[T, k]`` top-k affinities with
    ``return_eager_affi``)."""
    x = nv.require_device_tensor(x, "x")
    w = nv.require_device_tensor(w, "w")
    kernel_assert(x.dim() == 2 and w.dim() == 2, "x and w must be 2-D")
    kernel_assert(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "x and w must be bfloat16")
    if int(x_hbm_layout) == 0:
        x = x.t().contiguous()  # [H, T] -> [T, H]: the GEMM reads token rows
    T, H = x.shape
    kernel_assert(w.shape[0] == H, f"w must be [H, E] with H = {H} but got {tuple(w.shape)}")
    E = w.shape[1]
    kernel_assert(1 <= int(k) <= 8 and int(k) <= E, f"k must be in [1, min(8, E)] but got {k}")
    kernel_assert(E <= 512, f"E must be <= 512 but got {E}")
    kernel_assert(H % 128 == 0, f"H must be a multiple of 128 but got {H}")
    act = RouterActFnType(act_fn) if not isinstance(act_fn, RouterActFnType) else act_fn
    dev = x.device
    bias = None
    if w_bias is not None:
        bias = nv.require_device_tensor(w_bias, "w_bias").reshape(-1)
        kernel_assert(bias.numel() == E, f"w_bias must hold E = {E} values")
    rows = T + (1 if _pad_row else 0)
    if expert_affinities is None:
        expert_affinities = torch.empty((rows, E), dtype=torch.bfloat16, device=dev)
    kernel_assert(expert_affinities.is_contiguous() and expert_affinities.numel() == rows * E,
                  "expert_affinities must be a contiguous [T, E] tensor")
    if router_logits is None and not skip_store_router_logits:
        router_logits = torch.empty((T, E), dtype=torch.bfloat16, device=dev)
    if expert_index is None and not skip_store_expert_index:
        expert_index = torch.empty((T, int(k)), dtype=torch.int32, device=dev)
    if expert_index is not None:
        kernel_assert(expert_index.dtype in (torch.int32, torch.uint32) and expert_index.is_contiguous(),
                      "expert_index must be a contiguous 32-bit integer tensor")
    topk_aff = torch.empty((T, int(k)), dtype=torch.float32, device=dev) if return_eager_affi else None
    L = nv.lib()
    wsb = L.moe_router_topk_workspace_bytes(H, E)
    ws = nv.workspace(dev, wsb)
    rc = L.moe_router_topk(
        nv.ptr(x), nv.ptr(w), nv.ptr(bias), nv.dtype_code(bias, "w_bias") if bias is not None else 0, T, H, E, int(k),
        act.value, int(bool(router_pre_norm)), int(bool(norm_topk_prob)), int(bool(_mask_to_topk)), int(bool(_pad_row)),
        None if skip_store_router_logits else nv.ptr(router_logits),
        nv.dtype_code(router_logits, "router_logits") if router_logits is not None else 0,
        None if skip_store_expert_index else nv.ptr(expert_index), nv.ptr(expert_affinities),
        nv.dtype_code(expert_affinities, "expert_affinities"), nv.ptr(topk_aff), nv.ptr(ws), ws.numel(),
        nv.stream_ptr(dev))
    nv.check(rc, "router_topk")
    outs = [router_logits, expert_index, expert_affinities]
    if return_eager_affi:
        outs.append(topk_aff)
    return outs


router_topk = KernelEntry(_router_topk)


def route_for_moe(x, w, w_bias, k, act_fn=RouterActFnType.SOFTMAX, norm_topk_prob=False):
    """Hidden states ``[T+1, H]`` (last row = the padding token, as ``moe_cte`` takes them) -> what ``moe_cte`` and
    ``build_token_blocks`` consume: top-k ids ``[T, k]`` int32 and the masked affinity table ``[T+1, E]`` bf16
    (zero outside the top-k, zero padding row)."""
    T = x.shape[0] - 1
    _, idx, aff = _router_topk(x[:T], w, w_bias, None, None, None, act_fn, k, x_hbm_layout=1, router_pre_norm=True,
                               norm_topk_prob=norm_topk_prob, skip_store_router_logits=True, _mask_to_topk=True,
                               _pad_row=True)
    return idx, aff
