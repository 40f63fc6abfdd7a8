"""Token -> block index construction on the GPU.

The reference builds ``token_position_to_id`` / ``block_to_expert`` / ``conditions`` on the
host in its test helper ``generate_token_position_to_id_and_experts``
(test/integration/nkilib/core/moe/moe_cte/test_moe_cte_common.py:199-264); callers of
``moe_cte`` must produce exactly that layout.  This module produces it on the device from the
router's top-k expert ids, bit exact with the helper.
"""

import math
import weakref

import torch

from .... import _native as nv
from ...utils.kernel_assert import kernel_assert


def get_n_blocks(T, TOPK, E, B, n_block_per_iter=1):
    """Worst-case number of blocks (test_moe_cte_common.py:95-98)."""
    N = math.ceil((T * TOPK - (E - 1)) / B) + E - 1
    return n_block_per_iter * math.ceil(N / n_block_per_iter)


# The block build also leaves the blockwise layer its bookkeeping (valid rows per block, every token's slots, the
# expert chunks and work queues of the GEMM launches: moe_build_blocks_plan), which moe_cte otherwise derives from
# token_position_to_id in four small launches.  The plan lies in the same allocation as the three tables and is found
# again through it; ``block_plans = False`` builds the tables alone.
block_plans = True
_plans = {}


def plan_for(tp2id, b2e, cond, B, N, T1):
    """(address, bytes) of the plan that the block build left for exactly these tables, or None: they must be the tensors
    ``build_token_blocks`` returned (views of them count), unchanged since (torch's version counter, which views
    share), used with the same block size, block count and token count, and with its ``conditions`` or none."""
    ent = _plans.get(tp2id.untyped_storage().data_ptr())
    if ent is None:
        return None
    st, version, ptrs, shape, plan = ent
    if st() is not tp2id.untyped_storage() or tp2id._version != version or shape != (B, N, T1):
        return None
    if tp2id.data_ptr() != ptrs[0] or b2e.data_ptr() != ptrs[1] or b2e.untyped_storage() is not st():
        return None
    if cond is not None and (cond.data_ptr() != ptrs[2] or cond.numel() != ptrs[3] or cond.untyped_storage() is not st()):
        return None
    return plan


def build_token_blocks(topk_ids: torch.Tensor, E: int, B: int, N: int = None, skip_token: bool = False,
                       use_split_padding: bool = False, n_conditions: int = None, check: bool = False):
    """topk_ids int32 ``[T, k]`` (distinct expert ids per row) ->
    (token_position_to_id int32 ``[N*B]``, block_to_expert int32 ``[N]``, conditions int32 ``[n_conditions]``).

    ``n_conditions`` defaults to ``N + 1`` (the non-block-parallel form); pass ``N + 2`` for the MX
    block-parallel form.  ``check=True`` synchronises and raises if N is too small for the routing.
    """
    L = nv.lib()
    ids = nv.require_device_tensor(topk_ids, "topk_ids")
    kernel_assert(ids.dim() == 2 and ids.dtype == torch.int32, "topk_ids must be int32 [T, k]")
    T, k = ids.shape
    if N is None:
        N = get_n_blocks(T, k, E, B)
    if n_conditions is None:
        n_conditions = N + 1
    dev = ids.device
    # one allocation for the plan, the three outputs, the status word (always written by the layout step) and the
    # int32 workspace: at decode sizes the host side of this call costs more than its kernels
    ws_words = (L.moe_build_blocks_workspace_bytes(E) + 3) // 4
    plan_words = 0
    if block_plans and not use_split_padding and T >= 1 and T * k <= N * B and E <= 512:
        plan_words = L.moe_block_plan_bytes(T, B, N, 1 if skip_token else 0) // 4  # (a multiple of 256 bytes)
    buf = torch.empty(plan_words + N * B + N + n_conditions + 1 + ws_words, dtype=torch.int32, device=dev)
    plan, tp2id, b2e, cond, status, ws = torch.split(buf, [plan_words, N * B, N, n_conditions, 1, ws_words])
    with torch.cuda.device(dev):
        if plan_words:
            rc = L.moe_build_blocks_plan(nv.ptr(ids), T, k, E, B, N, 1 if skip_token else 0,
                                         1 if use_split_padding else 0, nv.ptr(tp2id), nv.ptr(b2e), nv.ptr(cond),
                                         n_conditions, nv.ptr(ws), ws.numel() * 4, nv.ptr(status), nv.ptr(plan),
                                         plan.numel() * 4, nv.stream_ptr(dev))
        else:
            rc = L.moe_build_blocks(nv.ptr(ids), T, k, E, B, N, 1 if skip_token else 0, 1 if use_split_padding else 0,
                                    nv.ptr(tp2id), nv.ptr(b2e), nv.ptr(cond), n_conditions, nv.ptr(ws), ws.numel() * 4,
                                    nv.ptr(status), nv.stream_ptr(dev))
    nv.check(rc, "build_token_blocks")
    if check:
        kernel_assert(int(status.item()) == 0, f"N={N} blocks cannot hold this routing")
    if plan_words:
        st = buf.untyped_storage()
        key = st.data_ptr()
        if len(_plans) >= 256:
            _plans.pop(next(iter(_plans)))
        # (no reference to the allocation is kept: the entry goes when the caller drops the tables)
        _plans[key] = (weakref.ref(st, lambda _ref, key=key: _plans.pop(key, None)), buf._version,
                       (tp2id.data_ptr(), b2e.data_ptr(), cond.data_ptr(), cond.numel()),
                       (B, N, T if skip_token else T + 1), (plan.data_ptr(), plan.numel() * 4))
    return tp2id, b2e, cond
