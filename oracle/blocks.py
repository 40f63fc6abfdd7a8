"""Token -> block index construction (integer, bit exact).  Oracle: test infrastructure only.

Restates, from test/integration/nkilib/core/moe/moe_cte/test_moe_cte_common.py:
  * ``get_n_blocks``                                   :95-98
  * ``get_router_with_controlled_distribution``        :173-196
  * ``generate_token_position_to_id_and_experts``      :199-264

The reference has no device kernel for this step; its test helper is the only
statement of the layout the MoE kernels consume, so it is the specification.
"""

import math

import numpy as np


def get_n_blocks(T, TOPK, E, B, n_block_per_iter=1):
    """Worst-case block count: every expert may leave one partially filled block."""
    N = math.ceil((T * TOPK - (E - 1)) / B) + E - 1
    N = n_block_per_iter * math.ceil(N / n_block_per_iter)
    return N


def router_with_controlled_distribution(T, TOPK, E, alpha=None):
    """Seeded synthetic top-k routing table [T, min(E, TOPK)] of expert ids.

    Uses the legacy ``np.random.seed(0)`` global stream exactly like the reference
    so that the same (T, TOPK, E, alpha) reproduces the reference's routing.
    """
    actual_k = min(E, TOPK)
    router = np.zeros((T, actual_k))
    np.random.seed(0)
    if alpha is None:
        n_pick = E if E < TOPK else TOPK
        for i in range(T):
            router[i] = np.random.choice(range(E), (n_pick), replace=False)
    elif alpha == -1:
        p_of_e = np.random.dirichlet(np.ones(E) * 0.001)
        for i in range(0, T):
            router[i] = np.random.choice(range(E), (actual_k), replace=False, p=p_of_e)
    else:
        for i in range(E):
            router[i] = np.arange(i, (i + actual_k) % T)
        p_of_e = np.random.dirichlet(np.ones(E) * alpha)
        for i in range(E, T):
            router[i] = np.random.choice(range(E), (actual_k), replace=False, p=p_of_e)
    return router


def expert_mask_from_router(router, E):
    """[T, k] expert ids -> dense 0/1 mask [T, E] (test_moe_cte_common.py:217-221)."""
    T, k = router.shape
    mask = np.zeros((T, E))
    one_hot = np.arange(E)
    for i in range(k):
        mask += np.expand_dims(router[:, i], 1) == np.expand_dims(one_hot, 0)
    return mask


def build_token_blocks(
    token_experts,
    B,
    N,
    skip_token=False,
    use_split_padding=False,
    n_block_per_iter=1,
    vnc_degree=1,
    is_block_parallel=False,
    is_mx=False,
):
    """Sort (token, expert) pairs by expert into fixed-size blocks.

    token_experts: 0/1 mask [T, E].  Returns (token_position_to_id int32[N*B],
    block_to_expert int32[N], conditions int32[...]).

    Layout (test_moe_cte_common.py:223-249): expert e owns ceil(count_e / B) blocks;
    every spare block is given to the last expert (or split between experts
    (E-1)//2 and E-1); expert regions are laid out in expert order; inside a region
    tokens appear in ascending id from the region's first slot; every other slot
    holds the padding id T (or -1 when skip_token).
    """
    token_experts = np.asarray(token_experts)
    T, E = token_experts.shape
    blocks_per_expert = np.ceil(token_experts.sum(0) / B).astype(np.int32)
    n_padding_block = N - np.sum(blocks_per_expert)
    assert n_padding_block >= 0, "N too small for this routing"
    if use_split_padding:
        blocks_per_expert[(E - 1) // 2] += n_padding_block // 2
        blocks_per_expert[E - 1] += n_padding_block - n_padding_block // 2
    else:
        blocks_per_expert[E - 1] += n_padding_block

    cumulative = np.cumsum(blocks_per_expert)
    block_to_expert = np.arange(E).repeat(blocks_per_expert).astype(np.int32)

    # 1-based position of every routed (token, expert) pair in the flat slot array
    pos = np.cumsum(token_experts, axis=0)
    offsets = cumulative * B
    pos[:, 1:] += offsets[:-1]
    pos = np.where(token_experts, pos, 0).astype(np.int32)

    pad_id = -1 if skip_token else T
    tp2id = np.full((int(N * B + 1),), pad_id)
    tp2id[pos] = np.expand_dims(np.arange(T), 1)
    tp2id = tp2id[1:].astype(np.int32)

    if not is_block_parallel:
        n_condition = n_block_per_iter * math.ceil(N / n_block_per_iter)
        conditions = np.ones((n_condition + 1,), dtype=np.int32)
        conditions[-(n_padding_block + 1) :] = 0
    elif is_mx:
        assert n_block_per_iter == 1
        conditions = np.ones((N + 2,), dtype=np.int32)
        conditions[-(n_padding_block + 2) :] = 0
    else:
        conditions = np.ones((math.ceil(N / vnc_degree) + 1,), dtype=np.int32)
        conditions[-(math.ceil(n_padding_block / vnc_degree) + 1) :] = 0
    return tp2id, block_to_expert, conditions


def generate_token_position_to_id_and_experts(
    T, TOPK, E, B, skip_token, N, use_split_padding=False, n_block_per_iter=1, vnc_degree=1, alpha=None,
    is_block_parallel=False, is_mx=False,
):
    """Reference-equivalent convenience: seeded router -> (mask, tp2id, b2e, conditions)."""
    if n_block_per_iter > 1:
        assert vnc_degree == 1
    router = router_with_controlled_distribution(T, TOPK, E, alpha)
    mask = expert_mask_from_router(router, E)
    tp2id, b2e, cond = build_token_blocks(
        mask, B, N, skip_token, use_split_padding, n_block_per_iter, vnc_degree, is_block_parallel, is_mx
    )
    return mask, tp2id, b2e, cond
