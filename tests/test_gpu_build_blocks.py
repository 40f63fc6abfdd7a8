"""GPU parity: token -> block index construction, bit exact against the oracle
(reference helper: test/integration/nkilib/core/moe/moe_cte/test_moe_cte_common.py:199-264)."""

import numpy as np
import pytest

from helpers import i32_tensor
from oracle import blocks as ob

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize(
    "T,k,E,B,skip,split,alpha",
    [
        (5, 2, 3, 2, False, False, None),
        (256, 2, 8, 128, False, False, None),
        (1024, 4, 16, 256, True, False, None),
        (4096, 2, 8, 128, False, True, None),
        (8192, 8, 128, 128, False, False, 0.3),   # skewed loads
        (8192, 8, 256, 128, False, False, None),
        (1, 8, 256, 128, False, False, None),     # decode-shaped: every expert block almost empty
        (128, 8, 256, 128, True, False, None),
        (1000, 1, 7, 128, False, False, None),
    ],
)
def test_build_blocks_bit_exact(T, k, E, B, skip, split, alpha):
    import torch
    from nkilib.core.moe.moe_cte import build_token_blocks, get_n_blocks

    router = ob.router_with_controlled_distribution(T, k, E, alpha).astype(np.int32)
    mask = ob.expert_mask_from_router(router, E)
    N = ob.get_n_blocks(T, k, E, B)
    assert N == get_n_blocks(T, k, E, B)
    g_tp, g_b2e, g_cond = ob.build_token_blocks(mask, B, N, skip_token=skip, use_split_padding=split)
    dev = torch.device("cuda:0")
    tp, b2e, cond = build_token_blocks(i32_tensor(router, dev), E, B, N, skip_token=skip, use_split_padding=split,
                                       check=True)
    assert np.array_equal(tp.cpu().numpy(), g_tp)
    assert np.array_equal(b2e.cpu().numpy(), g_b2e)
    assert np.array_equal(cond.cpu().numpy(), g_cond)
    # MX block-parallel form of conditions: N + 2 entries
    _, _, g_cond2 = ob.build_token_blocks(mask, B, N, skip_token=skip, use_split_padding=split,
                                          is_block_parallel=True, is_mx=True)
    _, _, cond2 = build_token_blocks(i32_tensor(router, dev), E, B, N, skip_token=skip, use_split_padding=split,
                                     n_conditions=N + 2)
    assert np.array_equal(cond2.cpu().numpy(), g_cond2)
