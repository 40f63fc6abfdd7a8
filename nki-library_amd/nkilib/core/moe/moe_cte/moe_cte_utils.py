"""Configuration types shared by the MoE CTE kernels
(src/nkilib_src/nkilib/core/moe/moe_cte/moe_cte_utils.py:65-95)."""

from enum import Enum


class SkipMode:
    """Controls how padding slots are marked.

    skip_token: padding slots carry id -1 and the token tables have T rows (no zero row T).
    skip_weight: accepted for compatibility; weight reloads are irrelevant on the GPU.
    """

    def __init__(self, skip_token: bool = False, skip_weight: bool = False):
        self.skip_token = skip_token
        self.skip_weight = skip_weight

    def __repr__(self):
        return f"SkipMode(skip_token={self.skip_token}, skip_weight={self.skip_weight})"


class BlockShardStrategy(Enum):
    """Block distribution over two NeuronCores in the reference; accepted and ignored on one GPU."""

    HI_LO = 0
    PING_PONG = 1
