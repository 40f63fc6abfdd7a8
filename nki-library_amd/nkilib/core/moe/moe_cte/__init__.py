"""MoE CTE (context encoding) blockwise matrix multiplication kernels for MI355X."""

from .block_index import build_token_blocks, get_n_blocks
from .moe_cte import (
    MoECTEImplementation,
    MoECTESpec,
    QuantizationConfig,
    ShardOnBlockConfig,
    ShardOnIConfig,
    moe_cte,
)
from .moe_cte_utils import BlockShardStrategy, SkipMode

__all__ = [
    "moe_cte",
    "MoECTESpec",
    "MoECTEImplementation",
    "ShardOnBlockConfig",
    "ShardOnIConfig",
    "QuantizationConfig",
    "BlockShardStrategy",
    "SkipMode",
    "build_token_blocks",
    "get_n_blocks",
]
