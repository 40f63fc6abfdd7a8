"""GPU parity of the dense (bf16 / fp8 weight-only) blockwise kind on the reference's own table
(test/integration/nkilib/core/moe/moe_cte/test_moe_cte.py:44-133): hidden size 3072 (a large-tile shape), block
sizes 512 and 256, intermediate sizes 192 .. 3072, 8 / 64 / 128 experts, Swish with the clamps (7, None, 8, -9),
skip modes 0 / 1 / 3, fp8 weights, the E < top_k rows, the activation-checkpoint ("training") rows and a
token-dropping row, against ``moe_blockwise_ref`` at the reference's tolerance (2e-2 max-abs-rel, `:246`).

Inputs follow the reference's generator (hidden states uniform in [0, 1), weights uniform in (-0.1, 0.1),
test_moe_cte_common.py:554-711).  Rows whose (E, I) pair would need gigabytes of host-side weights keep the row's
E and block structure with a smaller I of the table; the docstring of each case names the reference row.
"""

import numpy as np
import pytest

from helpers import dense_case, from_bf16_tensor
from oracle import moe as omoe
from test_gpu_moe import _check, _golden_dense, _run_checkpointed, _run_dense

pytestmark = pytest.mark.gpu

SWISH, SILU = 3, 0
POST = 1
CL = dict(gate_clamp_upper_limit=7.0, up_clamp_upper_limit=8.0, up_clamp_lower_limit=-9.0)   # (7, None, 8, -9)
CL7 = dict(gate_clamp_upper_limit=7.0, up_clamp_upper_limit=7.0, up_clamp_lower_limit=-7.0)  # (7, None, 7, -7)

# impl, H, T, E, B, k, I, skip, bias, fp8, act, clamps        (reference row it stands for)
FORWARD = [
    ("shard_on_i", 3072, 1024, 8, 512, 4, 2048, 0, True, False, SILU, None),       # :46
    ("shard_on_i", 3072, 1024, 64, 512, 8, 384, 0, True, False, SILU, None),       # :55-56 (E=64 top-8; I of :95)
    ("shard_on_i", 3072, 1024, 8, 512, 4, 3072, 1, True, False, SWISH, None),      # :82
    ("shard_on_i", 3072, 1024, 8, 512, 4, 1536, 1, True, True, SWISH, CL7),        # :92 at T=1024: fp8 weights
    ("shard_on_block", 3072, 1024, 8, 512, 4, 384, 1, True, False, SWISH, CL),     # :95
    ("shard_on_block", 3072, 1024, 8, 512, 4, 192, 3, True, False, SWISH, CL),     # :98
    ("shard_on_block", 3072, 1024, 8, 256, 4, 384, 3, True, False, SWISH, CL),     # :100
    ("shard_on_block", 3072, 1024, 8, 256, 4, 1536, 1, True, False, SWISH, CL),    # :103
    ("shard_on_block", 3072, 1024, 8, 512, 4, 3072, 1, True, False, SWISH, CL),    # :106
    ("shard_on_block", 3072, 10240, 128, 256, 4, 192, 3, True, False, SWISH, CL),  # :107
    ("shard_on_i", 4096, 10240, 4, 512, 8, 768, 1, False, False, SILU, None),      # :125  E < top_k
    ("shard_on_i_hybrid", 4096, 10240, 4, 512, 8, 768, 1, False, False, SILU, None),   # :126  E < top_k (the reference's hardware-loop variant)
]


@pytest.mark.parametrize("impl,H,T,E,B,k,I,skip,bias,fp8,act,clamps", FORWARD)
def test_dense_reference_table(impl, H, T, E, B, k, I, skip, bias, fp8, act, clamps):
    c = dense_case(T, H, I, E, k, B, seed=11, skip_token=bool(skip & 1), bias=bias, quant=fp8)
    out = _run_dense(c, impl=impl, act=act, mode=POST, clamps=clamps, fp8_weights=fp8)
    o = from_bf16_tensor(out)
    if o.ndim == 3:
        assert not o[:, 1].any(), "second shard slot must stay zero"
        o = o[:, 0]
    g = _golden_dense(c, act=act, mode=POST, clamps=clamps, fp8_weights=fp8)
    _check(o[:T], g[:T], f"reference table {impl} H={H} T={T} E={E} B={B} top-{k} I={I} skip={skip}")


# the activation-checkpoint rows (`:108-123`): H=3072, T=1024, B=512; (E, top_k, act); I, skip, multiply_on_I
TRAINING = [
    (8, 4, SWISH, 2048, 0, True),    # :110
    (8, 4, SWISH, 3072, 1, True),    # :115
    (8, 4, SWISH, 2048, 0, False),   # :118
    (64, 8, SILU, 384, 1, False),    # :120 (E=64 top-8; I of :95)
]


@pytest.mark.parametrize("E,k,act,I,skip,on_I", TRAINING)
def test_dense_reference_table_checkpoints(E, k, act, I, skip, on_I):
    H, T, B = 3072, 1024, 512
    c = dense_case(T, H, I, E, k, B, seed=13, skip_token=bool(skip))
    outs = _run_checkpointed(c, "shard_on_i", act, POST, None, on_I)
    assert len(outs) == (2 if on_I else 3)
    g_out, g_gu, g_d = omoe.moe_blockwise_ref(c["hidden"], c["aff"], c["gate_up_w"], c["down_w"], c["tp2id"], c["b2e"], B,
                                              activation_function=act, skip_token=bool(skip),
                                              expert_affinities_scaling_mode=POST, checkpoint_activation=True)
    _check(from_bf16_tensor(outs[0])[:T], g_out[:T], "training row: output")
    _check(from_bf16_tensor(outs[1]), g_gu, "training row: gate_up_activations_T")
    if not on_I:
        _check(from_bf16_tensor(outs[2]), g_d, "training row: down_activations")


@pytest.mark.parametrize("on_I", [True, False])
def test_dense_reference_table_dropping(on_I):
    """`:128,131`: H=2048, T=2048, E=2, B=1024 (= capacity), top-2, I=8192: every token selects both experts, each
    keeps its first 1024."""
    H, T, E, B, k, I = 2048, 2048, 2, 1024, 2, 8192
    c = dense_case(T, H, I, E, k, B, seed=17)
    tp = np.full((E, B), T, dtype=np.int32)
    for e in range(E):
        ids = np.flatnonzero(c["mask"][:, e])[:B]
        tp[e, : ids.size] = ids
    assert (c["mask"].sum(0) > B).any(), "the case must actually drop tokens"
    b2e = np.arange(E, dtype=np.int32)
    outs = _run_checkpointed(c, "shard_on_i_dropping", mode=POST, on_I=on_I, tp2id=tp.reshape(-1), b2e=np.zeros(E, np.int32))
    g_out, g_gu, g_d = omoe.moe_blockwise_ref(c["hidden"], c["aff"], c["gate_up_w"], c["down_w"], tp.reshape(-1), b2e, B,
                                              expert_affinities_scaling_mode=POST, checkpoint_activation=True)
    _check(from_bf16_tensor(outs[0])[:T], g_out[:T], "dropping row: output")
    _check(from_bf16_tensor(outs[1]), g_gu, "dropping row: gate_up_activations_T")
    if not on_I:
        _check(from_bf16_tensor(outs[2]), g_d, "dropping row: down_activations")
