"""Pins of the token-generation MoE oracle (oracle/moe.py::moe_tkg_ref, ::moe_tkg_mx_ref): a closed form, the two
modes against each other, and the independently restated context-encoding goldens on the equivalent routing."""

import numpy as np

from helpers import dense_case, mx_case
from oracle import moe as omoe
from oracle.compare import max_abs_rel
from oracle.numerics import to_bf16


def _topk(mask, k):
    return np.stack([np.flatnonzero(r)[:k] for r in mask]).astype(np.int32)


def test_closed_form_constant_gate():
    """Gate weights zero and gate bias c: every expert is the linear map act(c) * (x Wu + bu) Wd + bd."""
    rng = np.random.default_rng(0)
    T, H, I, E, K = 5, 32, 16, 4, 2
    x = to_bf16(rng.standard_normal((T, H)).astype(np.float32))
    w_gu = to_bf16(rng.uniform(-0.2, 0.2, (E, H, 2, I)).astype(np.float32))
    w_gu[:, :, 0, :] = 0
    w_d = to_bf16(rng.uniform(-0.2, 0.2, (E, I, H)).astype(np.float32))
    b_gu = to_bf16(rng.uniform(-1, 1, (E, 2, I)).astype(np.float32))
    b_gu[:, 0, :] = 0.75
    b_d = to_bf16(rng.uniform(-1, 1, (E, H)).astype(np.float32))
    aff = to_bf16(rng.uniform(0.1, 1, (T, E)).astype(np.float32))
    idx = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    got = omoe.moe_tkg_ref(x, w_gu, w_d, aff, idx, False, b_gu, b_d, expert_affinities_scaling_mode=omoe.POST_SCALE)
    silu_c = 0.75 / (1 + np.exp(-0.75))
    want = np.zeros((T, H))
    for t in range(T):
        for e in idx[t]:
            y = silu_c * (x[t].astype(np.float64) @ w_gu[e, :, 1, :] + b_gu[e, 1]) @ w_d[e] + b_d[e]
            want[t] += aff[t, e] * y
    assert max_abs_rel(got, want.astype(np.float32)) < 2e-2  # three bf16 roundings per term
    # without scaling the affinities do not enter
    got0 = omoe.moe_tkg_ref(x, w_gu, w_d, aff * 0 + 7, idx, False, b_gu, b_d)
    want0 = np.zeros((T, H))
    for t in range(T):
        for e in idx[t]:
            want0[t] += silu_c * (x[t].astype(np.float64) @ w_gu[e, :, 1, :] + b_gu[e, 1]) @ w_d[e] + b_d[e]
    assert max_abs_rel(got0, want0.astype(np.float32)) < 2e-2


def test_modes_agree_on_one_hot_affinities():
    """All-expert mode with a one-hot table of ones equals selective mode with K = 1, bit for bit."""
    c = dense_case(24, 64, 32, 6, 1, 8, seed=1, skip_token=True, hidden_std=1.0)
    idx = _topk(c["mask"], 1)
    one_hot = np.zeros((24, 6), np.float32)
    one_hot[np.arange(24), idx[:, 0]] = 1
    a = omoe.moe_tkg_ref(c["hidden"], c["gate_up_w"], c["down_w"][:, :32], one_hot, idx, True,
                         expert_affinities_scaling_mode=omoe.POST_SCALE)
    s = omoe.moe_tkg_ref(c["hidden"], c["gate_up_w"], c["down_w"][:, :32], one_hot, idx, False,
                         expert_affinities_scaling_mode=omoe.POST_SCALE)
    assert np.array_equal(a, s)


def test_selective_matches_context_encoding_golden():
    """Same routing through generate_blockwise_numpy_golden's restatement: the two goldens round at different
    points (bf16 after the affinity there, before it here), hence a tolerance."""
    c = dense_case(40, 64, 48, 8, 2, 8, seed=2, skip_token=True, bias=True, hidden_std=1.0)
    idx = _topk(c["mask"], 2)
    tkg = omoe.moe_tkg_ref(c["hidden"], c["gate_up_w"], c["down_w"][:, :48], c["aff"], idx, False, c["gate_up_bias"],
                           c["down_bias"], expert_affinities_scaling_mode=omoe.POST_SCALE)
    cte = omoe.moe_blockwise_ref(c["hidden"], c["aff"], c["gate_up_w"], c["down_w"], c["tp2id"], c["b2e"], 8,
                                 gate_up_proj_bias=c["gate_up_bias"], down_proj_bias=c["down_bias"], skip_token=True)
    assert max_abs_rel(tkg, cte) < 2e-2
    # a wrong expert or a dropped term is far outside that
    wrong = omoe.moe_tkg_ref(c["hidden"], c["gate_up_w"], c["down_w"][:, :48], c["aff"], (idx + 1) % 8, False,
                             c["gate_up_bias"], c["down_bias"], expert_affinities_scaling_mode=omoe.POST_SCALE)
    assert max_abs_rel(wrong, cte) > 0.2


def test_mx_matches_index_formula_reference():
    """moe_tkg_mx_ref against moe_mx_token_ref, which shares no reshape / fold code with it."""
    c = mx_case(6, 512, 512, 4, 2, 128, seed=3, skip_token=True, hidden_std=1.0)
    idx = _topk(c["mask"], 2)
    got = omoe.moe_tkg_mx_ref(c["hidden"], c["gate_up_q"], c["down_q"], c["gate_up_s"], c["down_s"], c["aff"], idx,
                              False, expert_affinities_scaling_mode=omoe.POST_SCALE)
    for t in range(6):
        want = omoe.moe_mx_token_ref(c["hidden"][t], list(idx[t]), c["aff"][t], c["gate_up_q"], c["gate_up_s"],
                                     c["down_q"], c["down_s"])
        assert max_abs_rel(got[t], want.astype(np.float32)) < 2e-2
    # all-expert mode = selective mode listing every expert (fp32 sums in ascending expert order both ways)
    every = np.tile(np.arange(4, dtype=np.int32), (6, 1))
    a = omoe.moe_tkg_mx_ref(c["hidden"], c["gate_up_q"], c["down_q"], c["gate_up_s"], c["down_s"], c["aff"], every,
                            True, expert_affinities_scaling_mode=omoe.POST_SCALE)
    s = omoe.moe_tkg_mx_ref(c["hidden"], c["gate_up_q"], c["down_q"], c["gate_up_s"], c["down_s"], c["aff"], every,
                            False, expert_affinities_scaling_mode=omoe.POST_SCALE)
    assert max_abs_rel(a, s) < 1e-2  # quantisation blocks are per token either way; only the batch shape differs
