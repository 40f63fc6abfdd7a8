"""GPU parity of the router top-k front end (through the C ABI) against oracle/router.py.

Bars: expert indices identical wherever the k-th and (k+1)-th logits are further apart than the fp32 GEMM's
reordering noise (1e-5; otherwise either expert is a correct answer) and in descending-logit order; logits within
bf16 rounding (output dtype) of the fp64-accumulated oracle; affinities max-abs-rel <= 1e-2 (bf16 output).
"""

import numpy as np
import pytest

from oracle import router as orr
from oracle.compare import max_abs_rel
from oracle.numerics import bf16_from_bits

pytestmark = pytest.mark.gpu


def _np(t):
    import torch

    if t.dtype == torch.bfloat16:
        return bf16_from_bits(t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16))
    return t.cpu().numpy()


@pytest.mark.parametrize(
    "T,H,E,k,act,pre,norm,bias,layout",
    [
        (300, 512, 64, 2, 1, True, False, True, 1),     # softmax over all experts, unmasked (reference default)
        (1000, 7168, 256, 8, 0, True, True, False, 1),  # DeepSeek-V3 shape: sigmoid, top-8, renormalised
        (257, 1024, 100, 4, 1, False, False, True, 0),  # activation after the selection, E not a multiple of 16, x [H, T]
        (64, 256, 512, 8, 0, False, False, False, 1),   # E = 512
        (5, 128, 8, 8, 1, True, True, True, 1),         # k == E, ragged T
    ],
)
def test_router_topk_matches_oracle(T, H, E, k, act, pre, norm, bias, layout):
    import torch
    from nkilib.core.router_topk import router_topk
    from nkilib.core.utils.common_types import RouterActFnType

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(11)
    x = torch.empty((T, H), device=dev).uniform_(-1, 1, generator=g).to(torch.bfloat16)
    w = torch.empty((H, E), device=dev).uniform_(-0.1, 0.1, generator=g).to(torch.bfloat16)
    b = torch.empty((1, E), device=dev).uniform_(-0.5, 0.5, generator=g).to(torch.bfloat16) if bias else None
    xin = x if layout == 1 else x.t().contiguous()
    outs = router_topk[2](xin, w, b, None, None, None, RouterActFnType(act), k, layout, 0, router_pre_norm=pre,
                          norm_topk_prob=norm, return_eager_affi=True)
    torch.cuda.synchronize()
    logits, idx, aff, topk_aff = outs
    r = orr.router_topk_ref(_np(x), _np(w), None if b is None else _np(b).reshape(-1), act, k, router_pre_norm=pre,
                            norm_topk_prob=norm)
    lg = _np(logits)
    assert np.abs(lg - r["router_logits"]).max() <= 2 ** -8 * np.abs(r["router_logits"]).max() + 1e-6
    gap = orr.topk_gap(r["router_logits"], k)
    safe = gap > 1e-5
    gi = idx.cpu().numpy()
    assert safe.mean() > 0.95
    assert np.array_equal(np.sort(gi[safe], axis=1), np.sort(r["expert_index"][safe], axis=1))
    # order: descending logits (compare through the oracle's logits; equal logits may swap)
    picked = np.take_along_axis(r["router_logits"], gi.astype(np.int64), axis=1)
    assert (np.diff(picked, axis=1) <= 1e-5).all()
    a = _np(aff)
    err = max_abs_rel(a[safe], r["expert_affinities"][safe])
    print(f"router T={T} E={E} k={k}: affinity max-abs-rel {err:.2e}, {100 * (1 - safe.mean()):.2f}% near-ties", flush=True)
    assert err <= 1e-2
    ta = topk_aff.cpu().numpy()
    want = np.take_along_axis(r["expert_affinities"], gi.astype(np.int64), axis=1)
    assert np.abs(ta[safe] - want[safe]).max() <= 1e-5 + 1e-4 * np.abs(want).max()


def test_route_for_moe_feeds_the_block_build():
    """Masked table + ids from hidden states: zero outside the top-k, zero padding row, ids usable as they are."""
    import torch
    from nkilib.core.moe.moe_cte import build_token_blocks, get_n_blocks
    from nkilib.core.router_topk import route_for_moe
    from nkilib.core.utils.common_types import RouterActFnType

    dev = torch.device("cuda:0")
    T, H, E, k, B = 512, 1024, 32, 4, 128
    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn((T + 1, H), generator=g, device=dev).to(torch.bfloat16)
    x[T] = 0
    w = (torch.randn((H, E), generator=g, device=dev) * 0.05).to(torch.bfloat16)
    ids, aff = route_for_moe(x, w, None, k, RouterActFnType.SIGMOID, norm_topk_prob=True)
    torch.cuda.synchronize()
    a = _np(aff)
    assert a.shape == (T + 1, E) and not a[T].any()
    assert ((a[:T] > 0).sum(axis=1) == k).all()
    np.testing.assert_allclose(a[:T].sum(axis=1), 1.0, atol=2e-2)
    rows = np.arange(T)[:, None]
    assert (a[rows, ids.cpu().numpy()] > 0).all()
    N = get_n_blocks(T, k, E, B, n_block_per_iter=2)
    tp2id, b2e, _ = build_token_blocks(ids, E, B, N, n_conditions=N + 2)
    assert int((tp2id.reshape(-1) < T).sum()) == T * k
