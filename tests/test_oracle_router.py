"""Pins of the router top-k oracle (oracle/router.py) that do not retype its formulas: torch's own softmax / sigmoid /
topk on the same inputs, closed forms, and a brute-force scalar loop written like the reference's scatter loops."""

import numpy as np
import torch

from oracle import router as orr


def _inputs(T, H, E, seed, bias=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.empty((T, H)).uniform_(-0.1, 0.1, generator=g).to(torch.bfloat16).float()
    w = torch.empty((H, E)).uniform_(-0.1, 0.1, generator=g).to(torch.bfloat16).float()
    b = torch.empty((E,)).uniform_(-0.1, 0.1, generator=g).to(torch.bfloat16).float() if bias else None
    return x, w, b


def test_against_torch_routines():
    x, w, b = _inputs(37, 128, 24, 0)
    logits = x.double() @ w.double() + b.double()
    for act, tact in ((orr.SOFTMAX, lambda z: torch.softmax(z, -1)), (orr.SIGMOID, torch.sigmoid)):
        r = orr.router_topk_ref(x.numpy(), w.numpy(), b.numpy(), act, 4, router_pre_norm=True, norm_topk_prob=False)
        np.testing.assert_allclose(r["router_logits"], logits.float().numpy(), rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(r["expert_affinities"], tact(logits).float().numpy(), rtol=2e-6, atol=1e-8)
        tv, ti = torch.topk(logits, 4, dim=-1)
        assert np.array_equal(r["expert_index"], ti.numpy().astype(np.int32))  # no exact ties in fp64 logits
        # activation after the selection
        r2 = orr.router_topk_ref(x.numpy(), w.numpy(), b.numpy(), act, 4, router_pre_norm=False)
        want = torch.zeros_like(logits).scatter_(1, ti, tact(tv))
        np.testing.assert_allclose(r2["expert_affinities"], want.float().numpy(), rtol=2e-6, atol=1e-8)


def test_norm_topk_prob_closed_forms():
    x, w, b = _inputs(16, 64, 12, 1, bias=False)
    r = orr.router_topk_ref(x.numpy(), w.numpy(), None, orr.SIGMOID, 3, router_pre_norm=True, norm_topk_prob=True)
    a = r["expert_affinities"]
    np.testing.assert_allclose(a.sum(axis=1), 1.0, rtol=1e-6)
    assert ((a > 0).sum(axis=1) == 3).all()
    # k == E with softmax: renormalising the full softmax changes nothing
    r = orr.router_topk_ref(x.numpy(), w.numpy(), None, orr.SOFTMAX, 12, router_pre_norm=True, norm_topk_prob=True)
    full = orr.router_topk_ref(x.numpy(), w.numpy(), None, orr.SOFTMAX, 12)["expert_affinities"]
    np.testing.assert_allclose(r["expert_affinities"], full, rtol=1e-6)
    # softmax over the selected logits == renormalised full softmax restricted to them (shift invariance)
    r1 = orr.router_topk_ref(x.numpy(), w.numpy(), None, orr.SOFTMAX, 3, router_pre_norm=False)
    r2 = orr.router_topk_ref(x.numpy(), w.numpy(), None, orr.SOFTMAX, 3, router_pre_norm=True, norm_topk_prob=True)
    np.testing.assert_allclose(r1["expert_affinities"], r2["expert_affinities"], rtol=1e-5, atol=1e-8)


def test_ties_go_to_the_lower_index_and_order_is_descending():
    x = np.zeros((2, 64), np.float32)
    w = np.zeros((64, 8), np.float32)
    b = np.array([0.5, 1.0, 1.0, 0.25, 1.0, 0.0, 0.5, 0.75], np.float32)
    r = orr.router_topk_ref(x, w, b, orr.SIGMOID, 5)
    assert r["expert_index"].tolist() == [[1, 2, 4, 7, 0]] * 2
    assert np.isinf(orr.topk_gap(np.zeros((1, 3)), 3)).all() and orr.topk_gap(b[None], 3)[0] == 0.25


def test_scalar_loop_restatement():
    """The reference's explicit scatter loops (router_topk_torch.py:97-105, :110-129), token by token."""
    x, w, b = _inputs(9, 64, 10, 3)
    k = 2
    logits = (x.double() @ w.double() + b.double()).float().numpy()
    r = orr.router_topk_ref(x.numpy(), w.numpy(), b.numpy(), orr.SIGMOID, k, router_pre_norm=True, norm_topk_prob=True)
    for t in range(9):
        order = sorted(range(10), key=lambda e: (-logits[t, e], e))[:k]
        assert r["expert_index"][t].tolist() == order
        sel = np.zeros(10)
        for e in order:
            sel[e] = 1.0 / (1.0 + np.exp(-np.float64(logits[t, e])))
        np.testing.assert_allclose(r["expert_affinities"][t], sel / sel.sum(), rtol=1e-5)
