"""Pins oracle/blocks.py: closed form for N, the worked example, invariants of the layout, brute force on
tiny routings, and the committed C1 fixture (seeded legacy numpy stream)."""

import math
import os

import numpy as np
import pytest

from oracle import blocks as ob

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def test_n_blocks_closed_form():
    # BASELINE configs (test_moe_cte_common.py:95-98): C1 11, C2 71, C3 639, C4 766
    assert ob.get_n_blocks(256, 2, 8, 128) == 11
    assert ob.get_n_blocks(4096, 2, 8, 128) == 71
    assert ob.get_n_blocks(8192, 8, 128, 128) == 639
    assert ob.get_n_blocks(8192, 8, 256, 128) == 766
    assert ob.get_n_blocks(8192, 8, 256, 128, n_block_per_iter=4) == 768
    for T, k, E, B in [(5, 2, 3, 2), (100, 4, 7, 16), (1, 8, 256, 128)]:
        assert ob.get_n_blocks(T, k, E, B) == math.ceil((T * k - (E - 1)) / B) + E - 1


def test_worked_example():
    router = np.array([[0, 1], [0, 2], [1, 2], [0, 1], [0, 2]])
    mask = ob.expert_mask_from_router(router, 3)
    tp, b2e, cond = ob.build_token_blocks(mask, 2, 6)
    assert tp.tolist() == [0, 1, 3, 4, 0, 2, 3, 5, 1, 2, 4, 5]
    assert b2e.tolist() == [0, 0, 1, 1, 2, 2]
    assert cond.tolist() == [1, 1, 1, 1, 1, 1, 0]
    tp, _, _ = ob.build_token_blocks(mask, 2, 6, skip_token=True)
    assert tp.tolist() == [0, 1, 3, 4, 0, 2, 3, -1, 1, 2, 4, -1]


def _brute_force(mask, B, N, pad):
    T, E = mask.shape
    slots, b2e = [], []
    counts = [int(mask[:, e].sum()) for e in range(E)]
    nb = [math.ceil(c / B) for c in counts]
    nb[E - 1] += N - sum(nb)
    for e in range(E):
        toks = [t for t in range(T) if mask[t, e]]
        region = toks + [pad] * (nb[e] * B - len(toks))
        slots += region
        b2e += [e] * nb[e]
    return np.array(slots, np.int32), np.array(b2e, np.int32)


@pytest.mark.parametrize("seed", range(8))
def test_brute_force_tiny(seed):
    rng = np.random.default_rng(seed)
    T, E, k, B = int(rng.integers(1, 9)), int(rng.integers(1, 4)), 1, 2
    k = int(rng.integers(1, E + 1))
    router = np.stack([rng.choice(E, size=k, replace=False) for _ in range(T)])
    mask = ob.expert_mask_from_router(router, E)
    N = ob.get_n_blocks(T, k, E, B)
    tp, b2e, cond = ob.build_token_blocks(mask, B, N)
    want_tp, want_b2e = _brute_force(mask, B, N, T)
    assert np.array_equal(tp, want_tp) and np.array_equal(b2e, want_b2e)
    n_pad = N - sum(math.ceil(int(mask[:, e].sum()) / B) for e in range(E))
    assert cond.tolist() == [1] * (N - n_pad) + [0] * (n_pad + 1)


@pytest.mark.parametrize("T,k,E,B,alpha", [(256, 2, 8, 128, None), (1024, 8, 64, 128, 0.3), (512, 4, 16, 256, -1)])
def test_invariants(T, k, E, B, alpha):
    N = ob.get_n_blocks(T, k, E, B)
    mask, tp, b2e, cond = ob.generate_token_position_to_id_and_experts(T, k, E, B, False, N, alpha=alpha)
    tpb = tp.reshape(N, B)
    assert (np.diff(b2e) >= 0).all()
    seen = set()
    for b in range(N):
        e = b2e[b]
        for t in tpb[b][tpb[b] < T]:
            assert mask[t, e] and (t, e) not in seen
            seen.add((int(t), int(e)))
    assert len(seen) == int(mask.sum())  # every routed pair exactly once
    for e in range(E):  # per expert: ascending ids packed from a B-aligned start, then only padding
        region = tpb[b2e == e].reshape(-1)
        real = region[region < T]
        assert (np.diff(real) > 0).all() and (region[: len(real)] == real).all() and (region[len(real):] == T).all()
    nz = np.nonzero(cond == 0)[0]
    assert (cond[: nz[0]] == 1).all() and (cond[nz[0]:] == 0).all()


def test_c1_fixture():
    """The legacy ``np.random.seed(0)`` + ``np.random.choice`` stream is frozen across numpy versions, so the
    reference's C1 routing is reproducible bit for bit; the vectors are committed."""
    fx = np.load(os.path.join(GOLDEN, "c1_blocks.npz"))
    N = ob.get_n_blocks(256, 2, 8, 128)
    mask, tp, b2e, cond = ob.generate_token_position_to_id_and_experts(256, 2, 8, 128, False, N)
    assert np.array_equal(tp, fx["token_position_to_id"])
    assert np.array_equal(b2e, fx["block_to_expert"])
    assert np.array_equal(cond, fx["conditions"])
    assert np.array_equal(ob.router_with_controlled_distribution(256, 2, 8).astype(np.int32), fx["router"])
