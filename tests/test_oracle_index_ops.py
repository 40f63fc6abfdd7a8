"""Pins of oracle/index_ops.py (find_nonzero_indices / indexed_flatten / cumsum restatements): hand-written
cases, library routines per column, and the chain against the independent layout statement in oracle/blocks.py."""

import numpy as np
import pytest

from oracle import blocks as ob
from oracle import index_ops as ox


def test_find_nonzero_indices_hand_case():
    x = np.array([[0, 2.5], [1, 0], [0, -0.0], [7, np.nan]], dtype=np.float32)
    r = ox.find_nonzero_indices_ref(x)
    assert r["indices"].tolist() == [[1, 3, -1, -1], [0, 3, -1, -1]]  # -0.0 is zero, NaN is not
    assert r["nonzero_counts"].tolist() == [2, 2]
    assert r["indices"].dtype == np.int32 and r["nonzero_counts"].dtype == np.int32


def test_find_nonzero_indices_matches_flatnonzero_and_column_window():
    rng = np.random.default_rng(0)
    x = (rng.random((97, 12)) < 0.2).astype(np.int32) * rng.integers(-3, 4, (97, 12)).astype(np.int32)
    r = ox.find_nonzero_indices_ref(x)
    for c in range(12):
        nz = np.flatnonzero(x[:, c])
        assert r["nonzero_counts"][c] == nz.size
        assert np.array_equal(r["indices"][c, : nz.size], nz)
        assert (r["indices"][c, nz.size:] == -1).all()
    w = ox.find_nonzero_indices_ref(x, col_start_id=np.array([5], np.int32), n_cols=4)
    assert np.array_equal(w["indices"], r["indices"][5:9]) and np.array_equal(w["nonzero_counts"], r["nonzero_counts"][5:9])


def test_indexed_flatten_hand_cases():
    x = np.arange(12, dtype=np.int32).reshape(2, 6)  # rows of 3 blocks of 2
    # disjoint placement
    out = ox.indexed_flatten_ref(x, 2, 16, np.array([4, 0], np.int32))["flattened_array"]
    assert out.tolist() == [6, 7, 8, 9, 10, 11, -1, -1, 0, 1, 2, 3, 4, 5, -1, -1]
    # overlap: the later row wins; blocks outside the output (negative, past the end) are dropped
    out = ox.indexed_flatten_ref(x, 2, 8, np.array([0, 1], np.int32))["flattened_array"]
    assert out.tolist() == [0, 1, 6, 7, 8, 9, 10, 11]
    out = ox.indexed_flatten_ref(x, 2, 8, np.array([-1, 3], np.int32), padding_val=-7)["flattened_array"]
    assert out.tolist() == [2, 3, 4, 5, -7, -7, 6, 7]
    # row_offsets_start selects a window of the offsets
    out = ox.indexed_flatten_ref(x, 2, 16, np.array([9, 9, 5, 1], np.int32), np.array([2], np.int32))["flattened_array"]
    assert out.tolist() == [-1, -1, 6, 7, 8, 9, 10, 11, -1, -1, 0, 1, 2, 3, 4, 5]


def test_indexed_flatten_reference_test_layout_is_a_plain_copy():
    """The reference's own test places row e at block e * (T // f_len): the output is the input followed by
    padding (test/integration/nkilib/core/subkernels/test_indexed_flatten.py:109-121)."""
    T, E, f = 256, 3, 32
    x = np.arange(E * T, dtype=np.int32).reshape(E, T)
    out_len = E * T + 1024
    out = ox.indexed_flatten_ref(x, f, out_len, np.arange(E, dtype=np.int32) * (T // f))["flattened_array"]
    assert np.array_equal(out[: E * T], x.reshape(-1)) and (out[E * T:] == -1).all()


def test_cumsum_closed_forms():
    assert ox.cumsum_ref(np.ones((2, 5), np.int32)).tolist() == [[1, 2, 3, 4, 5]] * 2
    n = np.arange(1, 101, dtype=np.int32)[None]
    assert np.array_equal(ox.cumsum_ref(n)[0], n[0] * (n[0] + 1) // 2)
    x = np.random.default_rng(1).standard_normal((3, 4, 50)).astype(np.float32)
    y = ox.cumsum_ref(x)
    assert y.shape == x.shape
    assert np.allclose(np.diff(y, axis=-1), x[..., 1:], atol=1e-12) and np.allclose(y[..., 0], x[..., 0])
    with pytest.raises(AssertionError):
        ox.cumsum_ref(x, axis=0)


@pytest.mark.parametrize("T,k,E,B,alpha", [(64, 2, 8, 16, None), (256, 2, 8, 128, None), (1000, 4, 16, 128, 0.3),
                                           (300, 8, 32, 32, None)])
def test_chain_reproduces_block_layout(T, k, E, B, alpha):
    """mask -> find_nonzero_indices -> ceil(count / B) -> cumsum -> indexed_flatten equals
    generate_token_position_to_id_and_experts with skip_token (padding -1): two independent statements of the
    same layout (one from the subkernel references, one from the MoE test helper)."""
    router = ob.router_with_controlled_distribution(T, k, E, alpha).astype(np.int32)
    mask = ob.expert_mask_from_router(router, E)
    N = ob.get_n_blocks(T, k, E, B)
    want, b2e, _ = ob.build_token_blocks(mask, B, N, skip_token=True)
    flat, counts, first = ox.block_index_chain(mask, B, N)
    assert np.array_equal(flat, want)
    assert np.array_equal(counts, mask.sum(0).astype(np.int32))
    # an expert's first block is where block_to_expert first names it
    for e in range(E):
        if counts[e]:
            assert b2e[first[e]] == e and (first[e] == 0 or b2e[first[e] - 1] != e)
