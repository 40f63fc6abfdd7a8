"""GPU parity, bit exact: find_nonzero_indices, indexed_flatten, cumsum through the C ABI against the oracle, on
the input shapes of the reference's tests (test/integration/nkilib/core/subkernels/test_find_nonzero_indices.py:
63-82, test_indexed_flatten.py:50-70, test/integration/nkilib/core/cumsum/test_cumsum.py:56-58)."""

import numpy as np
import pytest

from oracle import blocks as ob
from oracle import index_ops as ox

pytestmark = pytest.mark.gpu


def _sparse_input(T, E, top_k, dtype, seed):
    """K = T * top_k / E ones per column in random rows (test_find_nonzero_indices.py:38-45)."""
    rng = np.random.default_rng(seed)
    K = T * top_k // E
    flat = rng.permutation(np.concatenate([np.ones(K * E), np.zeros((T - K) * E)]))
    x = flat.reshape(E, T).T.astype(dtype)
    if dtype == np.float32:
        x[x > 0] = 0.1
    return np.ascontiguousarray(x)


def _fnz_fast(x, start=0, n=None):
    """Vectorised statement of the oracle's loops for the large cases (checked against them below)."""
    T, C = x.shape
    n = C if n is None else n
    idx = np.full((n, T), -1, np.int32)
    cnt = np.zeros(n, np.int32)
    for c in range(n):
        nz = np.flatnonzero(x[:, start + c])
        idx[c, : nz.size] = nz
        cnt[c] = nz.size
    return idx, cnt


@pytest.mark.parametrize("T,E,top_k,dtype", [(4096, 128, 8, "int32"), (4096, 128, 8, "float32"),
                                             (10240, 128, 4, "float32"), (65536, 128, 4, "int32"),
                                             (1000, 37, 4, "bfloat16"), (513, 256, 8, "float16"), (7, 3, 1, "int32")])
def test_find_nonzero_indices_bit_exact(T, E, top_k, dtype):
    import torch
    from nkilib.core.subkernels import find_nonzero_indices

    np_dt = np.float32 if dtype in ("bfloat16", "float16") else getattr(np, dtype)
    x = _sparse_input(T, E, top_k, np_dt, seed=T + E)
    if dtype != "int32":
        x[0, 0], x[min(1, T - 1), 0] = -0.0, 1.0  # negative zero is zero
    want_idx, want_cnt = _fnz_fast(x)
    if T * E <= 40000:
        r = ox.find_nonzero_indices_ref(x)
        assert np.array_equal(r["indices"], want_idx) and np.array_equal(r["nonzero_counts"], want_cnt)
    xt = torch.from_numpy(x).to("cuda:0").to(getattr(torch, dtype))
    idx, cnt = find_nonzero_indices[2](xt, chunk_size=T)
    torch.cuda.synchronize()
    assert idx.dtype == torch.int32 and tuple(idx.shape) == (E, T)
    assert np.array_equal(cnt.cpu().numpy(), want_cnt)
    assert np.array_equal(idx.cpu().numpy(), want_idx)


@pytest.mark.parametrize("T,E,top_k,E_offset,E_local", [(4096, 128, 8, 0, 4), (10240, 128, 4, 16, 16),
                                                        (10240, 128, 4, 120, 8), (777, 40, 4, 33, 7)])
def test_find_nonzero_indices_column_window(T, E, top_k, E_offset, E_local):
    import torch
    from nkilib.core.subkernels import find_nonzero_indices

    x = _sparse_input(T, E, top_k, np.float32, seed=3)
    want_idx, want_cnt = _fnz_fast(x, E_offset, E_local)
    dev = torch.device("cuda:0")
    idx, cnt = find_nonzero_indices(torch.from_numpy(x).to(dev), col_start_id=torch.tensor([E_offset], dtype=torch.int32,
                                                                                           device=dev), n_cols=E_local)
    assert np.array_equal(cnt.cpu().numpy(), want_cnt) and np.array_equal(idx.cpu().numpy(), want_idx)


@pytest.mark.parametrize("T,E,f_len", [(4096, 1, 128), (4096, 3, 128), (4096, 2, 256), (10240, 17, 128),
                                       (65536, 4, 256), (4096, 256, 128), (96, 5, 8)])
def test_indexed_flatten_reference_layout(T, E, f_len):
    import torch
    from nkilib.core.subkernels import indexed_flatten

    x = np.arange(E * T, dtype=np.int32).reshape(E, T)
    offs = (np.arange(E) * (T // f_len)).astype(np.int32)
    out_len = -(-(E * T + 1024) // 128) * 128
    out_len = -(-out_len // f_len) * f_len
    want = ox.indexed_flatten_ref(x, f_len, out_len, offs)["flattened_array"]
    dev = torch.device("cuda:0")
    got = indexed_flatten[2](torch.from_numpy(x).to(dev), f_len, out_len, torch.from_numpy(offs).to(dev))
    assert np.array_equal(got.cpu().numpy(), want)


def test_indexed_flatten_overlap_window_and_bounds():
    import torch
    from nkilib.core.subkernels import indexed_flatten

    dev = torch.device("cuda:0")
    rng = np.random.default_rng(5)
    E, T, f = 9, 64, 8
    x = rng.integers(0, 1000, (E, T)).astype(np.int32)
    for start in (None, 3):
        n_off = E if start is None else E + 5
        offs = rng.integers(-4, 40, n_off).astype(np.int32)  # overlapping, partly outside the output
        st = None if start is None else np.array([start], np.int32)
        want = ox.indexed_flatten_ref(x, f, 256, offs, st, padding_val=-9)["flattened_array"]
        got = indexed_flatten(torch.from_numpy(x).to(dev), f, 256, torch.from_numpy(offs).to(dev),
                              None if st is None else torch.from_numpy(st).to(dev), padding_val=-9)
        assert np.array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("shape,dtype", [((1, 256), "float32"), ((64, 3, 1024), "bfloat16"), ((128, 2048), "float32"),
                                         ((5, 8192), "float16"), ((256, 1000), "int32"), ((3, 1), "int32")])
def test_cumsum(shape, dtype):
    import torch
    from nkilib.core.cumsum import cumsum

    rng = np.random.default_rng(2)
    if dtype == "int32":
        x = rng.integers(-1000, 1000, shape).astype(np.int32)
        xt = torch.from_numpy(x).to("cuda:0")
    else:
        xt = torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).to("cuda:0").to(getattr(torch, dtype))
        x = xt.float().cpu().numpy()
    got = cumsum[1](xt, axis=-1)
    assert got.dtype == xt.dtype and got.shape == xt.shape
    want = ox.cumsum_ref(x)
    if dtype == "int32":
        assert np.array_equal(got.cpu().numpy(), want)  # exact
    else:
        # fp32 accumulation in tree order against the float64 sum: error <= a few ulp of the running |sum| bound,
        # plus the rounding of the result to the element type
        bound = np.cumsum(np.abs(x.astype(np.float64)), axis=-1)
        ulp = {"float32": 2.0 ** -23, "bfloat16": 2.0 ** -8, "float16": 2.0 ** -10}[dtype]
        err = np.abs(got.float().cpu().numpy().astype(np.float64) - want)
        assert (err <= 16 * 2.0 ** -23 * bound + ulp * np.abs(want) + 1e-30).all()
    with pytest.raises(AssertionError):
        cumsum(xt, axis=0) if xt.dim() > 1 else cumsum(xt, axis=1)


@pytest.mark.parametrize("T,k,E,B,alpha", [(8192, 8, 256, 128, None), (8192, 8, 128, 128, 0.3), (300, 2, 8, 32, None)])
def test_chain_builds_token_position_to_id(T, k, E, B, alpha):
    """router mask -> find_nonzero_indices -> blocks per expert -> cumsum -> indexed_flatten on the device equals the
    block layout of generate_token_position_to_id_and_experts (skip_token form), bit exact."""
    import torch
    from nkilib.core.cumsum import cumsum
    from nkilib.core.subkernels import find_nonzero_indices, indexed_flatten

    router = ob.router_with_controlled_distribution(T, k, E, alpha).astype(np.int32)
    mask = ob.expert_mask_from_router(router, E)
    N = ob.get_n_blocks(T, k, E, B)
    want, _, _ = ob.build_token_blocks(mask, B, N, skip_token=True)
    dev = torch.device("cuda:0")
    T_pad = -(-T // B) * B
    m = torch.zeros((T_pad, E), dtype=torch.float32, device=dev)
    m[:T] = torch.from_numpy(mask.astype(np.float32)).to(dev)
    idx, cnt = find_nonzero_indices(m)
    blocks = (cnt + (B - 1)) // B
    first = (cumsum(blocks.reshape(1, E)) - blocks.reshape(1, E)).reshape(E).to(torch.int32)
    flat = indexed_flatten(idx, B, N * B, first)
    assert np.array_equal(flat.cpu().numpy(), want)
