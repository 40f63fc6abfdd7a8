"""find_nonzero_indices / indexed_flatten / cumsum (integer, bit exact).  Oracle: test infrastructure only.

Restates, as numpy loops:
  * ``find_nonzero_indices_torch_ref``  src/nkilib_src/nkilib/core/subkernels/find_nonzero_indices_torch.py:20-63
  * ``indexed_flatten_torch_ref``       src/nkilib_src/nkilib/core/subkernels/indexed_flatten_torch.py:18-66
  * ``cumsum_torch_ref``                src/nkilib_src/nkilib/core/cumsum/cumsum_torch.py:20-32

Pinned in tests/test_oracle_index_ops.py: hand-written small cases, ``np.flatnonzero`` / ``np.cumsum`` per
column, and the chain mask -> indices -> block offsets -> flat list against ``oracle.blocks`` (an independent
statement of the same layout, from the MoE test helper).
"""

import numpy as np


def find_nonzero_indices_ref(input_tensor, col_start_id=None, n_cols=None):
    """[T, C] -> indices int32 [C_out, T] (ascending row numbers of the nonzero elements of each column, then
    -1) and nonzero_counts int32 [C_out]  (find_nonzero_indices_torch.py:43-63)."""
    x = np.asarray(input_tensor)
    T, C_full = x.shape
    if col_start_id is not None:
        start, C_out = int(np.asarray(col_start_id).reshape(-1)[0]), int(n_cols)
    else:
        start, C_out = 0, C_full
    indices = np.full((C_out, T), -1, dtype=np.int32)
    counts = np.zeros(C_out, dtype=np.int32)
    for c in range(C_out):
        n = 0
        for t in range(T):
            if x[t, start + c] != 0:
                indices[c, n] = t
                n += 1
        counts[c] = n
    return {"indices": indices, "nonzero_counts": counts}


def indexed_flatten_ref(input_tensor, f_len, output_len, row_offsets, row_offsets_start=None, padding_val=-1):
    """[E, T] seen as [E, T // f_len, f_len]: block p of row e is written to output block
    ``row_offsets[start + e] + p`` when that is inside the output, rows in ascending order (later rows overwrite
    earlier ones); the rest is ``padding_val``  (indexed_flatten_torch.py:45-66)."""
    x = np.asarray(input_tensor)
    E, T = x.shape
    per_row = T // f_len
    n_blocks = output_len // f_len
    start = 0 if row_offsets_start is None else int(np.asarray(row_offsets_start).reshape(-1)[0])
    out = np.full((output_len,), padding_val, dtype=x.dtype)
    blocks = out.reshape(n_blocks, f_len)
    xr = x.reshape(E, per_row, f_len)
    for e in range(E):
        off = int(row_offsets[start + e])
        for p in range(per_row):
            b = off + p
            if 0 <= b < n_blocks:
                blocks[b, :] = xr[e, p, :]
    return {"flattened_array": out}


def cumsum_ref(x, axis=-1):
    """Inclusive prefix sum along the last axis, sequential, in the element type for integers and in float64
    (rounded once to the element type) for floats: the kernel's fp32 accumulation is compared with a tolerance
    (cumsum.py:54-55 states ~1e-2 absolute error for long rows)."""
    x = np.asarray(x)
    assert axis in (-1, x.ndim - 1)
    if np.issubdtype(x.dtype, np.integer):
        return np.cumsum(x, axis=-1, dtype=x.dtype)
    return np.cumsum(x.astype(np.float64), axis=-1)


def block_index_chain(expert_mask, B, N):
    """The reference's device-side route to ``token_position_to_id``: mask [T, E] -> per-expert token lists
    (find_nonzero_indices) -> blocks per expert ``ceil(count / B)`` -> exclusive cumsum = first block of each
    expert -> indexed_flatten with ``f_len = B`` into ``N * B`` slots, -1 in the unused ones."""
    mask = np.asarray(expert_mask)
    T, E = mask.shape
    T_pad = -(-T // B) * B
    r = find_nonzero_indices_ref(mask)
    idx = np.full((E, T_pad), -1, dtype=np.int32)
    idx[:, :T] = r["indices"]
    blocks = (r["nonzero_counts"].astype(np.int64) + B - 1) // B
    first = (cumsum_ref(blocks.astype(np.int32)) - blocks).astype(np.int32)
    flat = indexed_flatten_ref(idx, B, N * B, first)["flattened_array"]
    return flat, r["nonzero_counts"], first
