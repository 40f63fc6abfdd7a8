"""``find_nonzero_indices`` on the MI355X: the reference operator
(src/nkilib_src/nkilib/core/subkernels/find_nonzero_indices.py:34-110) over ``moe_find_nonzero_indices`` of the
C ABI.  Semantics are those of ``find_nonzero_indices_torch_ref``
(src/nkilib_src/nkilib/core/subkernels/find_nonzero_indices_torch.py:20-63), bit exact.
"""

import torch

from ... import _native as nv
from ..._entry import KernelEntry
from ..utils.kernel_assert import kernel_assert


def _find_nonzero_indices(input_tensor, col_start_id=None, n_cols=None, chunk_size=None, index_dtype=torch.int32):
    """Same arguments as the reference kernel.  ``input_tensor`` ``[T, C]`` (int32, float32, bfloat16 or float16);
    ``col_start_id`` an optional ``[1]`` int32 device tensor (it is read on the device: no synchronisation), with
    which only ``n_cols`` columns from there on are processed.  ``chunk_size`` is a Trainium memory knob: checked
    like the reference does (it must divide T) and otherwise without effect.  Returns ``(indices [C_out, T],
    nonzero_counts [C_out])``, both int32: per column the ascending row numbers of its nonzero elements followed by
    -1."""
    x = nv.require_device_tensor(input_tensor, "input_tensor")
    kernel_assert(x.dim() == 2, f"input_tensor must be [T, C] but got {tuple(x.shape)}")
    kernel_assert(index_dtype in (torch.int32, "int32"), f"index_dtype must be int32 but got {index_dtype}")
    T, C_full = x.shape
    if chunk_size is not None:
        kernel_assert(T % int(chunk_size) == 0, f"chunk_size ({chunk_size}) must divide T ({T}) evenly")
    if col_start_id is not None:
        kernel_assert(n_cols is not None, "n_cols is required when col_start_id is given")
        start = nv.require_device_tensor(col_start_id, "col_start_id").reshape(-1)
        kernel_assert(start.dtype == torch.int32 and start.numel() == 1, "col_start_id must be a [1] int32 tensor")
        C_out = int(n_cols)
        kernel_assert(1 <= C_out <= C_full, f"n_cols must be in [1, {C_full}] but got {n_cols}")
    else:
        start, C_out = None, C_full
    dev = x.device
    indices = torch.empty((C_out, T), dtype=torch.int32, device=dev)
    counts = torch.empty((C_out,), dtype=torch.int32, device=dev)
    L = nv.lib()
    ws = nv.workspace(dev, L.moe_find_nonzero_indices_workspace_bytes(T, C_out))
    rc = L.moe_find_nonzero_indices(nv.ptr(x), nv.index_dtype_code(x, "input_tensor"), T, C_full, nv.ptr(start), C_out,
                                    nv.ptr(indices), nv.ptr(counts), nv.ptr(ws), ws.numel(), nv.stream_ptr(dev))
    nv.check(rc, "find_nonzero_indices")
    return indices, counts


find_nonzero_indices = KernelEntry(_find_nonzero_indices)
