"""``indexed_flatten`` on the MI355X: the reference operator
(src/nkilib_src/nkilib/core/subkernels/indexed_flatten.py:28-86) over ``moe_indexed_flatten`` of the C ABI.
Semantics are those of ``indexed_flatten_torch_ref``
(src/nkilib_src/nkilib/core/subkernels/indexed_flatten_torch.py:18-66), bit exact.
"""

import torch

from ... import _native as nv
from ..._entry import KernelEntry
from ..utils.kernel_assert import kernel_assert


def _indexed_flatten(input_tensor, f_len, output_len, row_offsets, row_offsets_start=None, padding_val=-1):
    """Same arguments as the reference kernel.  ``input_tensor`` int32 ``[E, T]`` is seen as ``[E, T // f_len,
    f_len]``; block p of row e goes to output block ``row_offsets[start + e] + p`` when that lies inside the
    output (``start = row_offsets_start[0]``, read on the device, 0 when ``None``); where rows overlap the later
    row wins; everything else is ``padding_val``.  Returns the int32 ``[output_len]`` array.  The reference's
    Trainium-only rules (``output_len % 128``, ``(T // f_len) % 16``) do not apply here."""
    x = nv.require_device_tensor(input_tensor, "input_tensor")
    offs = nv.require_device_tensor(row_offsets, "row_offsets").reshape(-1)
    kernel_assert(x.dim() == 2 and x.dtype == torch.int32, "input_tensor must be an int32 [E, T] tensor")
    kernel_assert(offs.dtype == torch.int32, "row_offsets must be int32")
    E, T = x.shape
    f_len, output_len = int(f_len), int(output_len)
    kernel_assert(output_len % f_len == 0, f"output_len must be divisible by f_len, got {output_len=}, {f_len=}")
    kernel_assert(T % f_len == 0, f"T must be divisible by f_len, got {T=}, {f_len=}")
    N = offs.numel()
    if row_offsets_start is None:
        kernel_assert(N == E, f"When row_offsets_start is None, N ({N}) must equal E ({E})")
        start = None
    else:
        kernel_assert(N >= E, f"When row_offsets_start is provided, N ({N}) must be >= E ({E})")
        start = nv.require_device_tensor(row_offsets_start, "row_offsets_start").reshape(-1)
        kernel_assert(start.dtype == torch.int32 and start.numel() == 1, "row_offsets_start must be a [1] int32 tensor")
    out = torch.empty((output_len,), dtype=torch.int32, device=x.device)
    rc = nv.lib().moe_indexed_flatten(nv.ptr(x), E, T, f_len, output_len, nv.ptr(offs), N, nv.ptr(start),
                                      int(padding_val), nv.ptr(out), nv.stream_ptr(x.device))
    nv.check(rc, "indexed_flatten")
    return out


indexed_flatten = KernelEntry(_indexed_flatten)
