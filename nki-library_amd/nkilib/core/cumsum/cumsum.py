"""``cumsum`` on the MI355X: the reference operator (src/nkilib_src/nkilib/core/cumsum/cumsum.py:30-75) over
``moe_cumsum`` of the C ABI; semantics ``cumsum_torch_ref`` (src/nkilib_src/nkilib/core/cumsum/cumsum_torch.py:20-32).
"""

import torch

from ... import _native as nv
from ..._entry import KernelEntry
from ..utils.kernel_assert import kernel_assert


def _cumsum(x, axis=-1):
    """Inclusive prefix sum along the last axis of ``x`` (any rank >= 1; int32, float32, bfloat16 or float16).
    Like the reference, only the last axis is supported.  Floats accumulate in fp32 and the result is rounded to
    the element type; int32 is exact."""
    x = nv.require_device_tensor(x, "x")
    rank = x.dim()
    kernel_assert(rank >= 1, "x must have at least one axis")
    ax = axis + rank if axis < 0 else axis
    kernel_assert(ax == rank - 1, f"cumsum only supports the last axis, got axis={axis} for rank {rank}")
    H = x.shape[-1]
    y = torch.empty_like(x)
    if x.numel() == 0:
        return y
    rc = nv.lib().moe_cumsum(nv.ptr(x), nv.ptr(y), nv.index_dtype_code(x, "x"), x.numel() // H, H,
                             nv.stream_ptr(x.device))
    nv.check(rc, "cumsum")
    return y


cumsum = KernelEntry(_cumsum)
