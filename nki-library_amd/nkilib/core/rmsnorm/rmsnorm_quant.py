"""RMSNorm + fp8 quantisation (ROW / STATIC): host side of the gfx950 kernel.

Same call signature, argument dataclass, output convention and validation
messages as the reference kernel
(src/nkilib_src/nkilib/core/rmsnorm/rmsnorm_quant.py:41-92,174-262).
"""

from dataclasses import dataclass
from typing import Optional

import torch

from ... import _native as nv
from ..._entry import KernelEntry
from ..utils.common_types import NormType, QuantizationType
from ..utils.kernel_assert import kernel_assert

MAX_S = 32768
MAX_H = 16384
MAX_B = 2
DEQUANT_SCALE_SIZE = 4  # fp32 scale stored as 4 fp8-sized elements at the end of each row


@dataclass(frozen=True)
class RmsNormQuantKernelArgs:
    """Kernel arguments (rmsnorm_quant.py:41-83)."""

    lower_bound: float = 0.0
    norm_type: NormType = NormType.RMS_NORM
    quantization_type: QuantizationType = QuantizationType.ROW
    eps: float = 1e-6

    def __post_init__(self):
        kernel_assert(
            self.quantization_type in (QuantizationType.ROW, QuantizationType.STATIC),
            f"{self.quantization_type.name} quantization is not supported",
        )
        kernel_assert(
            self.norm_type == NormType.NO_NORM or self.norm_type == NormType.RMS_NORM,
            f"{self.norm_type.name} normalization is not supported",
        )
        kernel_assert(self.lower_bound >= 0, f"Lower bound must be positive but got {self.lower_bound}")
        kernel_assert(self.eps >= 0, f"Epsilon must be positive but got {self.eps}")

    def needs_rms_normalization(self) -> bool:
        return self.norm_type == NormType.RMS_NORM

    def has_lower_bound(self) -> bool:
        return self.lower_bound is not None and self.lower_bound > 0.000001

    def is_row_quant(self) -> bool:
        return self.quantization_type == QuantizationType.ROW

    def is_static_quant(self) -> bool:
        return self.quantization_type == QuantizationType.STATIC


def _validate(hidden, ln_w, input_sc, kargs):
    """Shape checks of the reference (_validate_kernel_input, rmsnorm_quant.py:174-262)."""
    kernel_assert(len(hidden.shape) >= 2, f"Rank of hidden must be at least 2 but got {len(hidden.shape)}")
    H = hidden.shape[-1]
    if kargs.is_static_quant():
        kernel_assert(input_sc is not None, "input_dequant_scale must be provided for static quantization")
        kernel_assert(
            tuple(input_sc.shape) == (128, 1),
            f"static input dequant scale shape must be broadcasted to (128, 1) but got {tuple(input_sc.shape)}",
        )
    if kargs.needs_rms_normalization():
        kernel_assert(ln_w is not None, "ln_w must be provided for RMS normalization")
        kernel_assert(len(ln_w.shape) in (1, 2), f"Rank of ln_w must be 1 or 2 but got {len(ln_w.shape)}")
        kernel_assert(ln_w.shape[-1] == H, f"ln_w vector length must equal {H} but got {ln_w.shape[-1]}")
        if len(ln_w.shape) == 2:
            kernel_assert(ln_w.shape[0] <= 1, f"ln_w first dimension {ln_w.shape[0]} must be at most 1")
    if len(hidden.shape) >= 3:
        kernel_assert(hidden.shape[0] <= MAX_B, f"Batch dimension {hidden.shape[0]} exceeds maximum {MAX_B}")
        kernel_assert(hidden.shape[1] <= MAX_S, f"Sequence length {hidden.shape[1]} exceeds maximum {MAX_S}")
        kernel_assert(hidden.shape[2] <= MAX_H, f"Hidden dimension {hidden.shape[2]} exceeds maximum {MAX_H}")
    else:
        kernel_assert(H <= MAX_H, f"Processing dimension {H} exceeds maximum {MAX_H}")
        kernel_assert(
            hidden.shape[0] <= MAX_B * MAX_S,
            f"Outer dimension {hidden.shape[0]} exceeds maximum {MAX_B * MAX_S} (MAX_B * MAX_S)",
        )


def _rmsnorm_quant_kernel(
    hidden: torch.Tensor,
    ln_w: Optional[torch.Tensor],
    kargs: RmsNormQuantKernelArgs,
    input_dequant_scale: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Optional RMSNorm followed by fp8-e4m3 quantisation along the last dimension.

    Returns a ``torch.float8_e4m3fn`` tensor of shape ``[..., H+4]`` (ROW: the last 4
    bytes of every row are the little-endian fp32 dequantisation scale) or ``[..., H]``
    (STATIC).  Values are quantised to the range +-240 of the reference's float8_e4m3,
    whose bit patterns coincide with e4m3fn on that range.
    """
    _validate(hidden, ln_w, input_dequant_scale, kargs)
    L = nv.lib()
    hidden = nv.require_device_tensor(hidden, "hidden")
    H = hidden.shape[-1]
    rows = hidden.numel() // H
    do_norm = 1 if kargs.needs_rms_normalization() else 0
    gamma = nv.require_device_tensor(ln_w, "ln_w") if do_norm else None
    x_dt = nv.dtype_code(hidden, "hidden")
    g_dt = nv.dtype_code(gamma, "ln_w") if gamma is not None else nv.DT_BF16
    stream = nv.stream_ptr(hidden.device)
    with torch.cuda.device(hidden.device):
        if kargs.is_row_quant():
            out = torch.empty((*hidden.shape[:-1], H + DEQUANT_SCALE_SIZE), dtype=torch.uint8, device=hidden.device)
            lb = float(kargs.lower_bound) if kargs.has_lower_bound() else 0.0
            rc = L.moe_rmsnorm_quant_fp8_row(nv.ptr(hidden), x_dt, nv.ptr(gamma), g_dt, nv.ptr(out), rows, H,
                                             float(kargs.eps), lb, do_norm, stream)
        else:
            sc = nv.require_device_tensor(input_dequant_scale, "input_dequant_scale").to(torch.float32)
            out = torch.empty(tuple(hidden.shape), dtype=torch.uint8, device=hidden.device)
            rc = L.moe_rmsnorm_quant_fp8_static(nv.ptr(hidden), x_dt, nv.ptr(gamma), g_dt, nv.ptr(sc), nv.ptr(out),
                                                rows, H, float(kargs.eps), do_norm, stream)
    nv.check(rc, "rmsnorm_quant_kernel")
    return out.view(torch.float8_e4m3fn)


rmsnorm_quant_kernel = KernelEntry(_rmsnorm_quant_kernel)


def split_row_record(out: torch.Tensor):
    """[..., H+4] ROW output -> (fp8 codes [..., H], fp32 dequant scale [..., 1]).

    The consumer-side split the reference uses for pre-quantised inputs
    (test/integration/nkilib/core/mlp/test_mlp_common.py:1061-1069).
    """
    raw = out.view(torch.uint8)
    H = raw.shape[-1] - DEQUANT_SCALE_SIZE
    scale = raw[..., H:].contiguous().view(torch.float32)
    return raw[..., :H].view(torch.float8_e4m3fn), scale
