"""Fused RMSNorm -> MXFP8 quantisation: host side of the gfx950 kernel.

Mirrors ``rmsnorm_mx_quantize_tkg``
(src/nkilib_src/nkilib/core/subkernels/rmsnorm_mx_quantize_tkg.py:29-40): the caller
passes pre-allocated outputs, which are filled and returned.  With ``residual`` the
kernel normalises ``input + residual`` (rounded to the input type) and writes that
sum to ``output_residual`` in the same pass over the row (`:214-232`, golden
test/integration/nkilib/core/subkernels/test_rmsnorm_mx_quantize_tkg.py:104-117).
"""

from typing import Optional

import torch

from ... import _native as nv
from ..utils.kernel_assert import kernel_assert


def rmsnorm_mx_quantize_tkg(
    input: torch.Tensor,
    gamma: torch.Tensor,
    output: Optional[torch.Tensor],
    output_quant: torch.Tensor,
    output_scale: torch.Tensor,
    residual: Optional[torch.Tensor] = None,
    output_residual: Optional[torch.Tensor] = None,
    eps: float = 1e-6,
    hidden_actual: Optional[int] = None,
    hidden_dim_tp: bool = True,
):
    """input [B, S, H]; gamma [1, H]; output bf16 [128, B*S, H/128] (or None);
    output_quant 4-byte elements [128, H/512, B*S] (or uint8 [128, H/512, B*S, 4]);
    output_scale uint8 [16, H/512, B*S] (dense) or [128, H/512, B*S] (the reference's
    strided form: scale s lives in row (s//4)*32 + s%4, other rows are left untouched).
    residual [B, S, H] with output_residual [B*S, H] (both of input's dtype): fused residual add; the result is then
    (output, output_quant, output_scale, output_residual) as in the reference.
    """
    # the reference has no other layout either (validate_shapes_quantize_mx, norm_tkg_utils.py:467)
    kernel_assert(hidden_dim_tp, "Only hidden_dim_tp=True is supported")
    kernel_assert(len(input.shape) == 3, f"input must be [B, S, H] but got {tuple(input.shape)}")
    B, S, H = input.shape
    BxS = B * S
    if residual is not None:
        # norm_tkg_utils.py:473-476 (the reference's BxS >= 256 / H1 % 8 rules come from its transposes on the
        # tensor engine and have no counterpart here)
        kernel_assert(tuple(input.shape) == tuple(residual.shape), "input and residual shapes must match")
        kernel_assert(output_residual is not None, "output_residual required when residual provided")
        kernel_assert(tuple(output_residual.shape) == (BxS, H), f"expected output_residual shape (B*S, H)={(BxS, H)}")
        kernel_assert(residual.dtype == input.dtype and output_residual.dtype == input.dtype,
                      "residual and output_residual must have the input's dtype")
    else:
        kernel_assert(output_residual is None, "output_residual given without residual")
    kernel_assert(H % 512 == 0, f"H must be divisible by 512, got {H}")
    kernel_assert(gamma.shape[-1] == H, f"gamma length must equal {H} but got {gamma.shape[-1]}")
    nT = H // 512
    kernel_assert(output_quant.numel() * output_quant.element_size() == 128 * nT * BxS * 4,
                  f"output_quant must hold [128, {nT}, {BxS}] x4 elements")
    kernel_assert(output_scale.dtype == torch.uint8, "output_scale must be uint8")
    if output_scale.shape[0] == 16:
        layout = nv.MX_REF_DENSE
    else:
        kernel_assert(output_scale.shape[0] == 128, "output_scale first dimension must be 16 or 128")
        layout = nv.MX_REF_STRIDED
    kernel_assert(tuple(output_scale.shape[1:]) == (nT, BxS), f"output_scale must be [*, {nT}, {BxS}]")
    if output is not None:
        kernel_assert(tuple(output.shape) == (128, BxS, H // 128) and output.dtype == torch.bfloat16,
                      f"output must be bf16 [128, {BxS}, {H // 128}]")
    L = nv.lib()
    x = nv.require_device_tensor(input, "input")
    g = nv.require_device_tensor(gamma, "gamma")
    r = nv.require_device_tensor(residual, "residual") if residual is not None else None
    for t, n in ((output, "output"), (output_quant, "output_quant"), (output_scale, "output_scale"),
                 (output_residual, "output_residual")):
        if t is not None:
            kernel_assert(t.is_cuda and t.is_contiguous(), f"{n} must be a contiguous device tensor")
    with torch.cuda.device(x.device):
        rc = L.moe_rmsnorm_quant_mxfp8(nv.ptr(x), nv.dtype_code(x, "input"), nv.ptr(r), nv.ptr(output_residual), nv.ptr(g),
                                       nv.dtype_code(g, "gamma"), nv.ptr(output_quant), nv.ptr(output_scale),
                                       nv.ptr(output), BxS, H, float(eps), int(hidden_actual or H), 1, layout,
                                       nv.stream_ptr(x.device))
    nv.check(rc, "rmsnorm_mx_quantize_tkg")
    if residual is not None:
        return output, output_quant, output_scale, output_residual
    return output, output_quant, output_scale


def rmsnorm_mx_quantize(hidden: torch.Tensor, gamma: Optional[torch.Tensor], eps: float = 1e-6, do_norm: bool = True,
                        residual: Optional[torch.Tensor] = None):
    """Token-major front end for the MoE path: [T, H] -> (uint8 codes [T, H] in k' order, uint8 scales [T, H/32]).

    This is the pre-quantised activation format ``moe_cte`` accepts through
    ``hidden_states_scale`` (k' = tile*512 + p*4 + q for h = q*(H/4) + tile*128 + p).
    With ``residual`` ([T, H], hidden's dtype) the row ``hidden + residual`` (rounded to that dtype) is what is
    normalised and quantised, and it is returned as a third result: the layer's new residual stream.
    """
    kernel_assert(len(hidden.shape) == 2, f"hidden must be [T, H] but got {tuple(hidden.shape)}")
    T, H = hidden.shape
    kernel_assert(H % 512 == 0, f"H must be divisible by 512, got {H}")
    L = nv.lib()
    x = nv.require_device_tensor(hidden, "hidden")
    g = nv.require_device_tensor(gamma, "gamma") if do_norm else None
    q = torch.empty((T, H), dtype=torch.uint8, device=x.device)
    s = torch.empty((T, H // 32), dtype=torch.uint8, device=x.device)
    r = out_r = None
    if residual is not None:
        r = nv.require_device_tensor(residual, "residual")
        kernel_assert(tuple(r.shape) == (T, H) and r.dtype == x.dtype, "residual must match hidden in shape and dtype")
        out_r = torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = L.moe_rmsnorm_quant_mxfp8(nv.ptr(x), nv.dtype_code(x, "hidden"), nv.ptr(r), nv.ptr(out_r), nv.ptr(g),
                                       nv.dtype_code(g, "gamma") if g is not None else nv.DT_BF16, nv.ptr(q), nv.ptr(s),
                                       None, T, H, float(eps), H, 1 if do_norm else 0, nv.MX_TOKEN_MAJOR,
                                       nv.stream_ptr(x.device))
    nv.check(rc, "rmsnorm_mx_quantize")
    if residual is not None:
        return q, s, out_r
    return q, s
