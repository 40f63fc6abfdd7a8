"""RMSNorm + quantisation goldens.  Oracle: test infrastructure only.

Restates
  * ``rmsnorm_quant_ref``  test/integration/nkilib/core/rmsnorm/test_rmsnorm_quant.py:46-97
  * ``rms_norm``           test/integration/nkilib/utils/test_kernel_common.py:26-41
  * RMSNorm -> MXFP8 golden  test/integration/nkilib/core/subkernels/test_rmsnorm_mx_quantize_tkg.py:100-137

Two deliberate points where the *kernel* (not the test golden) is followed,
because the golden is undefined there:
  * ROW quantisation clamps the dequant scale to >= 1e-6
    (src/nkilib_src/nkilib/core/rmsnorm/rmsnorm_quant.py:597-604); the golden divides
    by zero for an all-zero row.  Identical whenever amax/240 >= 1e-6.
"""

import numpy as np

from .mx import quantize_mx
from .numerics import NEURON_E4M3_MAX, e4m3fn_encode, to_bf16

FP8_RANGE = NEURON_E4M3_MAX  # 240: Neuron float8_e4m3
MIN_DEQUANT_SCALE = 1e-6


def rmsnorm_quant_ref(inp, gamma, input_dequant_scale, lower_bound, quant_only, quant_type, eps=1e-6):
    """inp [..., H] (any float, computed in fp32) -> (uint8 e4m3 codes [..., H], fp32 dequant scale [..., 1] | None).

    quant_type: "row" or "static".
    """
    inp = np.asarray(inp, dtype=np.float32)
    if quant_only:
        norm = inp
    else:
        gamma = np.asarray(gamma, dtype=np.float32).reshape(-1)
        rms = np.sqrt(np.mean(np.square(inp), axis=-1, keepdims=True))
        norm = inp * np.reciprocal(rms + np.float32(eps))
        norm = norm * gamma

    if quant_type == "row":
        amax = np.abs(norm).max(axis=-1, keepdims=True)
        if lower_bound > 0:
            amax = np.clip(amax, a_min=None, a_max=np.float32(lower_bound))
            norm = np.clip(norm, a_min=-np.float32(lower_bound), a_max=np.float32(lower_bound))
        dequant_scale = (amax / np.float32(FP8_RANGE)).astype(np.float32)
        dequant_scale = np.maximum(dequant_scale, np.float32(MIN_DEQUANT_SCALE))
        quant_scale = np.reciprocal(dequant_scale)
        q = norm * quant_scale
        return e4m3fn_encode(q), dequant_scale
    elif quant_type == "static":
        s = np.asarray(input_dequant_scale, dtype=np.float32).reshape(-1)[0]
        q = norm * np.reciprocal(s)
        q = np.clip(q, -FP8_RANGE, FP8_RANGE)
        return e4m3fn_encode(q), None
    raise ValueError(quant_type)


def pack_row_record(codes, dequant_scale):
    """[..., H] codes + [..., 1] fp32 scale -> the kernel's single output buffer [..., H+4] uint8.

    Bytes [H:H+4] are the little-endian fp32 dequant scale
    (src/nkilib_src/nkilib/core/rmsnorm/rmsnorm_quant.py:389-403).
    """
    scale_bytes = np.ascontiguousarray(dequant_scale.astype("<f4")).view(np.uint8).reshape(*codes.shape[:-1], 4)
    return np.concatenate([codes, scale_bytes], axis=-1)


def rms_norm(hidden, gamma, eps=1e-6, hidden_actual=None):
    """RMSNorm with eps inside the sqrt (the variant the MX front end uses)."""
    hidden = np.asarray(hidden, dtype=np.float32)
    if hidden_actual is not None:
        ss = np.sum(np.square(hidden), axis=-1, keepdims=True)
        rms = np.sqrt(ss / np.float32(hidden_actual) + np.float32(eps)).astype(np.float32)
    else:
        rms = np.sqrt(np.mean(np.square(hidden), axis=-1, keepdims=True) + np.float32(eps)).astype(np.float32)
    norm = hidden * np.reciprocal(rms)
    if gamma is not None:
        norm = norm * np.asarray(gamma, dtype=np.float32).reshape(-1)
    return norm


def mx_k_order(H):
    """Permutation perm[k'] = h with k' = tile*512 + p*4 + q and h = q*(H/4) + tile*128 + p.

    This is the order in which the MX kernels contract the hidden dimension
    (test/integration/nkilib/core/mlp/test_mlp_common.py:587; kernel view
    src/nkilib_src/nkilib/core/moe/moe_cte/bwmm_shard_on_block_mx.py:271).
    """
    assert H % 512 == 0
    nt = H // 512
    tile, p, q = np.meshgrid(np.arange(nt), np.arange(128), np.arange(4), indexing="ij")
    return (q * (H // 4) + tile * 128 + p).reshape(-1)


def rmsnorm_mx_quant_ref(inp, gamma, eps=1e-6, hidden_actual=None, do_norm=True, residual=None):
    """[T, H] -> dict of the RMSNorm->MXFP8 front end outputs.

    Returns
      out        float32 (bf16-valued) [128, T, H/128]   normalised rows, h = h1*128 + p
      out_quant  uint8 [128, H/512, T, 4]  (== x4 [128, H/512, T]), element k' = tile*512 + p*4 + q
      out_scale  uint8 [16, H/512, T]      one E8M0 per 32 consecutive k' of a token
      tok_quant  uint8 [T, H] / tok_scale uint8 [T, H/32]: the same data token-major in k' order

    The normalised value is rounded to bf16 before quantisation, as in the golden
    (``.astype(out_dtype)`` at test_rmsnorm_mx_quantize_tkg.py:118).

    residual ([T, H], bf16-valued like inp): the golden's residual branch (`:104-109`): ``hidden = inp + residual`` as a
    sum of two bf16 arrays, i.e. rounded to bf16, replaces inp and is returned as "out_residual" [T, H].
    """
    inp = np.asarray(inp, dtype=np.float32)
    out_residual = None
    if residual is not None:
        inp = to_bf16(inp + np.asarray(residual, dtype=np.float32))
        out_residual = inp
    T, H = inp.shape
    nt = H // 512
    norm = rms_norm(inp, gamma, eps, hidden_actual) if do_norm else inp
    norm = to_bf16(norm)
    out = norm.reshape(T, H // 128, 128).transpose(2, 0, 1)
    # [p, T, q, tile] -> [p, tile, T, q] -> [128, tile*T*4]
    q_in = out.reshape(128, T, 4, nt).transpose(0, 3, 1, 2).reshape(128, -1)
    data, scale = quantize_mx(q_in)
    data = data.reshape(128, nt, T, 4)
    scale = scale.reshape(16, nt, T)
    tok_quant = data.transpose(2, 1, 0, 3).reshape(T, H)
    tok_scale = scale.transpose(2, 1, 0).reshape(T, H // 32)
    res = {"out": out, "out_quant": data, "out_scale": scale, "tok_quant": tok_quant, "tok_scale": tok_scale}
    if out_residual is not None:
        res["out_residual"] = out_residual
    return res
