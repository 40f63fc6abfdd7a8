"""OCP-MX goldens on the reference's [P, F] "8 partitions x 4 free" block form.

Oracle: test infrastructure only.  Restates
  * ``quantize_mx_golden``     test/utils/mx_utils.py:55-95 (dup. test/integration/nkilib/core/mlp/test_mlp_common.py:363-409)
  * ``quantize_to_mx``         src/nkilib_src/nkilib/core/utils/mx_torch_common.py:157-221
  * ``dequantize_mx_golden``   test/utils/mx_utils.py:195-246
  * ``nc_matmul_mx_golden``    test/utils/mx_utils.py:109-178  (== ``mx_matmul`` mx_torch_common.py:134-154)

An "x4" tensor of shape [P, F/4] (4 fp8 bytes per element, element q = byte q of
the little-endian uint32, mx_torch_common.py:114-123) is carried here as a uint8
array [P, F]; the memory image is identical.

Block scale rule (exponent-field arithmetic, not log2): per 8x4 block
``e = max fp32 exponent field``, ``scale_u8 = e - 8`` for e4m3fn, values are
divided by ``2**(scale_u8 - 127)``, clipped to +-448, cast RNE.

Blocks whose amax is below 2**-119 (e < 8; includes all-zero blocks): the two
reference statements disagree on the scale byte (mx_torch_common.py:213 clips to
0, mx_utils.py:78 wraps uint8 to 248+e) and both produce data that does not
dequantise to the input.  The oracle emits scale byte 0 and divides by
2**(0-127), which is self-consistent (dequantise(quantise(x)) ~= x) and equals
both goldens for all-zero blocks' data (zeros).  Parity unpinned for
0 < amax < 2**-119; tests never put values there.
"""

import numpy as np

from .numerics import (E2M1_MAX, E4M3FN_MAX, E5M2_MAX, e2m1_decode, e2m1_encode, e4m3fn_decode, e4m3fn_encode,
                       e5m2_decode, e5m2_encode, float32_exponent_field)

Q_HEIGHT = 8  # partitions per block
Q_WIDTH = 4  # packed free elements per block
E4M3_MAX_EXP = 8  # 448 = 1.75 * 2**8
# element formats of an MXFP8 tensor: (largest exponent, largest value, encode, decode), the table of
# mx_torch_common.py:190-198
FORMATS = {
    "e4m3": (E4M3_MAX_EXP, E4M3FN_MAX, e4m3fn_encode, e4m3fn_decode),
    "e5m2": (15, E5M2_MAX, e5m2_encode, e5m2_decode),
    "e2m1": (2, E2M1_MAX, e2m1_encode, e2m1_decode),  # MXFP4: one 4-bit pattern per uint8 here
}


def quantize_mx(x, fmt="e4m3"):
    """[P, F] float -> (uint8 data [P, F], uint8 scale [P/8, F/4]) as MXFP8 (e4m3fn unless fmt says e5m2)."""
    max_exp, max_val, encode, _ = FORMATS[fmt]
    x = np.ascontiguousarray(x, dtype=np.float32)
    P, F = x.shape
    assert P % Q_HEIGHT == 0 and F % Q_WIDTH == 0, (P, F)
    SP, SF = P // Q_HEIGHT, F // Q_WIDTH
    exp = float32_exponent_field(x).reshape(SP, Q_HEIGHT, SF, Q_WIDTH)
    emax = exp.max(axis=(1, 3)).astype(np.int32)
    scale_u8 = np.clip(emax - max_exp, 0, 255).astype(np.uint8)
    factor = np.power(2.0, scale_u8.astype(np.float64) - 127.0)
    factor = np.repeat(np.repeat(factor, Q_HEIGHT, axis=0), Q_WIDTH, axis=1)
    v = np.clip(x.astype(np.float64) / factor, -max_val, max_val).astype(np.float32)
    return encode(v), scale_u8


def dequantize_mx(data_u8, scale_u8, fmt="e4m3"):
    """Inverse of quantize_mx: uint8 [P, F], uint8 [P/8, F/4] -> float32 [P, F] (exact)."""
    decode = FORMATS[fmt][3]
    P, F = data_u8.shape
    assert scale_u8.shape == (P // Q_HEIGHT, F // Q_WIDTH), (data_u8.shape, scale_u8.shape)
    factor = np.power(2.0, np.clip(scale_u8.astype(np.int32) - 127, -127, 127).astype(np.float64))
    factor = np.repeat(np.repeat(factor, Q_HEIGHT, axis=0), Q_WIDTH, axis=1)
    return (decode(data_u8).astype(np.float64) * factor).astype(np.float32)


def mx_matmul(stationary_u8, moving_u8, stationary_scale, moving_scale, stationary_fmt="e4m3", moving_fmt="e4m3"):
    """Block-scaled matmul golden.

    stationary [K/4 (P), M*4] bytes + scale [K/32, M]; moving [K/4, N*4] bytes +
    scale [K/32, N].  Contraction runs over the partition axis and the packed q:
    ``out[i, j] = sum_{k, q} S[k, i, q] * Mv[k, j, q]`` (einsum "kiq,kjq->ij").
    Operands are dequantised exactly to fp32 and multiplied/accumulated in fp32
    like the golden's float32 einsum (summation order is BLAS's, as unspecified
    there as in numpy's einsum).
    """
    s = dequantize_mx(stationary_u8, stationary_scale, stationary_fmt)
    m = dequantize_mx(moving_u8, moving_scale, moving_fmt)
    KP = s.shape[0]
    s = s.reshape(KP, -1, Q_WIDTH)
    m = m.reshape(KP, -1, Q_WIDTH)
    # [M, K*4] @ [K*4, N]
    s2 = s.transpose(1, 0, 2).reshape(s.shape[1], -1)
    m2 = m.transpose(1, 0, 2).reshape(m.shape[1], -1)
    return (s2 @ m2.T).astype(np.float32)
