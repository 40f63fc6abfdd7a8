"""Low-precision number formats used by the goldens (oracle: test infrastructure only).

The reference casts through ``neuron_dtypes.static_cast`` (third party, absent,
unpinned).  These are the published formats restated from first principles:

* bfloat16: fp32 with the low 16 mantissa bits dropped, round-to-nearest-even.
* float8 e4m3fn (OCP): 1-4-3, bias 7, no inf, max 448, only S.1111.111 is NaN.
  Decode closed form as in ``src/nkilib_src/nkilib/core/utils/mx_torch_common.py:109-131``.
* Neuron ``float8_e4m3`` (max 240, ``src/nkilib_src/nkilib/core/rmsnorm/rmsnorm_quant_constants.py:84-87``)
  has the same bit patterns as e4m3fn for every |v| <= 240, so one codec serves both.
* E8M0: uint8 biased exponent, value 2**(byte - 127).

Everything takes / returns numpy arrays.  bf16 values are carried as float32
arrays whose low 16 bits are zero.
"""

import numpy as np

E4M3FN_MAX = 448.0
NEURON_E4M3_MAX = 240.0


def to_bf16(x):
    """Round float32 values to the nearest bfloat16 (ties to even); result stays float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    rounded = bits + 0x7FFF + ((bits >> 16) & 1)
    out = (rounded & 0xFFFF0000).astype(np.uint32)
    # NaN stays NaN (quiet), do not let the carry turn it into inf / another number.
    nan = np.isnan(x)
    if nan.any():
        out = np.where(nan, np.uint32(0x7FC00000), out)
    return out.view(np.float32).reshape(x.shape)


def bf16_bits(x):
    """uint16 bit patterns of to_bf16(x)."""
    return (to_bf16(x).view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def _build_e4m3fn_table():
    codes = np.arange(256, dtype=np.int64)
    sign = (codes >> 7) & 1
    exp = (codes >> 3) & 0xF
    man = codes & 0x7
    sub = (man / 8.0) * 2.0**-6
    nor = (1.0 + man / 8.0) * np.power(2.0, exp - 7.0)
    val = np.where(exp == 0, sub, nor)
    val = np.where(sign == 1, -val, val)
    val[0x7F] = np.nan
    val[0xFF] = np.nan
    return val.astype(np.float32)


E4M3FN_TABLE = _build_e4m3fn_table()


def e4m3fn_decode(codes):
    """uint8 bit patterns -> float32 (exact)."""
    return E4M3FN_TABLE[np.asarray(codes, dtype=np.uint8)]


def e4m3fn_encode(x):
    """float32 -> uint8 e4m3fn bit patterns, round-to-nearest-even, saturating at +-448.

    The goldens clip to the format maximum before the cast
    (``test/utils/mx_utils.py:91-93``), so saturation only matters for values the
    caller failed to clip.  NaN encodes as 0x7F.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    sign = ((bits >> 31) & 1).astype(np.uint8)
    a = np.abs(x)
    abits = (bits & 0x7FFFFFFF).astype(np.uint64)
    # normal path: keep 3 mantissa bits, RNE on the 20 dropped bits
    r = (abits + 0x7FFFF + ((abits >> 20) & 1)) >> 20  # (exp8 << 3) | man3
    code_n = r.astype(np.int64) - (120 << 3)  # rebias 127 -> 7
    # subnormal path (|x| < 2**-6): multiples of 2**-9, RNE; 8 == smallest normal
    code_s = np.rint(a.astype(np.float64) * 512.0).astype(np.int64)
    code = np.where(a < 2.0**-6, code_s, code_n)
    code = np.clip(code, 0, 0x7E)
    code = np.where(np.isnan(x), 0x7F, code)
    return (code.astype(np.uint8) | (sign << 7)).reshape(x.shape)


def _build_e5m2_table():
    """All 256 e5m2 bit patterns as the reference decodes them
    (src/nkilib_src/nkilib/core/utils/mx_torch_common.py:87-111): S(1) E(5) M(2), bias 15; the
    exponent field 31 is decoded like any other (no inf / NaN), codes the quantiser never emits."""
    codes = np.arange(256, dtype=np.int64)
    sign = (codes >> 7) & 1
    exp = (codes >> 2) & 0x1F
    man = codes & 0x3
    sub = (man / 4.0) * 2.0**-14
    nor = (1.0 + man / 4.0) * np.power(2.0, exp - 15.0)
    val = np.where(exp == 0, sub, nor)
    return np.where(sign == 1, -val, val).astype(np.float32)


E5M2_TABLE = _build_e5m2_table()
E5M2_MAX = 57344.0


def e5m2_decode(codes):
    """uint8 bit patterns -> float32 (exact)."""
    return E5M2_TABLE[np.asarray(codes, dtype=np.uint8)]


def e5m2_encode(x):
    """float32 -> uint8 e5m2 bit patterns, round-to-nearest-even, saturating at +-57344 (the callers
    clip first, like the goldens: mx_torch_common.py:216-219)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    sign = ((bits >> 31) & 1).astype(np.uint8)
    a = np.abs(x)
    abits = (bits & 0x7FFFFFFF).astype(np.uint64)
    # normal path: keep 2 mantissa bits, RNE on the 21 dropped bits
    r = (abits + 0xFFFFF + ((abits >> 21) & 1)) >> 21  # (exp8 << 2) | man2
    code_n = r.astype(np.int64) - (112 << 2)  # rebias 127 -> 15
    # subnormal path (|x| < 2**-14): multiples of 2**-16, RNE; 4 == smallest normal
    code_s = np.rint(a.astype(np.float64) * 65536.0).astype(np.int64)
    code = np.where(a < 2.0**-14, code_s, code_n)
    code = np.clip(code, 0, 0x7B)
    return (code.astype(np.uint8) | (sign << 7)).reshape(x.shape)


# float4_e2m1fn: S(1) E(2) M(1), bias 1, no inf / NaN; index = 4-bit pattern
# (src/nkilib_src/nkilib/core/utils/mx_torch_common.py:32-66)
E2M1_TABLE = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0],
                      dtype=np.float32)
E2M1_MAX = 6.0


def e2m1_decode(codes):
    """4-bit patterns (one per uint8, values 0..15) -> float32 (exact)."""
    return E2M1_TABLE[np.asarray(codes, dtype=np.uint8) & 0xF]


def e2m1_encode(x):
    """float32 -> 4-bit patterns (one per uint8), nearest value, ties to the even mantissa, saturating at
    +-6.  Only used to make test weights: the reference packs with the absent ``neuron_dtypes.static_cast``,
    whose tie rule is unknown; what both sides of a parity test consume are the codes."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    a = np.minimum(np.abs(x).astype(np.float64), 6.0)
    mag = E2M1_TABLE[:8].astype(np.float64)
    # midpoints between neighbours; a tie goes to the neighbour with even code (mantissa bit 0)
    mids = (mag[:-1] + mag[1:]) / 2
    idx = np.searchsorted(mids, a, side="left")  # a == mid -> lower neighbour
    tie = np.isin(a, mids)
    lower_even = (idx % 2) == 0
    idx = np.where(tie & ~lower_even, idx + 1, idx)
    sign = (np.signbit(x)).astype(np.uint8)
    return (idx.astype(np.uint8) | (sign << 3)).reshape(x.shape)


def pack_e2m1_x4(codes):
    """[..., 4] 4-bit patterns -> uint16 x4 elements, value q in bits 4q..4q+3 (mx_torch_common.py:69-81)."""
    c = np.asarray(codes, dtype=np.uint16)
    assert c.shape[-1] == 4
    return (c[..., 0] | (c[..., 1] << 4) | (c[..., 2] << 8) | (c[..., 3] << 12)).astype(np.uint16)


def e8m0_decode(b):
    """uint8 E8M0 -> float64 power of two, 2**(b-127)."""
    return np.power(2.0, np.asarray(b).astype(np.int32) - 127)


def float32_exponent_field(x):
    """Biased exponent field of float32 values (``test/utils/mx_utils.py:42-45``)."""
    return (np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) >> 23) & 0xFF
