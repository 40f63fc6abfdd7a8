"""Pins oracle/mx.py with the OCP-MX closed forms, the reference generator's round-trip invariant, brute
force on one block, and single-non-zero probes of the layout maps."""

import numpy as np
import pytest

from oracle import moe as omoe
from oracle import mx
from oracle.numerics import e4m3fn_decode


def test_known_answers():
    d, s = mx.quantize_mx(np.ones((8, 4), np.float32))
    assert s[0, 0] == 119 and (d == 0x78).all()  # 1.0 = 256 * 2^(119-127)
    for sh in (-20, -3, 0, 5, 40):
        x = np.full((8, 4), 0.001 * 2.0**sh, np.float32)
        x[3, 2] = 448.0 * 2.0**sh  # amax = 1.75 * 2^(sh+8)
        d, s = mx.quantize_mx(x)
        assert s[0, 0] == 127 + sh and d[3, 2] == 0x7E
        x[3, 2] = 1.9 * 2.0 ** (sh + 8)  # 486.4 * 2^sh saturates to 448
        d, s = mx.quantize_mx(x)
        assert s[0, 0] == 127 + sh and d[3, 2] == 0x7E
    # closed form: scale byte = floor(log2(amax)) + 127 - 8
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((64, 64)) * np.exp(rng.uniform(-20, 20, (64, 64)))).astype(np.float32)
    _, s = mx.quantize_mx(x)
    am = np.abs(x).reshape(8, 8, 16, 4).max(axis=(1, 3))
    assert np.array_equal(s, (np.floor(np.log2(am)) + 127 - 8).astype(np.uint8))


def test_powers_of_two_are_exact_and_zero_block():
    x = np.zeros((8, 8), np.float32)
    x[:, :4] = 2.0 ** np.arange(-3, 5, dtype=np.float32)[:, None]
    d, s = mx.quantize_mx(x)
    assert np.array_equal(mx.dequantize_mx(d, s), x)
    assert s[0, 1] == 0 and (d[:, 4:] == 0).all()  # all-zero block: scale byte 0, data 0


def test_roundtrip_invariant_of_the_reference_generator():
    """quantize(dequantize(q, s)) == (q, s) whenever each block holds an element with the maximum exponent
    (test/integration/nkilib/utils/tensor_generators.py:386-399,416)."""
    rng = np.random.default_rng(2)
    P, F = 64, 128
    q = rng.integers(0, 0x77, size=(P, F)).astype(np.uint8) | (rng.integers(0, 2, size=(P, F)).astype(np.uint8) << 7)
    for i in range(0, P, 8):
        for j in range(0, F, 4):
            q[i + rng.integers(0, 8), j + rng.integers(0, 4)] = 0x78 + rng.integers(0, 5)  # 256..384: exponent 8
    s = rng.integers(100, 140, size=(P // 8, F // 4)).astype(np.uint8)
    q2, s2 = mx.quantize_mx(mx.dequantize_mx(q, s))
    assert np.array_equal(s2, s)
    assert np.array_equal(e4m3fn_decode(q2), e4m3fn_decode(q))  # +-0 aside, identical codes


def test_mx_matmul_brute_force_one_block():
    rng = np.random.default_rng(3)
    K4, M, N = 16, 3, 5  # K = 64: two 32-blocks
    sq = rng.integers(0, 0x7E, size=(K4, M * 4)).astype(np.uint8)
    mq = rng.integers(0, 0x7E, size=(K4, N * 4)).astype(np.uint8)
    ss = rng.integers(120, 130, size=(K4 // 8, M)).astype(np.uint8)
    ms = rng.integers(120, 130, size=(K4 // 8, N)).astype(np.uint8)
    got = mx.mx_matmul(sq, mq, ss, ms)
    want = np.zeros((M, N))
    for i in range(M):
        for j in range(N):
            for k in range(K4):
                for q in range(4):
                    a = float(e4m3fn_decode(sq[k, i * 4 + q])) * 2.0 ** (int(ss[k // 8, i]) - 127)
                    b = float(e4m3fn_decode(mq[k, j * 4 + q])) * 2.0 ** (int(ms[k // 8, j]) - 127)
                    want[i, j] += a * b
    assert np.allclose(got, want, rtol=1e-6)


@pytest.mark.parametrize("H,I", [(512, 512), (1024, 768)])
def test_layout_maps_single_nonzero(H, I):
    """k' = tile*512 + p*4 + q <-> h = q*(H/4) + tile*128 + p, and gate/up column i lands at
    [p, t, b, q] with i = t*512 + q*(rows/4) + p: move one weight and watch which output moves."""
    rng = np.random.default_rng(4)
    nH = H // 512
    B = 4
    for _ in range(6):
        p, t, q, i = rng.integers(128), rng.integers(nH), rng.integers(4), rng.integers(I)
        w = np.zeros((128, nH, I, 4), np.uint8)
        w[p, t, i, q] = 0x38  # 1.0
        ws = np.full((16, nH, I), 127, np.uint8)
        h = q * (H // 4) + t * 128 + p
        x = np.zeros((B, H), np.float32)
        x[:, h] = np.arange(1, B + 1)
        x[0, (h + 1) % H] = 99.0  # must not leak into column i
        res = omoe.gate_up_proj_mx(x, w, ws, None, H, I, B)
        ti = i // 512
        rows = 512 if (ti < I // 512) else I % 512
        qi, pi = divmod(i - ti * 512, rows // 4)
        expect = np.zeros_like(res)
        expect[pi, ti, :, qi] = np.arange(1, B + 1)
        assert np.array_equal(res, expect)


def test_dequant_helpers_agree_with_block_form():
    """mx_dequant_gate_up / mx_dequant_down (explicit index formulas) == the 8x4 block golden path."""
    rng = np.random.default_rng(5)
    H, I, B = 512, 512, 8
    w = rng.integers(0, 0x7E, size=(128, 2, 1, I, 4)).astype(np.uint8)
    s = rng.integers(118, 126, size=(16, 2, 1, I)).astype(np.uint8)
    dense = omoe.mx_dequant_gate_up(w, s)  # [2, K', I]
    x = np.zeros((B, H), np.float32)
    kp = rng.integers(0, H, size=B)
    tile, p, q = kp // 512, (kp % 512) // 4, kp % 4
    x[np.arange(B), q * (H // 4) + tile * 128 + p] = 1.0  # exactly representable: row b picks K' index kp[b]
    res = omoe.gate_up_proj_mx(x, w[:, 0], s[:, 0], None, H, I, B)  # [128, 1, B, 4]
    got = res[:, 0].transpose(2, 0, 1).reshape(I, B)  # i = q*128 + p
    assert np.allclose(got.T, dense[0][kp], rtol=0, atol=0)


def test_e5m2_block_scale_closed_forms_and_round_trip():
    """e5m2 target (mx_torch_common.py:190-198: largest exponent 15, largest value 57344): an all-ones block gets
    scale byte 127 - 15 and the code of 2**15; values already on the e5m2 grid of their block survive a round trip."""
    d, s = mx.quantize_mx(np.ones((8, 4), np.float32), fmt="e5m2")
    assert s[0, 0] == 112 and (d == 0x78).all()
    assert np.array_equal(mx.dequantize_mx(d, s, fmt="e5m2"), np.ones((8, 4), np.float32))
    rng = np.random.default_rng(5)
    codes = rng.integers(0, 0x7C, size=(64, 32)).astype(np.uint8) | (rng.integers(0, 2, size=(64, 32)).astype(np.uint8) << 7)
    codes.reshape(8, 8, 8, 4)[:, 0, :, 0] = 0x7B  # every block holds the format maximum: scale == the one given
    sc = rng.integers(100, 150, size=(8, 8)).astype(np.uint8)
    x = mx.dequantize_mx(codes, sc, fmt="e5m2")
    q, s2 = mx.quantize_mx(x, fmt="e5m2")
    assert np.array_equal(s2, sc) and np.array_equal(mx.dequantize_mx(q, s2, fmt="e5m2"), x)


def test_mx_matmul_mixed_formats_is_the_plain_product():
    """e5m2 stationary x e4m3 moving equals the fp64 product of the dequantised operands."""
    rng = np.random.default_rng(6)
    a = (rng.standard_normal((32, 16 * 4)) * 0.1).astype(np.float32)
    b = rng.standard_normal((32, 8 * 4)).astype(np.float32)
    aq, asc = mx.quantize_mx(a, fmt="e5m2")
    bq, bsc = mx.quantize_mx(b)
    got = mx.mx_matmul(aq, bq, asc, bsc, stationary_fmt="e5m2")
    ad = mx.dequantize_mx(aq, asc, fmt="e5m2").astype(np.float64).reshape(32, 16, 4)
    bd = mx.dequantize_mx(bq, bsc).astype(np.float64).reshape(32, 8, 4)
    want = np.einsum("kiq,kjq->ij", ad, bd)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)


def test_e2m1_block_scale_closed_forms():
    """MXFP4 target (largest exponent 2, largest value 6): ones -> scale byte 127 - 2, code of 4.0; the format maximum
    times 2**n survives a round trip with scale 127 - 2 + n."""
    d, s = mx.quantize_mx(np.ones((8, 4), np.float32), fmt="e2m1")
    assert s[0, 0] == 125 and (d == 0x6).all()
    assert np.array_equal(mx.dequantize_mx(d, s, fmt="e2m1"), np.ones((8, 4), np.float32))
    x = np.zeros((8, 4), np.float32)
    x[0, 0], x[1, 1], x[2, 2] = 6 * 2.0**-3, -1.5 * 2.0**-3, 0.5 * 2.0**-3
    d, s = mx.quantize_mx(x, fmt="e2m1")
    assert s[0, 0] == 127 - 3 and d[0, 0] == 0x7 and d[1, 1] == 0xB and d[2, 2] == 0x1
    assert np.array_equal(mx.dequantize_mx(d, s, fmt="e2m1"), x)
