"""Pins oracle/numerics.py against an independent library routine (torch's float8 / bfloat16 casts)
and the formats' closed forms."""

import numpy as np
import torch

from oracle import numerics as nm


def test_e4m3fn_decode_is_the_closed_form_and_matches_torch():
    codes = np.arange(256, dtype=np.uint8)
    v = nm.e4m3fn_decode(codes)
    tv = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    ok = ~np.isnan(tv)
    assert np.array_equal(v[ok], tv[ok]) and np.isnan(v[~ok]).all()
    assert v[0x7E] == 448.0 and v[0x77] == 240.0 and v[0x78] == 256.0 and v[0x01] == 2.0**-9 and v[0x08] == 2.0**-6


def test_e4m3fn_encode_matches_torch_rne_on_random_and_boundaries():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(400000) * rng.choice([1e-4, 1e-2, 1.0, 30.0, 300.0], 400000)).astype(np.float32)
    x = np.clip(x, -448, 448)
    # every midpoint between adjacent representable values (ties) and its fp32 neighbours
    v = np.sort(nm.e4m3fn_decode(np.arange(0, 0x7F, dtype=np.uint8)))
    mids = ((v[:-1].astype(np.float64) + v[1:]) / 2).astype(np.float32)
    ties = np.concatenate([mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)), -mids])
    x = np.concatenate([x, ties, v, -v])
    ours = nm.e4m3fn_encode(x)
    theirs = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(ours, theirs)


def test_e4m3fn_roundtrip_every_code():
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    assert np.array_equal(nm.e4m3fn_encode(nm.e4m3fn_decode(codes)), codes)


def test_e5m2_decode_is_the_closed_form_and_matches_torch():
    codes = np.arange(256, dtype=np.uint8)
    v = nm.e5m2_decode(codes)
    tv = torch.from_numpy(codes).view(torch.float8_e5m2).float().numpy()
    finite = ((codes >> 2) & 0x1F) != 31  # torch reads exponent field 31 as inf / NaN, the reference as 2**16 * (1 + m/4)
    assert np.array_equal(v[finite], tv[finite])
    assert v[0x7B] == 57344.0 and v[0x3C] == 1.0 and v[0x01] == 2.0**-16 and v[0x04] == 2.0**-14 and v[0x7C] == 65536.0


def test_e5m2_encode_matches_torch_rne_on_random_and_boundaries():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(400000) * rng.choice([1e-6, 1e-4, 1.0, 300.0, 30000.0], 400000)).astype(np.float32)
    x = np.clip(x, -57344, 57344)
    v = np.sort(nm.e5m2_decode(np.arange(0, 0x7C, dtype=np.uint8)))
    mids = ((v[:-1].astype(np.float64) + v[1:]) / 2).astype(np.float32)
    ties = np.concatenate([mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)), -mids])
    x = np.concatenate([x, ties, v, -v])
    ours = nm.e5m2_encode(x)
    theirs = torch.from_numpy(x).to(torch.float8_e5m2).view(torch.uint8).numpy()
    assert np.array_equal(ours, theirs)
    codes = np.array([c for c in range(256) if ((c >> 2) & 0x1F) != 31], dtype=np.uint8)
    assert np.array_equal(nm.e5m2_encode(nm.e5m2_decode(codes)), codes)


def test_e2m1_table_is_the_closed_form_and_encode_is_nearest():
    codes = np.arange(16, dtype=np.uint8)
    s_, e_, m_ = (codes >> 3) & 1, (codes >> 1) & 3, codes & 1
    closed = np.where(e_ == 0, m_ * 0.5, (1 + m_ / 2) * 2.0 ** (e_.astype(np.float64) - 1)) * np.where(s_ == 1, -1.0, 1.0)
    assert np.array_equal(nm.e2m1_decode(codes), closed.astype(np.float32))
    assert np.array_equal(nm.e2m1_encode(nm.e2m1_decode(codes)) & 7, codes & 7)
    rng = np.random.default_rng(4)
    x = np.concatenate([rng.uniform(-7, 7, 20000), [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -2.5]]).astype(np.float32)
    got = nm.e2m1_decode(nm.e2m1_encode(x)).astype(np.float64)
    best = np.abs(nm.E2M1_TABLE[None, :8].astype(np.float64) - np.minimum(np.abs(x), 6.0)[:, None].astype(np.float64)).min(axis=1)
    assert np.allclose(np.abs(np.abs(got) - np.minimum(np.abs(x), 6.0)), best) and np.array_equal(np.signbit(got), np.signbit(x))
    # ties go to the even mantissa: 0.25 -> 0, 0.75 -> 1, 1.25 -> 1, 1.75 -> 2, 2.5 -> 2, 3.5 -> 4, 5 -> 4
    assert list(nm.e2m1_decode(nm.e2m1_encode(np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], np.float32)))) == [0, 1, 1, 2, 2, 4, 4]
    # packing: value q in bits 4q..4q+3, the inverse of the reference's unpack
    p = nm.pack_e2m1_x4(np.array([[1, 2, 3, 15]], np.uint8))
    assert p[0] == (1 | 2 << 4 | 3 << 8 | 15 << 12)
    assert [(int(p[0]) >> (4 * q)) & 0xF for q in range(4)] == [1, 2, 3, 15]


def test_bf16_round_matches_torch():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(300000) * rng.choice([1e-20, 1e-3, 1.0, 1e4, 1e30], 300000)).astype(np.float32)
    half = np.array([1.00390625, 1.01171875, -3.0078125], np.float32)  # exact ties between bf16 neighbours
    x = np.concatenate([x, half])
    assert np.array_equal(nm.to_bf16(x), torch.from_numpy(x).bfloat16().float().numpy())
    assert np.array_equal(nm.bf16_from_bits(nm.bf16_bits(x)), nm.to_bf16(x))


def test_e8m0_matches_torch():
    b = np.arange(0, 255, dtype=np.uint8)
    ours = nm.e8m0_decode(b)
    theirs = torch.from_numpy(b).view(torch.float8_e8m0fnu).to(torch.float64).numpy()
    ok = theirs > 0  # byte 0 (2^-127) is subnormal in fp32 and may flush in torch's cast
    assert np.array_equal(ours[ok], theirs[ok]) and ours[127] == 1.0 and ours[0] == 2.0**-127
