"""Seeded input builders shared by the parity tests.

They follow the reference's own generators so that the parity tests read like its tests:
  bf16 / fp8-weight cases  build_bwmm_inputs, test/integration/nkilib/core/moe/moe_cte/test_moe_cte_common.py:554-711
  MX cases                 build_moe_bwmm_mx_cte, test/integration/nkilib/core/moe/moe_cte/test_utils.py:221-471
Everything is numpy; ``to_dev`` moves a case to the GPU as torch tensors.
"""

import math

import numpy as np

from oracle import blocks as ob
from oracle import mx as omx
from oracle.numerics import bf16_bits, e4m3fn_decode, e4m3fn_encode, to_bf16


def routing(T, k, E, B, skip_token=False, alpha=None, n_block_per_iter=1, is_block_parallel=False, is_mx=False,
            vnc_degree=1):
    N = ob.get_n_blocks(T, k, E, B, n_block_per_iter=n_block_per_iter)
    mask, tp2id, b2e, cond = ob.generate_token_position_to_id_and_experts(
        T, k, E, B, skip_token, N, alpha=alpha, is_block_parallel=is_block_parallel, is_mx=is_mx,
        vnc_degree=vnc_degree)
    return N, mask, tp2id, b2e, cond


def affinities(rng, T, E, mask, skip_token):
    if skip_token:
        a = to_bf16(rng.random((T, E)).astype(np.float32)) * mask
    else:
        a = to_bf16(rng.random((T + 1, E)).astype(np.float32))
        a[:T] = a[:T] * mask
        a[T] = 0
    return to_bf16(a.astype(np.float32))


def dense_case(T, H, I, E, k, B, seed=0, skip_token=False, bias=False, quant=False, alpha=None, hidden_std=None):
    """bf16 (or fp8-weight when quant) blockwise case; weights uniform(-0.1, 0.1) like the reference."""
    rng = np.random.default_rng(seed)
    N, mask, tp2id, b2e, cond = routing(T, k, E, B, skip_token, alpha)
    T1 = T if skip_token else T + 1
    if hidden_std is None:
        hs = to_bf16(rng.random((T1, H)).astype(np.float32))
    else:
        hs = to_bf16((rng.standard_normal((T1, H)) * hidden_std).astype(np.float32))
    if not skip_token:
        hs[T] = 0
    c = {"T": T, "T1": T1, "H": H, "I": I, "E": E, "k": k, "B": B, "N": N, "skip_token": skip_token,
         "hidden": hs, "aff": affinities(rng, T, E, mask, skip_token), "tp2id": tp2id, "b2e": b2e, "cond": cond,
         "mask": mask}
    I_pad = math.ceil(I / 16) * 16
    if quant:
        gq = rng.integers(-240, 240, size=(E, H, 2, I)).astype(np.float32)
        dq = rng.integers(-240, 240, size=(E, I_pad, H)).astype(np.float32)
        c["gate_up_q"] = e4m3fn_encode(gq)
        c["down_q"] = e4m3fn_encode(dq)
        c["gate_up_w"] = e4m3fn_decode(c["gate_up_q"])
        c["down_w"] = e4m3fn_decode(c["down_q"])
        # keep products O(1): the reference draws scales in (-0.1, 0.1) for 0..1 inputs of unit-range weights;
        # here the fp8 integers are O(100), so scale them down further
        c["gate_up_scale"] = rng.uniform(-1e-3, 1e-3, size=(E, 1, 2 * I)).astype(np.float32)
        c["down_scale"] = rng.uniform(-1e-3, 1e-3, size=(E, 1, H)).astype(np.float32)
    else:
        c["gate_up_w"] = to_bf16(rng.uniform(-0.1, 0.1, size=(E, H, 2, I)).astype(np.float32))
        c["down_w"] = to_bf16(rng.uniform(-0.1, 0.1, size=(E, I_pad, H)).astype(np.float32))
    if bias:
        c["gate_up_bias"] = to_bf16(rng.uniform(-1, 1, size=(E, 2, I)).astype(np.float32))
        c["down_bias"] = to_bf16(rng.uniform(-1.632, 1.4375, size=(E, H)).astype(np.float32))
    return c


def mx_weights(rng, E, H, I, std=0.02, fmt="e4m3"):
    """Random MXFP8 expert weights (element format ``fmt``) in the reference's x4 layouts (byte axis last)."""
    nH, nI = H // 512, math.ceil(I / 512)
    pI = 128 if I > 512 else I // 4
    gu_fp = (rng.standard_normal((E * 128, 2 * nH * I * 4)) * std).astype(np.float32)
    gu_q, gu_s = omx.quantize_mx(gu_fp, fmt)
    gu_q = gu_q.reshape(E, 128, 2, nH, I, 4)
    gu_s = gu_s.reshape(E, 16, 2, nH, I)
    d_fp = (rng.standard_normal((E, pI, nI, H, 4)) * std).astype(np.float32)
    tail = I % 512
    if tail and I > 512:
        d_fp[:, tail // 4:, nI - 1] = 0  # zero padded partitions of the last tile (test_mlp_common.py:343-358)
    pI8 = math.ceil(pI / 8) * 8
    d2 = np.zeros((E, pI8, nI, H, 4), np.float32)
    d2[:, :pI] = d_fp
    d_q, d_s = omx.quantize_mx(d2.reshape(E * pI8, nI * H * 4), fmt)
    d_q = d_q.reshape(E, pI8, nI, H, 4)[:, :pI].copy()
    d_s = d_s.reshape(E, pI8 // 8, nI, H)
    return gu_q, gu_s, d_q, d_s


_CODE_POOLS = {}


def _random_codes(rng, shape, fmt):
    """Random element codes of an MX format whose VALUES are (nearly) uniform over the format's range, like the
    reference's ``(np.random.random(shape) * 2 - 1) * max_val`` cast to the format (tensor_generators.py:381-384):
    one random byte per element picks a sign and one of 128 magnitudes on an even grid over (0, max)."""
    from oracle.numerics import e2m1_encode, e5m2_encode

    if fmt not in _CODE_POOLS:
        enc, vmax = {"e4m3": (e4m3fn_encode, 448.0), "e5m2": (e5m2_encode, 57344.0), "e2m1": (e2m1_encode, 6.0)}[fmt]
        mag = enc(((np.arange(128, dtype=np.float64) + 0.5) * (vmax / 128)).astype(np.float32))
        sign_bit = 0x08 if fmt == "e2m1" else 0x80
        _CODE_POOLS[fmt] = np.concatenate([mag, mag | np.uint8(sign_bit)])
    return _CODE_POOLS[fmt][rng.integers(0, 256, size=shape, dtype=np.uint8)]


def mx_weights_random_codes(rng, E, H, I, fmt="e4m3", gate_rms=3.0):
    """Expert weights drawn directly in the quantised domain, the way the reference's generator does it
    (generate_stabilized_mx_data, test/integration/nkilib/utils/tensor_generators.py:351-418: element values
    uniform over the format's range, random E8M0 scales over a window of 11 exponents below an upper bound).  The
    upper bound is chosen so that a projection of unit-variance inputs has a root mean square of about
    ``gate_rms``.  Fast enough for the reference's own table shapes (no floating-point quantisation pass over
    hundreds of millions of elements)."""
    nH, nI = H // 512, math.ceil(I / 512)
    pI = 128 if I > 512 else I // 4
    pI8 = math.ceil(pI / 8) * 8
    rms_code = {"e4m3": 448.0, "e5m2": 57344.0, "e2m1": 6.0}[fmt] / math.sqrt(3.0)  # uniform over [-max, max]

    def scales(shape, K):
        # E[4^(s - hi)] over the 11 exponents of the window = 0.1212: weights have rms_code * 2^(hi-127) * 0.348
        hi = int(round(127 + math.log2(gate_rms / (rms_code * 0.348 * math.sqrt(K)))))
        return rng.integers(hi - 10, hi + 1, size=shape, dtype=np.uint8)

    gu_q = _random_codes(rng, (E, 128, 2, nH, I, 4), fmt)
    gu_s = scales((E, 16, 2, nH, I), H)
    d_q = _random_codes(rng, (E, pI, nI, H, 4), fmt)
    d_s = scales((E, pI8 // 8, nI, H), I)
    tail = I % 512
    if tail and I > 512:
        d_q[:, tail // 4:, nI - 1] = 0
    return gu_q, gu_s, d_q, d_s


def mx_case(T, H, I, E, k, B, seed=0, skip_token=False, bias=False, alpha=None, hidden_std=1.0, weight_std=0.05,
            dynamic=False, weight_format="e4m3", random_codes=False):
    rng = np.random.default_rng(seed)
    N, mask, tp2id, b2e, cond = routing(T, k, E, B, skip_token, alpha, n_block_per_iter=2, is_block_parallel=True,
                                        is_mx=True)
    T1 = T if skip_token else T + 1
    hs = to_bf16((rng.standard_normal((T1, H)) * hidden_std).astype(np.float32))
    if not skip_token:
        hs[T] = 0
    if random_codes:
        gu_q, gu_s, d_q, d_s = mx_weights_random_codes(rng, E, H, I, weight_format)
    else:
        gu_q, gu_s, d_q, d_s = mx_weights(rng, E, H, I, weight_std, weight_format)
    c = {"T": T, "T1": T1, "H": H, "I": I, "E": E, "k": k, "B": B, "N": N, "skip_token": skip_token,
         "hidden": hs, "aff": affinities(rng, T, E, mask, skip_token), "tp2id": tp2id, "b2e": b2e,
         "cond": cond if dynamic else None, "mask": mask, "weight_format": weight_format,
         "gate_up_q": gu_q, "gate_up_s": gu_s, "down_q": d_q, "down_s": d_s}
    if bias:
        nI = math.ceil(I / 512)
        pI = 128 if I > 512 else I // 4
        c["gate_up_bias"] = to_bf16(rng.uniform(-2.0625, 0.52, size=(E, pI, 2, nI, 4)).astype(np.float32))
        c["down_bias"] = to_bf16(rng.uniform(-1.632, 1.4375, size=(E, H)).astype(np.float32))
    return c


# ---------------------------------------------------------------- torch side


def bf16_tensor(x, dev):
    import torch

    return torch.from_numpy(bf16_bits(x).view(np.int16)).view(torch.bfloat16).to(dev)


def from_bf16_tensor(t):
    import torch

    return (t.detach().cpu().view(torch.int16).numpy().view(np.uint16).astype(np.uint32) << 16).view(np.float32)


def u8_tensor(x, dev):
    import torch

    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.uint8)).to(dev)


def i32_tensor(x, dev):
    import torch

    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.int32)).to(dev)


def f32_tensor(x, dev):
    import torch

    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dev)


def dirty_device_memory(nbytes, device="cuda:0"):
    """Leave a freed block of at least `nbytes` holding 0xff bytes in torch's caching allocator, so that the next
    torch.empty of that size comes back dirty: what a kernel is said to write must then really be written."""
    import torch

    t = torch.full((int(nbytes),), 0xFF, dtype=torch.uint8, device=device)
    torch.cuda.synchronize()
    del t
