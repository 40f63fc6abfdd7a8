"""Pins oracle/moe.py and oracle/rmsnorm.py: special cases that reduce to textbook / library routines,
brute force per token, invariants, the committed fixtures."""

import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import dense_case, mx_case
from oracle import moe as omoe
from oracle import rmsnorm as orn
from oracle.compare import fp8_codes_match_except_ties, max_abs_rel, max_all_close
from oracle.numerics import bf16_bits, e4m3fn_decode, e4m3fn_encode, to_bf16

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def test_single_expert_reduces_to_dense_swiglu():
    """E=1, k=1, B=T, affinity 1: the blockwise MoE is the dense SwiGLU MLP silu(x Wg) * (x Wu) Wd
    (GETTING_STARTED.md:25-35), checked against torch."""
    rng = np.random.default_rng(0)
    T, H, I = 64, 128, 96
    x = to_bf16(rng.standard_normal((T + 1, H)).astype(np.float32))
    x[T] = 0
    wgu = to_bf16(rng.uniform(-0.1, 0.1, (1, H, 2, I)).astype(np.float32))
    wd = to_bf16(rng.uniform(-0.1, 0.1, (1, I, H)).astype(np.float32))
    aff = np.ones((T + 1, 1), np.float32)
    aff[T] = 0
    out = omoe.moe_blockwise_ref(x, aff, wgu, wd, np.arange(T, dtype=np.int32), np.zeros(1, np.int32), T)
    xt = torch.from_numpy(x[:T]).double()
    want = (F.silu(xt @ torch.from_numpy(wgu[0, :, 0]).double()) * (xt @ torch.from_numpy(wgu[0, :, 1]).double())) @ \
        torch.from_numpy(wd[0]).double()
    assert max_abs_rel(out[:T], want.numpy()) < 2.0**-8  # one bf16 rounding of the result
    assert not out[T].any()


@pytest.mark.parametrize("act", [0, 1, 2, 3])
def test_activations_match_torch(act):
    x = np.linspace(-6, 6, 1001).astype(np.float32)
    xt = torch.from_numpy(x).double()
    want = {0: F.silu(xt), 1: F.gelu(xt), 2: F.gelu(xt, approximate="tanh"), 3: xt * torch.sigmoid(1.702 * xt)}[act]
    assert np.allclose(omoe.act_fn(x, act), want.numpy(), atol=1e-6)


@pytest.mark.parametrize("mode,bias", [(1, False), (2, False), (1, True)])
def test_blockwise_equals_per_token_sum(mode, bias):
    """sum over selected experts of aff * MLP_e(x_t), evaluated token by token in fp64, order independent."""
    c = dense_case(96, 64, 48, 4, 2, 16, seed=1, bias=bias, hidden_std=1.0)
    out = omoe.moe_blockwise_ref(c["hidden"], c["aff"], c["gate_up_w"], c["down_w"], c["tp2id"], c["b2e"], c["B"],
                                 gate_up_proj_bias=c.get("gate_up_bias"), down_proj_bias=c.get("down_bias"),
                                 expert_affinities_scaling_mode=mode)
    T, I = c["T"], c["I"]
    want = np.zeros((T, c["H"]))
    for t in range(T):
        for e in np.nonzero(c["mask"][t])[0]:
            a = float(c["aff"][t, e])
            x = c["hidden"][t].astype(np.float64) * (a if mode == 2 else 1.0)
            g = x @ c["gate_up_w"][e, :, 0].astype(np.float64)
            u = x @ c["gate_up_w"][e, :, 1].astype(np.float64)
            if bias:
                g, u = g + c["gate_up_bias"][e, 0], u + c["gate_up_bias"][e, 1]
            d = (g / (1 + np.exp(-g)) * u) @ c["down_w"][e, :I].astype(np.float64)
            if bias:
                d = d + c["down_bias"][e]
            want[t] += d * (a if mode == 1 else 1.0)
    assert max_all_close(out[:T], want, rtol=2.0**-7, atol=1e-5)  # k bf16 roundings
    if not bias:
        assert not out[T].any()  # padding row stays zero under zero affinity / zero hidden


def test_token_permutation_permutes_outputs():
    c = dense_case(64, 64, 32, 4, 2, 16, seed=2, hidden_std=1.0)
    out = omoe.moe_blockwise_ref(c["hidden"], c["aff"], c["gate_up_w"], c["down_w"], c["tp2id"], c["b2e"], c["B"])
    T = c["T"]
    perm = np.random.default_rng(3).permutation(T)
    inv = np.argsort(perm)
    hs = np.concatenate([c["hidden"][:T][perm], c["hidden"][T:]])
    aff = np.concatenate([c["aff"][:T][perm], c["aff"][T:]])
    from oracle import blocks as ob

    tp, b2e, _ = ob.build_token_blocks(c["mask"][perm], c["B"], c["N"])
    out2 = omoe.moe_blockwise_ref(hs, aff, c["gate_up_w"], c["down_w"], tp, b2e, c["B"])
    assert np.array_equal(out2[:T][inv], out[:T])  # same per-token block order -> bit identical


def test_conditions_and_skip_token():
    c = dense_case(64, 64, 32, 4, 2, 16, seed=4, hidden_std=1.0)
    full = omoe.moe_blockwise_ref(c["hidden"], c["aff"], c["gate_up_w"], c["down_w"], c["tp2id"], c["b2e"], c["B"])
    cond = c["cond"]
    assert np.array_equal(full, omoe.moe_blockwise_ref(c["hidden"], c["aff"], c["gate_up_w"], c["down_w"], c["tp2id"],
                                                       c["b2e"], c["B"], conditions=cond))  # padding blocks add 0
    s = dense_case(64, 64, 32, 4, 2, 16, seed=4, skip_token=True, hidden_std=1.0)
    out = omoe.moe_blockwise_ref(s["hidden"], s["aff"], s["gate_up_w"], s["down_w"], s["tp2id"], s["b2e"], s["B"],
                                 skip_token=True)
    assert out.shape == (64, 64) and (s["tp2id"].min() == -1)


def test_mx_block_golden_equals_independent_token_formulation():
    """The block golden (8x4 reshapes, fold/transposes) against explicit index formulas, token by token
    (the reference's own second formulation is _moe_tkg_mx_ref,
    src/nkilib_src/nkilib/core/moe/moe_tkg/moe_tkg_torch.py:299-442)."""
    c = mx_case(128, 1024, 512, 4, 2, 128, seed=5)
    out = omoe.moe_blockwise_mx_ref(c["hidden"], c["aff"], c["gate_up_q"], c["down_q"], c["gate_up_s"], c["down_s"],
                                    c["tp2id"], c["b2e"], c["B"])
    for t in (0, 31, 77, 127):
        es = np.nonzero(c["mask"][t])[0]
        want = omoe.moe_mx_token_ref(c["hidden"][t], es, c["aff"][t], c["gate_up_q"], c["gate_up_s"], c["down_q"],
                                     c["down_s"])
        assert max_abs_rel(out[t], want) < 2.0**-7


def test_grouped_expert_formulation_equals_token_formulation():
    """mx_expert_mlp_rows / moe_mx_tokens_ref (block scales taken out of the block sums, experts decoded once
    for all their rows) against moe_mx_token_ref (every weight scaled, fp64 throughout)."""
    c = mx_case(64, 1024, 1024, 6, 3, 64, seed=9)
    toks = [0, 5, 17, 40, 63]
    es = [list(np.nonzero(c["mask"][t])[0]) for t in toks]
    got = omoe.moe_mx_tokens_ref(c["hidden"][toks], es, [c["aff"][t][e] for t, e in zip(toks, es)],
                                 lambda e: (c["gate_up_q"][e], c["gate_up_s"][e], c["down_q"][e], c["down_s"][e]))
    for i, t in enumerate(toks):
        want = omoe.moe_mx_token_ref(c["hidden"][t], es[i], c["aff"][t], c["gate_up_q"], c["gate_up_s"], c["down_q"],
                                     c["down_s"])
        # the two differ only by fp32 vs fp64 sums inside a 32-element block, except where that moves an
        # intermediate value across an e4m3 rounding boundary of the re-quantisation (one step of one element)
        assert max_abs_rel(got[i], want) < 2e-3, (t, max_abs_rel(got[i], want))
    # one expert, activation other than SiLU
    one = omoe.mx_expert_mlp_rows(c["hidden"][:2], c["gate_up_q"][1], c["gate_up_s"][1], c["down_q"][1], c["down_s"][1],
                                  activation_function=omoe.ACT_SWISH)
    ref = omoe.moe_mx_token_ref(c["hidden"][1], [1], np.ones(6, np.float32), c["gate_up_q"], c["gate_up_s"], c["down_q"],
                                c["down_s"], activation_function=omoe.ACT_SWISH)
    assert max_abs_rel(one[1], ref) < 2e-3


def test_fp8_row_requant_known_answers():
    """Known answers for the fp8-row intermediate re-quantisation (test_mlp_common.py:978-986,1114-1116):
    the range is Neuron's 240, not OCP's 448, and the scale is floored at 1e-5."""
    for s in (2.0**-6, 1.0, 2.0**5):
        y = np.array([[240.0 * s, 9.0 * s, -120.0 * s, 0.0]], np.float32)
        codes, scale = omoe.fp8_row_requant(y)
        assert scale.dtype == np.float32 and scale[0, 0] == np.float32(s)
        # 240 = 1.875 * 2^7 -> 0x77; with amax/448 the first code would be 448 = 0x7E and the second 16.8 -> 16
        assert list(codes[0]) == [0x77, 0x51, 0xEF, 0x00]
    # amax below 240e-5: the scale is exactly the floor and the codes are y / 1e-5
    y = np.array([[1.2e-3, -6e-4, 0.0, 3e-4]], np.float32)
    codes, scale = omoe.fp8_row_requant(y)
    assert scale[0, 0] == np.float32(1e-5)
    assert list(codes[0]) == [0x6F, 0xE7, 0x00, 0x5F]  # 120, -60, 0, 30
    # an all-zero row does not divide by zero
    codes, scale = omoe.fp8_row_requant(np.zeros((1, 8), np.float32))
    assert scale[0, 0] == np.float32(1e-5) and not codes.any()


def test_fp8_row_golden_uses_the_requant_rule():
    """End to end through moe_blockwise_fp8_row_ref: one expert, gate = a constant, up = chosen values, down = a
    selector matrix, so out[h] = code(y_h / scale) * scale.  The ratio out[1] / out[0] is 9/240 under the 240 rule
    (9 is an e4m3 value) and 16/448 (5 % lower) had the range been 448."""
    H = I = 16
    x_codes = np.zeros((2, H), np.uint8)
    x_codes[0, 0] = 0x38  # 1.0 in column 0; row 1 is the padding token
    xs = np.array([1.0, 0.0], np.float32)
    gu = np.zeros((1, H, 2, I), np.uint8)
    gu[0, 0, 0, :] = 0x40  # gate = 2.0 everywhere
    up_vals = np.zeros(I, np.float32)
    up_vals[:3] = [240.0, 9.0, 120.0]
    gu[0, 0, 1, :] = e4m3fn_encode(up_vals)
    dw = np.zeros((1, I, H), np.uint8)
    dw[0, np.arange(I), np.arange(H)] = 0x38
    aff = np.array([[1.0], [0.0]], np.float32)
    out = omoe.moe_blockwise_fp8_row_ref(x_codes, xs, aff, gu, dw, np.ones((1, 1, 2 * I), np.float32),
                                         np.ones((1, 1, H), np.float32), np.array([0, 1], np.int32),
                                         np.array([0], np.int32), 2)
    silu2 = 2.0 / (1.0 + np.exp(-2.0))
    assert abs(out[0, 0] / (240.0 * silu2) - 1) < 2.0**-8           # bf16 output rounding
    assert abs(out[0, 1] / out[0, 0] - 9.0 / 240.0) < 9.0 / 240.0 * 2.0**-7
    assert abs(out[0, 2] / out[0, 0] - 0.5) < 2.0**-8


def test_fp8_row_reduces_to_dequantised_matmul():
    """With the intermediate re-quantisation removed from the picture (one token, tiny I) the fp8-row golden is
    (x_q*s_x) @ (W_q*s_w): check the projection rule on the gate/up half by making down an identity-like probe."""
    c = dense_case(32, 64, 16, 2, 1, 32, seed=6, quant=True, hidden_std=1.0)
    codes, scale = orn.rmsnorm_quant_ref(c["hidden"], np.ones((1, 64), np.float32), None, 0.0, True, "row")
    out = omoe.moe_blockwise_fp8_row_ref(codes, scale.reshape(-1), c["aff"], c["gate_up_q"], c["down_q"],
                                         c["gate_up_scale"], c["down_scale"], c["tp2id"], c["b2e"], c["B"])
    T, I = c["T"], c["I"]
    xd = e4m3fn_decode(codes).astype(np.float64) * scale.astype(np.float64)
    want = np.zeros((T, 64))
    for t in range(T):
        e = int(np.nonzero(c["mask"][t])[0][0])
        wgu = e4m3fn_decode(c["gate_up_q"][e]).astype(np.float64).reshape(64, 2 * I) * c["gate_up_scale"][e].reshape(-1)
        gu = xd[t] @ wgu
        y = gu[:I] / (1 + np.exp(-gu[:I])) * gu[I:]
        wd = e4m3fn_decode(c["down_q"][e]).astype(np.float64)[:I] * c["down_scale"][e].reshape(-1)
        want[t] = (y @ wd) * float(c["aff"][t, e])
    # the only difference is the fp8 re-quantisation of y: relative error <= 2^-4 per element, averaged over I
    assert max_abs_rel(out[:T], want) < 0.08


def test_rmsnorm_row_closed_forms():
    H = 4096
    x = np.ones((1, 5, H), np.float32)
    g = np.ones((1, H), np.float32)
    codes, dq = orn.rmsnorm_quant_ref(x, g, None, 0.0, False, "row")
    n = np.float32(1.0) * np.reciprocal(np.float32(1.0) + np.float32(1e-6))
    assert (codes == 0x77).all()  # every value quantises to 240
    assert np.array_equal(dq, np.full((1, 5, 1), n / np.float32(240.0), np.float32))
    rec = orn.pack_row_record(codes, dq)
    assert rec.shape == (1, 5, H + 4)
    assert np.array_equal(rec[0, 0, H:].tobytes(), np.float32(dq[0, 0, 0]).astype("<f4").tobytes())
    # duplicate rows -> identical records
    rng = np.random.default_rng(7)
    row = to_bf16(rng.standard_normal((1, 1, H)).astype(np.float32) / 100)
    c2, d2 = orn.rmsnorm_quant_ref(np.broadcast_to(row, (1, 9, H)), to_bf16(rng.random((1, H)).astype(np.float32)),
                                   None, 0.0, False, "row")
    assert (c2 == c2[:, :1]).all() and (d2 == d2[:, :1]).all()
    # against a float64 evaluation: same codes except near ties
    x = to_bf16(rng.standard_normal((1, 64, H)).astype(np.float32))
    gam = to_bf16(rng.random((1, H)).astype(np.float32))
    codes, dq = orn.rmsnorm_quant_ref(x, gam, None, 0.0, False, "row")
    x64 = x.astype(np.float64)
    n64 = x64 / (np.sqrt((x64**2).mean(-1, keepdims=True)) + 1e-6) * gam.astype(np.float64)
    q64 = n64 / (np.abs(n64).max(-1, keepdims=True) / 240.0)
    ok, n_bad, n_forgiven = fp8_codes_match_except_ties(codes, codes, q64)
    assert ok
    from oracle.numerics import e4m3fn_encode

    assert np.mean(e4m3fn_encode(q64.astype(np.float32)) != codes) < 1e-3
    # static: clip at +-240
    cs, none = orn.rmsnorm_quant_ref(x * 1000, gam, np.full((128, 1), 0.01, np.float32), 0.0, True, "static")
    assert none is None and np.abs(e4m3fn_decode(cs)).max() == 240.0
    # lower bound clips the scale
    cl, dl = orn.rmsnorm_quant_ref(x, gam, None, 0.5, True, "row")
    assert np.allclose(dl, 0.5 / 240.0)


def test_mx_front_end_is_norm_then_online_quantisation():
    """R3 == rms_norm (eps inside the sqrt) followed by the MoE's online quantisation of the same rows:
    MX blocks never span tokens, so quantise-then-gather == gather-then-quantise."""
    rng = np.random.default_rng(8)
    T, H = 16, 1024
    x = to_bf16(rng.standard_normal((T, H)).astype(np.float32))
    g = to_bf16(rng.random((1, H)).astype(np.float32) + 0.5)
    r = orn.rmsnorm_mx_quant_ref(x, g)
    normed = to_bf16(orn.rms_norm(x, g))
    # the gate/up golden quantises its [B, H] input online in the same [128, tile*B*4] form
    h = normed.reshape(T, 4, H // 512, 128).transpose(3, 2, 0, 1).reshape(128, -1)
    from oracle import mx

    hq, hs = mx.quantize_mx(h)
    assert np.array_equal(r["out_quant"].reshape(128, -1), hq)
    assert np.array_equal(r["out_scale"].reshape(16, -1), hs)
    # token-major view: k' = tile*512 + p*4 + q
    perm = orn.mx_k_order(H)
    deq = e4m3fn_decode(r["tok_quant"]) * np.repeat(np.power(2.0, r["tok_scale"].astype(np.float64) - 127), 32, 1)
    assert max_abs_rel(deq, normed[:, perm]) <= 0.125  # worst case: 1.99*2^8 saturates to 448
    # norm itself against float64
    x64 = x.astype(np.float64)
    n64 = x64 / np.sqrt((x64**2).mean(-1, keepdims=True) + 1e-6) * g.astype(np.float64)
    assert np.mean(bf16_bits(n64.astype(np.float32)) != bf16_bits(normed)) < 5e-3


def test_mx_front_end_residual_branch_closed_forms():
    """The residual branch of the RMSNorm -> MXFP8 golden (test_rmsnorm_mx_quantize_tkg.py:104-117): the new residual
    stream is bf16(x + r) -- checked against torch's bf16 addition, an independent routine -- and everything behind
    it equals the plain front end applied to that sum.  A branch that normalised x alone, or that kept the sum
    unrounded, fails one of the two."""
    import torch

    rng = np.random.default_rng(12)
    T, H = 12, 1024
    x = to_bf16(rng.standard_normal((T, H)).astype(np.float32))
    r = to_bf16((rng.standard_normal((T, H)) * 3).astype(np.float32))
    g = to_bf16(rng.random((1, H)).astype(np.float32) + 0.5)
    got = orn.rmsnorm_mx_quant_ref(x, g, residual=r)
    tsum = (torch.from_numpy(x).to(torch.bfloat16) + torch.from_numpy(r).to(torch.bfloat16)).float().numpy()
    assert np.array_equal(bf16_bits(got["out_residual"]), bf16_bits(tsum))
    assert (got["out_residual"] != (x + r)).any(), "the case must need the rounding"
    plain = orn.rmsnorm_mx_quant_ref(tsum, g)
    for k in ("out", "out_quant", "out_scale", "tok_quant", "tok_scale"):
        assert np.array_equal(got[k], plain[k]), k
    assert not np.array_equal(got["tok_quant"], orn.rmsnorm_mx_quant_ref(x, g)["tok_quant"])


def test_committed_fixtures():
    fx = np.load(os.path.join(GOLDEN, "small_cases.npz"))
    c = mx_case(128, 512, 512, 4, 2, 128, seed=21)
    out = omoe.moe_blockwise_mx_ref(c["hidden"], c["aff"], c["gate_up_q"], c["down_q"], c["gate_up_s"], c["down_s"],
                                    c["tp2id"], c["b2e"], c["B"])
    # BLAS summation order may differ between machines: compare at the parity tolerance, not bit-wise
    from oracle.numerics import bf16_from_bits

    assert max_all_close(out, bf16_from_bits(fx["mx_out_bits"]), rtol=2e-3)
    c2 = dense_case(128, 256, 256, 4, 2, 128, seed=22, hidden_std=1.0)
    out2 = omoe.moe_blockwise_ref(c2["hidden"], c2["aff"], c2["gate_up_w"], c2["down_w"], c2["tp2id"], c2["b2e"], c2["B"])
    assert max_all_close(out2, bf16_from_bits(fx["bf16_out_bits"]), rtol=2e-3)
    rng = np.random.default_rng(23)
    x = to_bf16(rng.standard_normal((4, 1024)).astype(np.float32))
    g = to_bf16(rng.random((1, 1024)).astype(np.float32))
    codes, scale = orn.rmsnorm_quant_ref(x, g, None, 0.0, False, "row")
    assert np.array_equal(orn.pack_row_record(codes, scale), fx["row_record"])
    mxq = orn.rmsnorm_mx_quant_ref(x, g)
    assert np.array_equal(mxq["tok_quant"], fx["mx_tok_quant"]) and np.array_equal(mxq["tok_scale"], fx["mx_tok_scale"])
