"""GPU parity: blockwise MoE through moe_cte -> C ABI -> HIP kernels vs the oracle.

Tolerances are the reference's (max-abs-rel, ``maxAllClose(mode="max")``): rtol 2e-2 for
bf16 (test/integration/nkilib/core/moe/moe_cte/test_moe_cte.py:246), and the stricter 2e-2
instead of the reference's 5e-2 for the quantised variants
(test/integration/nkilib/core/moe/moe_cte/test_moe_bwmm_mx_cte.py:287-288); atol 1e-5.
"""

import numpy as np
import pytest

from helpers import (affinities, bf16_tensor, dense_case, dirty_device_memory, f32_tensor, from_bf16_tensor, i32_tensor, mx_case,
                     mx_weights_random_codes, routing, u8_tensor)
from oracle.numerics import to_bf16
from oracle import moe as omoe
from oracle import rmsnorm as orn
from oracle.compare import max_abs_rel, max_all_close

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-2, 1e-5


def _spec(name):
    from nkilib.core.moe.moe_cte import MoECTEImplementation, MoECTESpec

    return MoECTESpec(implementation=getattr(MoECTEImplementation, name))


def _run_dense(c, impl="shard_on_block", act=0, mode=1, clamps=None, conditions=None, fp8_weights=False):
    import torch
    from nkilib.core.moe.moe_cte import QuantizationConfig, SkipMode, moe_cte
    from nkilib.core.utils.common_types import ActFnType, ExpertAffinityScaleMode

    dev = torch.device("cuda:0")
    kw = {}
    if fp8_weights:
        gu = u8_tensor(c["gate_up_q"], dev).view(torch.float8_e4m3fn)
        dw = u8_tensor(c["down_q"], dev).view(torch.float8_e4m3fn)
        kw["quantization_config"] = QuantizationConfig(f32_tensor(c["gate_up_scale"], dev),
                                                       f32_tensor(c["down_scale"], dev))
    else:
        gu, dw = bf16_tensor(c["gate_up_w"], dev), bf16_tensor(c["down_w"], dev)
    if "gate_up_bias" in c:
        kw["gate_and_up_proj_bias"] = bf16_tensor(c["gate_up_bias"], dev)
        kw["down_proj_bias"] = bf16_tensor(c["down_bias"], dev)
    if clamps:
        kw.update(clamps)
    if conditions is not None:
        kw["conditions"] = i32_tensor(conditions, dev)
    out = moe_cte[2](
        bf16_tensor(c["hidden"], dev), bf16_tensor(c["aff"].reshape(-1, 1), dev), gu, dw,
        i32_tensor(c["tp2id"], dev), i32_tensor(c["b2e"].reshape(-1, 1), dev), c["B"], _spec(impl),
        activation_function=ActFnType(act), skip_dma=SkipMode(c["skip_token"], False),
        is_tensor_update_accumulating=c["k"] != 1, expert_affinities_scaling_mode=ExpertAffinityScaleMode(mode), **kw)
    torch.cuda.synchronize()
    return out


def _golden_dense(c, act=0, mode=1, clamps=None, conditions=None, fp8_weights=False):
    clamps = clamps or {}
    return omoe.moe_blockwise_ref(
        c["hidden"], c["aff"], c["gate_up_w"], c["down_w"], c["tp2id"], c["b2e"], c["B"], conditions=conditions,
        gate_up_proj_bias=c.get("gate_up_bias"), down_proj_bias=c.get("down_bias"),
        gate_up_proj_scale=c["gate_up_scale"] if fp8_weights else None,
        down_proj_scale=c["down_scale"] if fp8_weights else None, activation_function=act,
        skip_token=c["skip_token"], expert_affinities_scaling_mode=mode,
        gate_clamp_upper_limit=clamps.get("gate_clamp_upper_limit"),
        gate_clamp_lower_limit=clamps.get("gate_clamp_lower_limit"),
        up_clamp_upper_limit=clamps.get("up_clamp_upper_limit"),
        up_clamp_lower_limit=clamps.get("up_clamp_lower_limit"))


def _check(actual, golden, what, rtol=RTOL):
    err = max_abs_rel(actual, golden)
    print(f"{what}: max-abs-rel {err:.3e} (rtol {rtol})", flush=True)
    assert max_all_close(actual, golden, rtol=rtol, atol=ATOL), f"{what}: max-abs-rel {err:.3e} > {rtol}"


def test_c1_tiny_bf16():
    """BASELINE config 1: T=256, H=512, I=1024, E=8, top-2, B=128, bf16, no quantisation."""
    c = dense_case(256, 512, 1024, 8, 2, 128, seed=0, hidden_std=1.0)
    dirty_device_memory(257 * 2 * 512 * 2)  # the result buffer starts as 0xff: its zeros are written, not inherited
    out = _run_dense(c)
    assert tuple(out.shape) == (257, 2, 512)
    o = from_bf16_tensor(out)
    assert not o[:, 1].any(), "second shard slot must stay zero"
    assert not o[256].any(), "padding token row must stay zero"
    _check(o[:, 0], _golden_dense(c), "C1 bf16")


@pytest.mark.parametrize(
    "T,H,I,E,k,B,impl,act,mode,bias,skip,clamp",
    [
        (512, 1024, 512, 4, 2, 256, "shard_on_block", 0, 1, False, False, False),
        (300, 512, 384, 8, 4, 128, "shard_on_block", 0, 1, True, False, False),
        (512, 768, 520, 8, 2, 128, "shard_on_i", 3, 2, False, False, True),    # Swish, PRE_SCALE, clamps, I%64 != 0
        (256, 512, 256, 8, 2, 128, "shard_on_i", 1, 1, True, True, False),     # GELU, bias, skip_token
        (256, 512, 256, 4, 1, 128, "shard_on_block", 2, 1, False, False, False),  # top-1: non accumulating
        (200, 256, 128, 3, 2, 64, "shard_on_i", 0, 0, False, False, False),    # NO_SCALE, B < 128
        # many rows per expert: the 256-row chunk tiles (a chunk of 300 rows = a full tile and a 44-row one; H and I
        # that are no multiples of the column tiles)
        (300, 512, 384, 2, 2, 128, "shard_on_block", 0, 1, True, False, False),
        (640, 576, 520, 2, 2, 128, "shard_on_i", 3, 2, False, False, True),
        (600, 512, 384, 2, 2, 128, "shard_on_block", 1, 1, True, True, False),
        # shapes of the large-tile kernels (H % 256 == 0, I % 128 == 0) with the options above: PRE_SCALE and clamps;
        # chunks of 257..320 rows (E = 2: 320 rows per expert); a short last intermediate tile (I = 640)
        (512, 768, 512, 8, 2, 128, "shard_on_i", 3, 2, False, False, True),
        (320, 512, 640, 2, 2, 64, "shard_on_block", 0, 1, True, False, True),
        (1100, 256, 128, 3, 2, 128, "shard_on_i", 2, 1, True, True, False),
    ],
)
def test_dense_variants(T, H, I, E, k, B, impl, act, mode, bias, skip, clamp):
    c = dense_case(T, H, I, E, k, B, seed=3, skip_token=skip, bias=bias, hidden_std=1.0)
    clamps = dict(gate_clamp_upper_limit=0.8, gate_clamp_lower_limit=-0.7, up_clamp_upper_limit=0.9,
                  up_clamp_lower_limit=-0.5) if clamp else None
    out = _run_dense(c, impl=impl, act=act, mode=mode, clamps=clamps)
    o = from_bf16_tensor(out)
    if impl == "shard_on_block" and k != 1:
        assert o.ndim == 3
        o = o[:, 0]
    g = _golden_dense(c, act=act, mode=mode, clamps=clamps)
    if not skip:
        # row T (padding token) is unspecified in the golden when a bias is scattered to it; the GPU keeps it zero
        assert not o[T].any()
        o, g = o[:T], g[:T]
    _check(o, g, f"dense {impl} act={act} mode={mode}")


@pytest.mark.parametrize("fp8_weights", [False, True])
def test_dense_down_weight_padded_on_I_large_tile_shape(fp8_weights):
    """down_proj_weight [E, I_pad, H] with I_pad > I (test_moe_cte_common.py:645,663) on a shape of the large-tile
    kernels: rows I.. of every expert's down weights hold junk that must not reach the result."""
    c = dense_case(256, 512, 128, 4, 2, 128, seed=21, quant=fp8_weights, hidden_std=1.0)
    rng = np.random.default_rng(21)
    pad = 32
    if fp8_weights:
        junk = rng.integers(0, 0x7e, size=(4, pad, 512)).astype(np.uint8)
        c["down_q"] = np.concatenate([c["down_q"], junk], axis=1)
        c["down_w"] = np.concatenate([c["down_w"], np.full((4, pad, 512), 3.0, np.float32)], axis=1)
    else:
        c["down_w"] = np.concatenate([c["down_w"], np.full((4, pad, 512), 3.0, np.float32)], axis=1)
    out = _run_dense(c, impl="shard_on_block", fp8_weights=fp8_weights)
    o = from_bf16_tensor(out)[:, 0]
    _check(o[:256], _golden_dense(c, fp8_weights=fp8_weights)[:256], f"padded I, fp8 weights {fp8_weights}")


def _run_checkpointed(c, impl, act=0, mode=1, clamps=None, on_I=False, tp2id=None, b2e=None, fp8_weights=False):
    import torch
    from nkilib.core.moe.moe_cte import (MoECTEImplementation, MoECTESpec, QuantizationConfig, ShardOnIConfig, SkipMode,
                                         moe_cte)
    from nkilib.core.utils.common_types import ActFnType, ExpertAffinityScaleMode

    dev = torch.device("cuda:0")
    kw = dict(clamps or {})
    if fp8_weights:
        gu = u8_tensor(c["gate_up_q"], dev).view(torch.float8_e4m3fn)
        dw = u8_tensor(c["down_q"], dev).view(torch.float8_e4m3fn)
        kw["quantization_config"] = QuantizationConfig(f32_tensor(c["gate_up_scale"], dev),
                                                       f32_tensor(c["down_scale"], dev))
    else:
        gu, dw = bf16_tensor(c["gate_up_w"], dev), bf16_tensor(c["down_w"], dev)
    if "gate_up_bias" in c:
        kw["gate_and_up_proj_bias"] = bf16_tensor(c["gate_up_bias"], dev)
        kw["down_proj_bias"] = bf16_tensor(c["down_bias"], dev)
    spec = MoECTESpec(implementation=getattr(MoECTEImplementation, impl),
                      shard_on_I=ShardOnIConfig(checkpoint_activation=True, expert_affinity_multiply_on_I=on_I))
    outs = moe_cte[2](
        bf16_tensor(c["hidden"], dev), bf16_tensor(c["aff"].reshape(-1, 1), dev), gu, dw,
        i32_tensor(c["tp2id"] if tp2id is None else tp2id, dev),
        i32_tensor((c["b2e"] if b2e is None else b2e).reshape(-1, 1), dev), c["B"], spec,
        activation_function=ActFnType(act), skip_dma=SkipMode(c["skip_token"], False),
        expert_affinities_scaling_mode=ExpertAffinityScaleMode(mode), **kw)
    torch.cuda.synchronize()
    return outs


@pytest.mark.parametrize(
    "T,H,I,E,k,B,act,mode,bias,skip,clamp,on_I",
    [
        (300, 512, 384, 4, 2, 128, 0, 1, False, False, False, False),  # ragged last blocks: padding rows are checkpointed too
        (300, 512, 256, 4, 2, 256, 3, 2, True, False, True, False),    # B = 2 tiles, PRE_SCALE, bias and clamps in the checkpoint
        (256, 256, 136, 8, 2, 64, 0, 1, True, True, False, True),      # skip_token, I % 64 != 0, affinity on I: no down checkpoint
    ],
)
def test_dense_checkpoint_activation(T, H, I, E, k, B, act, mode, bias, skip, clamp, on_I):
    """checkpoint_activation (bwmm_shard_on_I.py:160-176): gate_up_activations_T [N, 2, I, B] and down_activations
    [N, B, H] against the golden's (test_moe_cte_common.py:404-405,420-421), every row of every block."""
    c = dense_case(T, H, I, E, k, B, seed=7, skip_token=skip, bias=bias, hidden_std=1.0)
    clamps = dict(gate_clamp_upper_limit=0.8, gate_clamp_lower_limit=-0.7, up_clamp_upper_limit=0.9,
                  up_clamp_lower_limit=-0.5) if clamp else None
    outs = _run_checkpointed(c, "shard_on_i", act, mode, clamps, on_I)
    assert len(outs) == (2 if on_I else 3)
    cl = clamps or {}
    g_out, g_gu, g_d = omoe.moe_blockwise_ref(
        c["hidden"], c["aff"], c["gate_up_w"], c["down_w"], c["tp2id"], c["b2e"], B,
        gate_up_proj_bias=c.get("gate_up_bias"), down_proj_bias=c.get("down_bias"), activation_function=act,
        skip_token=skip, expert_affinities_scaling_mode=mode, checkpoint_activation=True,
        gate_clamp_upper_limit=cl.get("gate_clamp_upper_limit"), gate_clamp_lower_limit=cl.get("gate_clamp_lower_limit"),
        up_clamp_upper_limit=cl.get("up_clamp_upper_limit"), up_clamp_lower_limit=cl.get("up_clamp_lower_limit"))
    o = from_bf16_tensor(outs[0])
    rows = T
    _check(o[:rows], g_out[:rows], "checkpointed output")
    gu = from_bf16_tensor(outs[1])
    assert gu.shape == (c["N"], 2, I, B)
    _check(gu, g_gu, "gate_up_activations_T")
    if not on_I:
        d = from_bf16_tensor(outs[2])
        assert d.shape == (c["N"], B, H)
        _check(d, g_d, "down_activations")


def test_dense_checkpoint_activation_fp8_weights():
    """The checkpoints with fp8 weight-only quantisation (per-channel dequantisation scales,
    bwmm_shard_on_I.py:160-176 with gate_up_proj_scale / down_proj_scale): the checkpointed projections carry the
    scales, as the golden's in-place views do (test_moe_cte_common.py:383-405)."""
    T, H, I, E, k, B = 300, 512, 384, 4, 2, 128
    c = dense_case(T, H, I, E, k, B, seed=9, quant=True, bias=True, hidden_std=1.0)
    outs = _run_checkpointed(c, "shard_on_i", act=0, mode=2, fp8_weights=True)
    g_out, g_gu, g_d = omoe.moe_blockwise_ref(
        c["hidden"], c["aff"], c["gate_up_w"], c["down_w"], c["tp2id"], c["b2e"], B,
        gate_up_proj_bias=c.get("gate_up_bias"), down_proj_bias=c.get("down_bias"),
        gate_up_proj_scale=c["gate_up_scale"], down_proj_scale=c["down_scale"], activation_function=0,
        expert_affinities_scaling_mode=2, checkpoint_activation=True)
    _check(from_bf16_tensor(outs[0])[:T], g_out[:T], "checkpointed output, fp8 weights")
    _check(from_bf16_tensor(outs[1]), g_gu, "gate_up_activations_T, fp8 weights")
    _check(from_bf16_tensor(outs[2]), g_d, "down_activations, fp8 weights")


@pytest.mark.parametrize("mode,on_I", [(2, False), (1, True)])
def test_dropping_variant(mode, on_I):
    """shard_on_i_dropping (bwmm_shard_on_I.py:2014-2159): one block per expert (block b = expert b, block_to_expert
    not read), tokens past an expert's capacity dropped by the caller; always returns the checkpoints."""
    T, H, I, E, k, B = 384, 512, 256, 8, 2, 64
    c = dense_case(T, H, I, E, k, B, seed=9, hidden_std=1.0)
    tp = np.full((E, B), T, dtype=np.int32)
    for e in range(E):
        ids = np.flatnonzero(c["mask"][:, e])[:B]  # capacity B: the rest is dropped
        tp[e, : ids.size] = ids
    assert (c["mask"].sum(0) > B).any(), "the case must actually drop tokens"
    b2e = np.arange(E, dtype=np.int32)
    outs = _run_checkpointed(c, "shard_on_i_dropping", mode=mode, on_I=on_I, tp2id=tp.reshape(-1),
                             b2e=np.zeros(E, np.int32))  # block_to_expert is ignored by this variant
    assert len(outs) == (2 if on_I else 3)
    g_out, g_gu, g_d = omoe.moe_blockwise_ref(c["hidden"], c["aff"], c["gate_up_w"], c["down_w"], tp.reshape(-1), b2e, B,
                                              expert_affinities_scaling_mode=mode, checkpoint_activation=True)
    assert tuple(outs[0].shape) == (T + 1, H)
    _check(from_bf16_tensor(outs[0])[:T], g_out[:T], "dropping output")
    _check(from_bf16_tensor(outs[1]), g_gu, "dropping gate_up_activations_T")
    if not on_I:
        _check(from_bf16_tensor(outs[2]), g_d, "dropping down_activations")


@pytest.mark.parametrize("fp8_row", [False, True])
def test_kmajor_weight_cache(fp8_row):
    """The K-contiguous weight copies kept across calls give the same bits as the copies a call makes for itself,
    and an in-place change of the weights remakes them."""
    import torch
    from nkilib.core.moe.moe_cte import MoECTEImplementation, MoECTESpec, QuantizationConfig, _launch, moe_cte
    from nkilib.core.rmsnorm import RmsNormQuantKernelArgs, rmsnorm_quant_kernel

    dev = torch.device("cuda:0")
    c = dense_case(256, 512, 384, 4, 2, 128, seed=11, quant=fp8_row, hidden_std=1.0)
    kw = {}
    if fp8_row:
        gu = u8_tensor(c["gate_up_q"], dev).view(torch.float8_e4m3fn)
        dw = u8_tensor(c["down_q"], dev).view(torch.float8_e4m3fn)
        kw["quantization_config"] = QuantizationConfig(f32_tensor(c["gate_up_scale"], dev), f32_tensor(c["down_scale"], dev))
        x = rmsnorm_quant_kernel(bf16_tensor(c["hidden"], dev), bf16_tensor(np.ones((1, 512), np.float32), dev),
                                 RmsNormQuantKernelArgs())
    else:
        gu, dw = bf16_tensor(c["gate_up_w"], dev), bf16_tensor(c["down_w"], dev)
        x = bf16_tensor(c["hidden"], dev)
    aff, tp, be = bf16_tensor(c["aff"].reshape(-1, 1), dev), i32_tensor(c["tp2id"], dev), i32_tensor(c["b2e"], dev)

    def run():
        o = moe_cte(x, aff, gu, dw, tp, be, 128, MoECTESpec(implementation=MoECTEImplementation.shard_on_i), **kw)
        torch.cuda.synchronize()
        return o.clone()

    _launch.clear_kmajor_weight_cache()
    try:
        _launch.kmajor_weight_cache = False
        plain = run()
        _launch.kmajor_weight_cache = True
        first, second = run(), run()
        assert len(_launch._kmajor) == 1
        assert torch.equal(first, plain) and torch.equal(second, plain)
        # a fresh view of the same allocations for every call finds the same entry
        kept = _launch._kmajor[next(iter(_launch._kmajor))][3]
        gu0, dw0 = gu, dw
        gu, dw = gu0.view(gu0.dtype)[:], dw0.view(dw0.dtype)[:]
        assert gu is not gu0 and torch.equal(run(), plain)
        assert len(_launch._kmajor) == 1 and _launch._kmajor[next(iter(_launch._kmajor))][3] is kept
        gu, dw = gu0, dw0
        # in-place change of one expert's down weights: the cached copies must not survive it
        if fp8_row:
            dw.view(torch.uint8)[0].bitwise_xor_(0x80)  # flips the sign of every weight of expert 0
        else:
            dw[0].neg_()
        changed = run()
        _launch.kmajor_weight_cache = False
        assert torch.equal(changed, run())
        assert not torch.equal(changed, plain)
    finally:
        _launch.kmajor_weight_cache = True
        _launch.clear_kmajor_weight_cache()


def test_dense_conditions_stop():
    """Hybrid variant: blocks from the first conditions[b] == 0 on are skipped."""
    c = dense_case(256, 512, 256, 8, 2, 128, seed=4, hidden_std=1.0)
    cond = c["cond"].copy()
    cond[3:] = 0  # stop early, in the middle of real blocks
    out = _run_dense(c, impl="shard_on_i_hybrid", conditions=cond)
    _check(from_bf16_tensor(out), _golden_dense(c, conditions=cond), "hybrid conditions")


def test_fp8_weight_only():
    """bf16 activations x fp8 weights with per-channel scales (the reference's own quantised moe_cte)."""
    c = dense_case(256, 512, 256, 4, 2, 128, seed=5, quant=True, hidden_std=1.0)
    out = _run_dense(c, impl="shard_on_i", fp8_weights=True)
    _check(from_bf16_tensor(out), _golden_dense(c, fp8_weights=True), "fp8 weight-only")


def _run_fp8_row(c, gamma, mode=1, clamps=None, act=0, shared_scales=False):
    import torch
    from nkilib.core.moe.moe_cte import QuantizationConfig, moe_cte
    from nkilib.core.rmsnorm import RmsNormQuantKernelArgs, rmsnorm_quant_kernel
    from nkilib.core.utils.common_types import ActFnType, ExpertAffinityScaleMode

    dev = torch.device("cuda:0")
    rec = rmsnorm_quant_kernel(bf16_tensor(c["hidden"], dev), bf16_tensor(gamma, dev), RmsNormQuantKernelArgs())
    kw = dict(clamps or {})
    if "gate_up_bias" in c:
        kw["gate_and_up_proj_bias"] = bf16_tensor(c["gate_up_bias"], dev)
        kw["down_proj_bias"] = bf16_tensor(c["down_bias"], dev)
    gs, ds = c["gate_up_scale"], c["down_scale"]
    if shared_scales:  # one set of channel scales for every expert: leading dimension 1
        gs, ds = gs[:1], ds[:1]
    out = moe_cte(
        rec, bf16_tensor(c["aff"].reshape(-1, 1), dev), u8_tensor(c["gate_up_q"], dev).view(torch.float8_e4m3fn),
        u8_tensor(c["down_q"], dev).view(torch.float8_e4m3fn), i32_tensor(c["tp2id"], dev),
        i32_tensor(c["b2e"], dev), c["B"], _spec("shard_on_block"),
        quantization_config=QuantizationConfig(f32_tensor(gs, dev), f32_tensor(ds, dev)),
        activation_function=ActFnType(act), expert_affinities_scaling_mode=ExpertAffinityScaleMode(mode), **kw)
    torch.cuda.synchronize()
    return rec, out


@pytest.mark.parametrize("T,H,I,E,k,B", [(256, 512, 512, 4, 2, 128), (384, 1024, 896, 8, 2, 128),
                                         (300, 512, 640, 2, 2, 128), (768, 1024, 896, 2, 2, 128),  # 256-row chunk tiles
                                         # shapes outside the large-tile kernels: the general tiled kernel
                                         (256, 512, 448, 4, 2, 128), (300, 768, 512, 4, 2, 128)])
def test_fp8_row_pipeline(T, H, I, E, k, B):
    """RMSNorm-Quant ROW -> fp8 x fp8 blockwise MoE with per-row / per-channel scales (BASELINE config 2 shape family)."""
    import torch

    c = dense_case(T, H, I, E, k, B, seed=6, quant=True, hidden_std=1.0)
    gamma = np.ones((1, H), np.float32)
    rec, out = _run_fp8_row(c, gamma)
    raw = rec.view(torch.uint8).cpu().numpy()
    codes, scale = raw[:, :H], raw[:, H:].copy().view(np.float32).reshape(-1)
    # the oracle consumes the GPU's own records: the front end is checked bit-wise in test_gpu_rmsnorm_quant
    g = omoe.moe_blockwise_fp8_row_ref(codes, scale, c["aff"], c["gate_up_q"], c["down_q"], c["gate_up_scale"],
                                       c["down_scale"], c["tp2id"], c["b2e"], c["B"])
    _check(from_bf16_tensor(out)[:, 0], g, "fp8 row")


@pytest.mark.parametrize("mode,clamp,act,I,shared", [(2, False, 0, 896, False), (1, True, 3, 896, True),
                                                     (2, True, 1, 896, False), (0, False, 0, 896, False),
                                                     (2, True, 3, 448, True)])  # I = 448: the general tiled kernel
def test_fp8_row_scale_modes_and_clamps(mode, clamp, act, I, shared):
    """PRE_SCALE (the affinity scales the token's row, i.e. its dequantisation scale), NO_SCALE and the four clamps on
    the fp8-row kind.  The reference has no kernel with fp8 activations on this path: the rule is the dense
    golden's (test_moe_cte_common.py:383-402) applied to the row-quantised operands."""
    import torch

    T, H, E, k, B = 384, 1024, 8, 2, 128
    c = dense_case(T, H, I, E, k, B, seed=16, quant=True, bias=True, hidden_std=1.0)
    clamps = dict(gate_clamp_upper_limit=0.6, gate_clamp_lower_limit=-0.5, up_clamp_upper_limit=0.7,
                  up_clamp_lower_limit=-0.4) if clamp else {}
    rec, out = _run_fp8_row(c, np.ones((1, H), np.float32), mode=mode, clamps=clamps, act=act, shared_scales=shared)
    raw = rec.view(torch.uint8).cpu().numpy()
    codes, scale = raw[:, :H], raw[:, H:].copy().view(np.float32).reshape(-1)
    gs, ds = c["gate_up_scale"], c["down_scale"]
    if shared:
        gs, ds = np.repeat(gs[:1], E, axis=0), np.repeat(ds[:1], E, axis=0)
    g = omoe.moe_blockwise_fp8_row_ref(codes, scale, c["aff"], c["gate_up_q"], c["down_q"], gs, ds, c["tp2id"],
                                       c["b2e"], c["B"], gate_up_proj_bias=c["gate_up_bias"],
                                       down_proj_bias=c["down_bias"], activation_function=act,
                                       expert_affinities_scaling_mode=mode, **clamps)
    o = from_bf16_tensor(out)[:, 0]
    # (the golden scatters the down bias to the padding token's row as well; the kernels leave that row zero)
    assert not o[T].any()
    _check(o[:T], g[:T], f"fp8 row mode={mode} clamp={clamp} act={act} I={I} shared={shared}")


@pytest.mark.parametrize("T,H,I,E,k,B,fmt", [(512, 1024, 640, 8, 2, 128, "e4m3"), (300, 512, 1024, 2, 2, 256, "e5m2"),
                                             (256, 512, 128, 4, 2, 128, "e4m3"), (512, 1024, 640, 8, 2, 128, "e2m1"),
                                             (300, 512, 1024, 2, 2, 256, "e2m1")])
def test_mx_weight_copies_are_bit_equal(T, H, I, E, k, B, fmt):
    """Copies of the MX weights in the kernels' read order (``_launch.mx_weight_copies``: gate/up for every format, down
    for 4-bit weights): same bits out as from the reference layout, for full and short intermediate tiles and several
    chunks per expert."""
    import torch
    from nkilib.core.moe.moe_cte import _launch

    c = mx_case(T, H, I, E, k, B, seed=51, bias=True, weight_format=fmt, random_codes=True)
    was = _launch.mx_weight_copies
    try:
        _launch.mx_weight_copies = False
        plain = _run_mx_options(c, 3, REF_MX_CLAMPS, False)
        _launch.clear_kmajor_weight_cache()
        _launch.mx_weight_copies = True
        first = _run_mx_options(c, 3, REF_MX_CLAMPS, False)
        assert torch.equal(first, plain)
    finally:
        _launch.mx_weight_copies = was
        _launch.clear_kmajor_weight_cache()
    _check(from_bf16_tensor(plain)[0, :T], _golden_mx_options(c, 3, REF_MX_CLAMPS)[:T], f"mx copies {fmt} I={I}")


def _run_mx(c, prequant=False, act=0, weight_dtype=None):
    import torch
    from nkilib.core.moe.moe_cte import QuantizationConfig, SkipMode, moe_cte
    from nkilib.core.subkernels.rmsnorm_mx_quantize_tkg import rmsnorm_mx_quantize
    from nkilib.core.utils.common_types import ActFnType

    dev = torch.device("cuda:0")
    kw = {}
    if "gate_up_bias" in c:
        kw["gate_and_up_proj_bias"] = bf16_tensor(c["gate_up_bias"], dev)
        kw["down_proj_bias"] = bf16_tensor(c["down_bias"], dev)
    if c["cond"] is not None:
        kw["conditions"] = i32_tensor(c["cond"], dev)
    hs = bf16_tensor(c["hidden"], dev)
    if prequant:
        q, s = rmsnorm_mx_quantize(hs, None, do_norm=False)
        hs = q
        kw["hidden_states_scale"] = s
    gu = torch.from_numpy(c["gate_up_q"].view(np.int32).reshape(c["gate_up_q"].shape[:-1])).to(dev)  # x4 container
    out = moe_cte[2](
        hs, bf16_tensor(c["aff"].reshape(-1, 1), dev), gu, u8_tensor(c["down_q"], dev),
        i32_tensor(c["tp2id"], dev), i32_tensor(c["b2e"], dev), c["B"], _spec("shard_on_block_mx"),
        quantization_config=QuantizationConfig(u8_tensor(c["gate_up_s"], dev), u8_tensor(c["down_s"], dev)),
        activation_function=ActFnType(act), skip_dma=SkipMode(c["skip_token"], False), **kw)
    torch.cuda.synchronize()
    return out


def _run_mx_direct(c, weight_dtype):
    """bwmm_shard_on_block_mx with an explicit weight_dtype for uint containers (the reference's use_uint_weights cases)."""
    import torch
    from nkilib.core.moe.moe_cte.bwmm_shard_on_block_mx import bwmm_shard_on_block_mx
    from nkilib.core.moe.moe_cte import SkipMode

    dev = torch.device("cuda:0")
    kw = {}
    if "gate_up_bias" in c:
        kw["gate_and_up_proj_bias"] = bf16_tensor(c["gate_up_bias"], dev)
        kw["down_proj_bias"] = bf16_tensor(c["down_bias"], dev)
    if c.get("weight_format") == "e2m1":  # one 4-bit pattern per byte in the case; 2-byte x4 elements on the device
        from oracle.numerics import pack_e2m1_x4
        gu = torch.from_numpy(pack_e2m1_x4(c["gate_up_q"]).view(np.int16)).to(dev)
        dw = torch.from_numpy(pack_e2m1_x4(c["down_q"]).view(np.int16)).to(dev)
    else:
        gu = torch.from_numpy(c["gate_up_q"].view(np.int32).reshape(c["gate_up_q"].shape[:-1])).to(dev)
        dw = torch.from_numpy(c["down_q"].view(np.int32).reshape(c["down_q"].shape[:-1])).to(dev)
    out = bwmm_shard_on_block_mx[2](
        bf16_tensor(c["hidden"], dev), bf16_tensor(c["aff"].reshape(-1, 1), dev), gu, dw,
        i32_tensor(c["tp2id"], dev), i32_tensor(c["b2e"], dev), gate_up_proj_scale=u8_tensor(c["gate_up_s"], dev),
        down_proj_scale=u8_tensor(c["down_s"], dev), block_size=c["B"], skip_dma=SkipMode(c["skip_token"], False),
        weight_dtype=weight_dtype, **kw)
    torch.cuda.synchronize()
    return out


def _golden_mx(c, act=0):
    return omoe.moe_blockwise_mx_ref(
        c["hidden"], c["aff"], c["gate_up_q"], c["down_q"], c["gate_up_s"], c["down_s"], c["tp2id"], c["b2e"], c["B"],
        conditions=c["cond"], gate_up_proj_bias=c.get("gate_up_bias"), down_proj_bias=c.get("down_bias"),
        activation_function=act, skip_token=c["skip_token"], weight_format=c.get("weight_format", "e4m3"))


@pytest.mark.parametrize(
    "T,H,I,E,k,B,bias,skip,dynamic,alpha,prequant",
    [
        (256, 512, 512, 8, 2, 128, False, False, False, None, False),
        (256, 1024, 1024, 8, 4, 128, True, False, False, None, False),
        (512, 2048, 768, 16, 8, 128, False, False, True, 0.3, True),    # Qwen3-MoE-like tail tile (I=768), skewed, dynamic
        (200, 512, 256, 4, 2, 128, False, True, False, None, False),   # I < 512, skip_token
        (256, 512, 96, 4, 2, 256, True, False, False, None, True),     # tiny I, B=256
        (300, 512, 256, 2, 2, 128, True, False, False, None, False),   # 300 rows per expert: one 320-row chunk each
        (330, 1024, 384, 2, 2, 128, False, False, False, None, False), # 330 rows per expert: chunks of 256 + 74
        (280, 512, 128, 2, 2, 128, True, False, False, None, False),    # one K slice in the down stage (fewer than the lookahead)
    ],
)
def test_mx_variants(T, H, I, E, k, B, bias, skip, dynamic, alpha, prequant):
    c = mx_case(T, H, I, E, k, B, seed=7, skip_token=skip, bias=bias, alpha=alpha, dynamic=dynamic)
    dirty_device_memory(2 * (T + 1) * H * 2)
    out = _run_mx(c, prequant=prequant)
    o = from_bf16_tensor(out)
    assert o.shape[0] == 2 and not o[1].any()
    g = _golden_mx(c)
    if not skip:
        assert not o[0, T].any()
        _check(o[0, :T], g[:T], f"mx H={H} I={I} E={E}")
    else:
        _check(o[0], g, f"mx H={H} I={I} E={E}")


@pytest.mark.parametrize("T,H,I,E,k,B,bias", [(256, 512, 512, 8, 2, 128, False), (300, 1024, 384, 2, 2, 128, True)])
def test_mx_e5m2_weights(T, H, I, E, k, B, bias):
    """MXFP8 weights in e5m2 (nl.float8_e5m2_x4; test_moe_bwmm_mx_cte.py:74-76, :80): uint32 containers + weight_dtype."""
    c = mx_case(T, H, I, E, k, B, seed=11, bias=bias, weight_format="e5m2")
    o = from_bf16_tensor(_run_mx_direct(c, "float8_e5m2_x4"))
    g = _golden_mx(c)
    _check(o[0, :T], g[:T], f"mx e5m2 H={H} I={I} E={E}")
    # the same bytes read as e4m3 give a different answer: the format switch is what the result depends on
    o4 = from_bf16_tensor(_run_mx_direct(c, "float8_e4m3fn_x4"))
    assert max_abs_rel(o4[0, :T], g[:T]) > 0.1


@pytest.mark.parametrize("T,H,I,E,k,B,bias,wd", [
    (256, 512, 512, 8, 2, 128, False, "float4_e2m1fn_x4"),
    (300, 1024, 384, 2, 2, 128, True, None),           # 300-row chunks; format inferred from the 2-byte elements
    (512, 2048, 768, 16, 4, 256, True, "float4_e2m1fn_x4"),
])
def test_mx_fp4_weights(T, H, I, E, k, B, bias, wd):
    """MXFP4 weights (nl.float4_e2m1fn_x4, the first ten cases of test_moe_bwmm_mx_cte.py:60-70): 2-byte x4 elements,
    E8M0 scales as for MXFP8, activations and intermediate in MXFP8 e4m3."""
    c = mx_case(T, H, I, E, k, B, seed=12, bias=bias, weight_format="e2m1", weight_std=0.5)
    o = from_bf16_tensor(_run_mx_direct(c, wd))
    g = _golden_mx(c)
    _check(o[0, :T], g[:T], f"mx fp4 H={H} I={I} E={E}")


def _run_mx_options(c, act, clamps, uint_containers, prequant=False):
    """bwmm_shard_on_block_mx with every option of the reference's MX table: activation, clamps, bias, conditions,
    skip_token, and the weights either in typed containers (1-byte float8 elements with a trailing axis of 4, or
    2-byte elements for MXFP4: the format is read off the tensor) or in the uint32 / uint16 containers of
    convert_mx_weights_to_uint_dtype (test_moe_bwmm_mx_cte.py:113-133) with the format in ``weight_dtype``."""
    import torch
    from nkilib.core.moe.moe_cte import SkipMode
    from nkilib.core.moe.moe_cte.bwmm_shard_on_block_mx import bwmm_shard_on_block_mx
    from nkilib.core.subkernels.rmsnorm_mx_quantize_tkg import rmsnorm_mx_quantize
    from nkilib.core.utils.common_types import ActFnType

    dev = torch.device("cuda:0")
    fmt = c["weight_format"]
    kw = dict(clamps or {})
    if "gate_up_bias" in c:
        kw["gate_and_up_proj_bias"] = bf16_tensor(c["gate_up_bias"], dev)
        kw["down_proj_bias"] = bf16_tensor(c["down_bias"], dev)
    if c["cond"] is not None:
        kw["conditions"] = i32_tensor(c["cond"], dev)
    if fmt == "e2m1":
        from oracle.numerics import pack_e2m1_x4
        gu = torch.from_numpy(pack_e2m1_x4(c["gate_up_q"]).view(np.int16)).to(dev)
        dw = torch.from_numpy(pack_e2m1_x4(c["down_q"]).view(np.int16)).to(dev)
        if uint_containers:
            gu, dw = gu.view(torch.uint16), dw.view(torch.uint16)
            kw["weight_dtype"] = "float4_e2m1fn_x4"
    elif uint_containers:
        gu = torch.from_numpy(c["gate_up_q"].view(np.uint32).reshape(c["gate_up_q"].shape[:-1])).to(dev)
        dw = torch.from_numpy(c["down_q"].view(np.uint32).reshape(c["down_q"].shape[:-1])).to(dev)
        kw["weight_dtype"] = "float8_e5m2_x4" if fmt == "e5m2" else "float8_e4m3fn_x4"
    else:
        tdt = torch.float8_e5m2 if fmt == "e5m2" else torch.float8_e4m3fn
        gu, dw = u8_tensor(c["gate_up_q"], dev).view(tdt), u8_tensor(c["down_q"], dev).view(tdt)
    hs = bf16_tensor(c["hidden"], dev)
    if prequant:
        hs, kw["hidden_states_scale"] = rmsnorm_mx_quantize(hs, None, do_norm=False)
    out = bwmm_shard_on_block_mx[2](
        hs, bf16_tensor(c["aff"].reshape(-1, 1), dev), gu, dw, i32_tensor(c["tp2id"], dev),
        i32_tensor(c["b2e"], dev), gate_up_proj_scale=u8_tensor(c["gate_up_s"], dev),
        down_proj_scale=u8_tensor(c["down_s"], dev), block_size=c["B"], activation_function=ActFnType(act),
        skip_dma=SkipMode(c["skip_token"], False), **kw)
    torch.cuda.synchronize()
    return out


def _golden_mx_options(c, act, clamps):
    cl = clamps or {}
    return omoe.moe_blockwise_mx_ref(
        c["hidden"], c["aff"], c["gate_up_q"], c["down_q"], c["gate_up_s"], c["down_s"], c["tp2id"], c["b2e"], c["B"],
        conditions=c["cond"], gate_up_proj_bias=c.get("gate_up_bias"), down_proj_bias=c.get("down_bias"),
        activation_function=act, skip_token=c["skip_token"], weight_format=c["weight_format"],
        gate_clamp_upper_limit=cl.get("gate_clamp_upper_limit"), gate_clamp_lower_limit=cl.get("gate_clamp_lower_limit"),
        up_clamp_upper_limit=cl.get("up_clamp_upper_limit"), up_clamp_lower_limit=cl.get("up_clamp_lower_limit"))


# The reference's own clamp set for every row of its MX tables (test_moe_bwmm_mx_cte.py:59-106).
REF_MX_CLAMPS = dict(gate_clamp_upper_limit=7.0, up_clamp_upper_limit=7.0, up_clamp_lower_limit=-7.0)


@pytest.mark.parametrize(
    "H,T,I,E,B,k,act,fmt,skip,dynamic,uint",
    [
        # a covering selection of moe_bwmm_mx_cte_unit_perms (test_moe_bwmm_mx_cte.py:59-86) at the table's own small
        # token count: H=3072, (I, E) in {(384, 128), (1536, 32)}, top-4 (top-2 in the uint-container rows), B in
        # {256, 512}, Swish, bias, skip_token 0/1, static / dynamic conditions, MXFP4 / e4m3 / e5m2 weights
        (3072, 1024, 384, 128, 256, 4, 3, "e2m1", True, False, False),
        (3072, 1024, 384, 128, 512, 4, 3, "e4m3", False, True, False),
        (3072, 1024, 384, 128, 256, 2, 3, "e5m2", True, False, True),
        (3072, 1024, 1536, 32, 256, 4, 3, "e2m1", False, True, True),
        (3072, 1024, 1536, 32, 512, 4, 3, "e4m3", True, False, True),
        (3072, 1024, 1536, 32, 512, 4, 3, "e5m2", False, False, False),
        (3072, 1024, 384, 128, 512, 4, 3, "e2m1", True, True, False),
        (3072, 1024, 384, 128, 256, 4, 3, "e4m3", True, False, False),
        (3072, 1024, 1536, 32, 256, 4, 3, "e5m2", True, True, False),
        # the n_static_blocks rows (:83-85): few experts, so every expert holds several 256-row chunks
        (4096, 1024, 1536, 2, 256, 2, 0, "e4m3", True, True, False),
        (4096, 1024, 1024, 4, 256, 4, 0, "e4m3", True, True, False),
        (3072, 1024, 384, 2, 256, 2, 0, "e4m3", True, True, False),
    ],
)
def test_mx_reference_table(H, T, I, E, B, k, act, fmt, skip, dynamic, uint):
    """The large-tile MX kernels on the reference's own shard-on-block MX configurations: clamps 7 / +-7, bias, Swish
    (SiLU in the n_static_blocks rows), B = 256 / 512."""
    c = mx_case(T, H, I, E, k, B, seed=21, skip_token=skip, bias=True, dynamic=dynamic, weight_format=fmt,
                random_codes=True)
    out = _run_mx_options(c, act, REF_MX_CLAMPS, uint)
    o = from_bf16_tensor(out)
    assert o.shape[0] == 2 and not o[1].any()
    g = _golden_mx_options(c, act, REF_MX_CLAMPS)
    rows = T  # row T (the padding token, absent with skip_token) stays zero here; the golden scatters the bias to it
    if not skip:
        assert not o[0, T].any()
    _check(o[0, :rows], g[:rows], f"mx table H={H} I={I} E={E} B={B} {fmt}")


@pytest.mark.parametrize("fmt", ["e5m2", "e2m1"])
@pytest.mark.parametrize("I,B,uint", [(96, 128, False), (544, 256, True), (160, 128, True), (1056, 128, False)])
def test_mx_weight_formats_outside_the_large_tile_shapes(fmt, I, B, uint):
    """e5m2 and MXFP4 weights where I is not a multiple of 128 (the reference takes any I % 16 == 0 whose tail past a
    multiple of 512 is a multiple of 32, bwmm_shard_on_block_mx.py:620-633): the general tiled kernel, with the
    reference table's options (Swish, bias, clamps)."""
    T, H, E, k = 256, 1024, 8, 2
    c = mx_case(T, H, I, E, k, B, seed=41, bias=True, weight_format=fmt, random_codes=True)
    out = _run_mx_options(c, 3, REF_MX_CLAMPS, uint)
    o = from_bf16_tensor(out)
    assert o.shape[0] == 2 and not o[1].any() and not o[0, T].any()
    _check(o[0, :T], _golden_mx_options(c, 3, REF_MX_CLAMPS)[:T], f"mx general kernel I={I} B={B} {fmt}")


@pytest.mark.parametrize("I", [512, 96, 544])  # large-tile kernels; general tiled kernel (I % 128 != 0), with a tail tile
@pytest.mark.parametrize(
    "act,clamps",
    [
        (0, None), (1, None), (2, None), (3, None),
        (3, dict(gate_clamp_upper_limit=0.6)),
        (3, dict(gate_clamp_lower_limit=-0.4)),
        (3, dict(up_clamp_upper_limit=0.5)),
        (3, dict(up_clamp_lower_limit=-0.3)),
        (1, dict(gate_clamp_upper_limit=0.6, gate_clamp_lower_limit=-0.4, up_clamp_upper_limit=0.5, up_clamp_lower_limit=-0.3)),
    ],
)
def test_mx_activation_and_clamp_options(I, act, clamps):
    """Every ActFnType and every clamp limit on its own (limits small enough to cut a large share of the values)
    through both MX code paths, with bias."""
    T, H, E, k, B = 256, 512, 8, 2, 128
    c = mx_case(T, H, I, E, k, B, seed=31, bias=True, weight_std=0.05)
    out = _run_mx_options(c, act, clamps, uint_containers=False, prequant=(act == 2))
    o = from_bf16_tensor(out)
    g = _golden_mx_options(c, act, clamps)
    assert not o[0, T].any()
    _check(o[0, :T], g[:T], f"mx I={I} act={act} clamps={sorted((clamps or {}).keys())}")
    if clamps and len(clamps) == 1:
        # the limit must matter: without it the result is measurably different
        assert max_abs_rel(_golden_mx_options(c, act, None)[:T], g[:T]) > 2 * RTOL


@pytest.mark.parametrize(
    "H,T,I,E,B,k,fmt,dynamic,uint,via_moe_cte",
    [
        # the small-token rows of moe_bwmm_mx_shard_I_unit_perms (test_moe_bwmm_mx_cte.py:92-108): Swish, bias, clamps,
        # skip_token, top-4 / top-8 over 8 experts with B = 256
        (3072, 1024, 2048, 8, 256, 4, "e2m1", False, False, False),
        (3072, 1024, 2048, 8, 256, 4, "e2m1", True, False, True),
        (7168, 1024, 1024, 8, 256, 8, "e4m3", False, False, True),
        (7168, 1024, 1024, 8, 256, 8, "e4m3", True, False, False),
        (3072, 1024, 2048, 8, 256, 8, "e5m2", True, True, False),
    ],
)
def test_mx_shard_on_i_entry_points(H, T, I, E, B, k, fmt, dynamic, uint, via_moe_cte):
    """blockwise_mm_shard_intermediate_mx / _hybrid (bwmm_shard_on_I_mx.py:95-117, :400-426): the shard-on-block MX
    golden, result in the shape of hidden_states, conditions with one entry per block plus one."""
    import torch
    from nkilib.core.moe.moe_cte import MoECTEImplementation, MoECTESpec, QuantizationConfig, SkipMode, moe_cte
    from nkilib.core.moe.moe_cte.bwmm_shard_on_I_mx import (blockwise_mm_shard_intermediate_mx,
                                                            blockwise_mm_shard_intermediate_mx_hybrid)
    from nkilib.core.utils.common_types import ActFnType, ExpertAffinityScaleMode

    dev = torch.device("cuda:0")
    rng = np.random.default_rng(41)
    N, mask, tp2id, b2e, cond = routing(T, k, E, B, skip_token=True)  # not block parallel: conditions has N + 1 entries
    assert cond.size == N + 1
    hs = to_bf16(rng.standard_normal((T, H)).astype(np.float32))
    gu_q, gu_s, d_q, d_s = mx_weights_random_codes(rng, E, H, I, fmt)
    nI = I // 512
    gub = to_bf16(rng.uniform(-2.0625, 0.52, size=(E, 128, 2, nI, 4)).astype(np.float32))
    db = to_bf16(rng.uniform(-1.632, 1.4375, size=(E, H)).astype(np.float32))
    aff = affinities(rng, T, E, mask, True)
    if fmt == "e2m1":
        from oracle.numerics import pack_e2m1_x4
        gu = torch.from_numpy(pack_e2m1_x4(gu_q).view(np.int16)).to(dev)
        dw = torch.from_numpy(pack_e2m1_x4(d_q).view(np.int16)).to(dev)
        wd = None
    elif uint:
        gu = torch.from_numpy(gu_q.view(np.uint32).reshape(gu_q.shape[:-1])).to(dev)
        dw = torch.from_numpy(d_q.view(np.uint32).reshape(d_q.shape[:-1])).to(dev)
        wd = "float8_e5m2_x4" if fmt == "e5m2" else "float8_e4m3fn_x4"
    else:
        tdt = torch.float8_e5m2 if fmt == "e5m2" else torch.float8_e4m3fn
        gu, dw, wd = u8_tensor(gu_q, dev).view(tdt), u8_tensor(d_q, dev).view(tdt), None
    common = dict(gate_and_up_proj_bias=bf16_tensor(gub, dev), down_proj_bias=bf16_tensor(db, dev),
                  activation_function=ActFnType.Swish, skip_dma=SkipMode(True, False),
                  expert_affinities_scaling_mode=ExpertAffinityScaleMode.POST_SCALE, **REF_MX_CLAMPS)
    args = (bf16_tensor(hs, dev), bf16_tensor(aff.reshape(-1, 1), dev), gu, dw, i32_tensor(tp2id, dev),
            i32_tensor(b2e, dev))
    scales = (u8_tensor(gu_s, dev), u8_tensor(d_s, dev))
    if via_moe_cte:
        assert wd is None
        impl = MoECTEImplementation.shard_on_i_mx_hybrid if dynamic else MoECTEImplementation.shard_on_i_mx
        out = moe_cte[2](*args, B, MoECTESpec(implementation=impl), conditions=i32_tensor(cond, dev) if dynamic else None,
                         quantization_config=QuantizationConfig(*scales), **common)
    elif dynamic:
        out = blockwise_mm_shard_intermediate_mx_hybrid[2](i32_tensor(cond, dev), *args, gate_up_proj_scale=scales[0],
                                                           down_proj_scale=scales[1], block_size=B, weight_dtype=wd,
                                                           **common)
    else:
        out = blockwise_mm_shard_intermediate_mx[2](*args, gate_up_proj_scale=scales[0], down_proj_scale=scales[1],
                                                    block_size=B, weight_dtype=wd, **common)
    torch.cuda.synchronize()
    assert tuple(out.shape) == (T, H)
    g = omoe.moe_blockwise_mx_ref(hs, aff, gu_q, d_q, gu_s, d_s, tp2id, b2e, B, conditions=cond if dynamic else None,
                                  gate_up_proj_bias=gub, down_proj_bias=db, activation_function=3, skip_token=True,
                                  weight_format=fmt, **REF_MX_CLAMPS)
    _check(from_bf16_tensor(out), g, f"mx shard-on-I H={H} I={I} {fmt}")


def test_mx_prequantised_equals_online():
    """Quantise-then-gather == gather-then-quantise: MX blocks never span tokens, so both entry forms agree bit-wise."""
    c = mx_case(256, 1024, 512, 8, 2, 128, seed=8)
    a = from_bf16_tensor(_run_mx(c, prequant=False))
    b = from_bf16_tensor(_run_mx(c, prequant=True))
    assert np.array_equal(a, b)


@pytest.mark.parametrize("kind", ["bf16", "fp8_weights", "mx"])
def test_plain_gate_up_epilogue_equals_the_general_one(kind):
    """A SiLU layer without bias and clamps runs a form of the large-tile gate/up epilogue that leaves their adds and
    medians out; with biases of zero, or clamps that no value reaches, the same layer takes the general form.  All
    three must give the same rows (the reference applies bias and clamps only where given:
    test/integration/nkilib/core/moe/moe_cte/test_utils.py:474-735)."""
    import math

    big = {"gate_clamp_upper_limit": 1e30, "gate_clamp_lower_limit": -1e30, "up_clamp_upper_limit": 1e30,
           "up_clamp_lower_limit": -1e30}
    if kind == "mx":
        T, H, I, E, k, B = 300, 1024, 640, 4, 2, 128
        c = mx_case(T, H, I, E, k, B, seed=61)
        plain = from_bf16_tensor(_run_mx(c))
        nI, pI = math.ceil(I / 512), 128
        z = dict(c)
        z["gate_up_bias"] = to_bf16(np.zeros((E, pI, 2, nI, 4), np.float32))
        z["down_bias"] = to_bf16(np.zeros((E, H), np.float32))
        with_zero_bias = from_bf16_tensor(_run_mx(z))
        with_far_clamps = from_bf16_tensor(_run_mx_options(c, 0, big, False))
    else:
        T, H, I, E, k, B = 300, 1024, 640, 4, 2, 128
        fp8 = kind == "fp8_weights"
        c = dense_case(T, H, I, E, k, B, seed=62, quant=fp8, hidden_std=1.0)
        plain = from_bf16_tensor(_run_dense(c, fp8_weights=fp8))
        z = dict(c)
        z["gate_up_bias"] = to_bf16(np.zeros((E, 2, I), np.float32))
        z["down_bias"] = to_bf16(np.zeros((E, H), np.float32))
        with_zero_bias = from_bf16_tensor(_run_dense(z, fp8_weights=fp8))
        with_far_clamps = from_bf16_tensor(_run_dense(c, clamps=big, fp8_weights=fp8))
    assert np.abs(plain).max() > 0
    # (a padding token's row is zero in all of them; -0 and +0 compare equal)
    np.testing.assert_array_equal(plain, with_zero_bias)
    np.testing.assert_array_equal(plain, with_far_clamps)


def test_smoke_entry():
    import __graft_entry__ as ge

    ge.smoke()


@pytest.mark.parametrize("T,lo,hi", [(62000, 1900, 2048), (68000, 2049, 4096), (134000, 4097, 5000)])
def test_many_chunks_queue_paths(T, lo, hi):
    """The work-queue builder keeps the chunk list in LDS up to 2048 chunks and the chunks' sort keys up to 4096
    (beyond that the chunk-interleaved item order, which needs the keys, is switched off): one call on either side of
    both limits, on a small expert shape of the large-tile bf16 kernels (64 experts of about 1000 / 1060 / 2100
    rows each, i.e. several chunks per expert, the interleaved order where it applies), against the golden."""
    H, I, E, k, B = 256, 128, 64, 8, 128
    c = dense_case(T, H, I, E, k, B, seed=21)
    rows = c["mask"].sum(axis=0).astype(np.int64)
    n_chunks = int(sum(0 if r == 0 else 1 if r <= 320 else -(-(r - 320) // 256) + 1 for r in rows))
    assert lo <= n_chunks <= hi, f"T={T}: {n_chunks} chunks, meant to lie in [{lo}, {hi}]"
    out = from_bf16_tensor(_run_dense(c))
    assert not out[:, 1].any()
    g = _golden_dense(c)
    _check(out[:T, 0], g[:T], f"{n_chunks} chunks (T={T})")
