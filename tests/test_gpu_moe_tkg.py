"""GPU parity: moe_tkg (token-generation MoE) through the C ABI against the restatement of moe_tkg_torch_ref
(src/nkilib_src/nkilib/core/moe/moe_tkg/moe_tkg_torch.py).  Tolerance: max-abs-rel 2e-2 on the bf16 output (the
reference's own tests use rtol 2e-2 for bf16 and 5e-2 for MX)."""

import numpy as np
import pytest

from helpers import bf16_tensor, dense_case, f32_tensor, from_bf16_tensor, i32_tensor, mx_case, u8_tensor
from oracle import moe as omoe
from oracle.compare import max_abs_rel, max_all_close

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-2, 1e-5


def _topk(mask, k, rng):
    """The token's experts in a shuffled order: the order expert_index lists them in is the golden's summation order."""
    return np.stack([rng.permutation(np.flatnonzero(r)[:k]) for r in mask]).astype(np.int32)


def _check(actual, golden, what):
    err = max_abs_rel(actual, golden)
    print(f"{what}: max-abs-rel {err:.3e}", flush=True)
    assert max_all_close(actual, golden, rtol=RTOL, atol=ATOL), f"{what}: max-abs-rel {err:.3e} > {RTOL}"


@pytest.mark.parametrize("T,H,I,E,K,mode,bias,act", [
    (8, 512, 256, 16, 4, 1, True, 0),     # POST_SCALE, bias
    (1, 512, 256, 16, 4, 1, False, 0),    # a single token
    (128, 256, 128, 8, 2, 0, False, 3),   # NO_SCALE, Swish, the reference's largest selective T
    (300, 256, 128, 8, 2, 1, False, 0),   # beyond the reference's selective limit
])
def test_tkg_selective_dense(T, H, I, E, K, mode, bias, act):
    import torch
    from nkilib.core.moe.moe_tkg import moe_tkg
    from nkilib.core.utils.common_types import ActFnType, ExpertAffinityScaleMode

    c = dense_case(T, H, I, E, K, 128, seed=21, skip_token=True, bias=bias, hidden_std=1.0)
    idx = _topk(c["mask"], K, np.random.default_rng(1))
    dev = torch.device("cuda:0")
    kw = {}
    if bias:
        kw = dict(expert_gate_up_bias=bf16_tensor(c["gate_up_bias"], dev), expert_down_bias=bf16_tensor(c["down_bias"], dev))
    out = moe_tkg[2](bf16_tensor(c["hidden"], dev), bf16_tensor(c["gate_up_w"], dev), bf16_tensor(c["down_w"][:, :I], dev),
                     bf16_tensor(c["aff"], dev), i32_tensor(idx, dev), False,
                     expert_affinities_scaling_mode=ExpertAffinityScaleMode(mode), activation_fn=ActFnType(act), **kw)
    torch.cuda.synchronize()
    assert tuple(out.shape) == (T, H) and out.dtype == torch.bfloat16
    g = omoe.moe_tkg_ref(c["hidden"], c["gate_up_w"], c["down_w"][:, :I], c["aff"], idx, False, c.get("gate_up_bias"),
                         c.get("down_bias"), expert_affinities_scaling_mode=mode, activation_function=act)
    _check(from_bf16_tensor(out), g, f"tkg selective T={T} mode={mode}")


def test_tkg_selective_eager_affinities_and_output_dtype():
    import torch
    from nkilib.core.moe.moe_tkg import moe_tkg
    from nkilib.core.utils.common_types import ExpertAffinityScaleMode

    T, H, I, E, K = 16, 256, 128, 8, 2
    c = dense_case(T, H, I, E, K, 128, seed=22, skip_token=True, hidden_std=1.0)
    idx = _topk(c["mask"], K, np.random.default_rng(2))
    eager = np.take_along_axis(c["aff"], idx.astype(np.int64), axis=1)
    dev = torch.device("cuda:0")
    out = moe_tkg(bf16_tensor(c["hidden"], dev), bf16_tensor(c["gate_up_w"], dev), bf16_tensor(c["down_w"][:, :I], dev),
                  None, i32_tensor(idx, dev), False, expert_affinities_eager=bf16_tensor(eager, dev),
                  expert_affinities_scaling_mode=ExpertAffinityScaleMode.POST_SCALE, output_dtype=torch.float32)
    assert out.dtype == torch.float32
    g = omoe.moe_tkg_ref(c["hidden"], c["gate_up_w"], c["down_w"][:, :I], c["aff"], idx, False,
                         expert_affinities_scaling_mode=omoe.POST_SCALE)
    _check(out.cpu().numpy(), g, "tkg eager affinities")


@pytest.mark.parametrize("T,mask_unselected,mode", [(8, True, 1), (130, False, 1), (8, False, 0)])
def test_tkg_all_expert_dense(T, mask_unselected, mode):
    """All-expert mode on the local experts of rank 1 of 2: affinity columns [E_L, 2 E_L) of the global table,
    optionally masked to the experts expert_index lists (moe_tkg_affinity_masking.py:30-110)."""
    import torch
    from nkilib.core.moe.moe_tkg import moe_tkg
    from nkilib.core.utils.common_types import ExpertAffinityScaleMode

    H, I, E_L, K, rank = 256, 128, 4, 2, 1
    E = 2 * E_L
    rng = np.random.default_rng(23)
    c = dense_case(T, H, I, E_L, K, 128, seed=23, skip_token=True, hidden_std=1.0)
    aff = omoe.to_bf16(rng.uniform(0.05, 1.0, (T, E)).astype(np.float32))
    idx = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)  # global expert ids
    local = aff[:, rank * E_L:(rank + 1) * E_L].copy()
    if mask_unselected:
        chosen = np.zeros((T, E), bool)
        np.put_along_axis(chosen, idx.astype(np.int64), True, axis=1)
        local = np.where(chosen[:, rank * E_L:(rank + 1) * E_L], local, 0).astype(np.float32)
    dev = torch.device("cuda:0")
    out = moe_tkg(bf16_tensor(c["hidden"], dev), bf16_tensor(c["gate_up_w"], dev), bf16_tensor(c["down_w"][:, :I], dev),
                  bf16_tensor(aff, dev), i32_tensor(idx, dev), True,
                  rank_id=torch.tensor([[rank]], dtype=torch.int32, device=dev),
                  mask_unselected_experts=mask_unselected, expert_affinities_scaling_mode=ExpertAffinityScaleMode(mode))
    torch.cuda.synchronize()
    g = omoe.moe_tkg_ref(c["hidden"], c["gate_up_w"], c["down_w"][:, :I], local if mode else np.ones_like(local), idx,
                         True, expert_affinities_scaling_mode=mode)
    _check(from_bf16_tensor(out), g, f"tkg all-expert T={T} mask={mask_unselected} mode={mode}")


def test_tkg_fp8_row_weights():
    """fp8 weights with row scales [E, 2, I] / [E, H] (QuantizationType.ROW, moe_tkg.py:300-313)."""
    import torch
    from nkilib.core.moe.moe_tkg import moe_tkg
    from nkilib.core.utils.common_types import ExpertAffinityScaleMode

    T, H, I, E, K = 8, 512, 256, 4, 2
    c = dense_case(T, H, I, E, K, 128, seed=24, skip_token=True, quant=True, hidden_std=1.0)
    idx = _topk(c["mask"], K, np.random.default_rng(4))
    dev = torch.device("cuda:0")
    gs, ds = c["gate_up_scale"].reshape(E, 2, I), c["down_scale"].reshape(E, H)
    out = moe_tkg(bf16_tensor(c["hidden"], dev), u8_tensor(c["gate_up_q"], dev).view(torch.float8_e4m3fn),
                  u8_tensor(c["down_q"][:, :I], dev).view(torch.float8_e4m3fn), bf16_tensor(c["aff"], dev),
                  i32_tensor(idx, dev), False, expert_gate_up_weights_scale=f32_tensor(gs, dev),
                  expert_down_weights_scale=f32_tensor(ds, dev),
                  expert_affinities_scaling_mode=ExpertAffinityScaleMode.POST_SCALE)
    g = omoe.moe_tkg_ref(c["hidden"], c["gate_up_w"], c["down_w"][:, :I], c["aff"], idx, False,
                         expert_gate_up_weights_scale=gs, expert_down_weights_scale=ds,
                         expert_affinities_scaling_mode=omoe.POST_SCALE)
    _check(from_bf16_tensor(out), g, "tkg fp8 row weights")


@pytest.mark.parametrize("T,H,I,E,K,all_expert,bias", [(8, 512, 512, 8, 2, False, True), (1, 1024, 256, 8, 4, False, False),
                                                       (40, 512, 512, 4, 2, True, False)])
def test_tkg_mx(T, H, I, E, K, all_expert, bias):
    import torch
    from nkilib.core.moe.moe_tkg import moe_tkg
    from nkilib.core.utils.common_types import ExpertAffinityScaleMode

    c = mx_case(T, H, I, E, K, 128, seed=25, skip_token=True, bias=bias, hidden_std=1.0)
    rng = np.random.default_rng(5)
    idx = _topk(c["mask"], K, rng)
    aff = c["aff"] if not all_expert else omoe.to_bf16(rng.uniform(0.05, 1.0, (T, E)).astype(np.float32))
    dev = torch.device("cuda:0")
    kw = {}
    if bias:
        kw = dict(expert_gate_up_bias=bf16_tensor(c["gate_up_bias"], dev), expert_down_bias=bf16_tensor(c["down_bias"], dev))
    out = moe_tkg(bf16_tensor(c["hidden"], dev), u8_tensor(c["gate_up_q"], dev), u8_tensor(c["down_q"], dev),
                  bf16_tensor(aff, dev), i32_tensor(idx, dev), all_expert,
                  rank_id=torch.zeros((1, 1), dtype=torch.int32, device=dev) if all_expert else None,
                  expert_gate_up_weights_scale=u8_tensor(c["gate_up_s"], dev),
                  expert_down_weights_scale=u8_tensor(c["down_s"], dev),
                  expert_affinities_scaling_mode=ExpertAffinityScaleMode.POST_SCALE, **kw)
    torch.cuda.synchronize()
    g = omoe.moe_tkg_mx_ref(c["hidden"], c["gate_up_q"], c["down_q"], c["gate_up_s"], c["down_s"], aff, idx, all_expert,
                            c.get("gate_up_bias"), c.get("down_bias"), expert_affinities_scaling_mode=omoe.POST_SCALE)
    _check(from_bf16_tensor(out), g, f"tkg mx T={T} all_expert={all_expert}")


def test_tkg_rejects_what_the_reference_rejects():
    import torch
    from nkilib.core.moe.moe_tkg import moe_tkg
    from nkilib.core.utils.common_types import ExpertAffinityScaleMode

    dev = torch.device("cuda:0")
    x = torch.zeros((4, 256), dtype=torch.bfloat16, device=dev)
    wg = torch.zeros((2, 256, 2, 128), dtype=torch.bfloat16, device=dev)
    wd = torch.zeros((2, 128, 256), dtype=torch.bfloat16, device=dev)
    aff = torch.zeros((4, 2), dtype=torch.bfloat16, device=dev)
    idx = torch.zeros((4, 1), dtype=torch.int32, device=dev)
    with pytest.raises(AssertionError, match="pre-scale"):
        moe_tkg(x, wg, wd, aff, idx, False, expert_affinities_scaling_mode=ExpertAffinityScaleMode.PRE_SCALE)
    with pytest.raises(AssertionError, match="rank_id is required"):
        moe_tkg(x, wg, wd, aff, idx, True, expert_affinities_scaling_mode=ExpertAffinityScaleMode.POST_SCALE)
    with pytest.raises(AssertionError, match="Static quantization"):
        moe_tkg(x, wg, wd, aff, idx, False, gate_up_input_scale=aff, down_input_scale=aff)
    with pytest.raises(AssertionError, match="is_all_expert_dynamic=True requires is_all_expert=True"):
        moe_tkg(x, wg, wd, aff, idx, False, is_all_expert_dynamic=True, block_size=8)
