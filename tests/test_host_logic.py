"""Host-side mirror of the reference's operator interface: names, defaults, validation and error convention.
Runs without a GPU (nothing is launched)."""

import inspect

import pytest
import torch


def test_public_names_match_the_reference_package():
    import nkilib.core.moe.moe_cte as m

    # src/nkilib_src/nkilib/core/moe/moe_cte/__init__.py:17-36
    for n in ("moe_cte", "MoECTESpec", "MoECTEImplementation", "ShardOnBlockConfig", "ShardOnIConfig",
              "QuantizationConfig", "BlockShardStrategy", "SkipMode"):
        assert hasattr(m, n)
    assert [e.name for e in m.MoECTEImplementation] == [
        "shard_on_block", "shard_on_i", "shard_on_i_hybrid", "shard_on_i_dropping", "shard_on_block_mx",
        "shard_on_i_mx", "shard_on_i_mx_hybrid"]
    assert [e.value for e in m.MoECTEImplementation] == list(range(7))
    from nkilib.core.utils.common_types import ActFnType, ExpertAffinityScaleMode, NormType, QuantizationType

    assert ActFnType.SiLU.value == 0 and ActFnType.Swish.value == 3
    assert ExpertAffinityScaleMode.POST_SCALE.value == 1 and ExpertAffinityScaleMode.PRE_SCALE_DELAYED.value == 3
    assert NormType.RMS_NORM.value == 1 and QuantizationType.ROW.value == 2 and QuantizationType.STATIC.value == 1


def test_moe_cte_signature_is_the_reference_signature_plus_one_keyword():
    from nkilib.core.moe.moe_cte import moe_cte

    params = list(inspect.signature(moe_cte).parameters)
    # src/nkilib_src/nkilib/core/moe/moe_cte/moe_cte.py:253-277
    ref = ["hidden_states", "expert_affinities_masked", "gate_up_proj_weight", "down_proj_weight",
           "token_position_to_id", "block_to_expert", "block_size", "spec", "conditions", "gate_and_up_proj_bias",
           "down_proj_bias", "quantization_config", "gate_up_activations_T", "down_activations",
           "activation_function", "skip_dma", "compute_dtype", "is_tensor_update_accumulating",
           "expert_affinities_scaling_mode", "gate_clamp_upper_limit", "gate_clamp_lower_limit",
           "up_clamp_upper_limit", "up_clamp_lower_limit"]
    assert params[: len(ref)] == ref
    assert params[len(ref):] == ["hidden_states_scale"]
    assert moe_cte[2] is moe_cte  # kernel[lnc](...) launch syntax is accepted
    sig = inspect.signature(moe_cte)
    assert sig.parameters["is_tensor_update_accumulating"].default is True
    assert sig.parameters["expert_affinities_scaling_mode"].default.name == "POST_SCALE"


def test_spec_defaults():
    from nkilib.core.moe.moe_cte import (BlockShardStrategy, MoECTEImplementation, MoECTESpec, ShardOnBlockConfig,
                                         ShardOnIConfig)

    s = MoECTESpec(MoECTEImplementation.shard_on_block_mx)
    assert isinstance(s.shard_on_block, ShardOnBlockConfig) and s.shard_on_I is None
    assert s.shard_on_block.n_dynamic_blocks == 55 and s.shard_on_block.n_static_blocks == -1
    assert s.shard_on_block.block_sharding_strategy == BlockShardStrategy.PING_PONG
    s = MoECTESpec(MoECTEImplementation.shard_on_i_hybrid)
    assert isinstance(s.shard_on_I, ShardOnIConfig) and s.shard_on_I.num_static_block is None


def test_rmsnorm_args_validation():
    from nkilib.core.rmsnorm import RmsNormQuantKernelArgs, rmsnorm_quant_kernel
    from nkilib.core.utils.common_types import NormType, QuantizationType

    a = RmsNormQuantKernelArgs()
    assert a.lower_bound == 0.0 and a.eps == 1e-6 and a.is_row_quant() and a.needs_rms_normalization()
    with pytest.raises(AssertionError, match="NCC_INKI016"):
        RmsNormQuantKernelArgs(quantization_type=QuantizationType.MX)
    with pytest.raises(AssertionError):
        RmsNormQuantKernelArgs(norm_type=NormType.LAYER_NORM)
    with pytest.raises(AssertionError):
        RmsNormQuantKernelArgs(lower_bound=-1.0)
    # shape rules of the reference (rmsnorm_quant.py:174-262), raised before anything touches a device
    with pytest.raises(AssertionError, match="Rank of hidden"):
        rmsnorm_quant_kernel(torch.zeros(8), torch.zeros(8), a)
    with pytest.raises(AssertionError, match="exceeds maximum"):
        rmsnorm_quant_kernel(torch.zeros(1, 2, 16385), torch.zeros(16385), a)
    with pytest.raises(AssertionError, match="ln_w vector length"):
        rmsnorm_quant_kernel(torch.zeros(1, 2, 64), torch.zeros(32), a)
    with pytest.raises(AssertionError, match="input_dequant_scale must be provided"):
        rmsnorm_quant_kernel(torch.zeros(1, 2, 64), torch.zeros(64),
                             RmsNormQuantKernelArgs(quantization_type=QuantizationType.STATIC))


def test_no_cpu_fallback():
    """CPU tensors are rejected loudly; nothing silently computes on the host."""
    from nkilib._native import NativeLibraryError
    from nkilib.core.moe.moe_cte import MoECTEImplementation, MoECTESpec, moe_cte
    from nkilib.core.rmsnorm import RmsNormQuantKernelArgs, rmsnorm_quant_kernel

    with pytest.raises(NativeLibraryError, match="no CPU path"):
        rmsnorm_quant_kernel(torch.zeros(1, 2, 64, dtype=torch.bfloat16), torch.zeros(64, dtype=torch.bfloat16),
                             RmsNormQuantKernelArgs())
    with pytest.raises(NativeLibraryError, match="no CPU path"):
        moe_cte(torch.zeros(9, 64, dtype=torch.bfloat16), torch.zeros(18, 1, dtype=torch.bfloat16),
                torch.zeros(2, 64, 2, 32, dtype=torch.bfloat16), torch.zeros(2, 32, 64, dtype=torch.bfloat16),
                torch.zeros(16, dtype=torch.int32), torch.zeros(2, dtype=torch.int32), 8,
                MoECTESpec(MoECTEImplementation.shard_on_block))


def test_mx_shard_on_i_entry_points_validate_like_the_reference():
    """blockwise_mm_shard_intermediate_mx[_hybrid] exist under the reference's import path, refuse PRE_SCALE with the
    reference's message (bwmm_shard_on_I_mx.py:914-915) and are what the shard_on_i_mx enum members dispatch to."""
    from nkilib.core.moe.moe_cte import MoECTEImplementation, MoECTESpec, moe_cte
    from nkilib.core.moe.moe_cte.bwmm_shard_on_I_mx import (blockwise_mm_shard_intermediate_mx,
                                                            blockwise_mm_shard_intermediate_mx_hybrid)
    from nkilib.core.utils.common_types import ExpertAffinityScaleMode

    z = torch.zeros(1)
    with pytest.raises(AssertionError, match="PRE_SCALE mode not implemented"):
        blockwise_mm_shard_intermediate_mx[2](z, z, z, z, z, z, block_size=256)  # the default mode is PRE_SCALE
    with pytest.raises(AssertionError, match="conditions is required"):
        blockwise_mm_shard_intermediate_mx_hybrid(None, z, z, z, z, z, z, block_size=256)
    with pytest.raises(AssertionError, match="PRE_SCALE mode not implemented"):
        moe_cte(z, z, z, z, z, z, 256, MoECTESpec(MoECTEImplementation.shard_on_i_mx),
                expert_affinities_scaling_mode=ExpertAffinityScaleMode.PRE_SCALE)
    with pytest.raises(AssertionError, match="gate_up_proj_scale and down_proj_scale are required"):
        moe_cte(z, z, z, z, z, z, 256, MoECTESpec(MoECTEImplementation.shard_on_i_mx_hybrid), conditions=z)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from nkilib import _native as nv

    monkeypatch.setattr(nv, "_lib", None)
    monkeypatch.setattr(nv, "LIB_PATH", str(tmp_path / "absent.so"))
    with pytest.raises(nv.NativeLibraryError, match="no CPU fallback"):
        nv.lib()


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: --gpus N with N > 1 exits with a message that says so (before touching a GPU)."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)
    assert res.returncode != 0
    assert "one GPU" in res.stderr and res.stdout.strip() == ""
