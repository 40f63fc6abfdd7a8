"""Shared host driver of the blockwise MoE kernels: validates tensors the way the
reference kernels do (kernel_assert), allocates the output in the reference's
return shape, and calls ``moe_blockwise`` of libmoe_gfx950.so."""

import ctypes
import weakref
from typing import Optional

import torch

from .... import _native as nv
from ...utils.common_types import ActFnType, ExpertAffinityScaleMode
from ...utils.kernel_assert import kernel_assert
from .moe_cte_utils import SkipMode


# Profiling hook: when set to a callable, the pipeline is issued one stage per C-ABI call and
# ``stage_callback(name)`` runs after each stage has been enqueued (bench.py records a HIP event
# there).  The kernels and their order are identical to the single-call path.
stage_callback = None

_STAGES = (
    ("prep", nv.STAGE_PREP),
    ("act_quant", nv.STAGE_ACT_QUANT),
    ("gate_up", nv.STAGE_GATE_UP),
    ("requant", nv.STAGE_REQUANT),
    ("down", nv.STAGE_DOWN),
    ("combine", nv.STAGE_COMBINE),
)


# K-contiguous copies of the dense (bf16 / fp8) expert weights, kept per weight tensor pair: the GEMMs of the bf16
# and fp8-row kinds read both operands along K while the reference's layouts are N-contiguous, and the copies
# depend on the weights only.  An entry lives as long as both weight allocations do and is remade when either
# was modified in place (torch's version counter).  Costs one more copy of the weights in HBM (two for fp8 weights
# of the bf16 kind, which are widened); ``kmajor_weight_cache = False`` makes every call build its copies in the
# workspace instead.
kmajor_weight_cache = True
# The same mechanism for 8-bit MXFP8 weights on the large-tile shapes: copies in the order the kernels read them
# (contiguous 32 KB runs per workgroup and K slice instead of 128-byte pieces of the reference layout), of the
# gate/up weights only: that GEMM is 5 % faster at DeepSeek-V3's expert shape, the down GEMM was not.  A second
# copy of the gate/up weights in HBM, made on the first call with a weight tensor pair; ``mx_weight_copies =
# False`` reads the reference layout in place.
mx_weight_copies = True
# Measurement hook: an int64 device tensor of 4 elements that the large-tile GEMMs fill with the shader cycles and
# the 100 MHz ticks of their workgroup 0 (gate/up, then down): cycles / ticks * 0.1 = the clock in GHz under load.
gemm_clock_probe = None
# Measurement hook: seven ``torch.cuda.Event(enable_timing=True)`` (each recorded at least once before, so that its
# HIP event exists) which the library records on the stream on entry and after the bookkeeping, the activation
# quantisation, the gate/up GEMM, the fp8-row re-quantisation, the down GEMM and the combine of the next call.
stage_events = None
_KMAJOR_MAX_ENTRIES = 64
_kmajor = {}


def clear_kmajor_weight_cache():
    _kmajor.clear()


def _bytes_of(t):
    """Where a weight tensor's bytes are: (address of its storage, byte offset, byte length).  Views and casts of one
    allocation (``w.view(torch.int32)`` made anew for every call, say) name the same bytes."""
    return (t.untyped_storage().data_ptr(), t.storage_offset() * t.element_size(), t.numel() * t.element_size())


def _kmajor_weights(L, a, guw, dw, dev):
    """``guw`` / ``dw``: the weight tensors as the caller of the operator passed them.  An entry is found through the
    bytes the tensors name and how the call reads them (kind, weight type, expert shape), so a fresh view of the same
    allocation hits; it is valid while both allocations are alive (weak references to the storages: an address that
    was freed and handed out again is a different storage) and unchanged (torch's version counters, which views
    share with their base)."""
    st0, st1 = guw.untyped_storage(), dw.untyped_storage()
    key = (_bytes_of(guw), _bytes_of(dw), int(a.kind), int(a.weight_dtype), int(a.E), int(a.H), int(a.I), int(a.I_pad))
    sig = (guw._version, dw._version)
    ent = _kmajor.get(key)
    if ent is not None and ent[0]() is st0 and ent[1]() is st1 and ent[2] == sig:
        return ent[3], ent[4]
    n0 = L.moe_kmajor_weights_bytes(ctypes.byref(a), 0)
    n1 = L.moe_kmajor_weights_bytes(ctypes.byref(a), 1)
    if n0 == 0:
        return None, None
    k0 = torch.empty(n0, dtype=torch.uint8, device=dev)
    k1 = torch.empty(n1, dtype=torch.uint8, device=dev) if n1 else None  # (MXFP8: gate/up only)
    with torch.cuda.device(dev):
        nv.check(L.moe_prepare_kmajor_weights(ctypes.byref(a), nv.ptr(k0), nv.ptr(k1), nv.stream_ptr(dev)),
                 "moe_cte (K-contiguous weight copies)")
    if len(_kmajor) >= _KMAJOR_MAX_ENTRIES:
        _kmajor.pop(next(iter(_kmajor)))
    drop = lambda _ref, key=key: _kmajor.pop(key, None)
    _kmajor[key] = (weakref.ref(st0, drop), weakref.ref(st1, drop), sig, k0, k1)
    return k0, k1


def run_blockwise(
    kind: int,
    hidden_states: torch.Tensor,
    expert_affinities_masked: torch.Tensor,
    gate_up_proj_weight: torch.Tensor,
    down_proj_weight: torch.Tensor,
    token_position_to_id: torch.Tensor,
    block_to_expert: torch.Tensor,
    block_size: int,
    out_shape_kind: str,
    dims: dict,
    conditions: Optional[torch.Tensor] = None,
    gate_and_up_proj_bias: Optional[torch.Tensor] = None,
    down_proj_bias: Optional[torch.Tensor] = None,
    gate_up_proj_scale: Optional[torch.Tensor] = None,
    down_proj_scale: Optional[torch.Tensor] = None,
    hidden_states_scale: Optional[torch.Tensor] = None,
    activation_function: ActFnType = ActFnType.SiLU,
    skip_dma: SkipMode = None,
    expert_affinities_scaling_mode: ExpertAffinityScaleMode = ExpertAffinityScaleMode.POST_SCALE,
    gate_clamp_upper_limit: Optional[float] = None,
    gate_clamp_lower_limit: Optional[float] = None,
    up_clamp_upper_limit: Optional[float] = None,
    up_clamp_lower_limit: Optional[float] = None,
    weight_dtype: int = nv.DT_BF16,
    scale_experts: int = 0,
    checkpoint_gate_up: bool = False,
    checkpoint_down: bool = False,
    weight_objects=None,
):
    """dims: T1, H, I, E, I_pad.  out_shape_kind: "T2H" ([T1,2,H], slot 0), "2TH" ([2,T1,H], slot 0) or "TH".
    With ``checkpoint_gate_up`` / ``checkpoint_down`` (bf16 hidden states; bf16 or fp8 weight-only) the result is a tuple: the output, then
    ``gate_up_activations_T`` ``[N, 2, I, B]`` and / or ``down_activations`` ``[N, B, H]`` (bfloat16)."""
    L = nv.lib()
    skip_dma = skip_dma or SkipMode(False, False)
    T1, H, I, E = dims["T1"], dims["H"], dims["I"], dims["E"]
    B = int(block_size)
    dev = hidden_states.device
    kernel_assert(B > 0, f"block_size must be positive, got {B}")

    tp2id = nv.require_device_tensor(token_position_to_id, "token_position_to_id").reshape(-1)
    kernel_assert(tp2id.dtype == torch.int32, f"token_position_to_id must be int32 but got {tp2id.dtype}")
    kernel_assert(tp2id.numel() % B == 0, f"token_position_to_id length {tp2id.numel()} is not a multiple of B={B}")
    N = tp2id.numel() // B
    b2e = nv.require_device_tensor(block_to_expert, "block_to_expert").reshape(-1)
    kernel_assert(b2e.dtype == torch.int32, f"block_to_expert must be int32 but got {b2e.dtype}")
    kernel_assert(b2e.numel() == N, f"block_to_expert must have N={N} entries but got {b2e.numel()}")
    cond = None
    if conditions is not None:
        cond = nv.require_device_tensor(conditions, "conditions").reshape(-1)
        kernel_assert(cond.dtype == torch.int32, f"conditions must be int32 but got {cond.dtype}")

    aff = None
    if expert_affinities_scaling_mode != ExpertAffinityScaleMode.NO_SCALE:
        aff = nv.require_device_tensor(expert_affinities_masked, "expert_affinities_masked")
        kernel_assert(aff.numel() == T1 * E, f"expert_affinities_masked must hold (T+1)*E={T1 * E} values, got {aff.numel()}")
        kernel_assert(aff.dtype in (torch.bfloat16, torch.float32),
                      f"expert_affinities_masked must be bfloat16 or float32 but got {aff.dtype}")
    bias_dt = nv.DT_BF16
    gub = db = None
    if gate_and_up_proj_bias is not None or down_proj_bias is not None:
        kernel_assert(gate_and_up_proj_bias is not None and down_proj_bias is not None,
                      "gate_and_up_proj_bias and down_proj_bias must be given together")
        gub = nv.require_device_tensor(gate_and_up_proj_bias, "gate_and_up_proj_bias")
        db = nv.require_device_tensor(down_proj_bias, "down_proj_bias")
        kernel_assert(gub.dtype == db.dtype and gub.dtype in (torch.bfloat16, torch.float32),
                      "bias tensors must both be bfloat16 or both float32")
        bias_dt = nv.DT_BF16 if gub.dtype == torch.bfloat16 else nv.DT_FP32
        kernel_assert(db.numel() == E * H, f"down_proj_bias must be [E, H] but got {tuple(db.shape)}")

    # the combine stage writes every row of the result (zeros where a token has no contribution) and, through
    # output_shard1, zeros into the second shard slot, which the reference leaves zero after its reduction
    shard1_ptr = None
    if out_shape_kind == "T2H":
        out = torch.empty((T1, 2, H), dtype=torch.bfloat16, device=dev)
        shard1_ptr = out[:, 1].data_ptr()
        stride = 2 * H
    elif out_shape_kind == "2TH":
        out = torch.empty((2, T1, H), dtype=torch.bfloat16, device=dev)
        shard1_ptr = out[1].data_ptr()
        stride = H
    else:
        out = torch.empty((T1, H), dtype=torch.bfloat16, device=dev)
        stride = H

    a = nv.BwmmArgs()
    a.hidden_states = nv.ptr(hidden_states)
    a.hidden_states_scale = nv.ptr(hidden_states_scale)
    a.expert_affinities_masked = nv.ptr(aff)
    a.gate_up_proj_weight = nv.ptr(gate_up_proj_weight)
    a.down_proj_weight = nv.ptr(down_proj_weight)
    a.gate_up_proj_scale = nv.ptr(gate_up_proj_scale)
    a.down_proj_scale = nv.ptr(down_proj_scale)
    a.gate_and_up_proj_bias = nv.ptr(gub)
    a.down_proj_bias = nv.ptr(db)
    a.token_position_to_id = nv.ptr(tp2id)
    a.block_to_expert = nv.ptr(b2e)
    a.conditions = nv.ptr(cond)
    a.output = nv.ptr(out)
    a.output_shard1 = shard1_ptr
    a.T1, a.H, a.I, a.E, a.B, a.N = T1, H, I, E, B, N
    a.I_pad = dims.get("I_pad", I)
    a.n_conditions = cond.numel() if cond is not None else 0
    a.out_row_stride = stride
    a.scale_experts = scale_experts
    a.kind = kind
    a.weight_dtype = weight_dtype
    a.affinity_dtype = nv.DT_FP32 if (aff is not None and aff.dtype == torch.float32) else nv.DT_BF16
    a.bias_dtype = bias_dt
    a.act_fn = activation_function.value
    a.scaling_mode = expert_affinities_scaling_mode.value
    a.skip_token = 1 if skip_dma.skip_token else 0
    mask = 0
    for bit, v, name in (
        (nv.CLAMP_GATE_HI, gate_clamp_upper_limit, "gate_clamp_upper"),
        (nv.CLAMP_GATE_LO, gate_clamp_lower_limit, "gate_clamp_lower"),
        (nv.CLAMP_UP_HI, up_clamp_upper_limit, "up_clamp_upper"),
        (nv.CLAMP_UP_LO, up_clamp_lower_limit, "up_clamp_lower"),
    ):
        if v is not None:
            mask |= bit
            setattr(a, name, float(v))
    a.clamp_mask = mask
    ck_gu = ck_down = None
    if checkpoint_gate_up or checkpoint_down:
        kernel_assert(kind == nv.KIND_BF16, "activation checkpoints need bfloat16 hidden states")
    if checkpoint_gate_up:
        ck_gu = torch.empty((N, 2, I, B), dtype=torch.bfloat16, device=dev)
        a.gate_up_activations_T = nv.ptr(ck_gu)
    if checkpoint_down:
        ck_down = torch.empty((N, B, H), dtype=torch.bfloat16, device=dev)
        a.down_activations = nv.ptr(ck_down)

    plan = None
    if not (checkpoint_gate_up or checkpoint_down):
        from . import block_index

        plan = block_index.plan_for(tp2id, b2e, cond, B, N, T1)
        if plan is not None:
            a.block_plan, a.block_plan_bytes = plan
    if gemm_clock_probe is not None:
        kernel_assert(gemm_clock_probe.dtype == torch.int64 and gemm_clock_probe.numel() >= 4 and gemm_clock_probe.is_cuda,
                      "gemm_clock_probe must be a device int64 tensor of 4 elements")
        a.gemm_clocks = gemm_clock_probe.data_ptr()
    kmajor = (None, None)
    if (kmajor_weight_cache and kind in (nv.KIND_BF16, nv.KIND_FP8_ROW)) or (mx_weight_copies and kind == nv.KIND_MXFP8):
        # (weight_objects: the caller's own tensor objects where the operator had to make views of them)
        wo = weight_objects or (gate_up_proj_weight, down_proj_weight)
        kmajor = _kmajor_weights(L, a, wo[0], wo[1], dev)
        a.gate_up_proj_weight_kmajor = nv.ptr(kmajor[0])
        a.down_proj_weight_kmajor = nv.ptr(kmajor[1])

    ev_handles = None
    if stage_events is not None:
        kernel_assert(len(stage_events) == 7, "stage_events must hold seven events")
        # (entries may be None: that stage boundary is not recorded; the array is kept alive until the call returns)
        ev_handles = (ctypes.c_void_p * 7)(*[None if e is None else e.cuda_event for e in stage_events])
        a.stage_events = ctypes.cast(ev_handles, ctypes.c_void_p)
    need = L.moe_blockwise_workspace_bytes(ctypes.byref(a))
    if need == 0:
        # validation failed inside the library: run the call to obtain the precise code
        a.workspace = None
        a.workspace_bytes = 0
        nv.check(L.moe_blockwise(ctypes.byref(a), None) or -2, "moe_cte")
    ws = nv.workspace(dev, need)
    a.workspace = nv.ptr(ws)
    a.workspace_bytes = ws.numel()
    with torch.cuda.device(dev):
        if stage_callback is None:
            rc = L.moe_blockwise(ctypes.byref(a), nv.stream_ptr(dev))
        else:
            rc = 0
            for name, bit in _STAGES:
                if name == "act_quant" and not (kind == nv.KIND_MXFP8 and hidden_states_scale is None):
                    continue
                if name == "requant" and kind != nv.KIND_FP8_ROW:
                    continue
                rc = L.moe_blockwise_stages(ctypes.byref(a), bit, nv.stream_ptr(dev))
                if rc != 0:
                    break
                stage_callback(name)
    nv.check(rc, "moe_cte")
    if ck_gu is None and ck_down is None:
        return out
    return tuple(t for t in (out, ck_gu, ck_down) if t is not None)
