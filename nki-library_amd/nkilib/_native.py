"""ctypes binding of libmoe_gfx950.so (C ABI declared in include/moe_gfx950.h).

Loading is lazy and loud: if the shared library has not been built
(``python nki-library_amd/build.py``) every kernel entry point raises
``NativeLibraryError``.  There is no fallback path.
"""

import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p

import torch

from .core.utils.kernel_assert import kernel_assert

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_lib", "libmoe_gfx950.so")

# element types (MOE_DT_*)
DT_BF16, DT_FP16, DT_FP32, DT_FP8, DT_FP8_E5M2, DT_FP4_E2M1, DT_INT32 = 0, 1, 2, 3, 4, 5, 6
# MOE_KIND_*
KIND_BF16, KIND_FP8_ROW, KIND_MXFP8 = 0, 1, 2
# MOE_MX_LAYOUT_*
MX_TOKEN_MAJOR, MX_REF_DENSE, MX_REF_STRIDED = 0, 1, 2
CLAMP_GATE_HI, CLAMP_GATE_LO, CLAMP_UP_HI, CLAMP_UP_LO = 1, 2, 4, 8
# MOE_STAGE_*
STAGE_PREP, STAGE_ACT_QUANT, STAGE_GATE_UP, STAGE_REQUANT, STAGE_DOWN, STAGE_COMBINE, STAGE_ALL = 1, 2, 4, 8, 16, 32, 63

EXPORTED_SYMBOLS = (
    "moe_error_string",
    "moe_abi_version",
    "moe_check_device",
    "moe_rmsnorm_quant_fp8_row",
    "moe_rmsnorm_quant_fp8_static",
    "moe_rmsnorm_quant_mxfp8",
    "moe_build_blocks_workspace_bytes",
    "moe_build_blocks",
    "moe_build_blocks_static",
    "moe_block_plan_bytes",
    "moe_build_blocks_plan",
    "moe_find_nonzero_indices_workspace_bytes",
    "moe_find_nonzero_indices",
    "moe_indexed_flatten",
    "moe_cumsum",
    "moe_router_topk_workspace_bytes",
    "moe_router_topk",
    "moe_blockwise_workspace_bytes",
    "moe_blockwise",
    "moe_blockwise_stages",
    "moe_kmajor_weights_bytes",
    "moe_prepare_kmajor_weights",
)


class NativeLibraryError(RuntimeError):
    pass


class BwmmArgs(ctypes.Structure):
    """Mirror of ``struct moe_bwmm_args``; field order must match the header."""

    _fields_ = [
        ("hidden_states", c_void_p),
        ("hidden_states_scale", c_void_p),
        ("expert_affinities_masked", c_void_p),
        ("gate_up_proj_weight", c_void_p),
        ("down_proj_weight", c_void_p),
        ("gate_up_proj_scale", c_void_p),
        ("down_proj_scale", c_void_p),
        ("gate_and_up_proj_bias", c_void_p),
        ("down_proj_bias", c_void_p),
        ("token_position_to_id", c_void_p),
        ("block_to_expert", c_void_p),
        ("conditions", c_void_p),
        ("output", c_void_p),
        ("workspace", c_void_p),
        ("workspace_bytes", c_size_t),
        ("T1", c_int64),
        ("H", c_int64),
        ("I", c_int64),
        ("E", c_int64),
        ("B", c_int64),
        ("N", c_int64),
        ("I_pad", c_int64),
        ("n_conditions", c_int64),
        ("out_row_stride", c_int64),
        ("scale_experts", c_int32),
        ("kind", c_int32),
        ("weight_dtype", c_int32),
        ("affinity_dtype", c_int32),
        ("bias_dtype", c_int32),
        ("act_fn", c_int32),
        ("scaling_mode", c_int32),
        ("skip_token", c_int32),
        ("clamp_mask", c_int32),
        ("gate_clamp_upper", c_float),
        ("gate_clamp_lower", c_float),
        ("up_clamp_upper", c_float),
        ("up_clamp_lower", c_float),
        ("gate_up_activations_T", c_void_p),
        ("down_activations", c_void_p),
        ("gate_up_proj_weight_kmajor", c_void_p),
        ("down_proj_weight_kmajor", c_void_p),
        ("output_shard1", c_void_p),
        ("gemm_clocks", c_void_p),
        ("block_plan", c_void_p),
        ("block_plan_bytes", c_size_t),
        ("stage_events", c_void_p),
    ]


_lib = None


def lib():
    """The loaded shared library; raises NativeLibraryError if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NativeLibraryError(
            f"{LIB_PATH} not found: build it with `python nki-library_amd/build.py` (needs hipcc). "
            "There is no CPU fallback for these kernels."
        )
    try:
        L = ctypes.CDLL(LIB_PATH)
    except OSError as e:  # pragma: no cover - depends on the machine
        raise NativeLibraryError(f"cannot load {LIB_PATH}: {e}") from e
    L.moe_error_string.restype = c_char_p
    L.moe_error_string.argtypes = [c_int]
    L.moe_abi_version.restype = c_int
    L.moe_check_device.restype = c_int
    L.moe_rmsnorm_quant_fp8_row.restype = c_int
    L.moe_rmsnorm_quant_fp8_row.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int64, c_int64, c_float,
                                            c_float, c_int, c_void_p]
    L.moe_rmsnorm_quant_fp8_static.restype = c_int
    L.moe_rmsnorm_quant_fp8_static.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64,
                                               c_float, c_int, c_void_p]
    L.moe_rmsnorm_quant_mxfp8.restype = c_int
    L.moe_rmsnorm_quant_mxfp8.argtypes = [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                          c_void_p, c_int64, c_int64, c_float, c_int64, c_int, c_int, c_void_p]
    L.moe_build_blocks_workspace_bytes.restype = c_size_t
    L.moe_build_blocks_workspace_bytes.argtypes = [c_int64]
    L.moe_build_blocks.restype = c_int
    L.moe_build_blocks.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_void_p,
                                   c_void_p, c_void_p, c_int64, c_void_p, c_size_t, c_void_p, c_void_p]
    L.moe_build_blocks_static.restype = c_int
    L.moe_build_blocks_static.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_void_p,
                                          c_void_p, c_void_p, c_int64, c_void_p, c_void_p]
    L.moe_block_plan_bytes.restype = c_size_t
    L.moe_block_plan_bytes.argtypes = [c_int64, c_int64, c_int64, c_int]
    L.moe_build_blocks_plan.restype = c_int
    L.moe_build_blocks_plan.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_void_p,
                                        c_void_p, c_void_p, c_int64, c_void_p, c_size_t, c_void_p, c_void_p, c_size_t,
                                        c_void_p]
    L.moe_find_nonzero_indices_workspace_bytes.restype = c_size_t
    L.moe_find_nonzero_indices_workspace_bytes.argtypes = [c_int64, c_int64]
    L.moe_find_nonzero_indices.restype = c_int
    L.moe_find_nonzero_indices.argtypes = [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p,
                                           c_void_p, c_size_t, c_void_p]
    L.moe_indexed_flatten.restype = c_int
    L.moe_indexed_flatten.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p,
                                      c_int32, c_void_p, c_void_p]
    L.moe_cumsum.restype = c_int
    L.moe_cumsum.argtypes = [c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p]
    L.moe_router_topk_workspace_bytes.restype = c_size_t
    L.moe_router_topk_workspace_bytes.argtypes = [c_int64, c_int64]
    L.moe_router_topk.restype = c_int
    L.moe_router_topk.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int, c_int,
                                  c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                  c_size_t, c_void_p]
    L.moe_blockwise_workspace_bytes.restype = c_size_t
    L.moe_blockwise_workspace_bytes.argtypes = [POINTER(BwmmArgs)]
    L.moe_blockwise.restype = c_int
    L.moe_blockwise.argtypes = [POINTER(BwmmArgs), c_void_p]
    L.moe_kmajor_weights_bytes.restype = c_size_t
    L.moe_kmajor_weights_bytes.argtypes = [POINTER(BwmmArgs), c_int]
    L.moe_prepare_kmajor_weights.restype = c_int
    L.moe_prepare_kmajor_weights.argtypes = [POINTER(BwmmArgs), c_void_p, c_void_p, c_void_p]
    L.moe_blockwise_stages.restype = c_int
    L.moe_blockwise_stages.argtypes = [POINTER(BwmmArgs), ctypes.c_uint, c_void_p]
    _lib = L
    return L


def check(rc, what):
    """Map a negative return code to the reference's error convention (an AssertionError)."""
    if rc != 0:
        msg = lib().moe_error_string(int(rc)).decode()
        kernel_assert(False, f"{what}: {msg} (code {rc})")


def ptr(t):
    return None if t is None else c_void_p(t.data_ptr())


def stream_ptr(device):
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


_DT = {torch.bfloat16: DT_BF16, torch.float16: DT_FP16, torch.float32: DT_FP32}


def dtype_code(t, what):
    kernel_assert(t.dtype in _DT, f"{what} must be bfloat16, float16 or float32 but got {t.dtype}")
    return _DT[t.dtype]


def index_dtype_code(t, what):
    """Element type code for the index operators, which also take int32."""
    if t.dtype == torch.int32:
        return DT_INT32
    kernel_assert(t.dtype in _DT, f"{what} must be int32, bfloat16, float16 or float32 but got {t.dtype}")
    return _DT[t.dtype]


def require_device_tensor(t, what):
    kernel_assert(isinstance(t, torch.Tensor), f"{what} must be a torch.Tensor")
    if not t.is_cuda:
        raise NativeLibraryError(
            f"{what} lives on {t.device}: these kernels run on an MI355X (ROCm) device only; there is no CPU path"
        )
    return t.contiguous()


_workspaces = {}


def workspace(device, nbytes):
    """A per-device scratch tensor that only grows (uint8, 256-byte aligned by the allocator)."""
    key = (device.type, device.index)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        _workspaces[key] = None
        ws = torch.empty(int(nbytes), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws
