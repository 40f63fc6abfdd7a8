"""The C-ABI library loads, exports every function include/moe_gfx950.h declares, and its argument struct has
the layout the ctypes mirror assumes.  No compute calls (there is no GPU here)."""

import ctypes
import os
import re
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "moe_gfx950.h")


def _declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    names = re.findall(r"\b(moe_[a-z0-9_]+)\s*\(", src)
    return sorted(set(n for n in names if n != "moe_bwmm_args"))


def test_every_declared_symbol_is_exported():
    from nkilib import _native as nv

    L = nv.lib()
    declared = _declared_functions()
    assert len(declared) >= 10
    for name in declared:
        assert hasattr(L, name), f"{name} declared in the header but not exported"
    assert set(nv.EXPORTED_SYMBOLS) == set(declared)
    assert L.moe_abi_version() == 7
    assert b"workspace" in L.moe_error_string(-3)


def test_struct_layout_matches_ctypes_mirror():
    """Compile a probe with gcc against the header and compare sizeof / offsets with nkilib._native.BwmmArgs."""
    from nkilib._native import BwmmArgs

    fields = [f[0] for f in BwmmArgs._fields_]
    body = "\n".join(f'  printf("{f} %zu\\n", offsetof(moe_bwmm_args, {f}));' for f in fields)
    prog = f'#include <stdio.h>\n#include <stddef.h>\n#include "moe_gfx950.h"\nint main(void) {{\n' \
           f'  printf("sizeof %zu\\n", sizeof(moe_bwmm_args));\n{body}\n  return 0;\n}}\n'
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "probe.c")
        open(c, "w").write(prog)
        exe = os.path.join(d, "probe")
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), c, "-o", exe], check=True)
        out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()
    got = dict(zip(out[0::2], map(int, out[1::2])))
    assert got["sizeof"] == ctypes.sizeof(BwmmArgs)
    for f in fields:
        assert got[f] == getattr(BwmmArgs, f).offset, f


def test_argument_validation_runs_without_a_gpu():
    """Validation happens before any launch, so the error paths are reachable on the CPU."""
    from nkilib import _native as nv

    L = nv.lib()
    a = nv.BwmmArgs()
    assert L.moe_blockwise_workspace_bytes(ctypes.byref(a)) == 0
    assert L.moe_blockwise(ctypes.byref(a), None) == -1  # MOE_E_BAD_ARG: null tensors
    assert L.moe_rmsnorm_quant_fp8_row(None, 0, None, 0, None, 1, 8, 1e-6, 0.0, 0, None) == -1
    assert L.moe_rmsnorm_quant_mxfp8(ctypes.c_void_p(256), 0, None, None, None, 0, ctypes.c_void_p(256),
                                     ctypes.c_void_p(256), None, 4, 500, 1e-6, 500, 0, 0, None) == -2  # H % 512
    # a residual without a place for the sum (or the reverse) is refused
    assert L.moe_rmsnorm_quant_mxfp8(ctypes.c_void_p(256), 0, ctypes.c_void_p(256), None, None, 0, ctypes.c_void_p(256),
                                     ctypes.c_void_p(256), None, 4, 512, 1e-6, 512, 0, 0, None) == -1
    assert L.moe_rmsnorm_quant_fp8_row(ctypes.c_void_p(256), 0, None, 0, ctypes.c_void_p(256), 4, 32768, 1e-6, 0.0, 0,
                                       None) == -2  # H > 16384
    assert L.moe_build_blocks_workspace_bytes(256) >= 2 * 256 * 4
    with pytest.raises(AssertionError, match="NCC_INKI016"):
        nv.check(-2, "x")


def _valid_args(nv, kind, T1, H, I, E, B, N, weight_dtype=0):
    """An argument block that passes validation (pointers are never dereferenced by it)."""
    a = nv.BwmmArgs()
    fake = ctypes.c_void_p(4096)
    for f in ("hidden_states", "expert_affinities_masked", "gate_up_proj_weight", "down_proj_weight",
              "gate_up_proj_scale", "down_proj_scale", "token_position_to_id", "block_to_expert", "output"):
        setattr(a, f, fake)
    a.T1, a.H, a.I, a.E, a.B, a.N = T1, H, I, E, B, N
    a.out_row_stride = H
    a.scale_experts = E
    a.kind = kind
    a.weight_dtype = weight_dtype
    a.scaling_mode = 1
    return a


def test_shapes_beyond_the_32_bit_offsets_are_refused():
    """The kernels address rows with 32-bit offsets: tensors that outgrow them must be refused, not wrapped around
    (the reference states explicit limits too, bwmm_shard_on_block_mx.py:586-633)."""
    from nkilib import _native as nv

    L = nv.lib()
    ws = lambda a: L.moe_blockwise_workspace_bytes(ctypes.byref(a))
    rc = lambda a: L.moe_blockwise(ctypes.byref(a), None)
    BAD_SHAPE, WORKSPACE = -2, -3
    # MXFP8, DeepSeek-V3 experts: BASELINE config 4 passes
    ok = _valid_args(nv, nv.KIND_MXFP8, 8193, 7168, 2048, 256, 128, 766, nv.DT_FP8)
    assert ws(ok) > 0 and rc(ok) == WORKSPACE
    # hidden states of 2^32 bytes: (T+1) * H
    big_t = _valid_args(nv, nv.KIND_MXFP8, 2**32 // 7168 + 1, 7168, 2048, 256, 128, 766, nv.DT_FP8)
    assert ws(big_t) == 0 and rc(big_t) == BAD_SHAPE
    just_below = _valid_args(nv, nv.KIND_MXFP8, 2**32 // 7168, 7168, 2048, 256, 128, 766, nv.DT_FP8)
    assert ws(just_below) > 0
    # intermediate of 2^32 bytes: N * B * I (about 262k tokens top-8 at I = 2048)
    big_n = _valid_args(nv, nv.KIND_MXFP8, 8193, 7168, 2048, 256, 128, 2**32 // (128 * 2048), nv.DT_FP8)
    assert ws(big_n) == 0 and rc(big_n) == BAD_SHAPE
    # one expert's gate/up weights of 2 GiB: 2 * H * I bytes
    big_w = _valid_args(nv, nv.KIND_MXFP8, 129, 16384, 65536, 2, 128, 2, nv.DT_FP8)
    assert ws(big_w) == 0 and rc(big_w) == BAD_SHAPE
    # affinity table of 2^32 bytes: (T+1) * E fp32 or bf16 entries at 4-byte granularity
    big_aff = _valid_args(nv, nv.KIND_MXFP8, 2**21 + 1, 512, 512, 512, 128, 64, nv.DT_FP8)
    assert ws(big_aff) == 0 and rc(big_aff) == BAD_SHAPE
    # ... which 4-bit weights (half the bytes) still fit
    assert ws(_valid_args(nv, nv.KIND_MXFP8, 129, 16384, 65536, 2, 128, 2, nv.DT_FP4_E2M1)) > 0
    # dense kinds: 16 GiB per A operand
    assert ws(_valid_args(nv, nv.KIND_BF16, 4097, 4096, 14336, 8, 128, 71)) > 0
    big_bf16 = _valid_args(nv, nv.KIND_BF16, 2**34 // (4096 * 2), 4096, 1024, 8, 128, 71)
    assert ws(big_bf16) == 0 and rc(big_bf16) == BAD_SHAPE
    big_row = _valid_args(nv, nv.KIND_FP8_ROW, 4097, 4096, 14336, 8, 128, 2**34 // (128 * 14336) + 1)
    assert ws(big_row) == 0 and rc(big_row) == BAD_SHAPE


def test_static_scratch_entry_point_rejects_sizes_beyond_its_scratch():
    """moe_build_blocks_static checks its limit before it touches the device."""
    from nkilib import _native as nv

    L = nv.lib()
    fake = ctypes.c_void_p(4096)
    rc = L.moe_build_blocks_static(fake, 4, 2, 513, 128, 600, 0, 0, fake, fake, None, 0, None, None)
    assert rc == -7 and b"allocates nothing" in L.moe_error_string(rc)
    assert L.moe_build_blocks_static(None, 4, 2, 256, 128, 600, 0, 0, fake, fake, None, 0, None, None) == -1
    assert L.moe_build_blocks_workspace_bytes(512) == 133136  # MOE_BUILD_BLOCKS_STATIC_BYTES in the header


@pytest.mark.parametrize("kind,shape", [("KIND_FP8_ROW", (4096, 14336, 8)), ("KIND_BF16", (2048, 14336, 8))])
def test_kept_weight_copies_depend_on_the_expert_shape_only(kind, shape):
    """What a kept weight copy holds (x4 read order or K-contiguous rows) follows from kind, weight type and
    (H, I, E) alone.  A call whose activations outgrow the large-tile kernels' 32-bit row offsets must not change the
    meaning of the copies: it ignores them and plans K-contiguous copies of its own in the workspace."""
    from nkilib import _native as nv

    L = nv.lib()
    H, I, E = shape
    kind = getattr(nv, kind)
    es = 2 if kind == nv.KIND_BF16 else 1
    small = _valid_args(nv, kind, 4097, H, I, E, 128, 71)
    n_big = 2**32 // (128 * I * es) + 1  # N * B * I * es >= 2^32: past the large-tile kernels' offsets
    big = _valid_args(nv, kind, 150001, H, I, E, 128, n_big)
    nbytes = lambda a, which: L.moe_kmajor_weights_bytes(ctypes.byref(a), which)
    ws = lambda a: L.moe_blockwise_workspace_bytes(ctypes.byref(a))
    for which in (0, 1):
        assert nbytes(small, which) > 0
        assert nbytes(small, which) == nbytes(big, which)
        # the x4 copies carry their unit scale tables behind the weights: more bytes than bare K-contiguous rows
        assert nbytes(small, which) > E * (2 if which == 0 else 1) * I * H * es
    fake = ctypes.c_void_p(4096)
    ws_small, ws_big = ws(small), ws(big)
    for a in (small, big):
        a.gate_up_proj_weight_kmajor = fake
        a.down_proj_weight_kmajor = fake
    assert ws(small) < ws_small - 2 * E * I * H * es  # kept copies used: none planned in the workspace
    assert ws(big) == ws_big  # kept copies ignored: the call still plans its own
