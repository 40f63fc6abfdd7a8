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
    assert L.moe_abi_version() == 3
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
    assert L.moe_rmsnorm_quant_mxfp8(ctypes.c_void_p(256), 0, None, 0, ctypes.c_void_p(256), ctypes.c_void_p(256), None,
                                     4, 500, 1e-6, 500, 0, 0, None) == -2  # H % 512
    assert L.moe_rmsnorm_quant_fp8_row(ctypes.c_void_p(256), 0, None, 0, ctypes.c_void_p(256), 4, 32768, 1e-6, 0.0, 0,
                                       None) == -2  # H > 16384
    assert L.moe_build_blocks_workspace_bytes(256) >= 2 * 256 * 4
    with pytest.raises(AssertionError, match="NCC_INKI016"):
        nv.check(-2, "x")
