"""GPU parity: RMSNorm-Quant front end (fp8 ROW / STATIC, MXFP8) through the C ABI vs the oracle.

Shapes and generators follow the reference's own test table
(test/integration/nkilib/core/rmsnorm/test_rmsnorm_quant.py:286-304): H = 16384, S in {2, 160, 2048},
gaussian / duplicate-row / all-ones inputs, lower_bound in {0, 0.5}.
Bar: codes bit exact except round-half ties (decided by fp32 summation order), dequant scale
within 4 ulp of the oracle: the golden's fp32 pairwise ``np.mean`` and the kernel's correctly
rounded sum differ by an ulp or two, which the three following roundings (rms, reciprocal,
product with gamma) can stretch to 3-4 ulp of amax.  The reference's own bar is rtol 0.072 for
values and 0.007 (~6e4 ulp) for the scale (:260-266).
"""

import numpy as np
import pytest

from helpers import bf16_tensor, f32_tensor
from oracle import rmsnorm as orn
from oracle.compare import fp8_codes_match_except_ties
from oracle.numerics import to_bf16

pytestmark = pytest.mark.gpu


def _unrounded_row(inp, gamma, lower_bound, quant_only, eps=1e-6):
    """The oracle's value right before the fp8 cast (float64 view of its fp32 pipeline)."""
    inp = inp.astype(np.float32)
    if quant_only:
        norm = inp
    else:
        rms = np.sqrt(np.mean(np.square(inp), axis=-1, keepdims=True))
        norm = inp * np.reciprocal(rms + np.float32(eps)) * gamma.astype(np.float32)
    amax = np.abs(norm).max(axis=-1, keepdims=True)
    if lower_bound > 0:
        amax = np.minimum(amax, np.float32(lower_bound))
        norm = np.clip(norm, -np.float32(lower_bound), np.float32(lower_bound))
    dq = np.maximum((amax / np.float32(240.0)).astype(np.float32), np.float32(1e-6))
    return norm * np.reciprocal(dq)


def _gen(kind, rows, H, rng):
    if kind == "gauss":
        x = rng.normal(size=(1, rows, H))
    elif kind == "dup":
        x = np.broadcast_to(rng.normal(size=(1, 1, H)), (1, rows, H)) / 100.0
    else:
        x = np.ones((1, rows, H))
    g = np.ones((1, H)) if kind == "ones" else rng.random((1, H))
    return to_bf16(x.astype(np.float32)), to_bf16(g.astype(np.float32))


@pytest.mark.parametrize(
    "rows,H,quant_only,kind,lower_bound",
    [
        (2, 16384, True, "gauss", 0.0),
        (2, 16384, True, "gauss", 0.5),
        (2, 16384, False, "gauss", 0.0),
        (2, 16384, False, "gauss", 0.5),
        (2048, 16384, False, "gauss", 0.0),
        (160, 16384, False, "dup", 0.0),
        (160, 16384, False, "ones", 0.0),
        (160, 16384, True, "gauss", 0.0),
        (33, 4096, False, "gauss", 0.0),
        (5, 1000, False, "gauss", 0.0),   # H not a multiple of 8: scalar path
        (7, 7168, False, "gauss", 0.0),
    ],
)
def test_row_quant(rows, H, quant_only, kind, lower_bound):
    import torch
    from nkilib.core.rmsnorm import RmsNormQuantKernelArgs, rmsnorm_quant_kernel
    from nkilib.core.rmsnorm.rmsnorm_quant import split_row_record
    from nkilib.core.utils.common_types import NormType, QuantizationType

    rng = np.random.default_rng(0)
    x, g = _gen(kind, rows, H, rng)
    dev = torch.device("cuda:0")
    kargs = RmsNormQuantKernelArgs(lower_bound=lower_bound,
                                   norm_type=NormType.NO_NORM if quant_only else NormType.RMS_NORM,
                                   quantization_type=QuantizationType.ROW)
    out = rmsnorm_quant_kernel[2](bf16_tensor(x, dev), bf16_tensor(g, dev), kargs)
    assert tuple(out.shape) == (1, rows, H + 4) and out.dtype == torch.float8_e4m3fn
    codes_t, scale_t = split_row_record(out)
    codes = codes_t.view(torch.uint8).cpu().numpy()
    scale = scale_t.cpu().numpy()
    g_codes, g_scale = orn.rmsnorm_quant_ref(x, g, None, lower_bound, quant_only, "row")
    ulp = np.abs(scale.view(np.int32).astype(np.int64) - g_scale.view(np.int32).astype(np.int64))
    assert ulp.max() <= (0 if quant_only else 4), f"dequant scale differs by {ulp.max()} ulp"
    ok, n_bad, n_forgiven = fp8_codes_match_except_ties(codes, g_codes, _unrounded_row(x, g, lower_bound, quant_only))
    assert ok, f"{n_bad} mismatching codes, only {n_forgiven} are rounding ties"
    assert n_bad <= max(8, codes.size // 20000), f"too many tie flips: {n_bad} of {codes.size}"
    if kind == "ones":
        assert (codes == 0x77).all()  # 240.0


@pytest.mark.parametrize("rows,H,lower_bound", [(3, 512, 0.0), (130, 2048, 0.0), (257, 4096, 0.5), (33, 7168, 0.0),
                                                (9, 8200, 0.0), (17, 16384, 0.5)])
def test_row_quant_bf16_kernel_equals_the_general_one(rows, H, lower_bound):
    """bf16 input with bf16 gamma runs a specialised kernel; the same gamma values held as fp32 run the general one.
    Both do the same arithmetic in the same order: records equal byte for byte (codes and scale)."""
    import torch
    from nkilib.core.rmsnorm import RmsNormQuantKernelArgs, rmsnorm_quant_kernel

    rng = np.random.default_rng(7)
    x, g = _gen("gauss", rows, H, rng)
    x[0, 0, :5] = 0.0
    dev = torch.device("cuda:0")
    kargs = RmsNormQuantKernelArgs(lower_bound=lower_bound)
    xt, gt = bf16_tensor(x, dev), bf16_tensor(g, dev)
    fast = rmsnorm_quant_kernel(xt, gt, kargs).view(torch.uint8)
    general = rmsnorm_quant_kernel(xt, gt.float(), kargs).view(torch.uint8)
    assert torch.equal(fast, general)
    # the same pair of kernels with a static scale
    from nkilib.core.utils.common_types import QuantizationType
    kargs = RmsNormQuantKernelArgs(quantization_type=QuantizationType.STATIC)
    sc = f32_tensor(np.full((128, 1), 0.017, np.float32), dev)
    fast = rmsnorm_quant_kernel(xt, gt, kargs, sc).view(torch.uint8)
    general = rmsnorm_quant_kernel(xt, gt.float(), kargs, sc).view(torch.uint8)
    assert tuple(fast.shape)[-1] == H and torch.equal(fast, general)


@pytest.mark.parametrize("rows,H,quant_only", [(2, 16384, True), (160, 16384, False), (64, 4096, False)])
def test_static_quant(rows, H, quant_only):
    import torch
    from nkilib.core.rmsnorm import RmsNormQuantKernelArgs, rmsnorm_quant_kernel
    from nkilib.core.utils.common_types import NormType, QuantizationType

    rng = np.random.default_rng(1)
    x, g = _gen("gauss", rows, H, rng)
    sc = np.full((128, 1), 0.031, np.float32)
    dev = torch.device("cuda:0")
    kargs = RmsNormQuantKernelArgs(norm_type=NormType.NO_NORM if quant_only else NormType.RMS_NORM,
                                   quantization_type=QuantizationType.STATIC)
    out = rmsnorm_quant_kernel(bf16_tensor(x, dev), bf16_tensor(g, dev), kargs, f32_tensor(sc, dev))
    assert tuple(out.shape) == (1, rows, H)
    codes = out.view(torch.uint8).cpu().numpy()
    g_codes, _ = orn.rmsnorm_quant_ref(x, g, sc, 0.0, quant_only, "static")
    xf = x.astype(np.float32)
    if quant_only:
        norm = xf
    else:
        rms = np.sqrt(np.mean(np.square(xf), axis=-1, keepdims=True))
        norm = xf * np.reciprocal(rms + np.float32(1e-6)) * g.astype(np.float32)
    unr = np.clip(norm * np.reciprocal(np.float32(0.031)), -240, 240)
    ok, n_bad, n_forgiven = fp8_codes_match_except_ties(codes, g_codes, unr)
    assert ok, f"{n_bad} mismatching codes, only {n_forgiven} are rounding ties"


def test_zero_row_follows_kernel_rule():
    """All-zero row: dq = 1e-6 (the reference kernel's clamp), codes 0; no NaN."""
    import torch
    from nkilib.core.rmsnorm import RmsNormQuantKernelArgs, rmsnorm_quant_kernel
    from nkilib.core.rmsnorm.rmsnorm_quant import split_row_record
    from nkilib.core.utils.common_types import NormType

    dev = torch.device("cuda:0")
    x = torch.zeros((3, 512), dtype=torch.bfloat16, device=dev)
    out = rmsnorm_quant_kernel(x, None, RmsNormQuantKernelArgs(norm_type=NormType.NO_NORM))
    codes, scale = split_row_record(out)
    assert (codes.view(torch.uint8) == 0).all()
    assert torch.equal(scale.cpu(), torch.full((3, 1), 1e-6, dtype=torch.float32))


def _mx_blocks_explained_by_bf16_ties(norm32_k, q, s, g_q, g_s, window=8):
    """Every MX block (32 consecutive k') in which the kernel's codes or scale byte differ from the oracle's must be
    explained by a rounding tie: the oracle rounds its fp32 normalised value to bf16 before quantising, and a value
    within `window` fp32 ulps of a bf16 rounding boundary may legitimately round the other way when the row's sum of
    squares is accumulated in another order.  The fp8 rounding behind it is exact in both (a bf16 value times a power
    of two), so nothing else may differ: for each differing block some choice of "other neighbour" for its
    boundary values must reproduce the kernel's 32 codes and its scale byte exactly.

    norm32_k: the oracle's unrounded fp32 normalised values [T, H] in k' order.  Returns (number of differing blocks,
    number of differing codes, number of differing scale bytes, unexplained blocks)."""
    from oracle.mx import quantize_mx

    T, H = norm32_k.shape
    bits = norm32_k.view(np.uint32)
    low = (bits & 0xFFFF).astype(np.int64)
    near = np.abs(low - 0x8000) <= window
    trunc = bits & np.uint32(0xFFFF0000)
    up = trunc + np.uint32(0x10000)
    rne_up = (low > 0x8000) | ((low == 0x8000) & (((bits >> 16) & 1) == 1))
    b0 = np.where(rne_up, up, trunc).view(np.float32)
    b1 = np.where(rne_up, trunc, up).view(np.float32)
    diff_codes = q != g_q
    diff_scale = s != g_s
    blk = diff_codes.reshape(T, H // 32, 32).any(axis=2) | diff_scale
    unexplained = []
    for t, j in zip(*np.nonzero(blk)):
        sl = slice(32 * j, 32 * j + 32)
        cand = np.nonzero(near[t, sl])[0]
        ok = False
        if 0 < cand.size <= 8:
            for mask in range(1, 1 << cand.size):
                v = b0[t, sl].copy()
                for bit, idx in enumerate(cand):
                    if mask >> bit & 1:
                        v[idx] = b1[t, sl][idx]
                cq, cs = quantize_mx(v.reshape(8, 4))
                if np.array_equal(cq.reshape(-1), q[t, sl]) and cs.reshape(-1)[0] == s[t, j]:
                    ok = True
                    break
        if not ok:
            unexplained.append((int(t), int(j), int(cand.size)))
    return int(blk.sum()), int(diff_codes.sum()), int(diff_scale.sum()), unexplained


@pytest.mark.parametrize("T,H,do_norm", [(4, 512, True), (64, 2048, True), (33, 7168, True), (16, 16384, True),
                                          (40, 1024, False),
                                          # short rows share a workgroup (four of up to 64 MX blocks, two of up to
                                          # 128): row counts that leave the last workgroup partly empty
                                          (5, 1536, True), (7, 4096, True), (3, 3072, True),
                                          # BASELINE config 4's row length, a few hundred rows
                                          (300, 7168, True)])
def test_mx_front_end(T, H, do_norm):
    """RMSNorm -> MXFP8 (token-major and the reference's [128, H/512, T] layouts) vs the oracle: bit exact except
    where a bf16 rounding tie of the normalised value explains the difference, and those are counted."""
    import torch
    from nkilib.core.subkernels.rmsnorm_mx_quantize_tkg import rmsnorm_mx_quantize, rmsnorm_mx_quantize_tkg

    rng = np.random.default_rng(2)
    x = to_bf16((rng.standard_normal((T, H)) * rng.choice([0.01, 1.0, 30.0], size=(T, 1))).astype(np.float32))
    g = to_bf16(rng.random((1, H)).astype(np.float32) + 0.5)
    ref = orn.rmsnorm_mx_quant_ref(x, g if do_norm else None, do_norm=do_norm)
    dev = torch.device("cuda:0")
    q, s = rmsnorm_mx_quantize(bf16_tensor(x, dev), bf16_tensor(g, dev) if do_norm else None, do_norm=do_norm)
    q, s = q.cpu().numpy(), s.cpu().numpy()
    if not do_norm:
        # pure quantisation has no reduction: bit exact
        assert np.array_equal(q, ref["tok_quant"]) and np.array_equal(s, ref["tok_scale"])
        return
    norm32 = np.ascontiguousarray(orn.rms_norm(x, g)[:, orn.mx_k_order(H)], dtype=np.float32)
    n_blk, n_codes, n_scales, unexplained = _mx_blocks_explained_by_bf16_ties(norm32, q, s, ref["tok_quant"], ref["tok_scale"])
    print(f"MX front end T={T} H={H}: {n_codes} of {q.size} codes and {n_scales} of {s.size} scale bytes differ, in "
          f"{n_blk} blocks; unexplained: {len(unexplained)}", flush=True)
    assert not unexplained, f"blocks (token, block, boundary values) that no rounding tie explains: {unexplained[:8]}"
    assert n_codes <= max(8, q.size // 20000), f"too many tie flips: {n_codes} of {q.size} codes"
    assert n_scales <= max(2, s.size // 20000), f"too many scale bytes differ: {n_scales} of {s.size}"
    if T % 4 == 0:
        nT = H // 512
        out = torch.empty((128, T, H // 128), dtype=torch.bfloat16, device=dev)
        oq = torch.empty((128, nT, T), dtype=torch.int32, device=dev)
        osc = torch.zeros((128, nT, T), dtype=torch.uint8, device=dev)
        rmsnorm_mx_quantize_tkg(bf16_tensor(x.reshape(1, T, H), dev), bf16_tensor(g, dev), out, oq, osc)
        oq_b = oq.cpu().numpy().view(np.uint8).reshape(128, nT, T, 4)
        # same numbers as the token-major call, rearranged
        assert np.array_equal(oq_b.transpose(2, 1, 0, 3).reshape(T, H), q)
        rows = (np.arange(16) // 4) * 32 + np.arange(16) % 4
        assert np.array_equal(osc.cpu().numpy()[rows].transpose(2, 1, 0).reshape(T, H // 32), s)
        from helpers import from_bf16_tensor

        # the normalised bf16 copy: equal to the oracle's except at the same rounding boundaries
        o = from_bf16_tensor(out)                       # [128, T, H/128], h = h1*128 + p
        o_th = o.transpose(1, 2, 0).reshape(T, H)
        g_th = ref["out"].transpose(1, 2, 0).reshape(T, H)
        n32 = orn.rms_norm(x, g).astype(np.float32)
        low = (n32.view(np.uint32) & 0xFFFF).astype(np.int64)
        bad = o_th != g_th
        assert (np.abs(low[bad] - 0x8000) <= 8).all(), "a normalised value differs away from a bf16 rounding boundary"
        assert int(bad.sum()) <= max(8, o.size // 20000), f"{int(bad.sum())} of {o.size} normalised values differ"


@pytest.mark.parametrize("T,H,dtype", [(256, 2048, "bf16"), (260, 7168, "bf16"), (8, 16384, "bf16"), (12, 1024, "fp16"),
                                        (16, 1536, "fp32")])
def test_mx_front_end_residual(T, H, dtype):
    """Fused residual add (rmsnorm_mx_quantize_tkg.py:29-40; golden test_rmsnorm_mx_quantize_tkg.py:104-117), on the
    token-major layout and on the reference's [128, H/512, T] layout: output_residual is the sum rounded to the
    input type, bit for bit, and codes, scales and the normalised copy are bit-equal to the call without residual
    on that sum (the two calls run the same kernel arithmetic on the same row)."""
    import torch
    from helpers import from_bf16_tensor
    from nkilib.core.subkernels.rmsnorm_mx_quantize_tkg import rmsnorm_mx_quantize, rmsnorm_mx_quantize_tkg

    rng = np.random.default_rng(5)
    dev = torch.device("cuda:0")
    tdt = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[dtype]
    x = torch.from_numpy(rng.standard_normal((T, H)).astype(np.float32)).to(tdt).to(dev)
    r = torch.from_numpy((rng.standard_normal((T, H)) * 3).astype(np.float32)).to(tdt).to(dev)
    g = torch.from_numpy(rng.random((1, H)).astype(np.float32) + 0.5).to(tdt).to(dev)
    q, s, new_res = rmsnorm_mx_quantize(x, g, residual=r)
    want = x + r  # torch rounds the sum to the tensors' type
    assert new_res.dtype == tdt and torch.equal(new_res, want)
    q0, s0 = rmsnorm_mx_quantize(want, g)
    assert torch.equal(q, q0) and torch.equal(s, s0)
    if dtype == "bf16":
        # and against the oracle's residual branch, with the front end's tie rule
        xf, rf, gf = (from_bf16_tensor(t) for t in (x, r, g))
        ref = orn.rmsnorm_mx_quant_ref(xf, gf, residual=rf)
        assert np.array_equal(from_bf16_tensor(new_res), ref["out_residual"])
        norm32 = np.ascontiguousarray(orn.rms_norm(ref["out_residual"], gf)[:, orn.mx_k_order(H)], dtype=np.float32)
        n_blk, n_codes, n_scales, unexplained = _mx_blocks_explained_by_bf16_ties(
            norm32, q.cpu().numpy(), s.cpu().numpy(), ref["tok_quant"], ref["tok_scale"])
        print(f"residual front end T={T} H={H}: {n_codes} codes / {n_scales} scale bytes differ, unexplained {len(unexplained)}")
        assert not unexplained and n_codes <= max(8, q.numel() // 20000)
    if T % 4 == 0 and dtype != "fp32":
        nT = H // 512
        out = torch.empty((128, T, H // 128), dtype=torch.bfloat16, device=dev)
        oq = torch.empty((128, nT, T), dtype=torch.int32, device=dev)
        osc = torch.zeros((128, nT, T), dtype=torch.uint8, device=dev)
        ores = torch.empty((T, H), dtype=tdt, device=dev)
        res = rmsnorm_mx_quantize_tkg(x.reshape(1, T, H), g, out, oq, osc, residual=r.reshape(1, T, H), output_residual=ores)
        assert len(res) == 4 and res[3] is ores and torch.equal(ores, want)
        out0, oq0, osc0 = torch.empty_like(out), torch.empty_like(oq), torch.zeros_like(osc)
        rmsnorm_mx_quantize_tkg(want.reshape(1, T, H), g, out0, oq0, osc0)
        assert torch.equal(oq, oq0) and torch.equal(osc, osc0) and torch.equal(out, out0)
        oq_b = oq.cpu().numpy().view(np.uint8).reshape(128, nT, T, 4)
        assert np.array_equal(oq_b.transpose(2, 1, 0, 3).reshape(T, H), q.cpu().numpy())


def test_mx_front_end_residual_argument_rules():
    """The reference's argument rules for the residual pair (norm_tkg_utils.py:467,473-476)."""
    import torch
    from nkilib.core.subkernels.rmsnorm_mx_quantize_tkg import rmsnorm_mx_quantize_tkg

    dev = torch.device("cuda:0")
    T, H = 4, 512
    x = torch.zeros((1, T, H), dtype=torch.bfloat16, device=dev)
    g = torch.ones((1, H), dtype=torch.bfloat16, device=dev)
    out = torch.empty((128, T, H // 128), dtype=torch.bfloat16, device=dev)
    oq = torch.empty((128, 1, T), dtype=torch.int32, device=dev)
    osc = torch.zeros((128, 1, T), dtype=torch.uint8, device=dev)
    with pytest.raises(AssertionError, match="output_residual required"):
        rmsnorm_mx_quantize_tkg(x, g, out, oq, osc, residual=x)
    with pytest.raises(AssertionError, match="shapes must match"):
        rmsnorm_mx_quantize_tkg(x, g, out, oq, osc, residual=x[:, :2], output_residual=torch.empty((T, H), dtype=torch.bfloat16, device=dev))
    with pytest.raises(AssertionError, match="Only hidden_dim_tp=True is supported"):
        rmsnorm_mx_quantize_tkg(x, g, out, oq, osc, hidden_dim_tp=False)
