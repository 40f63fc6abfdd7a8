"""GPU parity at BASELINE's full sizes (config 4: T=8192, H=7168, I=2048, E=256, top-8, B=128, MXFP8).

The whole-layer golden takes hours on a CPU at this size, so the layer is checked through
  * sampled tokens against the oracle's per-token reference (explicit index formulas, fp64), which the
    CPU suite pins against the block-loop golden at small sizes;
  * properties that hold at any size: the padding row stays zero, a second run is bit-identical
    (no atomics anywhere), and permuting the tokens permutes the output rows bit-exactly (each token's
    contributions are accumulated in ascending expert order whatever slots they sit in).
Inputs are generated on the GPU by nkilib.synthetic, as in bench.py.
"""

import numpy as np
import pytest

from oracle import moe as omoe
from oracle import rmsnorm as orn
from oracle.compare import max_abs_rel, max_all_close
from oracle.numerics import bf16_from_bits

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-2, 1e-5


def _layer(t, cfg, ids, aff, x):
    import torch
    from nkilib.core.moe.moe_cte import (MoECTEImplementation, MoECTESpec, QuantizationConfig, build_token_blocks,
                                         get_n_blocks, moe_cte)
    from nkilib.core.subkernels.rmsnorm_mx_quantize_tkg import rmsnorm_mx_quantize

    T, E, k, B = cfg["T"], cfg["E"], cfg["k"], cfg["B"]
    N = get_n_blocks(T, k, E, B, n_block_per_iter=2)
    xq, xs = rmsnorm_mx_quantize(x, t["gamma"])
    tp2id, b2e, cond = build_token_blocks(ids, E, B, N, n_conditions=N + 2)
    gu_x4 = t["gu_q"].view(torch.int32).reshape(t["gu_q"].shape[:-1])
    out = moe_cte[2](xq, aff.reshape(-1, 1), gu_x4, t["d_q"], tp2id, b2e, B,
                     MoECTESpec(implementation=MoECTEImplementation.shard_on_block_mx), conditions=cond,
                     quantization_config=QuantizationConfig(t["gu_s"], t["d_s"]), hidden_states_scale=xs)
    torch.cuda.synchronize()
    return out


def _bf16_np(tensor):
    import torch

    return bf16_from_bits(tensor.contiguous().view(torch.int16).cpu().numpy().view(np.uint16))


_C4 = {}


def _c4_experts():
    """BASELINE config 4's expert weights (11 GB on the GPU), generated once for the tests of this module."""
    import torch
    from nkilib import synthetic as syn

    if not _C4:
        dev = torch.device("cuda:0")
        cfg = dict(syn.CONFIGS["c4"])
        gu_q, gu_s, d_q, d_s = syn.mx_expert_weights(cfg["E"], cfg["H"], cfg["I"], 0.02, dev, seed=0)
        _C4.update(cfg=cfg, t=dict(gu_q=gu_q, gu_s=gu_s, d_q=d_q, d_s=d_s,
                                   gamma=torch.ones((1, cfg["H"]), dtype=torch.bfloat16, device=dev)))
    return _C4["cfg"], _C4["t"]


def _check_tokens_against_oracle(t, x, ids, aff, out_rows, toks, what):
    """Rows `toks` of the layer's output against the grouped per-expert oracle (each expert decoded once for all
    the tokens that use it, experts spread over a thread pool)."""
    from concurrent.futures import ThreadPoolExecutor

    import torch

    H = x.shape[1]
    sel = torch.tensor(list(toks), device=x.device)
    x_np = _bf16_np(x[sel])
    aff_np = _bf16_np(aff[sel])
    ids_np = ids[sel].cpu().numpy()
    out_rows = out_rows[sel]
    experts = [sorted(int(e) for e in row) for row in ids_np]
    affs = [[aff_np[i, e] for e in es] for i, es in enumerate(experts)]
    normed = orn.to_bf16(orn.rms_norm(x_np, np.ones((1, H), np.float32)))

    def weights(e):
        return tuple(t[n][e].cpu().numpy() for n in ("gu_q", "gu_s", "d_q", "d_s"))

    with ThreadPoolExecutor(max_workers=8) as pool:
        want = omoe.moe_mx_tokens_ref(normed, experts, affs, weights, map_fn=pool.map)
    o = _bf16_np(out_rows)
    worst = 0.0
    for i, tok in enumerate(toks):
        err = max_abs_rel(o[i], want[i])
        worst = max(worst, err)
        assert max_all_close(o[i], want[i].astype(np.float32), rtol=RTOL, atol=ATOL), \
            f"{what} token {tok} (experts {experts[i]}): max-abs-rel {err:.3e}"
    n_exp = len({e for es in experts for e in es})
    print(f"{what}: {len(toks)} tokens over {n_exp} experts, worst max-abs-rel {worst:.3e} (rtol {RTOL})", flush=True)


def test_c4_sampled_tokens_and_invariants():
    import torch
    from nkilib import synthetic as syn

    dev = torch.device("cuda:0")
    cfg, t = _c4_experts()
    T, H, I, E, k = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["k"]
    ids, aff = syn.route(T, E, k, dev, seed=0, mode="sigmoid")
    x = syn.hidden_states(T, H, dev, seed=0)
    out = _layer(t, cfg, ids, aff, x)
    assert out.shape[0] == 2 and not bool(out[1].any()), "second output plane must stay zero"
    assert not bool(out[0, T].any()), "padding row must stay zero"

    # determinism: no atomics, fixed accumulation order
    out2 = _layer(t, cfg, ids, aff, x)
    assert torch.equal(out, out2), "two runs of the same layer differ"

    # the bookkeeping handed over by the block build (used above) and the one the layer derives itself: same bits
    from nkilib.core.moe.moe_cte import block_index
    block_index.block_plans = False
    try:
        out3 = _layer(t, cfg, ids, aff, x)
    finally:
        block_index.block_plans = True
    assert torch.equal(out, out3), "the layer's result depends on where its bookkeeping came from"

    # permutation of the tokens permutes the rows, bit for bit
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    perm = torch.randperm(T, generator=g, device=dev)
    xp = x.clone()
    xp[:T] = x[perm]
    affp = aff.clone()
    affp[:T] = aff[perm]
    outp = _layer(t, cfg, ids[perm].contiguous(), affp, xp)
    assert torch.equal(outp[0, :T], out[0, :T][perm]), "token permutation changed some output row"

    # Tokens against the oracle, chosen by construction: the first and the last token (in slot order) of
    #   expert 0, expert 255 (the last; its gate/up weights start 6.97 GiB into the tensor), an expert just past the
    #   4 GiB mark of the gate/up weights, an expert with more than 256 rows (one 320-row chunk: the last token sits in
    #   the row tiles that accumulate outside the accumulation registers) and one with at most 256 rows.
    ids_np = ids.cpu().numpy()
    counts = np.bincount(ids_np.reshape(-1), minlength=E)
    per_expert_bytes = 128 * 2 * (H // 512) * I * 4
    e_4g = int(np.ceil(2**32 / per_expert_bytes))
    e_big = int(np.flatnonzero((counts > 256) & (counts <= 320))[0])
    e_small = int(np.flatnonzero((counts > 128) & (counts <= 256))[0])
    targets = [0, E - 1, e_4g, e_big, e_small]
    toks = []
    for e in targets:
        users = np.flatnonzero((ids_np == e).any(axis=1))  # ascending token id == slot order within the expert
        toks += [int(users[0]), int(users[-1])]
    toks = sorted(set(toks))
    assert len(toks) >= 8
    print(f"c4 targets: experts {targets} (rows {[int(counts[e]) for e in targets]}), tokens {toks}", flush=True)
    _check_tokens_against_oracle(t, x, ids, aff, out[0], toks, "c4")


@pytest.mark.parametrize("T", [1, 8, 32, 128])
def test_c5_decode_shaped(T):
    """BASELINE config 5: T in {1, 8, 32, 128} tokens on config 4's experts, uniform random top-8 (most experts
    hold one partially filled block: the smallest row-tile variant, streamed weights, single-slab block build).
    Every token for T <= 8, 8 tokens for T >= 32, against the per-expert oracle; padding row zero; reruns bit-equal."""
    import torch
    from nkilib import synthetic as syn

    dev = torch.device("cuda:0")
    cfg4, t = _c4_experts()
    cfg = dict(cfg4, T=T)
    H, E, k = cfg["H"], cfg["E"], cfg["k"]
    ids, aff = syn.route(T, E, k, dev, seed=50 + T, uniform_random=True)
    x = syn.hidden_states(T, H, dev, seed=50 + T)
    out = _layer(t, cfg, ids, aff, x)
    assert tuple(out.shape) == (2, T + 1, H)
    assert not bool(out[1].any()), "second output plane must stay zero"
    assert not bool(out[0, T].any()), "padding row must stay zero"
    assert bool(out[0, :T].any(dim=1).all()), "every token must receive a contribution"
    assert torch.equal(out, _layer(t, cfg, ids, aff, x)), "two runs of the same layer differ"
    toks = list(range(T)) if T <= 8 else [int(v) for v in np.linspace(0, T - 1, 8).round()]
    _check_tokens_against_oracle(t, x, ids, aff, out[0], toks, f"c5 T={T}")


def _subset_problem(ids, aff, x, keep, experts=None):
    """The layer restricted to the tokens `keep` (and, if given, to the listed experts, renumbered)."""
    import torch

    dev = ids.device
    T2 = keep.numel()
    ids2 = ids[keep]
    aff2 = torch.zeros((T2 + 1, aff.shape[1]), dtype=aff.dtype, device=dev)
    aff2[:T2] = aff[keep]
    if experts is not None:
        lut = torch.full((aff.shape[1],), -1, dtype=torch.int32, device=dev)
        lut[experts] = torch.arange(experts.numel(), dtype=torch.int32, device=dev)
        ids2 = lut[ids2.long()]
        assert int(ids2.min()) >= 0
        aff2 = aff2[:, experts]
    x2 = torch.zeros((T2 + 1, x.shape[1]), dtype=x.dtype, device=dev)
    x2[:T2] = x[keep]
    return ids2.contiguous(), aff2.contiguous(), x2


def test_c3_skewed_subset_equals_golden_and_full_run():
    """BASELINE config 3 (Qwen3-MoE shape, I=768 with a short last tile, skewed router): a 192-token subset is
    checked against the block-loop golden, and the full 8192-token run must give those tokens the same rows
    bit for bit (a token's row depends on nothing but its own experts, in ascending expert order)."""
    import torch
    from nkilib import synthetic as syn
    from nkilib.core.moe.moe_cte import build_token_blocks, get_n_blocks

    dev = torch.device("cuda:0")
    cfg = dict(syn.CONFIGS["c3"])
    T, H, I, E, k, B = (cfg[n] for n in ("T", "H", "I", "E", "k", "B"))
    gu_q, gu_s, d_q, d_s = syn.mx_expert_weights(E, H, I, 0.02, dev, seed=3)
    ids, aff = syn.route(T, E, k, dev, seed=3, mode="softmax", expert_bias_std=0.5)
    x = syn.hidden_states(T, H, dev, seed=3)
    t = dict(gu_q=gu_q, gu_s=gu_s, d_q=d_q, d_s=d_s, gamma=torch.ones((1, H), dtype=torch.bfloat16, device=dev))
    out = _layer(t, cfg, ids, aff, x)
    assert not bool(out[0, T].any())

    keep = torch.arange(5, T, T // 192, device=dev)[:192]
    ids2, aff2, x2 = _subset_problem(ids, aff, x, keep)
    cfg2 = dict(cfg, T=keep.numel())
    out2 = _layer(t, cfg2, ids2, aff2, x2)
    assert torch.equal(out2[0, :keep.numel()], out[0][keep]), "rows of the full run differ from the subset run"

    T2 = keep.numel()
    N2 = get_n_blocks(T2, k, E, B, n_block_per_iter=2)
    tp2id, b2e, cond = build_token_blocks(ids2, E, B, N2, n_conditions=N2 + 2)
    normed = orn.to_bf16(orn.rms_norm(_bf16_np(x2), np.ones((1, H), np.float32)))
    normed[T2] = 0
    g = omoe.moe_blockwise_mx_ref(normed, _bf16_np(aff2), gu_q.cpu().numpy(), d_q.cpu().numpy(), gu_s.cpu().numpy(),
                                  d_s.cpu().numpy(), tp2id.cpu().numpy().reshape(-1), b2e.cpu().numpy().reshape(-1), B,
                                  conditions=cond.cpu().numpy().reshape(-1))
    o = _bf16_np(out2[0])
    err = max_abs_rel(o[:T2], g[:T2])
    print(f"c3 subset of {T2} tokens: max-abs-rel {err:.3e} (rtol {RTOL})", flush=True)
    assert max_all_close(o[:T2], g[:T2], rtol=RTOL, atol=ATOL)


def test_c2_fp8_row_subset_equals_golden_and_full_run():
    """BASELINE config 2 (Mixtral-8x7B shape, fp8 per-row activations x per-channel weights): the tokens routed
    to experts {0, 1} only are checked against the golden, and against their rows in the full 4096-token run."""
    import torch
    from nkilib import synthetic as syn
    from nkilib.core.moe.moe_cte import (MoECTEImplementation, MoECTESpec, QuantizationConfig, build_token_blocks,
                                         get_n_blocks, moe_cte)
    from nkilib.core.rmsnorm import RmsNormQuantKernelArgs, rmsnorm_quant_kernel

    dev = torch.device("cuda:0")
    cfg = dict(syn.CONFIGS["c2"])
    T, H, I, E, k, B = (cfg[n] for n in ("T", "H", "I", "E", "k", "B"))
    gu_q, gu_s, d_q, d_s = syn.fp8_channel_weights(E, H, I, 0.02, dev, seed=2)
    ids, aff = syn.route(T, E, k, dev, seed=2, mode="softmax")
    x = syn.hidden_states(T, H, dev, seed=2)
    gamma = torch.ones((1, H), dtype=torch.bfloat16, device=dev)

    def layer(ids_, aff_, x_, gu_q_, gu_s_, d_q_, d_s_):
        T_, E_ = x_.shape[0] - 1, aff_.shape[1]
        N = get_n_blocks(T_, k, E_, B, n_block_per_iter=2)
        rec = rmsnorm_quant_kernel(x_, gamma, RmsNormQuantKernelArgs())
        tp2id, b2e, cond = build_token_blocks(ids_, E_, B, N, n_conditions=N + 2)
        out_ = moe_cte(rec, aff_.reshape(-1, 1), gu_q_.view(torch.float8_e4m3fn), d_q_.view(torch.float8_e4m3fn),
                       tp2id, b2e, B, MoECTESpec(implementation=MoECTEImplementation.shard_on_block),
                       conditions=cond, quantization_config=QuantizationConfig(gu_s_, d_s_))
        torch.cuda.synchronize()
        return rec, out_, tp2id, b2e, cond

    _, out, _, _, _ = layer(ids, aff, x, gu_q, gu_s, d_q, d_s)
    assert not bool(out[T].any())

    experts = torch.tensor([0, 1], device=dev)
    keep = torch.nonzero((ids < 2).all(dim=1)).reshape(-1)
    assert keep.numel() >= 32, keep.numel()
    ids2, aff2, x2 = _subset_problem(ids, aff, x, keep, experts)
    rec2, out2, tp2id, b2e, cond = layer(ids2, aff2, x2, gu_q[:2].contiguous(), gu_s[:2].contiguous(),
                                         d_q[:2].contiguous(), d_s[:2].contiguous())
    T2 = keep.numel()
    assert torch.equal(out2[:T2], out[keep]), "rows of the full run differ from the subset run"

    raw = rec2.view(torch.uint8).cpu().numpy()
    codes, scale = raw[:, :H], raw[:, H:].copy().view(np.float32).reshape(-1)
    g = omoe.moe_blockwise_fp8_row_ref(codes, scale, _bf16_np(aff2), gu_q[:2].cpu().numpy(), d_q[:2].cpu().numpy(),
                                       gu_s[:2].cpu().numpy(), d_s[:2].cpu().numpy(), tp2id.cpu().numpy().reshape(-1),
                                       b2e.cpu().numpy().reshape(-1), B, conditions=cond.cpu().numpy().reshape(-1))
    o = _bf16_np(out2)[:, 0]
    err = max_abs_rel(o[:T2], g[:T2])
    print(f"c2 subset of {T2} tokens: max-abs-rel {err:.3e} (rtol {RTOL})", flush=True)
    assert max_all_close(o[:T2], g[:T2], rtol=RTOL, atol=ATOL)


def test_bf16_layer_subset_equals_golden_and_full_run():
    """The bf16 kind at the size bench.py's `--workload bf16` times (T=4096 H=2048 I=4096 E=8 top-2: 1024 rows per
    expert, i.e. four 256-row chunks of one expert side by side on the large-tile kernels): the tokens routed to
    experts {0, 1} only are checked against the golden, and against their rows in the full 4096-token run."""
    import torch
    from nkilib import synthetic as syn
    from nkilib.core.moe.moe_cte import MoECTEImplementation, MoECTESpec, build_token_blocks, get_n_blocks, moe_cte

    dev = torch.device("cuda:0")
    T, H, I, E, k, B = 4096, 2048, 4096, 8, 2, 128
    gen = torch.Generator(device=dev)
    gen.manual_seed(3)
    gu_w = (torch.randn((E, H, 2, I), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    d_w = (torch.randn((E, I, H), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    ids, aff = syn.route(T, E, k, dev, seed=3, mode="softmax")
    x = syn.hidden_states(T, H, dev, seed=3)

    def layer(ids_, aff_, x_, gu_, d_):
        T_, E_ = x_.shape[0] - 1, aff_.shape[1]
        N = get_n_blocks(T_, k, E_, B, n_block_per_iter=2)
        tp2id, b2e, cond = build_token_blocks(ids_, E_, B, N, n_conditions=N + 2)
        out_ = moe_cte(x_, aff_.reshape(-1, 1), gu_, d_, tp2id, b2e, B,
                       MoECTESpec(implementation=MoECTEImplementation.shard_on_block), conditions=cond)
        torch.cuda.synchronize()
        return out_, tp2id, b2e, cond

    out, _, _, _ = layer(ids, aff, x, gu_w, d_w)
    assert not bool(out[T].any())

    experts = torch.tensor([0, 1], device=dev)
    keep = torch.nonzero((ids < 2).all(dim=1)).reshape(-1)
    assert keep.numel() >= 32, keep.numel()
    ids2, aff2, x2 = _subset_problem(ids, aff, x, keep, experts)
    gu2, d2 = gu_w[:2].contiguous(), d_w[:2].contiguous()
    out2, tp2id, b2e, cond = layer(ids2, aff2, x2, gu2, d2)
    T2 = keep.numel()
    assert torch.equal(out2[:T2], out[keep]), "rows of the full run differ from the subset run"

    g = omoe.moe_blockwise_ref(_bf16_np(x2), _bf16_np(aff2), _bf16_np(gu2), _bf16_np(d2), tp2id.cpu().numpy().reshape(-1),
                               b2e.cpu().numpy().reshape(-1), B, conditions=cond.cpu().numpy().reshape(-1))
    o = _bf16_np(out2)[:, 0]
    err = max_abs_rel(o[:T2], g[:T2])
    print(f"bf16 subset of {T2} tokens: max-abs-rel {err:.3e} (rtol {RTOL})", flush=True)
    assert max_all_close(o[:T2], g[:T2], rtol=RTOL, atol=ATOL)
