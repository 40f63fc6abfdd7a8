#!/usr/bin/env python3
"""Benchmark of the MoE context-encoding hot path on one MI355X.

One "step" is one pass of the whole path over one batch of synthetic input that is already
resident in HBM: RMSNorm -> MXFP8 quantise of the hidden states, token -> block index build from
the router's top-k ids, gate/up GEMM with fused SiLU(gate)*up and MXFP8 re-quantisation, down
GEMM with fused affinity scaling, and the per-token combine into bf16 rows.

Default workload: BASELINE config 4, DeepSeek-V3-shaped routed experts (T=8192, H=7168, I=2048,
E=256, top-8, block 128, MXFP8 weights ~11 GB).  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c3|c5-<T>|c2|bf16] [--no-cpu-baseline]

`--workload c2` times BASELINE config 2 instead (fp8 activations with a per-row scale from RMSNorm-Quant, fp8
weights with per-channel scales, Mixtral-8x7B shape) through the same entry points.
"""

import argparse
import gc
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "nki-library_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

METRIC = "MoE layer TFLOP/s and tokens/s (fp8/MXFP8), % of MFMA peak, 1x MI355X"
PEAK_FP8_TFLOPS = 5000.0  # MI355X dense fp8 / MXFP8 MFMA peak
PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch of the gate/up kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch, scaled by
# the copy-kernel calibration: FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).  The figure is read from the profile summary
# that holds the runs it comes from, and only while the kernel sources still hash to what that summary was taken
# from: a kernel changed since then has no measured traffic until it is profiled again.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "mx_gemm_c4_moe_layer.md")
TRAFFIC_SOURCES = ("nki-library_amd/csrc/bwmm_mx.hip", "nki-library_amd/csrc/bwmm.hpp")


def profiled_traffic(workload, routing):
    import hashlib
    import re

    if (workload, routing) != ("c4", "router") or not os.path.exists(TRAFFIC_PROFILE):
        return None
    text = open(TRAFFIC_PROFILE).read()
    sha = re.search(r"sha256 of [^:]*: `([0-9a-f]{64})`", text)
    val = re.search(r"traffic_bytes_per_launch: (\d+)", text)
    if not sha or not val:
        return None
    h = hashlib.sha256()
    for f in TRAFFIC_SOURCES:
        h.update(open(os.path.join(ROOT, f), "rb").read())
    if h.hexdigest() != sha.group(1):
        return None
    # the clock the part held during the profiled gate/up launches (GRBM_GUI_ACTIVE over the launch time)
    ghz = re.search(r"`mx_gemm_kernel<1, 0>` \|[^\n]*\| ([0-9.]+) GHz \|", text)
    return int(val.group(1)), (float(ghz.group(1)) if ghz else None)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c4")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--sustain-seconds", type=float, default=2.0,
                    help="after the timed steps keep running the same step for at least this long and report its pace "
                         "and the shader clock the GEMMs held (extra keys; 0 skips it)")
    ap.add_argument("--graph", action="store_true",
                    help="also record the step into a HIP graph and time its replays (extra key graph_ms_per_step; on by "
                         "default for the decode-sized workloads c5-<T>, where the eager step is bound by the host's "
                         "launch path and not by the GPU)")
    ap.add_argument("--cpu-blocks", type=int, default=48, help="blocks of the workload timed on the CPU oracle (48: 10-20 s)")
    ap.add_argument("--with-router", action="store_true",
                    help="start from hidden states: time the router top-k front end (synthetic router weights) as a "
                         "stage of its own and route with its output; the headline metric stays the MoE layer")
    ap.add_argument("--weights", default="mxfp8", choices=["mxfp8", "mxfp4"],
                    help="mxfp8: e4m3 expert weights (the reported workload); mxfp4: float4_e2m1fn_x4 weights, same "
                         "layer (diagnostic: half the weight bytes; no CPU baseline)")
    ap.add_argument("--no-mx-weight-copies", action="store_true",
                    help="diagnostic: read the MXFP8 expert weights in the reference layout in place instead of the "
                         "copies in the kernels' read order that moe_cte makes once per weight tensor pair")
    ap.add_argument("--no-block-plans", action="store_true",
                    help="diagnostic: build_token_blocks makes the three tables only and moe_cte derives its chunk / "
                         "slot bookkeeping from them itself (four more small launches per step)")
    ap.add_argument("--routing", default="router", choices=["router", "balanced"],
                    help="router: top-k of synthetic scores (the reported workload); balanced: every expert gets "
                         "exactly T*k/E rows (diagnostic, shows the cost of ragged expert loads)")
    return ap.parse_args()


def build_workload(name, dev, routing="router", weights="mxfp8"):
    import torch
    from nkilib import synthetic as syn

    if name.startswith("c5"):
        cfg = dict(syn.CONFIGS["c4"])
        cfg["T"] = int(name.split("-")[1]) if "-" in name else 128
        router_kw = dict(uniform_random=True)
    else:
        cfg = dict(syn.CONFIGS[name])
        router_kw = dict(mode="sigmoid") if name == "c4" else dict(mode="softmax", expert_bias_std=0.5 if name == "c3" else 0.0)
    assert cfg["kind"] == "mxfp8", "bench.py times the MXFP8 layer (configs c3, c4, c5-<T>)"
    T, H, I, E, k, B = (cfg[x] for x in ("T", "H", "I", "E", "k", "B"))
    t0 = time.time()
    if weights == "mxfp4":
        gu_q, gu_s, d_q, d_s = syn.mx4_expert_weights(E, H, I, dev, seed=0)
    else:
        gu_q, gu_s, d_q, d_s = syn.mx_expert_weights(E, H, I, 0.02, dev, seed=0)
    ids, aff = syn.route(T, E, k, dev, seed=0, **router_kw)
    if routing == "balanced":
        tt = torch.arange(T, device=dev).reshape(T, 1)
        jj = torch.arange(k, device=dev).reshape(1, k)
        ids = ((tt + jj * (E // k)) % E).to(torch.int32).contiguous()
        aff = torch.zeros((T + 1, E), dtype=torch.float32, device=dev)
        aff[:T].scatter_(1, ids.long(), torch.full((T, k), 1.0 / k, device=dev))
        aff = aff.to(torch.bfloat16)
    x = syn.hidden_states(T, H, dev, seed=0)
    gamma = torch.ones((1, H), dtype=torch.bfloat16, device=dev)
    torch.cuda.synchronize()
    cfg["gen_seconds"] = time.time() - t0
    return cfg, dict(x=x, gamma=gamma, ids=ids, aff=aff, gu_q=gu_q, gu_s=gu_s, d_q=d_q, d_s=d_s)


def cpu_baseline(cfg, t, tp2id, b2e, n_blocks):
    """The CPU oracle (a port of the reference's numpy golden) on the first ``n_blocks`` non-empty blocks of the
    same workload: normalise, quantise online, MX gate/up, act, MX down, affinity, accumulate."""
    import numpy as np
    import torch
    from oracle import moe as omoe
    from oracle import rmsnorm as orn
    from oracle.numerics import bf16_from_bits

    T, H, I, E, B = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["B"]
    tp = tp2id.cpu().numpy()
    be = b2e.cpu().numpy()
    tpb = tp.reshape(-1, B)
    keep = [b for b in range(tpb.shape[0]) if (tpb[b] < T).any()][:n_blocks]
    experts = sorted(set(int(be[b]) for b in keep))
    remap = {e: i for i, e in enumerate(experts)}
    sel = torch.tensor(experts, device=t["gu_q"].device)
    gu_q = t["gu_q"][sel].cpu().numpy()
    gu_s = t["gu_s"][sel].cpu().numpy()
    d_q = t["d_q"][sel].cpu().numpy()
    d_s = t["d_s"][sel].cpu().numpy()
    x = bf16_from_bits(t["x"].view(torch.int16).cpu().numpy().view(np.uint16))
    aff_full = bf16_from_bits(t["aff"].view(torch.int16).cpu().numpy().view(np.uint16))
    aff = np.ascontiguousarray(aff_full[:, experts])
    tp_s = np.concatenate([tpb[b] for b in keep])
    be_s = np.array([remap[int(be[b])] for b in keep], dtype=np.int32)
    rows = int(sum((tpb[b] < T).sum() for b in keep))
    t0 = time.perf_counter()
    tok = np.unique(tp_s[tp_s < T])
    normed = np.zeros_like(x)
    normed[tok] = orn.to_bf16(orn.rms_norm(x[tok], np.ones((1, H), np.float32)))
    omoe.moe_blockwise_mx_ref(normed, aff, gu_q, d_q, gu_s, d_s, tp_s, be_s, B)
    dt = time.perf_counter() - t0
    flops = 6.0 * rows * H * I
    return {
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": os.cpu_count(),
        "kind": "port",
        "sample": f"first {len(keep)} non-empty blocks ({rows} routed rows, {len(experts)} experts) of the same workload, "
                  f"numpy oracle incl. RMSNorm of their tokens, {dt:.1f} s",
        "tokens_per_s": rows / cfg["k"] / dt,
    }


class StepEvents:
    """HIP events of one step: three recorded here (torch's current stream: the stream every kernel of the path is
    launched on) around the front end and the block build, seven recorded by the library itself between the stages
    of the one moe_blockwise call (moe_bwmm_args.stage_events), so that the step is the ordinary step.  An event
    costs the GPU 7-8 us on this part (a barrier and a timestamp in the queue), so the K timed steps carry only the
    two around the dominant kernel (``gemm_only``: the gate/up launch, which the roofline prices); the per-stage
    table comes from K more steps, run after the timed ones, that carry all ten."""

    def __init__(self, torch, gemm_only=False):
        self.py = [None if gemm_only else torch.cuda.Event(enable_timing=True) for _ in range(3)]
        self.lib = [torch.cuda.Event(enable_timing=True) if (not gemm_only or i in (2, 3)) else None for i in range(7)]
        for e in self.py + self.lib:
            if e is not None:
                e.record()  # creates the HIP event, whose handle the library is given

    def mark(self, i):
        if self.py[i] is not None:
            self.py[i].record()

    def gate_up_ms(self):
        return self.lib[2].elapsed_time(self.lib[3])

    def stage_ms(self, with_requant):
        t = lambda a, b: a.elapsed_time(b)
        out = {"norm_quant": t(self.py[0], self.py[1]), "build_blocks": t(self.py[1], self.py[2]),
               "prep": t(self.py[2], self.lib[2]), "gate_up": t(self.lib[2], self.lib[3])}
        if with_requant:
            out["requant"] = t(self.lib[3], self.lib[4])
            out["down"] = t(self.lib[4], self.lib[5])
        else:
            out["down"] = t(self.lib[3], self.lib[5])
        out["combine"] = t(self.lib[5], self.lib[6])
        return out


def bench_fp8_row(args):
    """BASELINE config 2: RMSNorm-Quant (fp8 rows + fp32 row scale) -> block build -> fp8-row blockwise layer.
    `--workload bf16` runs the same stages on the bf16 kind (bf16 hidden states and weights, no front end, no row
    re-quantisation) at T=4096 H=2048 I=4096 E=8 top-2: a diagnostic for the general tiled kernel."""
    import numpy as np
    import torch
    from nkilib import _native as nv
    from nkilib import synthetic as syn
    from nkilib.core.moe.moe_cte import (MoECTEImplementation, MoECTESpec, QuantizationConfig, build_token_blocks,
                                         get_n_blocks, moe_cte)
    from nkilib.core.moe.moe_cte import _launch
    from nkilib.core.moe.moe_cte import block_index
    block_index.block_plans = not args.no_block_plans
    from nkilib.core.rmsnorm import RmsNormQuantKernelArgs, rmsnorm_quant_kernel

    dev = torch.device("cuda:0")
    nv.check(nv.lib().moe_check_device(), "device check")
    bf16 = args.workload == "bf16"
    cfg = dict(T=4096, H=2048, I=4096, E=8, k=2, B=128) if bf16 else dict(syn.CONFIGS["c2"])
    T, H, I, E, k, B = (cfg[x] for x in ("T", "H", "I", "E", "k", "B"))
    if bf16:
        g = torch.Generator(device=dev)
        g.manual_seed(0)
        gu_w = (torch.randn((E, H, 2, I), generator=g, device=dev) * 0.02).to(torch.bfloat16)
        d_w = (torch.randn((E, I, H), generator=g, device=dev) * 0.02).to(torch.bfloat16)
        gu_q = gu_s = d_q = d_s = None
    else:
        gu_q, gu_s, d_q, d_s = syn.fp8_channel_weights(E, H, I, 0.02, dev, seed=0)
    ids, aff = syn.route(T, E, k, dev, seed=0, mode="softmax")
    x = syn.hidden_states(T, H, dev, seed=0)
    gamma = torch.ones((1, H), dtype=torch.bfloat16, device=dev)
    N = get_n_blocks(T, k, E, B)
    spec = MoECTESpec(implementation=MoECTEImplementation.shard_on_block)
    if bf16:
        kw, gu8, d8 = {}, gu_w, d_w
        names = ["norm_quant", "build_blocks", "prep", "gate_up", "down", "combine"]
    else:
        kw = {"quantization_config": QuantizationConfig(gu_s, d_s)}
        gu8, d8 = gu_q.view(torch.float8_e4m3fn), d_q.view(torch.float8_e4m3fn)
        names = ["norm_quant", "build_blocks", "prep", "gate_up", "requant", "down", "combine"]
    timed_events = [StepEvents(torch, gemm_only=True) for _ in range(args.steps)]
    events = [StepEvents(torch) for _ in range(args.steps)]

    def step(ev):
        if ev:
            ev.mark(0)
        recs = x if bf16 else rmsnorm_quant_kernel(x, gamma, RmsNormQuantKernelArgs())
        if ev:
            ev.mark(1)
        tp2id, b2e, cond = build_token_blocks(ids, E, B, N)
        if ev:
            ev.mark(2)
        _launch.stage_events = ev.lib if ev else None
        out = moe_cte[2](recs, aff.reshape(-1, 1), gu8, d8, tp2id, b2e, B, spec, **kw)
        _launch.stage_events = None
        return out, recs, tp2id, b2e

    for _ in range(args.warmup):
        step(None)
    torch.cuda.synchronize()
    gc.collect()
    gc.disable()  # (as timeit does: a collection in the middle of the timed steps is the host's time, not the path's)
    t0 = time.perf_counter()
    for i in range(args.steps):
        out, recs, tp2id, b2e = step(timed_events[i])
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    gc.enable()
    gate_up_timed_ms = sum(ev.gate_up_ms() for ev in timed_events) / args.steps
    for i in range(args.steps):  # the per-stage table: the same steps again, every stage boundary recorded
        step(events[i])
    torch.cuda.synchronize()
    stage_ms = {n: 0.0 for n in names}
    for ev in events:
        for n, v in ev.stage_ms(with_requant=not bf16).items():
            stage_ms[n] += v / args.steps
    stage_ms["gate_up"] = gate_up_timed_ms  # (the launch duration the roofline uses: from the timed steps)
    routed = int((tp2id.reshape(-1) < T).sum().item())
    flops_layer, flops_gu = 6.0 * routed * H * I, 4.0 * routed * H * I
    tflops = flops_layer / (ms_per_step * 1e-3) / 1e12
    gu_tflops = flops_gu / (stage_ms["gate_up"] * 1e-3) / 1e12
    # gate/up GEMM: the K-contiguous fp8 weights once (they are made on the first call and kept), the routed fp8
    # rows with their scale, the fp32 intermediate written
    # (bf16 kind: bf16 weights and rows, bf16 intermediate)
    gu_bytes = (E * 2 * H * I * 2 + routed * H * 2 + routed * I * 2) if bf16 else (
        E * 2 * H * I + routed * (H + 4) + routed * I * 4)
    peak = PEAK_BF16_TFLOPS if bf16 else PEAK_FP8_TFLOPS
    roofline = {"bound": "mfma", "achieved": round(gu_tflops, 2), "peak": peak, "unit": "TFLOP/s",
                "frac": round(gu_tflops / peak, 4), "traffic": None,
                "kernel": ("moe::mx_gemm_kernel<1, 4> (gate/up blockwise GEMM of the bf16 kind on the large-tile kernels with "
                           "fused act*up, on the x4-ordered weight copies kept from the first call)" if bf16 else
                           "moe::mx_gemm_kernel<1, 3> (gate/up blockwise GEMM of the fp8-row kind on the large-tile "
                           "kernels with fused scales and act*up, on the x4-ordered weight copies kept from the first "
                           "call)"),
                "algorithmic_bytes": int(gu_bytes), "algorithmic_flops": int(flops_gu),
                "avg_launch_ms": round(stage_ms["gate_up"], 4)}
    res = {
        "metric": METRIC, "value": round(tflops, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 (fp32 accumulate)" if bf16 else
                 "fp8_e4m3 (per-row activation scale, per-channel weight scale, fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": (f"bf16: bf16 blockwise MoE layer T={T} H={H} I={I} E={E} top-{k} B={B} (N={N} blocks, "
                                f"{routed} routed rows), block build + gate/up + down + combine" if bf16 else
                                f"c2: fp8-row blockwise MoE layer T={T} H={H} I={I} E={E} top-{k} B={B} (N={N} blocks, "
                                f"{routed} routed rows), RMSNorm-Quant front end + block build + gate/up + row "
                                f"re-quantise + down + combine"),
                   "T": T, "H": H, "I": I, "E": E, "top_k": k, "block_size": B},
        "tokens_per_s": round(T / (ms_per_step * 1e-3), 1),
        "pct_of_mfma_peak": round(100.0 * tflops / peak, 2),
        "stage_ms": {n: round(v, 4) for n, v in stage_ms.items()},
        "roofline": roofline,
    }
    if not args.no_cpu_baseline and not bf16:
        from oracle import moe as omoe

        tpb = tp2id.cpu().numpy().reshape(-1, B)
        be = b2e.cpu().numpy()
        keep = [b for b in range(tpb.shape[0]) if (tpb[b] < T).any()][:24]
        experts = sorted(set(int(be[b]) for b in keep))
        remap = {e: i for i, e in enumerate(experts)}
        sel = torch.tensor(experts, device=dev)
        raw = recs.view(torch.uint8).cpu().numpy()
        codes, scale = raw[:, :H], raw[:, H:].copy().view(np.float32).reshape(-1)
        aff_np = aff.float().cpu().numpy()[:, experts]
        tp_s = np.concatenate([tpb[b] for b in keep])
        be_s = np.array([remap[int(be[b])] for b in keep], dtype=np.int32)
        rows = int(sum((tpb[b] < T).sum() for b in keep))
        wq = [w[sel].cpu().numpy() for w in (gu_q, d_q, gu_s, d_s)]
        t0 = time.perf_counter()
        omoe.moe_blockwise_fp8_row_ref(codes, scale, aff_np, wq[0], wq[1], wq[2], wq[3], tp_s, be_s, B)
        dt = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": 6.0 * rows * H * I / dt / 1e12, "unit": "TFLOP/s", "cores": os.cpu_count(),
                               "kind": "port",
                               "sample": f"first {len(keep)} non-empty blocks ({rows} routed rows) of the same workload, "
                                         f"numpy oracle, {dt:.1f} s"}
    print(json.dumps(res), flush=True)


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this build has no multi-GPU path (got --gpus {args.gpus}); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.workload in ("c2", "bf16"):
        return bench_fp8_row(args)
    import torch

    from nkilib import _native as nv
    from nkilib.core.moe.moe_cte import (MoECTEImplementation, MoECTESpec, QuantizationConfig, build_token_blocks,
                                         get_n_blocks, moe_cte)
    from nkilib.core.moe.moe_cte import _launch
    _launch.mx_weight_copies = not args.no_mx_weight_copies
    from nkilib.core.moe.moe_cte import block_index
    block_index.block_plans = not args.no_block_plans
    from nkilib.core.subkernels.rmsnorm_mx_quantize_tkg import rmsnorm_mx_quantize

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    dev = torch.device("cuda:0")
    nv.check(nv.lib().moe_check_device(), "device check")
    cfg, t = build_workload(args.workload, dev, args.routing, args.weights)
    fp4 = args.weights == "mxfp4"
    wb = 0.5 if fp4 else 1.0  # bytes per weight value
    T, H, I, E, k, B = (cfg[x] for x in ("T", "H", "I", "E", "k", "B"))
    N = get_n_blocks(T, k, E, B, n_block_per_iter=2)
    spec = MoECTESpec(implementation=MoECTEImplementation.shard_on_block_mx)
    qcfg = QuantizationConfig(t["gu_s"], t["d_s"])
    gu_x4 = t["gu_q"] if fp4 else t["gu_q"].view(torch.int32).reshape(t["gu_q"].shape[:-1])

    names = ["norm_quant", "build_blocks", "prep", "gate_up", "down", "combine"]
    if args.with_router:
        from nkilib.core.router_topk import route_for_moe
        from nkilib.core.utils.common_types import RouterActFnType

        names = ["router"] + names
        g = torch.Generator(device=dev)
        g.manual_seed(77)
        w_router = (torch.randn((H, E), generator=g, device=dev) * 0.05).to(torch.bfloat16)
    timed_events = [StepEvents(torch, gemm_only=True) for _ in range(args.steps)]
    events = [StepEvents(torch) for _ in range(args.steps)]
    router_events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]

    def step(timed, i=0, all_stages=False):
        ev = (events[i] if all_stages else timed_events[i]) if timed else None
        if args.with_router:
            if all_stages:
                router_events[i][0].record()
            t["ids"], t["aff"] = route_for_moe(t["x"], w_router, None, k, RouterActFnType.SIGMOID, norm_topk_prob=True)
            if all_stages:
                router_events[i][1].record()
        if ev:
            ev.mark(0)
        xq, xs = rmsnorm_mx_quantize(t["x"], t["gamma"])
        if ev:
            ev.mark(1)
        tp2id, b2e, cond = build_token_blocks(t["ids"], E, B, N, n_conditions=N + 2)
        if ev:
            ev.mark(2)
        _launch.stage_events = ev.lib if ev else None
        out = moe_cte[2](xq, t["aff"].reshape(-1, 1), gu_x4, t["d_q"], tp2id, b2e, B, spec, conditions=cond,
                         quantization_config=qcfg, hidden_states_scale=xs)
        _launch.stage_events = None
        return out, tp2id, b2e

    for _ in range(args.warmup):
        step(False)
    torch.cuda.synchronize()
    gc.collect()
    gc.disable()  # (as timeit does: a collection in the middle of the timed steps is the host's time, not the path's)
    t0 = time.perf_counter()
    for i in range(args.steps):
        out, tp2id, b2e = step(True, i)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    gc.enable()
    ms_per_step = wall * 1e3 / args.steps

    gate_up_timed_ms = sum(ev.gate_up_ms() for ev in timed_events) / args.steps
    for i in range(args.steps):  # the per-stage table: the same steps again, every stage boundary recorded
        step(True, i, all_stages=True)
    torch.cuda.synchronize()
    stage_ms = {n: 0.0 for n in names}
    for i, ev in enumerate(events):
        for n, v in ev.stage_ms(with_requant=False).items():
            stage_ms[n] += v
        if args.with_router:
            stage_ms["router"] += router_events[i][0].elapsed_time(router_events[i][1])
    stage_ms = {n: v / args.steps for n, v in stage_ms.items()}
    stage_ms["gate_up"] = gate_up_timed_ms  # (the launch duration the roofline uses: from the timed steps)

    # Sustained pace: the same step, back to back, for at least --sustain-seconds more (the clock under load is a
    # power-management outcome with a time constant beyond the timed steps).  Workgroup 0 of each GEMM launch
    # reports its shader cycles and the ticks of the constant 100 MHz counter: their ratio is the clock it ran at.
    sustained = None
    if args.sustain_seconds > 0:
        clk = torch.zeros(4, dtype=torch.int64, device=dev)
        _launch.gemm_clock_probe = clk
        n_sus = 0
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        while True:
            for _ in range(args.steps):
                step(False)
            n_sus += args.steps
            torch.cuda.synchronize()
            if time.perf_counter() - t1 >= args.sustain_seconds:
                break
        sus_ms = (time.perf_counter() - t1) * 1e3 / n_sus
        _launch.gemm_clock_probe = None
        c = [int(v) for v in clk.cpu().tolist()]
        sustained = {"ms_per_step": sus_ms, "steps": n_sus,
                     "ghz_gate_up": (c[0] / c[1] * 0.1) if c[1] else None,
                     "ghz_down": (c[2] / c[3] * 0.1) if c[3] else None}

    # The step recorded once into a HIP graph and replayed: what a decode loop would run.  The library allocates
    # nothing on the device during a step (workspace and kept weight copies exist after the warm-up), so the recorded
    # launches are the eager ones; the result of every replay is compared with the eager result.
    graph_ms = None
    if (args.graph or args.workload.startswith("c5")) and not args.with_router:
        ref = out.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step(False)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            g_out = step(False)[0]
        for _ in range(max(args.warmup, 1)):
            graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_out, ref), "a graph replay differs from the eager step"
        t2 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t2) * 1e3 / args.steps
        assert torch.equal(g_out, ref), "a graph replay differs from the eager step"
        del graph

    routed = int((tp2id.reshape(-1) < T).sum().item())  # == T*k
    flops_layer = 6.0 * routed * H * I
    flops_gate_up = 4.0 * routed * H * I
    tflops = flops_layer / (ms_per_step * 1e-3) / 1e12
    gate_up_tflops = flops_gate_up / (stage_ms["gate_up"] * 1e-3) / 1e12
    e_hit = int(torch.unique(t["ids"]).numel())
    weight_bytes = e_hit * 3 * H * I * (wb + 1 / 32)
    # HBM-bound front end: bytes = rows*H*(2 in + 1 out) + scales
    nq_gbs = (T + 1) * H * (3 + 1 / 32) / (stage_ms["norm_quant"] * 1e-3) / 1e9
    comb_gbs = (routed * H * 2 + (T + 1) * H * 2) / (stage_ms["combine"] * 1e-3) / 1e9

    # Roofline of the dominant kernel, the gate/up GEMM (mx_gemm_kernel<1>).  Algorithmic work per launch:
    #   flops = 4 * routed_rows * H * I
    #   bytes = expert weights hit (2*H*I fp8 + E8M0 scales) + routed activation rows (H fp8 + scales)
    #           + re-quantised intermediate rows written (I fp8 + scales)
    # The roof that binds is the one with the larger time floor at MI355X's published peaks.
    gu_bytes = e_hit * 2 * H * I * (wb + 1 / 32) + routed * H * (1 + 1 / 32) + routed * I * (1 + 1 / 32)
    gu_s = stage_ms["gate_up"] * 1e-3
    floor_mfma = flops_gate_up / (PEAK_FP8_TFLOPS * 1e12)
    floor_hbm = gu_bytes / (PEAK_HBM_GBS * 1e9)
    prof = None if fp4 else profiled_traffic(args.workload, args.routing)
    measured, sclk_ghz = prof if prof else (None, None)
    if floor_hbm >= floor_mfma:
        roofline = {"bound": "hbm", "achieved": round(gu_bytes / gu_s / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": round(gu_bytes / gu_s / 1e9 / PEAK_HBM_GBS, 4)}
    else:
        roofline = {"bound": "mfma", "achieved": round(gate_up_tflops, 2), "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(gate_up_tflops / PEAK_FP8_TFLOPS, 4)}
    roofline.update({
        "traffic": measured,
        "kernel": "moe::mx_gemm_kernel<1> (gate/up blockwise MXFP8 GEMM, fused act*up + MX re-quantisation)",
        "algorithmic_bytes": int(gu_bytes),
        "algorithmic_flops": int(flops_gate_up),
        "avg_launch_ms": round(stage_ms["gate_up"], 4),
        "frac_of_mfma_peak": round(gate_up_tflops / PEAK_FP8_TFLOPS, 4),
        "frac_of_hbm_peak": round(gu_bytes / gu_s / 1e9 / PEAK_HBM_GBS, 4),
    })
    if sclk_ghz:
        # 256 CUs x 4 SIMDs, one 16x16x128 MFMA (65536 flop) per 32 cycles and SIMD
        roofline["sclk_ghz_profiled"] = sclk_ghz
        roofline["mfma_peak_at_that_clock_TFLOPs"] = round(1024 * 2048 * sclk_ghz / 1e3, 1)
    if sustained and sustained["ghz_gate_up"]:
        # the clock the gate/up launch itself reported at the end of the sustained run
        roofline["sclk_ghz_sustained"] = round(sustained["ghz_gate_up"], 3)
        roofline["mfma_peak_at_sustained_clock_TFLOPs"] = round(1024 * 2048 * sustained["ghz_gate_up"] / 1e3, 1)

    res = {
        "metric": METRIC,
        "value": round(tflops, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("mxfp8_e4m3 activations x mxfp4_e2m1 weights" if fp4 else "mxfp8_e4m3") + " (E8M0 block scales, fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: {'MXFP4-weight' if fp4 else 'MXFP8'} blockwise MoE layer T={T} H={H} I={I} E={E} top-{k} B={B} "
                               f"(N={N} blocks, {routed} routed rows), RMSNorm->MXFP8 front end + block build + "
                               f"gate/up + down + combine",
                   "T": T, "H": H, "I": I, "E": E, "top_k": k, "block_size": B},
        "tokens_per_s": round(T / (ms_per_step * 1e-3), 1),
        "experts_hit": e_hit,
        "expert_weight_bytes": int(weight_bytes),
        "gemm_phase_TFLOPs": round(flops_layer / ((stage_ms["gate_up"] + stage_ms["down"]) * 1e-3) / 1e12, 2),
        "pct_of_fp8_mfma_peak": round(100.0 * tflops / PEAK_FP8_TFLOPS, 2),
        "stage_ms": {n: round(v, 4) for n, v in stage_ms.items()},
        "stage_rates": {
            "gate_up_TFLOPs": round(gate_up_tflops, 2),
            "down_TFLOPs": round(2.0 * routed * H * I / (stage_ms["down"] * 1e-3) / 1e12, 2),
            "norm_quant_GBs": round(nq_gbs, 1),
            "combine_GBs": round(comb_gbs, 1),
            "weights_GBs_over_gemm_time": round(weight_bytes / ((stage_ms["gate_up"] + stage_ms["down"]) * 1e-3) / 1e9, 1),
        },
        "roofline": roofline,
    }
    if graph_ms is not None:
        res["graph_ms_per_step"] = round(graph_ms, 4)
        res["graph_TFLOPs"] = round(flops_layer / (graph_ms * 1e-3) / 1e12, 2)
    if sustained:
        res["sustained_ms_per_step"] = round(sustained["ms_per_step"], 4)
        res["sustained_steps"] = sustained["steps"]
        res["sustained_TFLOPs"] = round(flops_layer / (sustained["ms_per_step"] * 1e-3) / 1e12, 2)
        res["sustained_sclk_ghz"] = {"gate_up": round(sustained["ghz_gate_up"], 3) if sustained["ghz_gate_up"] else None,
                                     "down": round(sustained["ghz_down"], 3) if sustained["ghz_down"] else None}
    if not args.no_cpu_baseline and not fp4:
        res["cpu_baseline"] = cpu_baseline(cfg, t, tp2id, b2e, args.cpu_blocks)
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
