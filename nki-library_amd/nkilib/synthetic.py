"""Synthetic inputs of the BASELINE configurations, generated on the GPU with torch.

Used by ``bench.py`` and by the full-size parity tests.  Nothing here is on the hot path: the
generators only produce tensors in the layouts ``moe_cte`` / ``rmsnorm_quant_kernel`` consume
(reference generators: ``build_moe_bwmm_mx_cte``,
test/integration/nkilib/core/moe/moe_cte/test_utils.py:221-471; ``build_bwmm_inputs``,
test/integration/nkilib/core/moe/moe_cte/test_moe_cte_common.py:554-711).
"""

import math

import torch

CONFIGS = {
    # name: T, H, I, E, top_k, B, kind
    "c1": dict(T=256, H=512, I=1024, E=8, k=2, B=128, kind="bf16"),
    "c2": dict(T=4096, H=4096, I=14336, E=8, k=2, B=128, kind="fp8_row"),
    "c3": dict(T=8192, H=2048, I=768, E=128, k=8, B=128, kind="mxfp8"),
    "c4": dict(T=8192, H=7168, I=2048, E=256, k=8, B=128, kind="mxfp8"),
}


def mx_quantize_torch(x, block_dims):
    """OCP-MX e4m3 quantisation of ``x`` with blocks spanning ``block_dims`` (kept as size-1 dims in the scale).

    Same rule as the reference golden (test/utils/mx_utils.py:55-95): scale byte = max fp32 exponent
    field - 8 (clipped at 0), values divided by 2**(scale-127), clipped to +-448, cast RNE.
    Returns (uint8 codes shaped like x, uint8 scales with block dims reduced to 1).
    """
    x = x.to(torch.float32).contiguous()
    e = ((x.view(torch.int32) >> 23) & 0xFF).amax(dim=block_dims, keepdim=True)
    s = (e - 8).clamp_(min=0)
    inv = ((254 - s) << 23).to(torch.int32).view(torch.float32)
    q = (x * inv).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    return q, s.to(torch.uint8)


def mx_expert_weights(E, H, I, std, device, seed=0):
    """Random ~N(0, std) MXFP8 expert weights in the reference's x4 layouts.

    gate_up uint8 [E,128,2,H/512,I,4] + scale [E,16,2,H/512,I];
    down uint8 [E,p_I,ceil(I/512),H,4] + scale [E,ceil(p_I/8),ceil(I/512),H].
    """
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    nH, nI = H // 512, math.ceil(I / 512)
    pI = 128 if I > 512 else I // 4
    pI8 = math.ceil(pI / 8) * 8
    gu_q = torch.empty((E, 128, 2, nH, I, 4), dtype=torch.uint8, device=device)
    gu_s = torch.empty((E, 16, 2, nH, I), dtype=torch.uint8, device=device)
    d_q = torch.empty((E, pI, nI, H, 4), dtype=torch.uint8, device=device)
    d_s = torch.empty((E, pI8 // 8, nI, H), dtype=torch.uint8, device=device)
    tail = I % 512
    for e in range(E):
        w = torch.randn((16, 8, 2, nH, I, 4), generator=g, device=device) * std
        q, s = mx_quantize_torch(w, (1, 5))
        gu_q[e] = q.view(128, 2, nH, I, 4)
        gu_s[e] = s.view(16, 2, nH, I)
        w = torch.zeros((pI8, nI, H, 4), device=device)
        w[:pI] = torch.randn((pI, nI, H, 4), generator=g, device=device) * std
        if tail and I > 512:
            w[tail // 4:, nI - 1] = 0  # zero-padded partitions of the last intermediate tile
        q, s = mx_quantize_torch(w.view(pI8 // 8, 8, nI, H, 4), (1, 4))
        d_q[e] = q.view(pI8, nI, H, 4)[:pI]
        d_s[e] = s.view(pI8 // 8, nI, H)
    return gu_q, gu_s, d_q, d_s


def mx4_expert_weights(E, H, I, device, seed=0):
    """Random MXFP4 expert weights for timing runs: uniformly random 4-bit patterns in the reference's x4 layouts with
    2-byte elements (gate_up int16 [E,128,2,H/512,I], down int16 [E,p_I,ceil(I/512),H]) and one E8M0 scale
    (2**-8: values up to 6/256) everywhere."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    nH, nI = H // 512, math.ceil(I / 512)
    pI = 128 if I > 512 else I // 4
    pI8 = math.ceil(pI / 8) * 8
    gu_q = torch.randint(-32768, 32768, (E, 128, 2, nH, I), generator=g, device=device, dtype=torch.int16)
    d_q = torch.randint(-32768, 32768, (E, pI, nI, H), generator=g, device=device, dtype=torch.int16)
    gu_s = torch.full((E, 16, 2, nH, I), 119, dtype=torch.uint8, device=device)
    d_s = torch.full((E, pI8 // 8, nI, H), 119, dtype=torch.uint8, device=device)
    return gu_q, gu_s, d_q, d_s


def fp8_channel_weights(E, H, I, std, device, seed=0):
    """~N(0, std) weights quantised to e4m3 (range 240) with per-output-channel fp32 scales (BASELINE config 2)."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    gu_q = torch.empty((E, H, 2, I), dtype=torch.uint8, device=device)
    gu_s = torch.empty((E, 1, 2 * I), dtype=torch.float32, device=device)
    d_q = torch.empty((E, I, H), dtype=torch.uint8, device=device)
    d_s = torch.empty((E, 1, H), dtype=torch.float32, device=device)
    for e in range(E):
        w = torch.randn((H, 2, I), generator=g, device=device) * std
        sc = w.abs().amax(dim=0, keepdim=True) / 240.0
        gu_q[e] = (w / sc).clamp_(-240, 240).to(torch.float8_e4m3fn).view(torch.uint8)
        gu_s[e] = sc.reshape(1, 2 * I)
        w = torch.randn((I, H), generator=g, device=device) * std
        sc = w.abs().amax(dim=0, keepdim=True) / 240.0
        d_q[e] = (w / sc).clamp_(-240, 240).to(torch.float8_e4m3fn).view(torch.uint8)
        d_s[e] = sc.reshape(1, H)
    return gu_q, gu_s, d_q, d_s


def route(T, E, k, device, seed=0, mode="softmax", expert_bias_std=0.0, uniform_random=False):
    """Synthetic router: returns (topk_ids int32 [T,k], dense masked affinities bf16 [T+1,E], row T zero).

    mode "softmax": logits ~N(0,1) (+ per-expert bias), softmax, top-k, affinities = softmax probabilities of the
    selected experts.  mode "sigmoid": sigmoid scores, top-k, renormalised to sum to one
    (``norm_topk_prob`` path, src/nkilib_src/nkilib/core/router_topk/router_topk_torch.py:96-105).
    """
    g = torch.Generator(device=device)
    g.manual_seed(seed + 1000)
    if uniform_random:
        scores = torch.rand((T, E), generator=g, device=device)
        ids = scores.topk(k, dim=1).indices
        vals = torch.full((T, k), 1.0 / k, device=device)
    else:
        logits = torch.randn((T, E), generator=g, device=device)
        if expert_bias_std > 0:
            logits = logits + torch.randn((1, E), generator=g, device=device) * expert_bias_std
        if mode == "softmax":
            p = torch.softmax(logits, dim=1)
            vals, ids = p.topk(k, dim=1)
        else:
            p = torch.sigmoid(logits)
            vals, ids = p.topk(k, dim=1)
            vals = vals / vals.sum(dim=1, keepdim=True)
    aff = torch.zeros((T + 1, E), dtype=torch.float32, device=device)
    aff[:T].scatter_(1, ids, vals)
    return ids.to(torch.int32).contiguous(), aff.to(torch.bfloat16)


def hidden_states(T, H, device, seed=0):
    """bf16 ~N(0,1) [T+1, H] with the zero padding row T."""
    g = torch.Generator(device=device)
    g.manual_seed(seed + 2000)
    x = torch.randn((T + 1, H), generator=g, device=device).to(torch.bfloat16)
    x[T] = 0
    return x
