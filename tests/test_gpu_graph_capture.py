"""The whole layer (RMSNorm -> MXFP8 front end, block build, blockwise MoE) recorded into a HIP graph.

The library clears its counters and scratch tables with fill kernels and allocates nothing on the device itself, so
a caller may record the sequence once and replay it.  Each replay must reproduce the eager result bit for bit, also
with eager work of the same library (which shares the workspace and the kept weight copies) between the replays.
"""

import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind", ["mxfp8", "bf16"])
def test_layer_replays_from_a_graph(kind):
    import torch
    from nkilib import synthetic as syn
    from nkilib.core.moe.moe_cte import (MoECTEImplementation, MoECTESpec, QuantizationConfig, build_token_blocks,
                                         get_n_blocks, moe_cte)
    from nkilib.core.subkernels.rmsnorm_mx_quantize_tkg import rmsnorm_mx_quantize

    dev = torch.device("cuda:0")
    T, H, I, E, k, B = 700, 1024, 512, 4, 2, 128
    ids, aff = syn.route(T, E, k, dev, seed=5, mode="softmax")
    x = syn.hidden_states(T, H, dev, seed=5)
    N = get_n_blocks(T, k, E, B, n_block_per_iter=2)
    if kind == "mxfp8":
        gu_q, gu_s, d_q, d_s = syn.mx_expert_weights(E, H, I, 0.02, dev, seed=5)
        gu_x4 = gu_q.view(torch.int32).reshape(gu_q.shape[:-1])
        gamma = torch.ones((1, H), dtype=torch.bfloat16, device=dev)
        spec = MoECTESpec(implementation=MoECTEImplementation.shard_on_block_mx)
        qcfg = QuantizationConfig(gu_s, d_s)
    else:
        gen = torch.Generator(device=dev)
        gen.manual_seed(5)
        gu_w = (torch.randn((E, H, 2, I), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
        d_w = (torch.randn((E, I, H), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
        spec = MoECTESpec(implementation=MoECTEImplementation.shard_on_block)

    def layer():
        tp2id, b2e, cond = build_token_blocks(ids, E, B, N, n_conditions=N + 2)
        if kind == "mxfp8":
            xq, xs = rmsnorm_mx_quantize(x, gamma)
            return moe_cte[2](xq, aff.reshape(-1, 1), gu_x4, d_q, tp2id, b2e, B, spec, conditions=cond,
                              quantization_config=qcfg, hidden_states_scale=xs)
        return moe_cte(x, aff.reshape(-1, 1), gu_w, d_w, tp2id, b2e, B, spec, conditions=cond)

    for _ in range(2):  # the first call makes the kept weight copies and sizes the workspace
        eager = layer()
    torch.cuda.synchronize()
    eager = eager.clone()
    assert bool(eager.any())

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = layer()
    torch.cuda.synchronize()
    for replay in range(4):
        out.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {replay} differs from the eager result"
        assert torch.equal(layer(), eager)  # eager work between the replays
        torch.cuda.synchronize()
