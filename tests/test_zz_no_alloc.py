"""The entry point that allocates nothing, moe_build_blocks_static, against moe_build_blocks: same bits, on two calls
in a row (the second smaller, so that it runs on whatever the first left in the built-in scratch)."""

import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(L, nv, ids, E, B, N, skip_token, split, n_cond, dev):
    import torch

    T, k = ids.shape
    outs = []
    for static in (False, True):
        # poison the outputs so that a slot the kernels leave unwritten shows
        tp = torch.full((N * B,), -7, dtype=torch.int32, device=dev)
        b2e = torch.full((N,), -7, dtype=torch.int32, device=dev)
        cond = torch.full((n_cond,), -7, dtype=torch.int32, device=dev)
        status = torch.zeros(1, dtype=torch.int32, device=dev)
        s = nv.stream_ptr(dev)
        if static:
            rc = L.moe_build_blocks_static(nv.ptr(ids), T, k, E, B, N, int(skip_token), int(split), nv.ptr(tp),
                                           nv.ptr(b2e), nv.ptr(cond), n_cond, nv.ptr(status), s)
        else:
            ws = torch.empty(L.moe_build_blocks_workspace_bytes(E), dtype=torch.uint8, device=dev)
            rc = L.moe_build_blocks(nv.ptr(ids), T, k, E, B, N, int(skip_token), int(split), nv.ptr(tp), nv.ptr(b2e),
                                    nv.ptr(cond), n_cond, nv.ptr(ws), ws.numel(), nv.ptr(status), s)
        assert rc == 0, rc
        torch.cuda.synchronize()
        outs.append((tp.cpu().numpy(), b2e.cpu().numpy(), cond.cpu().numpy(), int(status.item())))
    return outs


def test_static_scratch_entry_point_equals_workspace_entry_point():
    import torch
    from nkilib import _native as nv
    from oracle import blocks as ob

    L = nv.lib()
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    # first a many-slab call with the largest expert count the built-in scratch takes, then a smaller, single-slab one
    for (T, k, E, B, skip, split) in [(8192, 8, 512, 128, False, False), (300, 4, 64, 128, True, True),
                                      (8192, 8, 256, 128, False, False), (8, 8, 256, 128, False, False)]:
        ids = torch.rand((T, E), generator=g, device=dev).topk(k, dim=1).indices.to(torch.int32).contiguous()
        N = ob.get_n_blocks(T, k, E, B, n_block_per_iter=2)
        ref, got = _both(L, nv, ids, E, B, N, skip, split, N + 2, dev)
        for a, b, what in zip(ref, got, ("token_position_to_id", "block_to_expert", "conditions", "status")):
            assert np.array_equal(a, b), f"T={T} E={E}: {what} differs"
        assert ref[3] == 0 and (ref[0] != -7).all() and (ref[1] != -7).all()
        # and both equal the oracle (the workspace entry point is checked against it elsewhere as well)
        mask = ob.expert_mask_from_router(ids.cpu().numpy(), E)
        tp_o, b2e_o, _ = ob.build_token_blocks(mask, B, N, skip, use_split_padding=split)[:3]
        assert np.array_equal(got[0], tp_o) and np.array_equal(got[1], b2e_o)


def test_static_scratch_limit_is_an_error():
    import torch
    from nkilib import _native as nv

    L = nv.lib()
    dev = torch.device("cuda:0")
    ids = torch.zeros((4, 2), dtype=torch.int32, device=dev)
    out = torch.zeros(1024 * 128, dtype=torch.int32, device=dev)
    rc = L.moe_build_blocks_static(nv.ptr(ids), 4, 2, 513, 128, 600, 0, 0, nv.ptr(out), nv.ptr(out), None, 0, None,
                                   nv.stream_ptr(dev))
    assert rc == -7 and b"allocates nothing" in L.moe_error_string(rc)


def test_static_scratch_entry_point_replays_from_a_graph_and_allocates_nothing():
    """After the per-device set-up (moe_check_device, outside any capture) the entry point can be recorded into a
    HIP graph: every replay gives the eager result, also with eager calls of the same entry point between the
    replays (they share the GPU's scratch in stream order), and an eager call changes neither the device's free memory nor
    torch's allocation count."""
    import torch
    from nkilib import _native as nv
    from oracle import blocks as ob

    L = nv.lib()
    dev = torch.device("cuda:0")
    assert L.moe_check_device() == 0
    T, k, E, B = 128, 8, 256, 128
    N = ob.get_n_blocks(T, k, E, B, n_block_per_iter=2)
    g = torch.Generator(device=dev)
    g.manual_seed(9)
    ids = torch.rand((T, E), generator=g, device=dev).topk(k, dim=1).indices.to(torch.int32).contiguous()
    ids2 = torch.rand((T, E), generator=g, device=dev).topk(k, dim=1).indices.to(torch.int32).contiguous()
    tp = torch.empty((N * B,), dtype=torch.int32, device=dev)
    b2e = torch.empty((N,), dtype=torch.int32, device=dev)
    cond = torch.empty((N + 2,), dtype=torch.int32, device=dev)
    tp2, b2e2, cond2 = torch.empty_like(tp), torch.empty_like(b2e), torch.empty_like(cond)

    def call(i, t, b, c):
        rc = L.moe_build_blocks_static(nv.ptr(i), T, k, E, B, N, 0, 0, nv.ptr(t), nv.ptr(b), nv.ptr(c), N + 2, None,
                                       nv.stream_ptr(dev))
        assert rc == 0, rc

    call(ids, tp, b2e, cond)  # warm-up: loads the kernels
    torch.cuda.synchronize()
    free0, alloc0 = torch.cuda.mem_get_info(dev)[0], torch.cuda.memory_allocated(dev)
    call(ids, tp, b2e, cond)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free0 and torch.cuda.memory_allocated(dev) == alloc0
    eager = (tp.clone(), b2e.clone(), cond.clone())
    mask = ob.expert_mask_from_router(ids.cpu().numpy(), E)
    tp_o, b2e_o, _ = ob.build_token_blocks(mask, B, N, False, use_split_padding=False)[:3]
    assert np.array_equal(eager[0].cpu().numpy(), tp_o) and np.array_equal(eager[1].cpu().numpy(), b2e_o)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(ids, tp, b2e, cond)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):  # (torch's own capture bookkeeping allocates a few bytes: not checked here)
        call(ids, tp, b2e, cond)
    torch.cuda.synchronize()
    for replay in range(3):
        tp.fill_(-7), b2e.fill_(-7), cond.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        for got, want, what in zip((tp, b2e, cond), eager, ("token_position_to_id", "block_to_expert", "conditions")):
            assert torch.equal(got, want), f"replay {replay}: {what} differs from the eager call"
        call(ids2, tp2, b2e2, cond2)  # an eager call on other ids between the replays
        torch.cuda.synchronize()
