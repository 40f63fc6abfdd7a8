"""The block build's hand-over of the blockwise layer's bookkeeping (moe_build_blocks_plan, moe_bwmm_args.block_plan).

No counterpart in the reference: what is checked is that the plan's tables say what token_position_to_id and
block_to_expert say (restated here from those tables alone), that the layer computes the same bits with and
without a plan, and that a plan is used only with the tables it was made for.
"""

import numpy as np
import pytest

from helpers import i32_tensor
from oracle import blocks as ob

pytestmark = pytest.mark.gpu

CHUNK_ROWS, CHUNK_ROWS_MAX, CLASSES = 256, 320, 12


def _al(nbytes):
    return (nbytes + 255) // 256 * 256


def _carve(plan, T1, N, B):
    """The regions of a plan, in the order the library lays them out (256-byte aligned each)."""
    max_chunks = N * ((B + CHUNK_ROWS - 1) // CHUNK_ROWS)
    sizes = [("n_active", 4), ("valid_rows", N), ("cnt", T1), ("cursor", T1), ("off", T1 + 1), ("list", N * B),
             ("n_chunks", 4), ("chunk_slot", max_chunks), ("chunk_rows", max_chunks), ("chunk_expert", max_chunks),
             ("chunk_xcd", max_chunks), ("q_chunk", None), ("q_off", 8 * (CLASSES + 1) + 1)]
    out, pos = {}, 0
    for name, words in sizes:
        if name == "q_chunk":
            nbytes = 2 * _al(max_chunks * 4)
            out[name] = plan[pos // 4: pos // 4 + 2 * max_chunks]
        else:
            nbytes = _al(words * 4)
            out[name] = plan[pos // 4: pos // 4 + words]
        pos += nbytes
    assert pos == plan.size * 4, (pos, plan.size * 4)
    return out


def _expected_chunks(tp, b2e, n_active, valid_rows, B, E):
    """Chunks as the blockwise layer cuts them: maximal runs of blocks of one expert, up to the run's last valid row,
    in pieces of 256 rows with a last piece of up to 320."""
    chunks, b = [], 0
    while b < n_active:
        e, j, last_end = b2e[b], b, -1
        while j < n_active and b2e[j] == e:
            if valid_rows[j] > 0:
                last_end = j * B + valid_rows[j]
            j += 1
        length = last_end - b * B
        if 0 <= e < E and length > 0:
            n = 1 if length <= CHUNK_ROWS_MAX else -(-(length - CHUNK_ROWS_MAX) // CHUNK_ROWS) + 1
            for c in range(n):
                s0 = b * B + c * CHUNK_ROWS
                chunks.append((s0, CHUNK_ROWS if c + 1 < n else last_end - s0, int(e)))
        b = j
    return chunks


@pytest.mark.parametrize(
    "T,k,E,B,skip,split,alpha,spoil",
    [
        (5, 2, 3, 2, False, False, None, False),
        (1, 8, 256, 128, False, False, None, False),        # decode: one launch builds tables and plan
        (128, 8, 256, 128, True, False, None, False),
        (700, 4, 16, 128, False, False, None, True),         # ids outside [0, E) and ids listed twice in a row
        (4096, 2, 8, 128, False, False, None, False),        # 1024 rows per expert: four chunks each
        (8192, 8, 128, 128, False, False, 0.3, False),       # skewed loads
        (8192, 8, 256, 128, False, False, None, True),
    ],
)
def test_plan_says_what_the_tables_say(T, k, E, B, skip, split, alpha, spoil):
    import torch
    from nkilib import _native as nv

    L = nv.lib()
    dev = torch.device("cuda:0")
    router = ob.router_with_controlled_distribution(T, k, E, alpha).astype(np.int32)
    if spoil:
        rng = np.random.default_rng(5)
        rows = rng.choice(T, size=T // 7, replace=False)
        router[rows, 0] = -1                      # no expert
        router[rows[: len(rows) // 2], 1] = E + 3   # out of range
        dup = rng.choice(T, size=T // 9, replace=False)
        router[dup, k - 1] = router[dup, k - 2]   # the same expert twice
    N = ob.get_n_blocks(T, k, E, B)
    T1 = T if skip else T + 1
    ids = i32_tensor(router, dev)

    def build(with_plan):
        tp = torch.full((N * B,), -7, dtype=torch.int32, device=dev)
        b2e = torch.full((N,), -7, dtype=torch.int32, device=dev)
        cond = torch.full((N + 2,), -7, dtype=torch.int32, device=dev)
        ws = torch.empty(L.moe_build_blocks_workspace_bytes(E), dtype=torch.uint8, device=dev)
        plan = None
        if with_plan:
            nbytes = L.moe_block_plan_bytes(T, B, N, int(skip))
            assert nbytes > 0 and nbytes % 256 == 0
            plan = torch.full((nbytes // 4,), -7, dtype=torch.int32, device=dev)
            rc = L.moe_build_blocks_plan(nv.ptr(ids), T, k, E, B, N, int(skip), int(split), nv.ptr(tp), nv.ptr(b2e),
                                         nv.ptr(cond), N + 2, nv.ptr(ws), ws.numel(), None, nv.ptr(plan), nbytes,
                                         nv.stream_ptr(dev))
        else:
            rc = L.moe_build_blocks(nv.ptr(ids), T, k, E, B, N, int(skip), int(split), nv.ptr(tp), nv.ptr(b2e),
                                    nv.ptr(cond), N + 2, nv.ptr(ws), ws.numel(), None, nv.stream_ptr(dev))
        assert rc == 0, rc
        torch.cuda.synchronize()
        return tp.cpu().numpy(), b2e.cpu().numpy(), cond.cpu().numpy(), None if plan is None else plan.cpu().numpy()

    tp0, b2e0, cond0, _ = build(False)
    tp, b2e, cond, plan = build(True)
    assert np.array_equal(tp, tp0) and np.array_equal(b2e, b2e0) and np.array_equal(cond, cond0)
    p = _carve(plan, T1, N, B)

    # blocks in use = those before the first zero condition; valid rows = 1 + last row that holds a token
    n_active = int(np.argmax(cond == 0)) if (cond == 0).any() else N
    assert int(p["n_active"][0]) == n_active
    tpb = tp.reshape(N, B)
    real = (tpb >= 0) & (tpb < T)
    want_valid = np.where(real.any(axis=1), B - np.argmax(real[:, ::-1], axis=1), 0)
    assert np.array_equal(p["valid_rows"], want_valid)
    assert not real[n_active:].any()

    # every (token, j): the slot that holds the token among its j-th expert's blocks, once per distinct valid expert
    assert np.array_equal(p["off"][: T + 1], np.arange(T + 1) * k)
    slot_of = {}
    expert_of_slot = np.repeat(b2e, B)
    for s in np.flatnonzero(real.reshape(-1)):
        slot_of[(int(tp[s]), int(expert_of_slot[s]))] = int(s)
    lst = p["list"][: T * k].reshape(T, k)
    want = np.full((T, k), -1, dtype=np.int64)
    for t in range(T):
        seen = set()
        for j in range(k):
            e = int(router[t, j])
            if 0 <= e < E and e not in seen:
                want[t, j] = slot_of[(t, e)]
                seen.add(e)
    assert np.array_equal(lst, want)
    assert len(slot_of) == int((want >= 0).sum())  # every slot that holds a token is listed exactly once

    # chunks in block order, and the eight XCD queues together hold each chunk once
    chunks = _expected_chunks(tp, b2e, n_active, want_valid, B, E)
    n = int(p["n_chunks"][0])
    assert n == len(chunks)
    got = list(zip(p["chunk_slot"][:n].tolist(), p["chunk_rows"][:n].tolist(), p["chunk_expert"][:n].tolist()))
    assert got == chunks
    q = p["q_chunk"][: 2 * n].reshape(n, 2)
    queued = sorted((int(s), int(w) & 0xffff, int(w) >> 16) for s, w in q)
    assert queued == sorted(chunks)
    qo = p["q_off"][: 8 * (CLASSES + 1)].reshape(8, CLASSES + 1)
    assert qo[0, 0] == 0 and qo[7, CLASSES] == n and (np.diff(qo.reshape(-1)) >= 0).all()
    assert 1 <= int(p["q_off"][8 * (CLASSES + 1)]) <= 8


def test_plan_refusals():
    import torch
    from nkilib import _native as nv

    L = nv.lib()
    dev = torch.device("cuda:0")
    ids = torch.zeros((4, 2), dtype=torch.int32, device=dev)
    buf = torch.zeros(1 << 16, dtype=torch.int32, device=dev)
    ws = torch.empty(L.moe_build_blocks_workspace_bytes(8), dtype=torch.uint8, device=dev)
    s = nv.stream_ptr(dev)
    need = L.moe_block_plan_bytes(4, 4, 4, 0)
    assert need > 0 and L.moe_block_plan_bytes(0, 4, 4, 0) == 0
    args = (nv.ptr(ids), 4, 2, 8, 4, 4, 0, 0, nv.ptr(buf), nv.ptr(buf), None, 0, nv.ptr(ws), ws.numel(), None)
    assert L.moe_build_blocks_plan(*args, None, need, s) == -1                       # no plan buffer
    assert L.moe_build_blocks_plan(*args, buf[1:].data_ptr(), need, s) == -1            # not 256-byte aligned
    assert L.moe_build_blocks_plan(*args, nv.ptr(buf), need - 256, s) == -3          # too small
    split = list(args)
    split[7] = 1
    assert L.moe_build_blocks_plan(*split, nv.ptr(buf), need, s) == -5               # split padding
    # more (token, j) pairs than slots: the lists would not fit
    args = (nv.ptr(ids), 4, 2, 8, 1, 4, 0, 0, nv.ptr(buf), nv.ptr(buf), None, 0, nv.ptr(ws), ws.numel(), None)
    assert L.moe_build_blocks_plan(*args, nv.ptr(buf), 1 << 18, s) == -2
    torch.cuda.synchronize()


def _mx_case(T, H, I, E, k, B, dev, seed=3):
    import torch
    from nkilib import synthetic as syn
    from nkilib.core.moe.moe_cte import MoECTEImplementation, MoECTESpec, QuantizationConfig

    ids, aff = syn.route(T, E, k, dev, seed=seed, mode="softmax", expert_bias_std=0.5)
    x = syn.hidden_states(T, H, dev, seed=seed)
    gu_q, gu_s, d_q, d_s = syn.mx_expert_weights(E, H, I, 0.02, dev, seed=seed)
    return dict(ids=ids, aff=aff, x=x, gu=gu_q.view(torch.int32).reshape(gu_q.shape[:-1]), d=d_q,
                spec=MoECTESpec(implementation=MoECTEImplementation.shard_on_block_mx),
                kw=dict(quantization_config=QuantizationConfig(gu_s, d_s)))


def _dense_case(T, H, I, E, k, B, dev, seed=4, impl="shard_on_block"):
    import torch
    from nkilib import synthetic as syn
    from nkilib.core.moe.moe_cte import MoECTEImplementation, MoECTESpec

    ids, aff = syn.route(T, E, k, dev, seed=seed, mode="softmax")
    x = syn.hidden_states(T, H, dev, seed=seed)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    gu = (torch.randn((E, H, 2, I), generator=g, device=dev) * 0.05).to(torch.bfloat16)
    d = (torch.randn((E, I, H), generator=g, device=dev) * 0.05).to(torch.bfloat16)
    return dict(ids=ids, aff=aff, x=x, gu=gu, d=d, spec=MoECTESpec(implementation=getattr(MoECTEImplementation, impl)),
                kw={})


@pytest.mark.parametrize("kind,T,H,I,E,k,B", [
    ("mx", 1500, 1024, 512, 8, 2, 128),      # large-tile MX kernels, several chunks per expert
    ("mx", 3, 1024, 512, 16, 4, 128),        # decode-sized
    ("mx", 600, 1024, 96, 4, 2, 128),        # general tiled kernel (I % 128 != 0)
    ("bf16", 900, 512, 256, 4, 2, 256),      # large-tile bf16 kernels
    ("bf16", 500, 320, 80, 4, 2, 64),        # general tiled kernel
])
def test_layer_is_bit_equal_with_and_without_a_plan(kind, T, H, I, E, k, B):
    import torch
    from nkilib.core.moe.moe_cte import block_index, build_token_blocks, get_n_blocks, moe_cte
    from nkilib.core.moe.moe_cte import _launch

    dev = torch.device("cuda:0")
    c = _mx_case(T, H, I, E, k, B, dev) if kind == "mx" else _dense_case(T, H, I, E, k, B, dev)
    ids = c["ids"].clone()
    # a few rows with a missing expert and with the same expert twice (their masked affinities say the same)
    ids[::11, 0] = -1
    ids[5::13, k - 1] = ids[5::13, k - 2]
    aff = c["aff"].clone()
    mask = torch.zeros_like(aff, dtype=torch.bool)
    rows = torch.arange(T, device=dev)
    for j in range(k):
        m = ids[:, j] >= 0
        mask[rows[m], ids[m, j].long()] = True
    aff = torch.where(mask, aff, torch.zeros_like(aff))
    N = get_n_blocks(T, k, E, B, n_block_per_iter=2)

    seen = []
    real_blockwise = _launch.nv.lib().moe_blockwise

    def layer(with_plan, conditions="own"):
        block_index.block_plans = with_plan
        try:
            tp, b2e, cond = build_token_blocks(ids, E, B, N, n_conditions=N + 2)
        finally:
            block_index.block_plans = True
        cnd = {"own": cond, "none": None, "copy": cond.clone()}[conditions]
        seen.append(block_index.plan_for(tp, b2e.reshape(-1), None if cnd is None else cnd.reshape(-1), B, N, T + 1))
        out = moe_cte[2](c["x"], aff.reshape(-1, 1), c["gu"], c["d"], tp, b2e, B, c["spec"], conditions=cnd, **c["kw"])
        torch.cuda.synchronize()
        return out.clone()

    base = layer(False)
    assert seen[-1] is None
    for conditions in ("own", "none"):
        got = layer(True, conditions)
        assert seen[-1] is not None, "the plan was not found for the tables it was made with"
        assert torch.equal(got, base), f"conditions={conditions}: the result differs with a plan"
    # another conditions array (equal contents, other memory) is not the plan's: the layer derives its own bookkeeping
    got = layer(True, "copy")
    assert seen[-1] is None and torch.equal(got, base)
    assert bool(base.any()) and real_blockwise is not None


def test_plan_is_dropped_when_the_tables_change_or_are_used_differently():
    import torch
    from nkilib.core.moe.moe_cte import block_index, build_token_blocks, get_n_blocks

    dev = torch.device("cuda:0")
    T, k, E, B = 300, 2, 8, 128
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    ids = torch.rand((T, E), generator=g, device=dev).topk(k, dim=1).indices.to(torch.int32).contiguous()
    N = get_n_blocks(T, k, E, B)
    tp, b2e, cond = build_token_blocks(ids, E, B, N)
    assert block_index.plan_for(tp, b2e, cond, B, N, T + 1) is not None
    assert block_index.plan_for(tp.view(N, B).reshape(-1), b2e.reshape(-1, 1).reshape(-1), None, B, N, T + 1) is not None
    assert block_index.plan_for(tp, b2e, cond, B, N, T) is None          # another token count
    assert block_index.plan_for(tp, b2e, cond, 64, 2 * N, T + 1) is None  # another block size
    assert block_index.plan_for(tp, b2e.clone(), cond, B, N, T + 1) is None
    assert block_index.plan_for(tp.clone(), b2e, cond, B, N, T + 1) is None
    b2e[0] = b2e[0]  # an in-place write bumps the version counter that the three tables share
    assert block_index.plan_for(tp, b2e, cond, B, N, T + 1) is None
    n_before = len(block_index._plans)
    del tp, b2e, cond
    assert len(block_index._plans) == n_before - 1  # the entry goes with the allocation
