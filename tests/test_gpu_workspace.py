"""What a workspace's head words promise, on the GPU: the plan a routed call leaves there is the oracle's; a bounded
wait that gives up leaves a fault the host can read, stores nothing, and hb_workspace_reset puts the workspace back in
service; calls in flight together on workspaces of their own share nothing (two streams, many iterations, bit for
bit the serial results); a graph replayed on changing inputs gives every replay the eager call's bits."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import layers
from tests.util import random_experts

pytestmark = pytest.mark.gpu


def _layout(st, m, topk, shared):
    from hibana_amd import _lib
    offsets = (C.c_int64 * 6)()
    _lib.check(_lib.lib().hb_debug_workspace_layout(m, topk, C.byref(st), int(shared), offsets), "layout")
    return list(offsets)


def _read_plan(ws: torch.Tensor, st, m, topk, shared):
    """(header, slot entries [slots, 4], order) a routed call left in its workspace."""
    plan_at, order_at, _, _, _, cap = _layout(st, m, topk, shared)
    words = ws.cpu().numpy().view(np.int32)
    head = words[plan_at // 4:plan_at // 4 + 16]
    slots = int(head[0])
    entries = words[plan_at // 4 + 16:plan_at // 4 + 16 + 4 * cap].reshape(cap, 4)
    order = words[order_at // 4:order_at // 4 + m * topk + (m if shared else 0)]
    return head, entries, slots, order


def _check_plan(head, entries, slots, order, ids, topk, e_lo, e_n, shared_rows, slot_rows=16):
    """The plan against the oracle's expert_plan: the sorted pair list is the stable sort's, the routed slots cover each
    distinct expert's run in order (16 rows a slot), the shared expert's slots come first and its rows last."""
    experts, starts, want_order = layers.expert_plan(ids, e_lo, e_n)
    kept = len(want_order)
    pairs = ids.size
    assert head[1] == len(experts) and head[2] == kept
    assert head[3] == 0 and head[4] == 0  # the ticket is back at zero, no fault
    assert np.array_equal(order[:kept], want_order)
    assert np.array_equal(order[kept:kept + shared_rows], pairs + np.arange(shared_rows))
    shared_slots = -(-shared_rows // slot_rows)
    for s in range(shared_slots):
        assert entries[s].tolist() == [-1, kept + s * slot_rows, min(slot_rows, shared_rows - s * slot_rows), 0]
    routed = entries[shared_slots:slots]
    assert (routed[:, 2] > 0).all() and (routed[:, 2] <= slot_rows).all()
    reach = min(pairs, pairs // slot_rows + e_n) + shared_slots  # the launches' grids: the plan's upper bound on the slots
    assert slots <= reach and (entries[slots:reach, 2] == 0).all()  # the entries they reach beyond the last slot say "no rows"
    # every distinct expert's run, cut into slots in order; heavily loaded experts (more than a quarter slot) first
    by_expert = {}
    for e, p0, rows, _ in routed.tolist():
        by_expert.setdefault(e, []).append((p0, rows))
    assert sorted(by_expert) == experts.tolist()
    for d, e in enumerate(experts.tolist()):
        runs = sorted(by_expert[e])
        count = int(starts[d + 1] - starts[d])
        assert runs[0][0] == starts[d] and sum(r for _, r in runs) == count
        assert all(r == slot_rows for _, r in runs[:-1]) and all(a + ra == b for (a, ra), (b, _) in zip(runs, runs[1:]))
    counts = {e: int(starts[d + 1] - starts[d]) for d, e in enumerate(experts.tolist())}
    heavy = [4 * counts[e] > slot_rows for e in routed[:, 0].tolist()]
    assert heavy == sorted(heavy, reverse=True)
    for group in (True, False):  # each class in ascending expert id
        ids_in = [e for e, h in zip(routed[:, 0].tolist(), heavy) if h == group]
        assert ids_in == sorted(ids_in)


@pytest.fixture(scope="module")
def small():
    ex, _ = random_experts(64, 256, 128, True, 21)
    sh, _ = random_experts(1, 256, 128, True, 22)
    return ex, sh


@pytest.mark.parametrize("m,topk,route_plan", [(32, 10, 0), (32, 10, 1), (64, 6, 0), (7, 10, 0), (100, 4, 0), (2, 10, 0)])
def test_plan_of_a_routed_call_is_the_oracles(small, m, topk, route_plan):
    """The layer from logits: in-kernel routing, then the plan (the last routing workgroup's, by rows or - route_plan 1,
    and beyond 64 rows - the general form; up to four rows the planning workgroup routes; one token plans inside fc1)."""
    from hibana_amd import _lib
    from hibana_amd.kernels import w3_moe
    ex, sh = small
    lib = _lib.lib()
    g = torch.Generator().manual_seed(m * 31 + topk)
    x = torch.randn(m, 256, generator=g).bfloat16().cuda()
    logits = (torch.randn(m, 64, generator=g) + torch.linspace(2, 0, 64)).cuda()  # skewed: some experts drawn by most rows
    assert lib.hb_tune(b"route_plan", route_plan) == 0
    try:
        _, ids, _ = w3_moe.moe_layer_logits(ex, x, logits, topk, shared=sh, return_routing=True)
    finally:
        lib.hb_tune(b"route_plan", 0)
    torch.cuda.synchronize()
    st = w3_moe._struct(ex)
    ws = _lib.workspace(x.device, 0)
    head, entries, slots, order = _read_plan(ws, st, m, topk, True)
    _check_plan(head, entries, slots, order, ids.cpu().numpy(), topk, 0, 64, m)


@pytest.mark.parametrize("base,count", [(0, 64), (16, 32)])
def test_plan_of_given_ids_with_an_expert_range(small, base, count):
    """hb_w3_moe on caller's ids (the general form; an expert named twice by a row; experts outside the rank's range)."""
    from hibana_amd import _lib
    from hibana_amd.kernels import w3_moe
    ex, _ = small
    part = w3_moe.W3Experts(ex.planes13[base:base + count], ex.scales13[base:base + count], ex.row13[base:base + count], ex.planes2[base:base + count],
                            ex.scales2[base:base + count], ex.row2[base:base + count], ex.codebook, ex.lut, ex.fc2_codebook, ex.fc2_lut, base=base)
    g = torch.Generator().manual_seed(base + 5)
    m, topk = 45, 10
    x = torch.randn(m, 256, generator=g).bfloat16().cuda()
    ids = torch.randint(0, 66, (m, topk), generator=g).to(torch.int32)  # 64, 65: no expert
    ids[3, 4] = ids[3, 1]
    weights = torch.rand(m, topk, generator=g)
    w3_moe.w3_moe(part, x, ids.cuda(), weights.cuda())
    torch.cuda.synchronize()
    st = w3_moe._struct(part)
    head, entries, slots, order = _read_plan(_lib.workspace(x.device, 0), st, m, topk, False)
    _check_plan(head, entries, slots, order, ids.numpy(), topk, base, count, 0)


def test_plan_of_a_prefill_sized_call_three_launches():
    """45 056 pairs (2048 rows x 22): the plan shared among workgroups (count / scan / place), slots of 128 rows."""
    from hibana_amd import _lib
    from hibana_amd.kernels import w3_moe
    ex, _ = random_experts(32, 128, 128, False, 23)
    g = torch.Generator().manual_seed(9)
    m, topk = 2048, 22
    x = torch.randn(m, 128, generator=g).bfloat16().cuda()
    ids = torch.stack([torch.randperm(32, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    weights = torch.rand(m, topk, generator=g)
    w3_moe.w3_moe(ex, x, ids.cuda(), weights.cuda())
    torch.cuda.synchronize()
    st = w3_moe._struct(ex)
    head, entries, slots, order = _read_plan(_lib.workspace(x.device, 0), st, m, topk, False)
    assert entries[:slots, 2].max() == 128  # the MFMA tile kernel's slots
    _check_plan(head, entries, slots, order, ids.numpy(), topk, 0, 32, 0, slot_rows=128)


def test_a_wait_that_gives_up_is_reported_and_reset_restores_service(small):
    """The fused fc1 + fc2 launch with a count its fc2 workgroups cannot reach and a bound of a few polls (forced from the
    host; every kernel exits normally): the fault word is set, fc2 stored nothing, hb_workspace_reset clears it and the
    next call is right."""
    from hibana_amd import _lib
    from hibana_amd.kernels import w3_moe
    ex, sh = small
    lib = _lib.lib()
    g = torch.Generator().manual_seed(77)
    m, topk = 12, 6
    x = torch.randn(m, 256, generator=g).bfloat16().cuda()
    ids = torch.stack([torch.randperm(64, generator=g)[:topk] for _ in range(m)]).to(torch.int32).cuda()
    weights = torch.rand(m, topk, generator=g).cuda()
    good = w3_moe.moe_layer(ex, x, ids, weights, shared=sh).clone()
    ws = _lib.workspace(x.device, 0)
    assert _lib.workspace_status(ws) == 0
    st = w3_moe._struct(ex)
    _, _, _, y_at, _, _ = _layout(st, m, topk, True)
    pair_bytes = (m * topk + m) * 256 * 4
    ws[y_at:y_at + pair_bytes].fill_(0x7f)  # what fc2 would overwrite
    assert lib.hb_tune(b"fault_inject", 1) == 0
    try:
        w3_moe.moe_layer(ex, x, ids, weights, shared=sh)
    finally:
        lib.hb_tune(b"fault_inject", 0)
    assert _lib.workspace_status(ws) == 1  # HB_FAULT_WAIT
    assert bool((ws[y_at:y_at + pair_bytes] == 0x7f).all())  # no workgroup of fc2 stored anything
    again = w3_moe.moe_layer(ex, x, ids, weights, shared=sh)  # the counters themselves are fine: a later call is right ...
    assert torch.equal(again, good)
    assert _lib.workspace_status(ws) == 1  # ... and the fault word stays until the caller has seen to it
    _lib.workspace_reset(ws)
    assert _lib.workspace_status(ws) == 0
    assert torch.equal(w3_moe.moe_layer(ex, x, ids, weights, shared=sh), good)
    # a ticket left standing by an aborted launch: the next call's last workgroup would not know itself; reset restores it
    logits = torch.randn(m, 64, generator=g).cuda()
    want = w3_moe.moe_layer_logits(ex, x, logits, topk, shared=sh).clone()
    torch.cuda.synchronize()
    ws.view(torch.int32)[3] = 5
    _lib.workspace_reset(ws)
    assert torch.equal(w3_moe.moe_layer_logits(ex, x, logits, topk, shared=sh), want)
    # the library's own scratch has the same two calls
    assert _lib.workspace_status(None) == 0
    _lib.workspace_reset(None)


def test_two_streams_with_workspaces_of_their_own_share_nothing():
    """Two verify-sized layer calls from logits (routing and plan in one launch: the arrival counter; fc1 and fc2 in one
    launch: the slots' counters) on two ordinary streams at once, and two NVFP4 products of 64 rows (tiles that share K:
    the tiles' counters), many iterations: every result is the serial call's, bit for bit."""
    from hibana_amd import _lib
    from hibana_amd.kernels import ops, w3_moe
    from tests.test_gpu_graph_capture import _nvfp4_linear
    ex, _ = random_experts(64, 512, 256, True, 41)
    sh, _ = random_experts(1, 512, 256, True, 42)
    lin = _nvfp4_linear(2048, 1024, 43)
    g = torch.Generator().manual_seed(3)
    cases = []
    for i in range(2):
        x = torch.randn(32, 512, generator=g).bfloat16().cuda()
        logits = torch.randn(32, 64, generator=g).cuda()
        xd = torch.randn(64, 1024, generator=g).bfloat16().cuda()
        cases.append((x, logits, xd))
    assert _lib.lib().hb_nvfp4_gemm_workspace_bytes(64, 2048, 1024) > 0
    serial = [(w3_moe.moe_layer_logits(ex, x, lg, 8, shared=sh).clone(), ops.nvfp4_linear(xd, lin).clone()) for x, lg, xd in cases]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]  # default priority both
    for it in range(40):
        outs = []
        for s, (x, lg, xd) in zip(streams, cases):
            with torch.cuda.stream(s):
                outs.append((w3_moe.moe_layer_logits(ex, x, lg, 8, shared=sh), ops.nvfp4_linear(xd, lin)))
        torch.cuda.synchronize()
        for (a, b), (wa, wb) in zip(outs, serial):
            assert torch.equal(a, wa) and torch.equal(b, wb), it
    with torch.cuda.stream(streams[0]):
        first = _lib.workspace(x.device, 0)
    with torch.cuda.stream(streams[1]):
        second = _lib.workspace(x.device, 0)
    assert first.data_ptr() != second.data_ptr()
    assert _lib.workspace_status(first) == 0 and _lib.workspace_status(second) == 0


def test_graph_replays_on_changing_inputs_follow_the_eager_results():
    """One captured verify step (routing + plan, fc1 + fc2 in one launch, combine) replayed on inputs rewritten in place
    between replays: every replay equals the eager call on the same inputs (fc2 reads the h of THIS replay's fc1, whatever
    an earlier replay left in the caches)."""
    from hibana_amd.kernels import w3_moe
    ex, _ = random_experts(48, 1024, 256, True, 61)
    sh, _ = random_experts(1, 1024, 256, True, 62)
    g = torch.Generator().manual_seed(5)
    m, topk = 32, 8
    x = torch.randn(m, 1024, generator=g).bfloat16().cuda()
    logits = torch.randn(m, 48, generator=g).cuda()
    w3_moe.moe_layer_logits(ex, x, logits, topk, shared=sh)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = w3_moe.moe_layer_logits(ex, x, logits, topk, shared=sh)
    for i in range(6):
        x.copy_(torch.randn(m, 1024, generator=g).bfloat16())
        logits.copy_(torch.randn(m, 48, generator=g))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = captured.clone()
        eager = w3_moe.moe_layer_logits(ex, x, logits, topk, shared=sh)
        assert torch.equal(got, eager), i


def test_trace_hook_records_within_its_capacity(small):
    """hb_debug_trace: records of the fused launch's workgroups up to the buffer's capacity, nothing beyond it."""
    from hibana_amd import _lib
    from hibana_amd.kernels import w3_moe
    ex, sh = small
    lib = _lib.lib()
    g = torch.Generator().manual_seed(8)
    m, topk = 16, 6
    x = torch.randn(m, 256, generator=g).bfloat16().cuda()
    ids = torch.stack([torch.randperm(64, generator=g)[:topk] for _ in range(m)]).to(torch.int32).cuda()
    weights = torch.rand(m, topk, generator=g).cuda()
    records = 24
    buf = torch.full((4 * records + 64,), -1, dtype=torch.int64, device="cuda")
    assert lib.hb_debug_trace(_lib.ptr(buf), -1) == _lib.HB_EINVAL
    assert lib.hb_debug_trace(_lib.ptr(buf), records) == 0
    try:
        w3_moe.moe_layer(ex, x, ids, weights, shared=sh)
        torch.cuda.synchronize()
    finally:
        assert lib.hb_debug_trace(None, 0) == 0
    host = buf.cpu().numpy()
    assert (host[4 * records:] == -1).all()  # nothing past the capacity
    rec = host[:4 * records].reshape(records, 4)
    used = rec[rec[:, 3] != -1]
    assert len(used) > 0 and (used[:, 2] >= used[:, 0]).all() and ((used[:, 3] & 0xffff) <= 16).all()
    w3_moe.moe_layer(ex, x, ids, weights, shared=sh)  # disarmed: nothing is written
    torch.cuda.synchronize()
    assert np.array_equal(buf.cpu().numpy(), host)
