"""The routed-expert kernels on the GPU against the oracle's layer math (weight-only, identity activation rounding):
one row to prefill-sized calls, fewer experts per row, unfilled slots, expert-parallel halves, pair outputs, the
shared expert and the gated combine, ReLU^2 experts. Mirrors tests/gpu/test_w3_moe.py and test_w3_moe_nemotron.py
of the reference."""
import numpy as np
import pytest
import torch

from oracle import layers
from tests.util import MAX_REL, NORM_REL, errors, oracle_expert_getter, random_experts

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["auto", "tile", "stream", "stream16", "apart", "planes"], autouse=True)
def kernel_choice(request):
    """Every case runs with the library's own choice between the 128-row MFMA tile kernel and the 16-row weight stream,
    with each of them forced, with the stream's body for slots of at most four rows switched off (so those slots
    take the sixteen-row body, as they do when the activation matrix is too large for a buffer descriptor), with fc1
    and fc2 of a call in launches of their own instead of one ("apart"), and with fc1's slots of at most four rows on the
    two-plane E4M3 form of the activations and the FP8 matrix cores ("planes")."""
    from hibana_amd import _lib
    knobs = {"auto": {}, "tile": {"w3_tile": 1}, "stream": {"w3_tile": 2}, "stream16": {"w3_tile": 2, "w3_few": 2},
             "apart": {"w3_tile": 2, "moe_fused": 2}, "planes": {"w3_tile": 2, "moe_split": 1}}[request.param]
    for key, value in knobs.items():
        assert _lib.lib().hb_tune(key.encode(), value) == 0
    yield request.param
    for key in knobs:
        _lib.lib().hb_tune(key.encode(), 0)

E, H, I, TOPK = 16, 256, 128, 10


@pytest.fixture(scope="module")
def gated():
    ex, per = random_experts(E, H, I, True, 5)
    return ex, oracle_expert_getter(per, True, I)


@pytest.fixture(scope="module")
def relu2():
    ex, per = random_experts(8, 256, 384, False, 6, codebook="lloyd", fc2_codebook="zero8")
    return ex, oracle_expert_getter(per, False, 384)


def _inputs(m, k, seed, experts=E):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, H, generator=g).bfloat16()
    x[:, ::97] *= 30
    ids = torch.stack([torch.randperm(experts, generator=g)[:k] for _ in range(m)]).to(torch.int32)
    weights = torch.softmax(torch.randn(m, k, generator=g), -1)
    return x, ids, weights


def _check(ex, get, x, ids, weights, is_gated=True, e_lo=0, e_n=None):
    from hibana_amd.kernels import w3_moe
    e_n = ex.experts if e_n is None else e_n
    want = layers.moe_layer_ref(x, ids.numpy(), weights, get, is_gated, e_lo=e_lo, e_n=e_n)
    got = w3_moe.w3_moe(ex, x.cuda(), ids.cuda(), weights.cuda())
    assert got.dtype == torch.bfloat16 and got.shape == want.shape
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    assert torch.equal(w3_moe.w3_moe(ex, x.cuda(), ids.cuda(), weights.cuda()), got)  # no atomics in the sums
    return got


@pytest.mark.parametrize("m", [1, 2, 5, 16, 32, 64, 200])
def test_kernel_matches_oracle(gated, m):
    _check(*gated, *_inputs(m, TOPK, m))


@pytest.mark.parametrize("k", [1, 5, 9])
@pytest.mark.parametrize("m", [1, 5, 64])
def test_fewer_experts_per_row(gated, m, k):
    _check(*gated, *_inputs(m, k, 100 * k + m))


@pytest.mark.parametrize("m", [2, 5, 16, 17, 80])
def test_ids_past_the_last_expert_add_nothing(gated, m):
    ex, get = gated
    from hibana_amd.kernels import w3_moe
    g = torch.Generator().manual_seed(300 + m)
    x = torch.randn(m, H, generator=g).bfloat16()
    ids = torch.full((m, TOPK), w3_moe.EXPERTS, dtype=torch.int32)
    weights = torch.zeros(m, TOPK)
    others = [e for e in range(E) if e != 3]
    for r in range(m):  # every row shares expert 3, with 1 to 9 unfilled slots
        n = 1 + r % 9
        ids[r, :n] = torch.tensor([3] + [others[i] for i in torch.randperm(len(others), generator=g)[:n - 1].tolist()], dtype=torch.int32)
        weights[r, :n] = torch.softmax(torch.randn(n, generator=g), -1)
    ids[-1], weights[-1] = w3_moe.EXPERTS, 0.0  # a padded row
    got = _check(ex, get, x, ids, weights)
    assert torch.isfinite(got.float()).all() and not got[-1].any()


@pytest.mark.parametrize("k", [TOPK, 5])
@pytest.mark.parametrize("m", [1, 5, 80])
def test_expert_parallel_halves_sum_to_the_whole(gated, m, k):
    from dataclasses import replace

    from hibana_amd.kernels import w3_moe
    ex, get = gated
    x, ids, weights = _inputs(m, k, 100 + m + k)
    half = E // 2

    def part(lo):
        return replace(ex, planes13=ex.planes13[lo:lo + half], scales13=ex.scales13[lo:lo + half], row13=ex.row13[lo:lo + half],
                       planes2=ex.planes2[lo:lo + half], scales2=ex.scales2[lo:lo + half], row2=ex.row2[lo:lo + half], base=lo,
                       tiled13=None, tiled2=None)

    whole = w3_moe.w3_moe(ex, x.cuda(), ids.cuda(), weights.cuda()).float()
    lo, hi = part(0), part(half)
    parts = w3_moe.w3_moe(lo, x.cuda(), ids.cuda(), weights.cuda()).float() + w3_moe.w3_moe(hi, x.cuda(), ids.cuda(), weights.cuda()).float()
    assert float((parts - whole).norm() / whole.norm()) < NORM_REL
    _check(hi, lambda e: get(e + half), x, ids, weights, e_lo=half, e_n=half)
    only = torch.full_like(ids, half)  # every pair on the second rank: the first rank's partial is zero
    assert not w3_moe.w3_moe(lo, x.cuda(), only.cuda(), weights.cuda()).any()


@pytest.mark.parametrize("m", [1, 5, 64, 200])
def test_pairs_then_combine_gives_the_same_bits(gated, m):
    """`w3_moe(..., pairs=True)` summed by `moe_combine_pairs` == the kernel's own combine; BF16 pairs are the FP32
    pairs rounded once (tests/gpu/test_w3_moe.py:132-186 of the reference)."""
    from hibana_amd.kernels import ops, w3_moe
    ex, get = gated
    x, ids, weights = _inputs(m, TOPK, 300 + m)
    ids[::3, -1] = w3_moe.EXPERTS
    xd, idd, wd = x.cuda(), ids.cuda(), weights.cuda()
    summed = w3_moe.w3_moe(ex, xd, idd, wd)
    pairs = w3_moe.w3_moe(ex, xd, idd, wd, pairs=True)
    assert pairs.dtype == torch.float32 and pairs.shape == (m * TOPK, H)
    assert torch.equal(ops.moe_combine_pairs(pairs, idd, wd, None, None, None, 0, E), summed)
    want_pairs = layers.routed_experts_ref(x, ids.numpy(), get, True, 0, E)
    local = (ids.reshape(-1) < E)
    mx, nr = errors(pairs[local.cuda()], want_pairs[local])
    assert mx < MAX_REL and nr < NORM_REL
    half = w3_moe.w3_moe(ex, xd, idd, wd, pairs=True, pairs_bf16=True)
    assert half.dtype == torch.bfloat16
    assert torch.equal(half[local.cuda()], pairs[local.cuda()].bfloat16())
    shared = torch.randn(m, H, generator=torch.Generator().manual_seed(1)).bfloat16()
    gate = torch.randn(H, generator=torch.Generator().manual_seed(2)) * 0.02
    fused = ops.moe_combine_pairs(pairs, idd, wd, shared.cuda(), xd, gate.cuda(), 0, E)
    want = layers.combine_shared_ref(summed.cpu(), shared, x, gate)
    assert errors(fused, want)[0] < 2 ** -7  # one BF16 rounding apart at most (the sigmoid's dot product order)
    assert torch.equal(ops.moe_combine_pairs(half, idd, wd, shared.cuda(), xd, gate.cuda(), 0, E),
                       ops.moe_combine_pairs(half.float(), idd, wd, shared.cuda(), xd, gate.cuda(), 0, E))


@pytest.mark.parametrize("m", [1, 7, 32, 100])
@pytest.mark.parametrize("with_gate", [False, True])
def test_layer_with_shared_expert(gated, m, with_gate):
    from hibana_amd.kernels import w3_moe
    ex, get = gated
    shared_ex, shared_per = random_experts(1, H, I, True, 77)
    shared_get = oracle_expert_getter(shared_per, True, I)
    x, ids, weights = _inputs(m, TOPK, 500 + m)
    gate = torch.randn(H, generator=torch.Generator().manual_seed(3)) * 0.05 if with_gate else None
    want = layers.moe_layer_ref(x, ids.numpy(), weights, get, True, shared=shared_get(0), gate_vec=gate, e_n=E)
    got = w3_moe.moe_layer(ex, x.cuda(), ids.cuda(), weights.cuda(), shared=shared_ex, gate_vec=None if gate is None else gate.cuda())
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    assert torch.equal(w3_moe.moe_layer(ex, x.cuda(), ids.cuda(), weights.cuda(), shared=shared_ex, gate_vec=None if gate is None else gate.cuda()), got)
    # the layer without a shared expert is the routed sum
    assert torch.equal(w3_moe.moe_layer(ex, x.cuda(), ids.cuda(), weights.cuda()), w3_moe.w3_moe(ex, x.cuda(), ids.cuda(), weights.cuda()))


@pytest.mark.parametrize("m", [1, 4, 5, 16, 17, 32, 200])
def test_layer_from_logits_is_route_then_layer(gated, m):
    """Routing inside the chain (in the planning workgroup up to four rows, its own launch beyond) gives the bits of
    ops.route_topk followed by moe_layer."""
    from hibana_amd.kernels import ops, w3_moe
    ex, _ = gated
    shared_ex, _ = random_experts(1, H, I, True, 78)
    g = torch.Generator().manual_seed(m)
    x = torch.randn(m, H, generator=g).bfloat16().cuda()
    logits = (torch.randn(m, E, generator=g) * 2).cuda()
    ids, wts = ops.route_topk(logits, TOPK)
    want = w3_moe.moe_layer(ex, x, ids, wts, shared=shared_ex)
    got, got_ids, got_w = w3_moe.moe_layer_logits(ex, x, logits, TOPK, shared=shared_ex, return_routing=True)
    assert torch.equal(got_ids, ids) and torch.equal(got_w, wts) and torch.equal(got, want)
    assert torch.equal(w3_moe.moe_layer_logits(ex, x, logits, TOPK), w3_moe.moe_layer(ex, x, ids, wts))


@pytest.mark.parametrize("m,steps", [(1, 1), (5, 5), (12, 3), (32, 8), (200, 1)])
def test_layer_under_a_budget_is_route_budget_then_layer(m, steps):
    """`moe_layer_budget`: the selection's second launch also plans the call; ids, weights and output are the bits of
    `ops.route_budget` followed by `moe_layer`, with padded requests, a cap per request, and a call of more pairs
    than one workgroup plans (the plan's own launches then follow)."""
    from hibana_amd.kernels import ops, w3_moe
    e = 32  # the selection takes a row's candidates from its 20 largest logits
    ex, _ = random_experts(e, H, I, True, 31)
    shared_ex, _ = random_experts(1, H, I, True, 78)
    g = torch.Generator().manual_seed(50 + m)
    x = torch.randn(m, H, generator=g).bfloat16().cuda()
    logits = (torch.randn(m, e, generator=g) * 1.5).bfloat16().cuda()
    slots = torch.ones(m // steps, dtype=torch.int32)
    if m // steps > 1:
        slots[-1] = 0
    topk = 10 if m < 200 else 20  # 200 x 20 pairs... below the wide plan; the wide case follows
    for keep, budget, per_request in [(2, 12, 0), (3, 24, 4), (0, 8, 0)]:
        ids, wts = ops.route_budget(logits, topk, keep, budget, slots.cuda(), steps, per_request=per_request, min_cap=6)
        want = w3_moe.moe_layer(ex, x, ids, wts, shared=shared_ex)
        got, got_ids, got_w = w3_moe.moe_layer_budget(ex, x, logits, topk, keep, budget, slots.cuda(), steps, per_request=per_request, min_cap=6,
                                                      shared=shared_ex, return_routing=True)
        assert torch.equal(got_ids, ids) and torch.equal(got_w, wts) and torch.equal(got, want)
    got = w3_moe.moe_layer_budget(ex, x, logits, topk, 2, 12)  # no slots, no shared expert
    ids, wts = ops.route_budget(logits, topk, 2, 12)
    assert torch.equal(got, w3_moe.moe_layer(ex, x, ids, wts))


def test_layer_under_a_budget_with_more_pairs_than_one_workgroup_plans():
    from hibana_amd.kernels import ops, w3_moe
    e, m, topk = 32, 900, 10  # 9000 pairs: the plan is shared among workgroups
    ex, _ = random_experts(e, H, I, True, 31)
    g = torch.Generator().manual_seed(9)
    x = torch.randn(m, H, generator=g).bfloat16().cuda()
    logits = (torch.randn(m, e, generator=g) * 1.5).bfloat16().cuda()
    ids, wts = ops.route_budget(logits, topk, 2, 24)
    got, got_ids, got_w = w3_moe.moe_layer_budget(ex, x, logits, topk, 2, 24, return_routing=True)
    assert torch.equal(got_ids, ids) and torch.equal(got_w, wts) and torch.equal(got, w3_moe.moe_layer(ex, x, ids, wts))


def _one_token_both_ways(call):
    """`call()` with one token's fc2 and combine as one launch (the library's choice) and as two."""
    from hibana_amd import _lib
    fused = call()
    assert _lib.lib().hb_tune(b"moe_one", 2) == 0
    try:
        apart = call()
    finally:
        _lib.lib().hb_tune(b"moe_one", 0)
    return fused, apart


@pytest.mark.parametrize("k", [1, 3, TOPK, 15])
@pytest.mark.parametrize("shape", ["routed", "shared", "gate"])
def test_one_token_fc2_and_combine_in_one_launch_give_the_bits_of_two(gated, k, shape):
    """A decode step (one token) runs fc2 and the combine as one launch: bit for bit what the two launches give, with
    and without the shared expert and its gate, with ids past the local experts, on an expert-parallel half, and when
    the caller names an expert twice or five times (slots of more than one row, and of more than the body's four)."""
    from hibana_amd.kernels import w3_moe
    ex, get = gated
    shared_ex, shared_per = random_experts(1, H, I, True, 79)
    shared_get = oracle_expert_getter(shared_per, True, I)
    gate = (torch.randn(H, generator=torch.Generator().manual_seed(4)) * 0.05).cuda()
    kw = {"routed": {}, "shared": {"shared": shared_ex}, "gate": {"shared": shared_ex, "gate_vec": gate}}[shape]
    x, ids, weights = _inputs(1, k, 900 + k)
    cases = [ids.clone()]
    if k > 1:
        cases.append(ids.clone())
        cases[-1][0, -1] = w3_moe.EXPERTS  # a pair without an expert
        cases.append(ids.clone())
        cases[-1][0, 1] = cases[-1][0, 0]  # an expert named twice
    if k >= 5:
        cases.append(ids.clone())
        cases[-1][0, :5] = 3
    for case in cases:
        fused, apart = _one_token_both_ways(lambda: w3_moe.moe_layer(ex, x.cuda(), case.cuda(), weights.cuda(), **kw))
        assert torch.equal(fused, apart)
        want = layers.moe_layer_ref(x, case.numpy(), weights, get, True, e_n=E, shared=shared_get(0) if kw else None,
                                    gate_vec=gate.cpu() if shape == "gate" else None)
        mx, nr = errors(fused, want)
        assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    from dataclasses import replace
    half = E // 2
    hi = replace(ex, planes13=ex.planes13[half:], scales13=ex.scales13[half:], row13=ex.row13[half:], planes2=ex.planes2[half:],
                 scales2=ex.scales2[half:], row2=ex.row2[half:], base=half, tiled13=None, tiled2=None)
    fused, apart = _one_token_both_ways(lambda: w3_moe.w3_moe(hi, x.cuda(), ids.cuda(), weights.cuda()))
    assert torch.equal(fused, apart)


def test_one_token_at_the_decode_geometry_and_relu2(relu2):
    """The same at the benchmark layer's geometry (fc2 of four chunks, 32 output blocks) and on ReLU^2 experts."""
    from hibana_amd.kernels import w3_moe
    ex, _ = random_experts(24, 2048, 512, True, 81)
    shared_ex, _ = random_experts(1, 2048, 512, True, 82)
    g = torch.Generator().manual_seed(83)
    x = torch.randn(1, 2048, generator=g).bfloat16().cuda()
    logits = torch.randn(1, 24, generator=g).cuda()
    gate = (torch.randn(2048, generator=g) * 0.02).cuda()
    fused, apart = _one_token_both_ways(lambda: w3_moe.moe_layer_logits(ex, x, logits, TOPK, shared=shared_ex, gate_vec=gate))
    assert torch.equal(fused, apart) and fused.float().abs().max() > 0
    rex, _ = relu2
    xr, ids, weights = _inputs(1, 6, 84, experts=8)
    fused, apart = _one_token_both_ways(lambda: w3_moe.w3_moe(rex, xr.cuda(), ids.cuda(), weights.cuda()))
    assert torch.equal(fused, apart)


@pytest.mark.parametrize("m", [1, 16, 150])
def test_relu2_experts_with_their_own_fc2_codebook(relu2, m):
    """The latent experts' geometry in small (fc1 = up alone, h = relu(up)^2, top 6 of 8, a zero level in fc2)."""
    ex, get = relu2
    from hibana_amd.kernels import w3_moe
    assert not w3_moe.gated(ex)
    g = torch.Generator().manual_seed(700 + m)
    x = (torch.randn(m, 256, generator=g) * 0.5).bfloat16()
    ids = torch.stack([torch.randperm(8, generator=g)[:6] for _ in range(m)]).to(torch.int32)
    ids[0, 2] = ids[0, 1]  # a duplicate expert in one row is legal: two pairs on one expert
    weights = torch.rand(m, 6, generator=g)
    _check(ex, get, x, ids, weights, is_gated=False)


@pytest.mark.parametrize("m", [1, 32])  # one token: fc2 and the combine are one launch
def test_graph_replay_gives_the_eager_bits(gated, m):
    from hibana_amd.kernels import w3_moe
    ex, _ = gated
    x, ids, weights = _inputs(m, TOPK, 900)
    xd, idd, wd = x.cuda(), ids.cuda(), weights.cuda()
    eager = w3_moe.w3_moe(ex, xd, idd, wd)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = w3_moe.w3_moe(ex, xd, idd, wd)
    for _ in range(3):
        captured.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager)


@pytest.mark.parametrize("m", [2, 5, 17, 32, 100])
def test_one_launch_for_fc1_and_fc2_gives_the_bits_of_two(gated, m):
    """fc1 and fc2 in one launch (fc2's workgroups wait for their slot's fc1 workgroups) against the two launches: the
    same sums in the same order."""
    from hibana_amd import _lib
    from hibana_amd.kernels import w3_moe
    ex, _ = gated
    shared_ex, _ = random_experts(1, H, I, True, 77)
    x, ids, weights = _inputs(m, TOPK, 40 + m)
    call = lambda: w3_moe.moe_layer(ex, x.cuda(), ids.cuda(), weights.cuda(), shared=shared_ex)  # noqa: E731
    _lib.lib().hb_tune(b"moe_fused", 0)
    one = call()
    for lag in (1, 16):  # fc2 of a slot right behind its fc1's successor, or far behind
        _lib.lib().hb_tune(b"moe_lag", lag)
        assert torch.equal(call(), one)
    _lib.lib().hb_tune(b"moe_lag", 0)
    _lib.lib().hb_tune(b"moe_fused", 2)
    two = call()
    _lib.lib().hb_tune(b"moe_fused", 0)
    assert torch.equal(one, two)


@pytest.mark.parametrize("m", [819, 820, 2000])
def test_plan_orders_many_pairs_on_the_device(gated, m):
    """8,190 pairs (the last count one workgroup plans alone), 8,200 and 20,000 (shared among 8 and 19 workgroups in
    three launches), sorted by the planning kernel itself, against the oracle."""
    _check(*gated, *_inputs(m, TOPK, 1234 + m))


def test_bad_calls_raise(gated):
    from hibana_amd.kernels import w3_moe
    ex, _ = gated
    x, ids, weights = _inputs(4, TOPK, 1)
    with pytest.raises(ValueError):
        w3_moe.w3_moe(ex, x.cuda().float(), ids.cuda(), weights.cuda())
    with pytest.raises(ValueError):
        w3_moe.w3_moe(ex, x.cuda()[:, :128], ids.cuda(), weights.cuda())
    with pytest.raises(ValueError):
        w3_moe.w3_moe(ex, x.cuda(), ids.cuda()[:2], weights.cuda())
    with pytest.raises(RuntimeError):
        w3_moe.w3_moe(ex, x, ids, weights)
