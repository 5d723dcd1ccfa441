"""Budgeted expert selection on the GPU (`ops.route_budget`, through hb_route_budget) against the oracle's rule. The
set's scores are FP32 sums of each side's own softmax, so the set is compared up to FP32 near-ties at its boundary, as
the reference's own GPU test does (tests/gpu/test_route_budget.py:46-63); given the set, ids are bitwise and weights
hold to rtol 1e-5. Inputs: router-like logits with a component the rows share, exact ties across the guarantee, rank-k
and rank-20 boundaries, logits on a coarse grid with both zeros, padded requests anywhere, a cap per request, expert
counts other than 512, and replays of a captured graph."""
import pytest
import torch

from hibana_amd.kernels import ops
from oracle import layers

pytestmark = pytest.mark.gpu
E, K, C = 512, 10, layers.ROUTE_CANDIDATES


def router_like(rows: int, seed: int, top: float = 3.0, common: float = 0.0, experts: int = E) -> torch.Tensor:
    """BF16 logits of about a router's spread whose row maximum is `top` (the BF16 spacing there sets how often logits
    tie exactly), with a part all rows share."""
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(rows, experts, generator=g) * 1.2 + common * torch.randn(1, experts, generator=g)
    return (z + (top - z.amax(-1, keepdim=True))).bfloat16()


def ties_at(lg: torch.Tensor, rank: int) -> torch.Tensor:
    """Exact ties across the boundary between ranks `rank` - 1 and `rank` of every row (one or two experts below it
    raised to the logit above it)."""
    out = lg.clone()
    order = torch.sort(lg.float(), dim=-1, descending=True, stable=True).indices
    for t in range(lg.shape[0]):
        for below in range(rank, rank + 1 + t % 2):
            out[t, order[t, below]] = lg[t, order[t, rank - 1]]
    return out


def on_a_grid(rows: int, seed: int, experts: int = E) -> torch.Tensor:
    """Multiples of 1/8 in [-3, 0] with zeros of both signs: most of a row's candidates tie."""
    g = torch.Generator().manual_seed(seed)
    v = torch.randint(0, 25, (rows, experts), generator=g).float() * -0.125
    flip = torch.rand(rows, experts, generator=g) < 0.5
    return torch.where(flip & (v == 0), torch.tensor(-0.0), v).bfloat16()


def paddings(requests: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    live = torch.randint(1, 1000, (requests,), generator=g, dtype=torch.int32)
    tail = live.clone()
    tail[requests - max(1, requests // 3):] = 0
    holes = torch.where(torch.arange(requests) % 3 == 0, torch.zeros_like(live), live)
    return [tail, holes, torch.zeros_like(live)]


def check(lg, keep, cap, slots=None, steps=1, per_request=0, repeat=False, min_cap=0, k=K):
    e = lg.shape[1]
    ids, w = ops.route_budget(lg.cuda(), k, keep, cap, None if slots is None else slots.cuda(), steps, repeat=repeat, per_request=per_request,
                              min_cap=min_cap)
    ids, w = ids.cpu(), w.cpu()
    real = [slots is None or int(slots[t // steps]) != 0 for t in range(lg.shape[0])]
    _, _, want, core, score = layers.route_budget_ref(lg, k, keep, cap, slots, steps, repeat, per_request, min_cap)
    if per_request:
        cap = min(cap, max(min_cap, per_request * sum(1 for t in range(0, len(real), steps) if real[t])))
    got = {int(x) for t, row in enumerate(ids.tolist()) if real[t] for x in row} - {e}
    assert core <= got and len(got) <= max(cap, len(core))
    differ = (got - core) ^ (want - core)
    if differ:  # only where the last places of the set tie up to FP32 rounding
        edge = [float(score[x]) for x in (got | want) - core]
        assert all(abs(float(score[x]) - min(edge)) <= 1e-5 * max(1.0, max(edge)) for x in differ), differ
    rids, rw, _, _, _ = layers.route_budget_ref(lg, k, keep, cap, slots, steps, repeat, given=got)
    assert torch.equal(ids, rids)
    torch.testing.assert_close(w, rw, rtol=1e-5, atol=0)
    return ids, got


@pytest.mark.parametrize("rows", [1, 5, 20, 64, 256])
@pytest.mark.parametrize("keep,cap", [(1, 8), (2, 16), (3, 24), (4, 64), (4, 512)])
def test_matches_the_rule(rows, keep, cap):
    seed = 1000 * keep + rows
    base = router_like(rows, seed, common=1.0)
    for lg in (base, router_like(rows, seed + 1, top=8.0), ties_at(base, keep), ties_at(base, K), ties_at(base, C), on_a_grid(rows, seed)):
        check(lg, keep, cap)


@pytest.mark.parametrize("steps", [1, 5])
@pytest.mark.parametrize("rows", [5, 20, 65, 320])
def test_padded_requests_score_nothing_and_name_no_expert(rows, steps):
    for i, slots in enumerate(paddings(rows // steps, 7 * rows + steps)):
        for lg in (ties_at(router_like(rows, i, common=1.0), 3), on_a_grid(rows, i)):
            ids, _ = check(lg, 3, 32, slots, steps)
            padded = ~(slots != 0).repeat_interleave(steps)
            assert (ids[padded] == E).all()
            rep, _ = check(lg, 3, 32, slots, steps, repeat=True)
            first = int(torch.sort(lg[0].float(), descending=True, stable=True).indices[0])
            assert (rep[padded] == first).all() and (rep < E).all()


def test_the_cap_per_request_counts_real_requests():
    lg = router_like(40, 11, common=0.5)  # eight requests of five rows
    two = torch.tensor([3, 4, 0, 0, 0, 0, 0, 0], dtype=torch.int32)
    assert len(check(lg, 1, 64, two, 5, per_request=6)[1]) <= 12
    assert 12 < len(check(lg, 1, 64, torch.arange(1, 9, dtype=torch.int32), 5, per_request=6)[1]) <= 48
    one = check(router_like(9, 12, common=0.5), 1, 64, torch.tensor([5], dtype=torch.int32), 9, per_request=12, min_cap=16)[1]
    assert 12 < len(one) <= 16  # a request alone takes the floor
    assert 16 < len(check(router_like(36, 13, common=0.5), 1, 64, torch.arange(1, 5, dtype=torch.int32), 9, per_request=12, min_cap=16)[1]) <= 48
    # more requests than one pass of the counting workgroup holds
    many = torch.arange(1, 1301, dtype=torch.int32) % 4
    assert len(check(router_like(1300, 14, common=0.5), 1, 400, many, 1, per_request=1)[1]) <= 400


@pytest.mark.parametrize("experts,k", [(20, 3), (64, 8), (100, 10), (384, 8), (1000, 20), (1024, 6)])
def test_other_expert_counts(experts, k):
    for rows, keep, cap in [(1, 1, 4), (9, 2, 12), (33, 3, 40)]:
        for lg in (router_like(rows, experts + rows, common=0.7, experts=experts), on_a_grid(rows, experts + rows, experts)):
            check(lg, min(keep, k), cap, k=k)
            check(lg, min(keep, k), experts, k=k, repeat=True)


def test_a_keep_of_none_and_a_budget_of_none():
    lg = router_like(12, 21, common=1.0)
    check(lg, 0, 16)          # nothing guaranteed: the set is the best-scoring experts alone
    ids, got = check(lg, 2, 0)  # no budget: the guaranteed experts alone
    assert (ids[:, 2:] == E).sum() > 0


def test_the_same_bits_on_every_run():
    lg = ties_at(router_like(64, 5, common=1.0), 4).cuda()
    first = ops.route_budget(lg, K, 4, 48)
    for _ in range(5):
        again = ops.route_budget(lg, K, 4, 48)
        assert torch.equal(first[0], again[0]) and torch.equal(first[1].view(torch.int32), again[1].view(torch.int32))


@pytest.mark.parametrize("rows,steps", [(5, 5), (20, 1), (320, 5)])
def test_graph_replay(rows, steps):
    n = rows // steps
    feeds = [(router_like(rows, 1, common=1.0), torch.arange(1, n + 1, dtype=torch.int32))]
    feeds += [(ties_at(router_like(rows, 2 + i), 4), s) for i, s in enumerate(paddings(n, rows))]
    lg, slots = feeds[0][0].cuda(), feeds[0][1].cuda()
    ops.route_budget(lg, K, 4, 64, slots, steps, per_request=12)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ids, w = ops.route_budget(lg, K, 4, 64, slots, steps, per_request=12)
    for logits, sl in feeds + feeds[:2]:
        lg.copy_(logits)
        slots.copy_(sl)
        graph.replay()
        torch.cuda.synchronize()
        eager = ops.route_budget(logits.cuda(), K, 4, 64, sl.cuda(), steps, per_request=12)
        assert torch.equal(ids, eager[0]) and torch.equal(w.view(torch.int32), eager[1].view(torch.int32))


def test_silu_mul_rounds_once():
    g = torch.Generator().manual_seed(3)
    for rows, inter, pairs in [(1, 64, 0), (7, 512, 0), (33, 1024, 32), (4, 96, 16)]:
        gu = (torch.randn(rows, 2 * inter, generator=g) * 2).bfloat16()
        got = ops.silu_mul(gu.cuda(), pairs).cpu()
        want = layers.silu_mul(gu, pairs)
        # the FP32 sigmoid of the two sides may differ in its last place: a BF16 result may then sit one step apart
        assert (got != want).float().mean() < 0.005
        torch.testing.assert_close(got.float(), want.float(), rtol=2.0 ** -7, atol=1e-30)


# ------------------------------------------------------------------ the latent MoE's form (sigmoid + bias ranking)

def check_sigmoid(fused, bias, k, latent, keep, cap, slots=None, steps=1, per_request=0, repeat=True, fallback=0):
    """The device ranks a row as its plain routing does (checked against the oracle on its own), so the candidates are
    the device's own top k: a last-bit difference between the two sides' sigmoids cannot reorder them."""
    from hibana_amd.model import nemotron_moe
    e = fused.shape[1] - latent
    dev = lambda t: None if t is None else t.cuda()  # noqa: E731
    ids, w, lat = nemotron_moe.route_budget(dev(fused), dev(bias), k, latent, keep, cap, dev(slots), steps, per_request, repeat, fallback)
    ids, w = ids.cpu(), w.cpu()
    cand = nemotron_moe.route_topk(dev(fused), dev(bias), k, latent)[0].cpu().tolist()
    real = [slots is None or int(slots[t // steps]) != 0 for t in range(fused.shape[0])]
    _, _, want, core, score, want_lat = layers.route_budget_sigmoid_ref(fused, bias, k, latent, keep, cap, slots, steps, per_request, repeat, fallback, cand=cand)
    if per_request:
        cap = min(cap, per_request * sum(1 for t in range(0, len(real), steps) if real[t]))
    got = {int(x) for t in range(len(real)) if real[t] for x, v in zip(ids[t].tolist(), w[t].tolist()) if v > 0}
    assert core <= got and len(got) <= max(cap, len(core))
    differ = (got - core) ^ (want - core)
    if differ:
        edge = [float(score[x]) for x in (got | want) - core]
        assert all(abs(float(score[x]) - min(edge)) <= 1e-5 * max(1.0, max(edge)) for x in differ), differ
    rids, rw, _, _, _, _ = layers.route_budget_sigmoid_ref(fused, bias, k, latent, keep, cap, slots, steps, 0, repeat, fallback, cand=cand, given=got)
    assert torch.equal(ids, rids)
    torch.testing.assert_close(w, rw, rtol=1e-5, atol=0)
    assert torch.equal(lat.cpu(), want_lat)
    return ids, w, got


@pytest.mark.parametrize("m,keep,cap", [(8, 6, 20), (32, 4, 48), (8, 6, 0), (8, 9, 512), (16, 3, 30)])
@pytest.mark.parametrize("repeat", [True, False])
def test_sigmoid_form_at_the_top_9_of_432(m, keep, cap, repeat):
    """The invariants of the reference's own test (tests/gpu/test_bolt_kernels.py:188-216) and, with every top 9 in the
    set, the plain routing's ids and weights bit for bit."""
    from hibana_amd.model import nemotron_moe
    g = torch.Generator().manual_seed(19 + m)
    experts, latent, k = 432, 1024, 9
    fused = torch.randn(m, experts + latent, generator=g) * 2
    bias = torch.randn(experts, generator=g) * 0.1
    slots = torch.tensor([1] * (m // 8 - 1) + [0], dtype=torch.int32)  # the last request padded
    ids, w, got = check_sigmoid(fused, bias, k, latent, min(keep, k), cap, slots, 8, repeat=repeat)
    real = m - 8
    order = nemotron_moe.route_topk(fused.cuda(), bias.cuda(), k, latent)[0].cpu()
    s = torch.sigmoid(fused[:, :experts])
    for t in range(real):
        live = w[t] > 0
        assert torch.equal(ids[t, :min(keep, k)], order[t, :min(keep, k)])
        picked = ids[t][live].long()
        torch.testing.assert_close(w[t][live], s[t, picked] / s[t, picked].sum(), rtol=2e-6, atol=1e-7)
        assert (ids[t][~live] == (ids[t, 0] if repeat else experts)).all()
    assert not w[real:].any() and (ids[real:] == (order[0, 0] if repeat else experts)).all()
    if cap >= real * k:
        plain = nemotron_moe.route_topk(fused.cuda(), bias.cuda(), k, latent, slots.cuda(), 8, repeat)
        assert torch.equal(ids, plain[0].cpu()) and torch.equal(w, plain[1].cpu())


@pytest.mark.parametrize("m,cap", [(4, 44), (16, 64), (16, 128), (1, 22), (64, 96)])
def test_sigmoid_form_at_the_top_22_of_512(m, cap):
    g = torch.Generator().manual_seed(1000 + m)
    experts, latent, k = 512, 1024, 22
    fused = torch.randn(m, experts + latent, generator=g) * 1.5
    bias = torch.randn(experts, generator=g) * 0.1
    keep = max(4, min(8, cap // m))
    slots = torch.tensor([1] * max(1, m - 1) + [0] * (m > 1), dtype=torch.int32)  # the last row padded
    check_sigmoid(fused, bias, k, latent, keep, cap, slots, 1)
    check_sigmoid(fused, bias, k, latent, keep, cap, None, 1, per_request=12)
    check_sigmoid(fused, bias, k, latent, keep, cap, slots, 1, repeat=False)


def test_sigmoid_form_falls_back_when_the_floors_exceed_the_cap():
    g = torch.Generator().manual_seed(5)
    experts, latent, k = 512, 64, 22
    fused = torch.randn(16, experts + latent, generator=g) * 1.5
    bias = torch.zeros(experts)
    full = check_sigmoid(fused, bias, k, latent, 12, 48)[2]           # sixteen rows' top 12: far more than 48 experts, all kept
    assert len(full) > 48
    capped = check_sigmoid(fused, bias, k, latent, 12, 48, fallback=2)[2]  # guaranteed only their top 2: the cap holds
    assert len(capped) == 48
    assert check_sigmoid(fused, bias, k, latent, 12, 0, fallback=2)[2] == check_sigmoid(fused, bias, k, latent, 12, 0)[2]  # no cap, no fallback
    roomy = check_sigmoid(fused[:2], bias, k, latent, 12, 48, fallback=2)[2]  # two rows' top 12 fit: the floors stand
    assert len(roomy) == 44  # their 44 candidates in all


@pytest.mark.parametrize("experts,k", [(32, 32), (100, 8), (1000, 32), (1024, 6)])
def test_sigmoid_form_at_other_expert_counts(experts, k):
    g = torch.Generator().manual_seed(experts)
    for m, keep, cap in [(1, 1, 4), (9, 2, 12), (33, 3, 40)]:
        fused = torch.randn(m, experts + 8, generator=g) * 2
        bias = torch.randn(experts, generator=g) * 0.1
        check_sigmoid(fused, bias, k, 8, min(keep, k), cap)


def test_sigmoid_form_graph_replay():
    from hibana_amd.model import nemotron_moe
    g = torch.Generator().manual_seed(2)
    experts, latent, k = 512, 256, 22
    feeds = [(torch.randn(16, experts + latent, generator=g) * 1.5, s) for s in paddings(4, 9) + [torch.arange(1, 5, dtype=torch.int32)]]
    bias = (torch.randn(experts, generator=g) * 0.1).cuda()
    fused, slots = feeds[0][0].cuda(), feeds[0][1].cuda()
    call = lambda f, s: nemotron_moe.route_budget(f, bias, k, latent, 6, 40, s, 4, per_request=16, fallback=2)  # noqa: E731
    call(fused, slots)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = call(fused, slots)
    for f, s in feeds + feeds[:2]:
        fused.copy_(f)
        slots.copy_(s)
        graph.replay()
        torch.cuda.synchronize()
        eager = call(f.cuda(), s.cuda())
        assert all(torch.equal(a.view(torch.int32) if a.dtype == torch.float32 else a, b.view(torch.int32) if b.dtype == torch.float32 else b)
                   for a, b in zip(out, eager))
