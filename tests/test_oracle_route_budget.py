"""Pins of the oracle's budgeted expert selection (oracle/layers.py `route_budget_ref`, following
hibana/kernels/flashnext_fused.py:322-502 and the rule of tests/unit/test_moe_selection.py:19-58): a hand-worked call,
the reduction to a sorted top-k, padded requests, exact ties, the cap per request, and the invariants the reference's
unit test states; the latent MoE's form (`route_budget_sigmoid_ref`, hibana/model/nemotron/moe.py:124-313) by a
hand-worked call, the reduction to plain sigmoid routing and the invariants of tests/gpu/test_bolt_kernels.py:188-216."""
import math

import numpy as np
import torch

from oracle import layers

E, K = 512, 10


def gaussian_logits(rows: int, seed: int, experts: int = E, sigma: float = 1.2) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(rows, experts, generator=g) * sigma).bfloat16()


def test_a_call_worked_by_hand():
    """24 experts, k = 3, every row guaranteed its top 1. Row 0 ranks 5 > 7 > 9, row 1 ranks 11 > 7 > 2 > 5; the four
    lowest logits of a row are no candidates of it (row 0: 11, 20, 21, 22)."""
    lg = torch.full((2, 24), -1.0)
    lg[0, [5, 7, 9]] = torch.tensor([3.0, 2.0, 1.0])
    lg[0, [11, 20, 21, 22]] = -8.0
    lg[1, [11, 7, 2, 5]] = torch.tensor([3.0, 2.5, 1.0, 0.5])
    lg[1, [20, 21, 22, 23]] = -8.0
    lg = lg.bfloat16()
    # cap 3: the guaranteed {5, 11} and the one expert both rows hold in their top 3
    ids, w, chosen, core, _ = layers.route_budget_ref(lg, 3, 1, 3)
    assert core == {5, 11} and chosen == {5, 7, 11}
    assert ids.tolist() == [[5, 7, 24], [11, 7, 5]]  # row 0 cannot take 11: not among its 20 candidates
    e = math.e
    assert np.allclose(w[0].numpy(), [e / (1 + e), 1 / (1 + e), 0.0], rtol=1e-6)
    z = e ** 3 + e ** 2.5 + e ** 0.5
    assert np.allclose(w[1].numpy(), [e ** 3 / z, e ** 2.5 / z, e ** 0.5 / z], rtol=1e-6)
    # cap 4: rank 3 of row 0 (expert 9) and of row 1 (expert 2) hold the same logit; row 0's softmax denominator is the
    # smaller one, so 9 scores more
    ids, _, chosen, _, score = layers.route_budget_ref(lg, 3, 1, 4)
    assert score[9] > score[2] > 0 and chosen == {5, 7, 9, 11}
    assert ids.tolist() == [[5, 7, 9], [11, 7, 5]]
    # a slot left over repeats the row's first choice
    assert layers.route_budget_ref(lg, 3, 1, 3, repeat=True)[0].tolist() == [[5, 7, 5], [11, 7, 5]]
    # a budget below the guaranteed experts keeps them all and adds nothing
    ids, w, chosen, _, _ = layers.route_budget_ref(lg, 3, 1, 1)
    assert chosen == {5, 11} and ids.tolist() == [[5, 24, 24], [11, 5, 24]]
    assert w[0].tolist() == [1.0, 0.0, 0.0]


def test_a_cap_above_the_rows_union_is_plain_top_k():
    for seed, rows in [(0, 1), (1, 7), (2, 40)]:
        lg = gaussian_logits(rows, seed)
        ids, w, _, _, _ = layers.route_budget_ref(lg, K, 2, E)
        order = torch.sort(lg.float(), dim=-1, descending=True, stable=True).indices[:, :K]
        assert torch.equal(ids.long(), order)
        p = torch.softmax(lg.float(), -1).gather(1, order)
        torch.testing.assert_close(w, p / p.sum(-1, keepdim=True), rtol=2e-6, atol=0)


def test_exact_ties_and_both_zeros_go_to_the_lower_expert():
    lg = torch.zeros(1, E)
    lg[0, 1::2] = -0.0
    lg[0, [9, 3, 400]] = 1.0
    lg[0, 30:] -= 2.0
    lg[0, [9, 3, 400]] = 1.0
    ids, _, _, _, _ = layers.route_budget_ref(lg.bfloat16(), K, 0, E)
    assert ids[0].tolist() == [3, 9, 400, 0, 1, 2, 4, 5, 6, 7]


def test_padded_requests_score_nothing_and_name_no_expert():
    lg = gaussian_logits(12, 4)
    slots = torch.tensor([5, 0, 9, 0], dtype=torch.int32)
    real = torch.tensor([bool(slots[t // 3]) for t in range(12)])
    ids, w, chosen, _, _ = layers.route_budget_ref(lg, K, 3, 16, slots, 3)
    alone = layers.route_budget_ref(lg[real], K, 3, 16)
    assert chosen == alone[2]
    assert torch.equal(ids[real], alone[0]) and torch.equal(w[real], alone[1])
    assert (ids[~real] == E).all() and not w[~real].any()
    rep = layers.route_budget_ref(lg, K, 3, 16, slots, 3, repeat=True)[0]
    first = int(torch.sort(lg[0].float(), descending=True, stable=True).indices[0])
    assert (rep[~real] == first).all()  # row 0's first choice


def test_the_set_and_the_rows():
    for seed, keep, cap in [(0, 2, 16), (1, 4, 12), (2, 3, 64), (3, 1, 8)]:
        lg = gaussian_logits(16, seed)
        ids, w, chosen, core, score = layers.route_budget_ref(lg, K, keep, cap)
        order = torch.sort(lg.float(), dim=-1, descending=True, stable=True).indices
        assert core == set(order[:, :keep].reshape(-1).tolist())
        assert core <= chosen and len(chosen) == max(cap, len(core))  # 16 rows of 10 hold more than the cap
        assert set(ids.reshape(-1).tolist()) <= chosen | {E}
        assert torch.equal(ids[:, :keep].long(), order[:, :keep])
        torch.testing.assert_close(w.sum(-1), torch.ones(16), rtol=1e-6, atol=0)
        # no expert outside the set outscores one of its non-guaranteed members
        inside = [float(score[x]) for x in chosen - core]
        outside = [float(score[x]) for x in range(E) if x not in chosen]
        assert not inside or min(inside) >= max(outside)
        # a row's experts are in rank order and skip only candidates outside the set
        for t in range(16):
            cand = order[t, :layers.ROUTE_CANDIDATES].tolist()
            assert [x for x in ids[t].tolist() if x != E] == [x for x in cand if x in chosen][:K]


def test_the_cap_per_request_counts_real_requests():
    lg = gaussian_logits(40, 11)
    two = torch.tensor([3, 4, 0, 0, 0, 0, 0, 0], dtype=torch.int32)
    chosen = layers.route_budget_ref(lg, K, 1, 64, two, 5, per_request=6)[2]
    assert len(chosen) == 12  # min(64, 6 x 2): ten rows of ten hold more
    chosen = layers.route_budget_ref(lg, K, 1, 64, torch.arange(1, 9, dtype=torch.int32), 5, per_request=6)[2]
    assert len(chosen) == 48
    chosen = layers.route_budget_ref(lg[:9], K, 1, 64, torch.tensor([5], dtype=torch.int32), 9, per_request=12, min_cap=16)[2]
    assert len(chosen) == 16  # max(16, 12 x 1)


def test_silu_mul_rounds_the_fp32_product_once():
    g = torch.Generator().manual_seed(0)
    gu = (torch.randn(5, 128, generator=g) * 2).bfloat16()
    gate, up = gu[:, :64].double(), gu[:, 64:].double()
    exact = gate / (1 + torch.exp(-gate)) * up
    got = layers.silu_mul(gu)
    # one BF16 rounding of the exact product (where the FP32 arithmetic does not sit on a rounding boundary)
    want = exact.float().bfloat16()
    assert (got != want).float().mean() < 0.01
    assert (got.double() - exact).abs().max() <= (exact.abs() * 2.0 ** -8 + 1e-30).max()
    pairs = layers.silu_mul(torch.cat((gu[:, :32], gu[:, 64:96], gu[:, 32:64], gu[:, 96:]), 1), 32)
    assert torch.equal(pairs, got)


def test_the_sigmoid_form_worked_by_hand():
    """Eight experts, k = 3. Sigmoids 0.9 / 0.75 / 0.5 / 0.1 from logits ln 9 / ln 3 / 0 / -ln 9; a bias of 1 puts
    expert 5 (sigmoid 0.1) first in both rows' choice, and its weight stays 0.1."""
    hi, mid, low = math.log(9.0), math.log(3.0), -math.log(9.0)
    fused = torch.full((2, 8), low)
    fused[0, [0, 1, 2]] = torch.tensor([hi, mid, 0.0])
    fused[1, [2, 1, 3]] = torch.tensor([hi, mid, 0.0])
    bias = torch.zeros(8)
    bias[5] = 1.0
    run = lambda **kw: layers.route_budget_sigmoid_ref(fused, bias, 3, 0, **kw)  # noqa: E731
    # the guaranteed expert 5 and the one expert both rows hold below it
    ids, w, chosen, core, score, _ = run(keep=1, budget=2)
    assert core == {5} and chosen == {1, 5}
    assert np.allclose(score[[0, 1, 2]], [0.9 / 1.75, 1.5 / 1.75, 0.9 / 1.75], rtol=1e-6) and score[0] == score[2]
    assert ids.tolist() == [[5, 1, 5], [5, 1, 5]]  # the slot left over repeats the row's first choice
    assert np.allclose(w.numpy(), [[0.1 / 0.85, 0.75 / 0.85, 0.0]] * 2, rtol=1e-6)
    # experts 0 and 2 score the same: the lower one takes the third place
    ids, w, chosen, _, _, _ = run(keep=1, budget=3)
    assert chosen == {0, 1, 5} and ids.tolist() == [[5, 0, 1], [5, 1, 5]]
    assert np.allclose(w[0].numpy(), np.array([0.1, 0.9, 0.75]) / 1.75, rtol=1e-6)
    assert run(keep=1, budget=3, repeat=False)[0].tolist() == [[5, 0, 1], [5, 1, 8]]
    # the rows' top 2 are three experts, above a cap of 2: they all stay, unless a fallback of 1 guarantees only expert 5
    assert run(keep=2, budget=2)[2] == {0, 2, 5}
    ids, _, chosen, core, _, _ = run(keep=2, budget=2, fallback=1)
    assert core == {5} and chosen == {1, 5} and ids.tolist() == [[5, 1, 5], [5, 1, 5]]
    assert run(keep=2, budget=0, fallback=1)[2] == {0, 2, 5}  # no cap: nothing to fall back from


def test_the_sigmoid_form_with_every_top_k_in_the_set_is_plain_routing():
    g = torch.Generator().manual_seed(8)
    e, k, latent = 432, 9, 16
    fused = torch.randn(16, e + latent, generator=g) * 2
    bias = torch.randn(e, generator=g) * 0.1
    slots = torch.tensor([1, 0], dtype=torch.int32)
    ids, w, _, _, _, lat = layers.route_budget_sigmoid_ref(fused, bias, k, latent, 6, 512, slots, 8, repeat=False)
    want_ids, want_w = layers.route_sigmoid_topk(fused[:8, :e], bias, k)
    assert torch.equal(ids[:8], want_ids)
    torch.testing.assert_close(w[:8], want_w, rtol=1e-6, atol=0)
    assert (ids[8:] == e).all() and not w[8:].any()
    assert torch.equal(lat, fused[:, e:].bfloat16())


def test_the_sigmoid_form_invariants():
    g = torch.Generator().manual_seed(19)
    e, k, latent = 432, 9, 0
    for m, keep, cap in [(8, 6, 20), (32, 4, 48), (8, 6, 0)]:
        fused = torch.randn(m, e, generator=g) * 2
        bias = torch.randn(e, generator=g) * 0.1
        slots = torch.tensor([1] * (m // 8 - 1) + [0], dtype=torch.int32)
        real = m - 8
        ids, w, chosen, core, _, _ = layers.route_budget_sigmoid_ref(fused, bias, k, latent, keep, cap, slots, 8)
        s = torch.sigmoid(fused)
        order = torch.sort(s + bias, dim=-1, descending=True, stable=True).indices[:, :k]
        assert core == set(order[:real, :keep].reshape(-1).tolist()) and len(chosen) <= max(cap, len(core))
        for t in range(real):
            live = w[t] > 0
            assert torch.equal(ids[t, :keep].long(), order[t, :keep])
            picked = ids[t][live].long()
            assert picked.tolist() == [x for x in order[t].tolist() if x in chosen]
            torch.testing.assert_close(w[t][live], s[t, picked] / s[t, picked].sum(), rtol=1e-6, atol=1e-7)
            assert (ids[t][~live] == ids[t, 0]).all()
        assert not w[real:].any() and (ids[real:] == order[0, 0]).all()
