"""Pins of the oracle's budgeted expert selection (oracle/layers.py `route_budget_ref`, following
hibana/kernels/flashnext_fused.py:322-502 and the rule of tests/unit/test_moe_selection.py:19-58): a hand-worked call,
the reduction to a sorted top-k, padded requests, exact ties, the cap per request, and the invariants the reference's
unit test states."""
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
