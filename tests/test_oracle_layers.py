"""The oracle's layer math against special cases, brute force and library routines (CPU)."""
import numpy as np
import torch

from oracle import layers as L


def _experts(e, inter, hidden, gated, seed):
    g = torch.Generator().manual_seed(seed)
    n1 = 2 * inter if gated else inter
    w13 = torch.randn(e, n1, hidden, generator=g) * 0.05
    w2 = torch.randn(e, hidden, inter, generator=g) * 0.05
    return lambda i: (w13[i].numpy(), w2[i].numpy()), w13, w2


def test_fc1_order_pairs_up_and_gate_rows():
    """tests/unit/test_w3_moe_pack.py:27-31 of the reference."""
    order = L.fc1_order(128)
    assert sorted(order.tolist()) == list(range(256))
    blocks = order.reshape(-1, 32)
    assert np.array_equal(blocks[:, 16:], blocks[:, :16] + 128)


def test_plan_is_a_stable_sort_with_csr_starts():
    g = np.random.default_rng(0)
    ids = g.integers(0, 20, (37, 6))
    ids[3, 2] = 512
    experts, starts, order = L.expert_plan(ids, 4, 10)
    flat = ids.reshape(-1) - 4
    key = np.where((flat >= 0) & (flat < 10), flat, 512)
    want = np.argsort(key, kind="stable")[:np.count_nonzero(key < 512)]
    assert np.array_equal(order, want)
    assert experts.tolist() == sorted(set(key[key < 512].tolist()))
    for d, e in enumerate(experts):
        assert (key[order[starts[d]:starts[d + 1]]] == e).all()
    assert starts[0] == 0 and starts[-1] == len(order)


def test_one_token_one_expert_reduces_to_two_dense_products():
    get, w13, w2 = _experts(3, 64, 128, True, 1)
    x = torch.randn(1, 128, generator=torch.Generator().manual_seed(2)).bfloat16()
    out = L.moe_layer_ref(x, np.array([[2]]), torch.ones(1, 1), get, True)
    h1 = (x.float() @ w13[2].T).bfloat16().float()
    h = (torch.nn.functional.silu(h1[:, 64:]) * h1[:, :64]).bfloat16()
    want = (h.float() @ w2[2].T).bfloat16()
    assert torch.allclose(out.float(), want.float(), rtol=2 ** -7, atol=1e-6)
    relu_get, r13, r2 = _experts(3, 64, 128, False, 4)
    out = L.moe_layer_ref(x, np.array([[1]]), torch.ones(1, 1), relu_get, False)
    h = torch.relu((x.float() @ r13[1].T).bfloat16().float()).square().bfloat16()
    assert torch.allclose(out.float(), (h.float() @ r2[1].T).bfloat16().float(), rtol=2 ** -7, atol=1e-6)


def test_matches_a_per_pair_loop_written_from_the_reference_formula():
    """hibana/kernels/w3_moe.py:205-213 with an identity activation rounding, one (row, slot) at a time."""
    import torch.nn.functional as F
    for gated in (True, False):
        get, w13, w2 = _experts(6, 32, 128, gated, 5)
        gen = torch.Generator().manual_seed(6)
        m, k, inter = 7, 3, 32
        x = torch.randn(m, 128, generator=gen).bfloat16()
        ids = torch.stack([torch.randperm(6, generator=gen)[:k] for _ in range(m)]).numpy()
        ids[2, 1] = 512  # an unfilled slot
        weights = torch.softmax(torch.randn(m, k, generator=gen), -1)
        out = torch.zeros(m, 128)
        for r in range(m):
            for s in range(k):
                e = int(ids[r, s])
                if e >= 6:
                    continue
                h1 = (x[r:r + 1].float() @ w13[e].T).to(torch.bfloat16).float()
                h = (F.silu(h1[:, inter:]) * h1[:, :inter] if gated else torch.relu(h1).square()).to(torch.bfloat16)
                out[r] += float(weights[r, s]) * (h.float() @ w2[e].T)[0]
        got = L.moe_layer_ref(x, ids, weights, get, gated, e_n=6)
        assert torch.allclose(got.float(), out.bfloat16().float(), rtol=2 ** -6, atol=1e-5)


def test_zero_weights_dropped_rows_and_slot_permutation():
    get, _, _ = _experts(4, 32, 128, True, 7)
    gen = torch.Generator().manual_seed(8)
    x = torch.randn(3, 128, generator=gen).bfloat16()
    ids = np.array([[0, 1], [2, 3], [512, 512]])
    assert not L.moe_layer_ref(x, ids, torch.zeros(3, 2), get, True, e_n=4).any()
    w = torch.full((3, 2), 0.5)
    a = L.moe_layer_ref(x, ids, w, get, True, e_n=4)
    b = L.moe_layer_ref(x, ids[:, ::-1].copy(), w, get, True, e_n=4)
    assert not a[2].any() and torch.allclose(a.float(), b.float(), rtol=2 ** -7, atol=1e-6)
    # expert-parallel halves add up to the whole (tests/gpu/test_w3_moe.py:84-105 of the reference)
    lo = L.moe_layer_ref(x, ids, w, get, True, e_lo=0, e_n=2)
    hi = L.moe_layer_ref(x, ids, w, lambda e: get(e + 2), True, e_lo=2, e_n=2)
    assert torch.allclose(lo.float() + hi.float(), a.float(), rtol=2 ** -6, atol=1e-5)


def test_shared_expert_and_gate():
    get, w13, w2 = _experts(4, 32, 128, True, 9)
    gen = torch.Generator().manual_seed(10)
    x = torch.randn(5, 128, generator=gen).bfloat16()
    ids = np.stack([np.array([0, 1]) for _ in range(5)])
    w = torch.full((5, 2), 0.5)
    routed = L.moe_layer_ref(x, ids, w, get, True, e_n=4)
    shared = L.moe_layer_ref(x, np.full((5, 1), 3), torch.ones(5, 1), get, True, e_n=4)
    both = L.moe_layer_ref(x, ids, w, get, True, shared=get(3), e_n=4)
    assert torch.equal(both, (routed.float() + shared.float()).bfloat16())
    gate = torch.randn(128, generator=gen) * 0.1
    gated = L.moe_layer_ref(x, ids, w, get, True, shared=get(3), gate_vec=gate, e_n=4)
    g = torch.sigmoid(x.float() @ gate)[:, None]
    assert torch.allclose(gated.float(), (routed.float() + g * shared.float()).bfloat16().float(), rtol=2 ** -7, atol=1e-6)


def test_routing_against_torch():
    gen = torch.Generator().manual_seed(11)
    logits = torch.randn(9, 64, generator=gen)
    ids, w = L.route_softmax_topk(logits, 5)
    sel = logits.gather(1, ids.long())
    assert torch.allclose(w, torch.softmax(sel, -1), atol=1e-6)  # renormalized softmax == softmax over the selection
    assert (sel[:, :-1] >= sel[:, 1:]).all()
    bias = torch.randn(64, generator=gen) * 0.1
    ids2, w2 = L.route_sigmoid_topk(logits, bias, 6, 2.5)
    want = torch.topk(torch.sigmoid(logits) + bias, 6).indices
    assert torch.equal(ids2.long().sort(-1).values, want.sort(-1).values)
    assert torch.allclose(w2.sum(-1), torch.full((9,), 2.5), atol=1e-5)
    tie = torch.zeros(1, 8)
    assert L.route_sigmoid_topk(tie, torch.zeros(8), 3)[0].tolist() == [[0, 1, 2]]


def test_latent_moe_single_expert_special_case():
    gen = torch.Generator().manual_seed(12)
    x = torch.randn(4, 64, generator=gen).bfloat16()
    fc1 = (torch.randn(32, 64, generator=gen) * 0.1).bfloat16()
    fc2 = (torch.randn(64, 32, generator=gen) * 0.1).bfloat16()
    up = torch.randint(-6, 7, (48, 32), generator=gen).float() * 0.5
    down = torch.randint(-6, 7, (32, 48), generator=gen).float() * 0.5
    got = L.latent_moe_ref(x, fc1, fc2, np.zeros((4, 1), np.int64), torch.full((4, 1), 0.75), lambda e: (up.numpy(), 0.01, down.numpy(), 0.02))
    lat = (x.float() @ fc1.float().T).bfloat16()
    h = torch.relu(((lat.float() @ up.T) * 0.01).bfloat16().float()).square().bfloat16()
    acc = (h.float() @ down.T) * 0.02 * 0.75
    want = (acc.bfloat16().float() @ fc2.float().T).bfloat16()
    assert torch.allclose(got.float(), want.float(), rtol=2 ** -6, atol=1e-6)


def test_silu_and_mul_layouts():
    gen = torch.Generator().manual_seed(13)
    gu = torch.randn(3, 256, generator=gen)
    plain = L.silu_and_mul(gu)
    assert torch.allclose(plain, torch.nn.functional.silu(gu[:, :128]) * gu[:, 128:])
    order = torch.arange(256).view(2, 2, 64).transpose(0, 1).reshape(-1)  # pair_order(256, 64)
    assert torch.allclose(L.silu_and_mul(gu[:, order], pairs=64), plain)


# ------------------------------------------------------------------------------------------ E4M3 activation rounding
def _e4m3_table():
    """Every finite E4M3 value from the bit fields (1 sign, 4 exponent bits with bias 7, 3 mantissa bits, no infinities,
    0x7f / 0xff NaN), written out here rather than taken from a dtype cast."""
    vals = []
    for byte in range(256):
        sign, exp, man = byte >> 7, (byte >> 3) & 15, byte & 7
        if exp == 15 and man == 7:
            vals.append(float("nan"))
            continue
        mag = man / 8.0 * 2.0 ** -6 if exp == 0 else (1 + man / 8.0) * 2.0 ** (exp - 7)
        vals.append(-mag if sign else mag)
    return np.array(vals, dtype=np.float64)


def _nearest_e4m3(v: float, table: np.ndarray) -> int:
    """The code whose value is nearest to v; of two equally near, the one with the even code (round to nearest even)."""
    dist = np.abs(table - v)
    dist[np.isnan(dist)] = np.inf
    best = np.flatnonzero(dist == dist.min())
    best = [b for b in best if (b < 128) == (v >= 0 or table[b] == 0)] or list(best)  # the zero of v's sign
    if v == 0:
        return 0x80 if np.signbit(v) else 0
    return int(min(best, key=lambda b: (b & 1, b)))


def test_quant_e4m3_groups_is_nearest_value_rounding_under_the_group_scale():
    table = _e4m3_table()
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(6, 96, generator=g) * torch.tensor([1e-3, 0.1, 1.0, 30.0, 3e3, 1.0])[:, None]).bfloat16()
    x[5, :32] = 0  # an all-zero group: scale 1e-12, codes zero
    x[5, 40] = -0.0
    q, s = L.quant_e4m3_groups(x)
    assert q.dtype == torch.uint8 and q.shape == (6, 96) and s.shape == (6, 3) and s.dtype == torch.float32
    xf = x.float().numpy()
    for r in range(6):
        for grp in range(3):
            vals = xf[r, 32 * grp:32 * grp + 32]
            amax = np.float32(np.abs(vals).max())
            scale = max(np.float32(amax / np.float32(448.0)), np.float32(1e-12))
            assert s[r, grp].item() == scale
            for i, v in enumerate(vals):
                ratio = float(np.float32(v) / scale)  # the FP32 quotient, as the definition divides in FP32
                want = _nearest_e4m3(min(max(ratio, -448.0), 448.0), table)
                got = int(q[r, 32 * grp + i])
                assert table[got] == table[want] and (got == want or table[got] == 0), (r, grp, i, v, got, want)
            if amax > 0:  # the group's largest magnitude lands on the largest code
                top = int(np.argmax(np.abs(vals)))
                assert abs(table[int(q[r, 32 * grp + top])]) == 448.0
    back = L.dequant_e4m3_groups(q, s)
    assert torch.all(back[5, :32] == 0)


def test_quant_e4m3_groups_keeps_what_is_already_representable():
    table = _e4m3_table()
    codes = torch.randint(0, 127, (4, 64), generator=torch.Generator().manual_seed(1))
    codes[:, 0] = 126  # 448 in every group: the scale is exactly the multiplier
    codes[:, 32] = 126
    vals = torch.tensor(table[codes.numpy()], dtype=torch.float32) * 0.25  # a power-of-two scale: bf16-exact
    q, s = L.quant_e4m3_groups(vals.bfloat16())
    assert torch.all(s == 0.25) and torch.equal(q.long(), codes)
    assert torch.equal(L.rounded_e4m3(vals.bfloat16()), vals)


def test_quant_e4m3_rows_is_the_same_rounding_with_one_scale_a_row():
    table = _e4m3_table()
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(5, 96, generator=g) * torch.tensor([1e-3, 0.1, 1.0, 300.0, 1.0])[:, None]).bfloat16()
    x[4] = 0  # an all-zero row: scale 1e-12, codes zero
    q, s = L.quant_e4m3_rows(x)
    assert q.dtype == torch.uint8 and q.shape == (5, 96) and s.shape == (5,) and s.dtype == torch.float32
    xf = x.float().numpy()
    for r in range(5):
        scale = max(np.float32(np.float32(np.abs(xf[r]).max()) / np.float32(448.0)), np.float32(1e-12))
        assert s[r].item() == scale
        for i, v in enumerate(xf[r]):
            want = _nearest_e4m3(min(max(float(np.float32(v) / scale), -448.0), 448.0), table)
            got = int(q[r, i])
            assert table[got] == table[want] and (got == want or table[got] == 0), (r, i, v, got, want)
    # a row that is one 32-group: the per-row and the per-group forms are the same function
    one = x[:, :32].contiguous()
    qg, sg = L.quant_e4m3_groups(one)
    qr, sr = L.quant_e4m3_rows(one)
    assert torch.equal(qg, qr) and torch.equal(sg.reshape(-1), sr)


def test_dense_a8_ref_is_the_dense_product_of_the_rounded_activations():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 64, generator=g).bfloat16()
    w = torch.randn(5, 64, generator=g)
    want = L.dense_ref(L.rounded_e4m3(x), w.numpy())  # rounded values are FP32: dense_ref takes any float x
    assert torch.equal(L.dense_a8_ref(x, w.numpy()), want)
    # one expert, one token, weight one: the routed sum with quant is two dense products with both inputs rounded
    w13, w2 = torch.randn(64, 64, generator=g), torch.randn(64, 32, generator=g)
    y = L.expert_pairs_ref(x[:1], np.array([0]), w13.numpy(), w2.numpy(), True, quant=L.rounded_e4m3)
    h1 = L.bf16((L.rounded_e4m3(x[:1]).double() @ w13.double().T).float()).float()
    h = L.bf16(torch.nn.functional.silu(h1[:, 32:]) * h1[:, :32])
    assert torch.equal(y, (L.rounded_e4m3(h).double() @ w2.double().T).float())
