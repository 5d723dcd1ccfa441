"""The E4M3 activation mode on the GPU: the activation rounding bit for bit against the oracle, the dense product and
the routed experts on rounded activations against the oracle's statement of the reference kernel's arithmetic
(hibana/kernels/w3_moe.py:182-214)."""
import numpy as np
import pytest
import torch

from oracle import layers, w3_format as ow3
from tests.util import MAX_REL, NORM_REL, errors, oracle_expert_getter, random_experts, random_w3, to_device_w3

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("m,k", [(1, 32), (3, 96), (17, 2048), (320, 512)])
def test_quant_groups_matches_the_oracle_bit_for_bit(m, k):
    from hibana_amd.kernels import w3
    g = torch.Generator().manual_seed(m + k)
    x = torch.randn(m, k, generator=g)
    x *= torch.logspace(-4, 4, m)[:, None]  # rows from tiny to large
    x[0, :32] = 0  # an all-zero group
    x[-1, -1] = 3.0e38  # near the top of the BF16 range
    x = x.bfloat16()
    want_q, want_s = layers.quant_e4m3_groups(x)
    q, s = w3.quant_groups(x.cuda())
    assert q.dtype == torch.float8_e4m3fn and q.shape == (m, k) and s.shape == (m, k // 32) and s.dtype == torch.float32
    assert torch.equal(s.cpu(), want_s)
    got = q.view(torch.uint8).cpu()
    same = (got == want_q) | (((got | want_q) & 0x7f) == 0)  # a zero of either sign is a zero
    assert bool(same.all()), int((~same).sum())


def test_quant_groups_rejects_what_it_cannot_take():
    from hibana_amd.kernels import w3
    with pytest.raises(ValueError):
        w3.quant_groups(torch.zeros(2, 48, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        w3.quant_groups(torch.zeros(2, 64, device="cuda"))
    with pytest.raises(RuntimeError):
        w3.quant_groups(torch.zeros(2, 64, dtype=torch.bfloat16))


@pytest.mark.parametrize("m", [1, 4, 5, 16, 33])
@pytest.mark.parametrize("n,k,codebook", [(128, 128, "uniform"), (256, 384, "lloyd"), (512, 2048, "zero8")])
def test_dense_product_on_rounded_activations(m, n, k, codebook):
    from hibana_amd import _lib
    from hibana_amd.kernels import w3
    packed, *_ = random_w3(n, k, 3, codebook)
    dev = to_device_w3(packed)
    x = torch.randn(m, k, generator=torch.Generator().manual_seed(m)).bfloat16()
    x[:, ::61] *= 20  # outlier channels: their groups get their own scales
    want = layers.dense_a8_ref(x, ow3.dequantize(packed))
    q, s = w3.quant_groups(x.cuda())
    try:
        for ks, nbw in ((0, 0), (1, 1), (2, 2), (3, 1)):
            if ks > k // 128:
                continue
            assert _lib.lib().hb_tune(b"w3_ksplit", ks) == 0 and _lib.lib().hb_tune(b"w3_nbw", nbw) == 0
            got = w3.w3_linear(q, dev, s)
            assert got.dtype == torch.bfloat16 and got.shape == (m, n)
            mx, nr = errors(got, want)
            assert mx < MAX_REL and nr < NORM_REL, (ks, nbw, mx, nr)
            assert torch.equal(w3.w3_linear(q, dev, s), got)  # bitwise repeatable
    finally:
        _lib.lib().hb_tune(b"w3_ksplit", 0)
        _lib.lib().hb_tune(b"w3_nbw", 0)


def test_scale_forms_and_bad_calls():
    from hibana_amd.kernels import w3
    packed, *_ = random_w3(128, 128, 4)
    dev = to_device_w3(packed)
    x = torch.randn(2, 128, generator=torch.Generator().manual_seed(0)).bfloat16()
    q, s = w3.quant_groups(x.cuda())
    one = torch.full((1,), 0.5, device="cuda")
    per_row = torch.tensor([0.5, 2.0], device="cuda")
    full = w3.w3_linear(q, dev, per_row[:, None].expand(2, 4).contiguous())
    assert torch.equal(w3.w3_linear(q, dev, per_row), full)
    assert torch.equal(w3.w3_linear(q[:1], dev, one), full[:1])
    with pytest.raises(ValueError):
        w3.w3_linear(q, dev)  # FP8 activations need their scale
    with pytest.raises(ValueError):
        w3.w3_linear(q, dev, torch.ones(3, device="cuda"))


@pytest.mark.parametrize("gated", [True, False])
@pytest.mark.parametrize("m,topk", [(1, 4), (9, 3), (40, 2)])
def test_routed_experts_on_rounded_activations(gated, m, topk):
    from hibana_amd.kernels import w3_moe
    e, hidden, inter = 6, 256, 128
    ex, per = random_experts(e, hidden, inter, gated, 31)
    g = torch.Generator().manual_seed(m)
    x = torch.randn(m, hidden, generator=g).bfloat16()
    ids = torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    ids[:, 0] = 1  # one loaded expert: slots of more than four rows take several passes
    wt = torch.rand(m, topk, generator=g) + 0.1
    get = oracle_expert_getter(per, gated, inter)
    pairs = layers.routed_experts_ref(x, ids.numpy(), get, gated, 0, e, quant=layers.rounded_e4m3)
    got_pairs = w3_moe.w3_moe(ex, x.cuda(), ids.cuda(), wt.cuda(), pairs=True, e4m3=True)
    mx, nr = errors(got_pairs, pairs)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    got = w3_moe.w3_moe(ex, x.cuda(), ids.cuda(), wt.cuda(), e4m3=True)
    mx, nr = errors(got, layers.combine_ref(pairs, ids.numpy(), wt, 0, e))
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    assert torch.equal(got, w3_moe.w3_moe(ex, x.cuda(), ids.cuda(), wt.cuda(), e4m3=True))
    # and it is a different function from the weight-only one: the rounding of x alone moves the result
    plain = w3_moe.w3_moe(ex, x.cuda(), ids.cuda(), wt.cuda())
    assert not torch.equal(plain, got)


@pytest.mark.parametrize("m,with_gate", [(1, False), (5, True), (33, True)])
def test_layer_with_shared_expert_on_rounded_activations(m, with_gate):
    """The whole layer in the E4M3 activation mode: the routed experts and the shared expert both round x and h."""
    from hibana_amd.kernels import w3_moe
    e, hidden, inter, topk = 8, 256, 128, 3
    ex, per = random_experts(e, hidden, inter, True, 41)
    shared_ex, shared_per = random_experts(1, hidden, inter, True, 42)
    get, shared_get = oracle_expert_getter(per, True, inter), oracle_expert_getter(shared_per, True, inter)
    g = torch.Generator().manual_seed(50 + m)
    x = torch.randn(m, hidden, generator=g).bfloat16()
    ids = torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    wt = torch.softmax(torch.randn(m, topk, generator=g), -1)
    gate = torch.randn(hidden, generator=g) * 0.05 if with_gate else None
    want = layers.moe_layer_ref(x, ids.numpy(), wt, get, True, shared=shared_get(0), gate_vec=gate, e_n=e, quant=layers.rounded_e4m3)
    run = lambda **kw: w3_moe.moe_layer(ex, x.cuda(), ids.cuda(), wt.cuda(), shared=shared_ex, gate_vec=None if gate is None else gate.cuda(), **kw)
    got = run(e4m3=True)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    assert torch.equal(run(e4m3=True), got)
    assert not torch.equal(run(), got)  # the weight-only layer is another function


@pytest.mark.parametrize("gated", [True, False])
def test_fc1_rounds_h_in_its_epilogue_under_every_split(gated):
    """h leaves fc1 as E4M3 codes: both bodies of the stream (expert 1 has twelve rows, the others at most four), K
    unsplit and split two to eight ways, one to four blocks a workgroup."""
    from hibana_amd import _lib
    from hibana_amd.kernels import w3_moe
    e, hidden, inter, m, topk = 4, 1024, 256, 12, 2
    ex, per = random_experts(e, hidden, inter, gated, 61)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(m, hidden, generator=g).bfloat16()
    x[:, ::53] *= 25
    ids = torch.stack([1 + torch.randperm(e - 1, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    ids[:, 0] = 1
    ids[:, 1] = torch.tensor([0, 2, 3] * 4)
    wt = torch.rand(m, topk, generator=g) + 0.1
    want = layers.routed_experts_ref(x, ids.numpy(), oracle_expert_getter(per, gated, inter), gated, 0, e, quant=layers.rounded_e4m3)
    try:
        for ks, nbw in ((1, 1), (1, 4), (2, 2), (3, 1), (4, 1), (5, 2), (8, 1), (0, 0)):
            assert _lib.lib().hb_tune(b"moe_fc1_ksplit", ks) == 0 and _lib.lib().hb_tune(b"moe_fc1_nbw", nbw) == 0
            got = w3_moe.w3_moe(ex, x.cuda(), ids.cuda(), wt.cuda(), pairs=True, e4m3=True)
            mx, nr = errors(got, want)
            assert mx < MAX_REL and nr < NORM_REL, (ks, nbw, mx, nr)
    finally:
        _lib.lib().hb_tune(b"moe_fc1_ksplit", 0)
        _lib.lib().hb_tune(b"moe_fc1_nbw", 0)


@pytest.mark.parametrize("m", [3, 4, 5, 16, 24])  # up to four rows the planning workgroup routes them itself
def test_layer_from_logits_on_rounded_activations(m):
    """Routing from the FP32 logits is the weight-only layer's; the experts then see rounded activations: the same
    output as the E4M3 layer called with the ids and weights the routing chose."""
    from hibana_amd.kernels import w3_moe
    e, hidden, inter, topk = 8, 256, 128, 3
    ex, _ = random_experts(e, hidden, inter, True, 41)
    shared_ex, _ = random_experts(1, hidden, inter, True, 42)
    g = torch.Generator().manual_seed(90 + m)
    x = torch.randn(m, hidden, generator=g).bfloat16().cuda()
    logits = torch.randn(m, e, generator=g).cuda()
    gate = (torch.randn(hidden, generator=g) * 0.05).cuda()
    got, ids, wt = w3_moe.moe_layer_logits(ex, x, logits, topk, shared=shared_ex, gate_vec=gate, return_routing=True, e4m3=True)
    _, ids_plain, wt_plain = w3_moe.moe_layer_logits(ex, x, logits, topk, shared=shared_ex, gate_vec=gate, return_routing=True)
    assert torch.equal(ids, ids_plain) and torch.equal(wt, wt_plain)
    assert torch.equal(got, w3_moe.moe_layer(ex, x, ids, wt, shared=shared_ex, gate_vec=gate, e4m3=True))


def test_many_pairs_on_rounded_activations_agree_with_the_call_in_halves():
    """From 8192 pairs the plan is shared among workgroups and the rounding of x is a launch of its own: the same rows
    as two calls of half the tokens, whose plans are one workgroup with the rounding beside it (the slots group the rows
    differently, so sums may differ in their last bits)."""
    from hibana_amd.kernels import w3_moe
    e, hidden, inter, m, topk = 8, 256, 128, 2048, 4
    ex, _ = random_experts(e, hidden, inter, True, 71)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(m, hidden, generator=g).bfloat16().cuda()
    ids = torch.stack([torch.randperm(e, generator=g)[:topk] for _ in range(m)]).to(torch.int32).cuda()
    wt = (torch.rand(m, topk, generator=g) + 0.1).cuda()
    whole = w3_moe.w3_moe(ex, x, ids, wt, e4m3=True)
    half = m // 2
    halves = torch.cat([w3_moe.w3_moe(ex, x[:half], ids[:half], wt[:half], e4m3=True), w3_moe.w3_moe(ex, x[half:], ids[half:], wt[half:], e4m3=True)])
    mx, nr = errors(whole, halves.cpu())
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    assert torch.equal(whole, w3_moe.w3_moe(ex, x, ids, wt, e4m3=True))
