"""The small ops either side of the experts on the GPU: per-row activation rounding, the standalone SiLU-gate, softmax
routing with a graph's padded rows, the gated-MoE block (`MoeLayer`), attaching calibrated copies to a model."""
import json
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import layers, w3_format as ow3
from tests.util import MAX_REL, NORM_REL, errors, oracle_expert_getter, random_experts, random_w3, to_device_w3

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("m,k", [(1, 32), (3, 104), (17, 2048), (64, 5120)])
def test_quant_rows_matches_the_oracle_bit_for_bit(m, k):
    from hibana_amd.kernels import w3
    g = torch.Generator().manual_seed(m + k)
    x = torch.randn(m, k, generator=g) * torch.logspace(-4, 4, m)[:, None]
    x[0] = 0 if m > 1 else x[0]  # an all-zero row
    x[-1, -1] = 3.0e38
    x = x.bfloat16()
    want_q, want_s = layers.quant_e4m3_rows(x)
    q, s = w3.quant_rows(x.cuda())
    assert q.dtype == torch.float8_e4m3fn and q.shape == (m, k) and s.shape == (m,) and s.dtype == torch.float32
    assert torch.equal(s.cpu(), want_s)
    got = q.view(torch.uint8).cpu()
    same = (got == want_q) | (((got | want_q) & 0x7f) == 0)  # a zero of either sign is a zero
    assert bool(same.all()), int((~same).sum())


def test_w3_linear_takes_per_row_scales():
    """w3_linear on quant_rows' output is the oracle's product of the row-rounded activations."""
    from hibana_amd.kernels import w3
    packed, *_ = random_w3(256, 384, 3)
    dev = to_device_w3(packed)
    x = torch.randn(5, 384, generator=torch.Generator().manual_seed(1)).bfloat16()
    q, s = w3.quant_rows(x.cuda())
    got = w3.w3_linear(q, dev, s)
    qo, so = layers.quant_e4m3_rows(x)
    rounded = qo.view(torch.float8_e4m3fn).float() * so[:, None]
    want = layers.dense_ref(rounded, ow3.dequantize(packed))
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)


@pytest.mark.parametrize("shape,pairs", [((3, 256), 0), ((3, 256), 64), ((2, 5, 1024), 0), ((7, 1024), 16), ((1, 4), 2)])
def test_silu_and_mul_matches_the_bf16_tensor_expression(shape, pairs):
    from hibana_amd.kernels import ops
    gu = (torch.randn(*shape, generator=torch.Generator().manual_seed(shape[-1] + pairs)) * 3).bfloat16()
    want = layers.silu_and_mul(gu, pairs)
    got = ops.silu_and_mul(gu.cuda(), pairs).cpu()
    assert got.dtype == torch.bfloat16 and got.shape == want.shape
    # the device exponential may differ from the host's in its last bit: one BF16 unit at most, and rarely
    off = got.view(torch.int16).int() - want.view(torch.int16).int()
    assert off.abs().max() <= 1 and (off != 0).float().mean() < 0.01
    # closed form in FP64 on a few values: silu(g) * u with the two BF16 roundings
    g64, u64 = (gu[..., :gu.shape[-1] // 2], gu[..., gu.shape[-1] // 2:]) if not pairs else (None, None)
    if g64 is not None:
        ref = ((g64.double() / (1 + torch.exp(-g64.double()))).bfloat16().double() * u64.double()).bfloat16()
        assert (got.view(torch.int16).int() - ref.view(torch.int16).int()).abs().max() <= 1


@pytest.mark.parametrize("m,inter,pairs", [(1, 64, 0), (5, 256, 0), (7, 512, 64), (33, 17408 // 8, 32)])
def test_silu_mul_quant_groups_is_the_two_ops_in_one_launch(m, inter, pairs):
    """Bit for bit `quant_groups(silu_and_mul(gu, pairs))` with `torch_chain` (the reference's statement of the fused
    kernel, hibana/kernels/flashnext_fused.py:842); the single-rounding product against the oracle's rounding of it."""
    from hibana_amd.kernels import ops, w3
    gu = (torch.randn(m, 2 * inter, generator=torch.Generator().manual_seed(m + inter)) * 2).bfloat16().cuda()
    q, s = ops.silu_mul_quant_groups(gu, pairs, torch_chain=True)
    q2, s2 = w3.quant_groups(ops.silu_and_mul(gu, pairs))
    assert q.dtype == torch.float8_e4m3fn and q.shape == (m, inter) and s.shape == (m, inter // 32)
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s, s2)
    # one rounding of the FP32 product: the oracle's quantizer on the device's own BF16 product (within one unit of the
    # host's, as for silu_and_mul), then the same bytes and scales
    q1, s1 = ops.silu_mul_quant_groups(gu, pairs)
    g = layers.silu_and_mul(gu.cpu().float(), pairs).bfloat16()  # FP32 product, one rounding
    wq, ws = layers.quant_e4m3_groups(g)
    same = (q1.view(torch.uint8).cpu() == wq).float().mean()
    assert same > 0.98 and torch.allclose(s1.cpu(), ws, rtol=1e-2)  # a last-bit exponential moves a code here and there
    with pytest.raises(ValueError):
        ops.silu_mul_quant_groups(gu[:, :-2], pairs)


def test_moe_combine_of_a_routed_sum_and_the_gated_shared_expert():
    from hibana_amd.kernels import ops
    g = torch.Generator().manual_seed(12)
    routed, shared = torch.randn(9, 256, generator=g).bfloat16(), torch.randn(9, 256, generator=g).bfloat16()
    x, gate = torch.randn(9, 256, generator=g).bfloat16(), torch.randn(256, generator=g) * 0.1  # the layer's input rows: the same width
    got = ops.moe_combine(routed.cuda(), shared.cuda(), x.cuda(), gate.cuda()).cpu()
    gv = torch.sigmoid((x.double() @ gate.double()))[:, None]
    want = (routed.double() + gv * shared.double()).float().bfloat16()
    # one BF16 unit at most, and rarely: the gate's dot product and exponential are FP32 on the device
    # (where the two terms cancel, the gate's last bits show against the small sum: an absolute term beside the relative)
    assert ((got.float() - want.float()).abs() <= want.float().abs() * 2.0 ** -7 + 1e-5 * (1 + shared.float().abs())).all()
    assert (got.view(torch.int16) != want.view(torch.int16)).float().mean() < 0.02


def test_relu2_in_place():
    from hibana_amd.model import nemotron_moe
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(37, 130, generator=g) * 3).bfloat16()
    x[0, :4] = torch.tensor([0.0, -0.0, float("inf"), -float("inf")]).bfloat16()
    want = (torch.relu(x).float() ** 2).bfloat16()
    y = x.cuda()
    assert nemotron_moe.relu2_(y) is y and torch.equal(y.cpu().view(torch.int16), want.view(torch.int16))
    wide = (torch.randn(5, 64, generator=g)).bfloat16().cuda()
    before = wide.cpu()
    nemotron_moe.relu2_(wide[:, :32])  # rows of a wider tensor: the columns beside them stay
    assert torch.equal(wide[:, 32:].cpu(), before[:, 32:])
    assert torch.equal(wide[:, :32].cpu(), (torch.relu(before[:, :32]).float() ** 2).bfloat16())
    with pytest.raises(ValueError):
        nemotron_moe.relu2_(torch.zeros(2, 3, dtype=torch.bfloat16).cuda())


def test_softmax_routing_with_padded_rows():
    from hibana_amd.kernels import ops
    g = torch.Generator().manual_seed(4)
    logits = torch.randn(6, 64, generator=g).cuda()
    k = 5
    plain_ids, plain_w = ops.route_topk(logits, k)
    ref_w, ref_ids = torch.topk(torch.softmax(logits.float().cpu(), -1), k)
    assert torch.equal(plain_ids.cpu().long(), ref_ids)
    assert torch.allclose(plain_w.cpu(), ref_w / ref_w.sum(-1, keepdim=True), rtol=1e-5)
    slots = torch.tensor([3, 0, 9], dtype=torch.int32).cuda()  # request 1 is a graph's padding: rows 2, 3 at two steps a request
    ids, w = ops.route_topk(logits, k, slots, 2)
    real = [0, 1, 4, 5]
    assert torch.equal(ids[real], plain_ids[real]) and torch.equal(w[real], plain_w[real])
    assert (ids[2:4] == 64).all() and (w[2:4] == 0).all()  # no expert
    ids, w = ops.route_topk(logits, k, slots, 2, repeat=True)
    assert (ids[2:4] == plain_ids[0, 0]).all() and (w[2:4] == 0).all()  # row 0's first choice at weight 0


@pytest.mark.parametrize("m,mode", [(1, "decode"), (6, "verify"), (40, "prefill")])
def test_moe_layer_block(m, mode):
    """`MoeLayer.__call__(x, ctx)`: router GEMM, routing (padded rows of a decode / verify graph name no expert), routed
    experts, the shared expert given as the reference holds it (two linears, rows [gate; up]), gated combine."""
    from hibana_amd.kernels import w3
    from hibana_amd.model.flashnext_moe import MoeLayer, shared_from_linears
    e, hidden, inter, topk = 16, 256, 128, 4
    ex, per = random_experts(e, hidden, inter, True, 61)
    get = oracle_expert_getter(per, True, inter)
    g = torch.Generator().manual_seed(62 + m)
    router = (torch.randn(e, hidden, generator=g) * 0.3).bfloat16()
    gate_vec = torch.randn(1, hidden, generator=g) * 0.05
    gate_up, *_ = random_w3(2 * inter, hidden, 63)  # rows [gate; up]
    down, *_ = random_w3(hidden, inter, 64)
    lin_gu = SimpleNamespace(w3=to_device_w3(gate_up))
    lin_d = SimpleNamespace(w3=to_device_w3(down))
    layer = MoeLayer(router.cuda(), gate_vec.cuda(), ex, topk, shared_gate_up=lin_gu, shared_down=lin_d)
    # the re-stored shared expert dequantizes to the same weights, rows moved
    fc1 = w3.dequantize(layer.shared.matrix(0, True)).cpu().numpy()
    gu = ow3.dequantize(gate_up)
    inverse = np.argsort(layers.fc1_order(inter))
    assert np.array_equal(fc1[inverse], np.concatenate([gu[inter:], gu[:inter]]))
    x = torch.randn(m, hidden, generator=g).bfloat16()
    steps = 2 if mode == "verify" else 1
    slots = None
    if mode != "prefill":
        slots = torch.ones(m // steps, dtype=torch.int32)
        if m > 1:
            slots[-1] = 0  # the last request is padding
    ctx = SimpleNamespace(mode=mode, slots=None if slots is None else slots.cuda(), seq_slots=None if slots is None else slots.cuda(), verify_steps=steps)
    got = layer(x.cuda(), ctx)
    ids, weights = layer.route(x.cuda(), ctx)
    logits = torch.mm(x.cuda(), router.cuda().T).float().cpu()
    ref_ids = torch.topk(torch.softmax(logits, -1), topk).indices
    pad = torch.zeros(m, dtype=torch.bool) if slots is None else (slots.repeat_interleave(steps) == 0)
    assert torch.equal(ids.cpu().long()[~pad], ref_ids[~pad]) and (ids.cpu()[pad] == e).all() and (weights.cpu()[pad] == 0).all()
    shared_w13 = np.concatenate([gu[inter:], gu[:inter]])  # checkpoint order [up; gate]
    want = layers.moe_layer_ref(x, ids.cpu().numpy(), weights.cpu(), get, True, shared=(shared_w13, ow3.dequantize(down)), gate_vec=gate_vec.reshape(-1), e_n=e)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    assert torch.equal(layer(x.cuda(), None), layer(x.cuda(), SimpleNamespace(mode="prefill")))


@pytest.mark.parametrize("m,decode", [(200, True), (40, False), (40, True)])
def test_moe_layer_runs_the_shared_expert_where_the_reference_does(m, decode):
    """The shared expert as the reference holds it - two NVFP4 linears with 3-bit copies attached: a call the reference
    serves from the copies (at most w3.MAX_ROWS rows with HIBANA_W3_DECODE on, ops.w3_decode) runs them inside the
    experts' launches; any other call (more rows, or the switch off) runs the NVFP4 linears and the combine over the
    pair outputs (hibana/model/flashnext/moe.py:181-189). Each against the oracle on the weights that call uses."""
    from hibana_amd.kernels import w3
    from hibana_amd.model.flashnext_moe import MoeLayer
    from hibana_amd.weights import modelopt
    from oracle import nvfp4_format as onv
    from tests.test_gpu_nvfp4_moe import _stack
    e, hidden, inter, topk = 16, 256, 128, 4
    ex, per = random_experts(e, hidden, inter, True, 91)
    get = oracle_expert_getter(per, True, inter)
    g = torch.Generator().manual_seed(92 + m)
    router = (torch.randn(e, hidden, generator=g) * 0.3).bfloat16()
    gate_vec = torch.randn(1, hidden, generator=g) * 0.05
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    lins, dense = [], []
    for rows, k, seed, copy_seed in ((2 * inter, hidden, 93, 95), (hidden, inter, 94, 96)):  # gate_up rows [gate; up], down
        (w, sc, g2) = _stack(1, rows, k, seed)
        lin = modelopt.Nvfp4Linear(dev(w[0]), dev(onv.swizzle_block_scales(sc[0])).view(torch.float8_e4m3fn), torch.tensor(float(g2[0])).cuda(),
                                   torch.tensor(1.0).cuda(), rows, k).tile()
        copy, *_ = random_w3(rows, k, copy_seed)  # any 3-bit matrix: the two paths must be told apart
        lin.w3 = to_device_w3(copy)
        lins.append(lin)
        dense.append((onv.unpack_fp4(w[0], sc[0]) * np.float32(g2[0]), ow3.dequantize(copy)))
    layer = MoeLayer(router.cuda(), gate_vec.cuda(), ex, topk, shared_gate_up=lins[0], shared_down=lins[1])
    x = torch.randn(m, hidden, generator=g).bfloat16()
    w3.set_enabled(decode)
    try:
        on_linears = layer.shared_on_linears(m)
        assert on_linears == (m > w3.MAX_ROWS or not decode)
        got = layer(x.cuda(), None)
        ids, weights = layer.route(x.cuda(), None)
    finally:
        w3.set_enabled(None)
    which = 0 if on_linears else 1
    gu, down = dense[0][which], dense[1][which]
    shared_w13 = np.concatenate([gu[inter:], gu[:inter]])  # checkpoint order [up; gate]
    want = layers.moe_layer_ref(x, ids.cpu().numpy(), weights.cpu(), get, True, shared=(shared_w13, down), gate_vec=gate_vec.reshape(-1), e_n=e)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)


def test_attach_model_takes_calibrated_copies(tmp_path):
    """attach_model with a W3 checkpoint: every projection gets the checkpoint's copy (tiled), the model's identity is
    the manifest's digest; a checkpoint that does not cover the model is refused; without one, nearest-level copies."""
    from hibana_amd.kernels import w3
    from hibana_amd.weights.w3_checkpoint import CalibratedWeights, save_weight
    names = ["layers.0.mlp.gate_up", "layers.0.mlp.down"]
    shapes = [(256, 128), (128, 256)]
    packed = [random_w3(n, k, 70 + i)[0] for i, (n, k) in enumerate(shapes)]
    entries = {name: save_weight(tmp_path / f"{i}.safetensors", to_device_w3(p, "cpu")) for i, (name, p) in enumerate(zip(names, packed))}
    (tmp_path / "manifest.json").write_text(json.dumps({"format": 1, "target_revision": "rev", "weights": entries}))

    class Lin:
        def __init__(self, n, k, deq):
            self.out_features, self.in_features, self.w3, self.weight = n, k, None, torch.zeros(1, device="cuda")
            self._deq = deq

        def dequantize(self):
            return torch.from_numpy(self._deq).cuda()

    def model():
        lins = [Lin(n, k, ow3.dequantize(p)) for (n, k), p in zip(shapes, packed)]
        return SimpleNamespace(linears=lambda: list(zip(names, lins)), revision="rev"), lins

    mdl, lins = model()
    report = w3.attach_model(mdl, log=lambda *_: None, checkpoint=tmp_path)
    assert report["matrices"] == 2 and mdl.w3_identity == CalibratedWeights(tmp_path, "rev").identity
    for lin, p in zip(lins, packed):
        assert lin.w3.tiled is not None
        assert np.array_equal(w3.dequantize(lin.w3).cpu().numpy().view(np.uint32), ow3.dequantize(p).view(np.uint32))
    mdl, lins = model()
    mdl.linears = lambda: list(zip(names[:1], lins[:1]))
    with pytest.raises(ValueError, match="every target layer projection"):
        w3.attach_model(mdl, log=lambda *_: None, checkpoint=tmp_path)
    mdl, lins = model()
    report = w3.attach_model(mdl, log=lambda *_: None, codebook="uniform")
    assert report["matrices"] == 2 and mdl.w3_identity == "nearest:uniform" and all(lin.w3.tiled is not None for lin in lins)


@pytest.mark.parametrize("m,mode,budget", [(6, "verify", 8), (5, "decode", 0), (1, "decode", 6)])
def test_moe_layer_block_under_a_budget(m, mode, budget):
    """Decode and verify forwards of a layer with a `keep`: the routing is `ops.route_budget`'s (or each token's top
    `keep` alone), slots left over name no expert, and the block is the oracle's on those ids; prefill routes top-k."""
    from hibana_amd.kernels import ops
    from hibana_amd.model.flashnext_moe import MoeLayer
    e, hidden, inter, topk, keep = 32, 256, 128, 4, 2
    ex, per = random_experts(e, hidden, inter, True, 71)
    shared, shared_per = random_experts(1, hidden, inter, True, 72)
    get = oracle_expert_getter(per, True, inter)
    g = torch.Generator().manual_seed(73 + m)
    router = (torch.randn(e, hidden, generator=g) * 0.3).bfloat16()
    gate_vec = torch.randn(1, hidden, generator=g) * 0.05
    layer = MoeLayer(router.cuda(), gate_vec.cuda(), ex, topk, shared=shared, keep=keep, budget=budget, per_request=3)
    x = torch.randn(m, hidden, generator=g).bfloat16()
    steps = 2 if mode == "verify" else 1
    slots = torch.ones(m // steps, dtype=torch.int32)
    if m > 1:
        slots[-1] = 0
    ctx = SimpleNamespace(mode=mode, slots=slots.cuda(), seq_slots=slots.cuda(), verify_steps=steps)
    ids, weights = layer.route(x.cuda(), ctx)
    logits = torch.mm(x.cuda(), router.cuda().T)
    if budget:
        want_ids, want_w = ops.route_budget(logits, topk, layer.guarantee(m, steps), budget, slots.cuda(), steps, per_request=3, min_cap=16)
        ref = layers.route_budget_ref(logits.cpu(), topk, layer.guarantee(m, steps), budget, slots, steps, per_request=3, min_cap=16)
        assert torch.equal(ids.cpu(), ref[0])
        torch.testing.assert_close(weights.cpu(), ref[1], rtol=1e-5, atol=0)
    else:
        want_ids, want_w = ops.route_topk(logits, keep)
        assert ids.shape == (m, keep)
    assert torch.equal(ids, want_ids) and torch.equal(weights, want_w)
    got = layer(x.cuda(), ctx)
    sh = oracle_expert_getter(shared_per, True, inter)(0)
    want = layers.moe_layer_ref(x, ids.cpu().numpy(), weights.cpu(), get, True, shared=sh, gate_vec=gate_vec.reshape(-1), e_n=e)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    served = layer.route(x.cuda(), SimpleNamespace(mode="prefill"))[0]
    assert served.shape == (m, topk) and (served < e).all()
