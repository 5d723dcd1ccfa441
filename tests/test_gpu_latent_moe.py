"""Sigmoid top-k routing and the latent-MoE block on the GPU against the oracle (the reference's statements:
hibana/model/nemotron/moe.py:75-121 for the routing, :508-517 and tests/nemotron_reference.py:568-593 for the block)."""
import numpy as np
import pytest
import torch

from oracle import layers, nvfp4_format as onv
from tests.test_gpu_nvfp4_moe import _experts, _stack
from tests.util import MAX_REL, NORM_REL, errors

pytestmark = pytest.mark.gpu


def _check_routing(fused, bias, k, latent, ids, w, lat):
    """The device exponential may differ from the host's in the last bit, so the selection is checked by its defining
    properties on the oracle's scores, with near-ties (1e-6) allowed to swap, and the weights by the formula on the
    device's own ids."""
    m = fused.shape[0]
    e = fused.shape[1] - latent
    s = torch.sigmoid(fused[:, :e].float())
    choice = (s + bias.float()).double()
    ids_c = ids.cpu().long()
    picked = choice.gather(1, ids_c)
    assert (picked[:, :-1] >= picked[:, 1:] - 1e-6).all()  # descending
    rest = choice.clone()
    rest.scatter_(1, ids_c, -np.inf)
    assert (picked.min(1).values >= rest.max(1).values - 1e-6).all()
    assert all(len(set(row.tolist())) == k for row in ids_c)
    sw = s.gather(1, ids_c)
    want_w = sw / (sw.sum(-1, keepdim=True) + 1e-20)
    assert torch.allclose(w.cpu(), want_w, rtol=2e-6, atol=1e-9)
    assert torch.equal(lat.cpu(), fused[:, e:].bfloat16())


@pytest.mark.parametrize("m,e,k,latent", [(1, 512, 22, 1024), (33, 512, 22, 256), (5, 128, 6, 64), (9, 100, 8, 0), (4, 1000, 64, 128)])
def test_sigmoid_routing(m, e, k, latent):
    from hibana_amd.model import nemotron_moe
    g = torch.Generator().manual_seed(e + m)
    fused = torch.randn(m, e + latent, generator=g) * 2
    bias = torch.randn(e, generator=g) * 0.1
    ids, w, lat = nemotron_moe.route_topk(fused.cuda(), bias.cuda(), k, latent)
    assert ids.dtype == torch.int32 and ids.shape == (m, k) and w.dtype == torch.float32 and lat.dtype == torch.bfloat16
    _check_routing(fused, bias, k, latent, ids, w, lat)
    want_ids, want_w = layers.route_sigmoid_topk(fused[:, :e], bias, k)
    assert (ids.cpu() == want_ids).float().mean() > 0.99  # bit-level ties aside, the oracle's ids in the oracle's order


def test_sigmoid_routing_ties_take_the_lower_id_and_strided_rows():
    from hibana_amd.model import nemotron_moe
    e, k = 64, 5
    wide = torch.zeros(3, e + 16 + 7)  # rows wider than E + latent: the stride is honoured
    wide[:, :e] = -1.0
    wide[0, [40, 3, 17, 5, 9, 60]] = 2.0        # six equal scores, five slots
    wide[1, 10] = 3.0                           # one winner, then the all-equal rest from id 0
    wide[2, :e] = torch.arange(e).float() / 8   # strictly increasing: the top five from the end
    fused = wide.cuda()[:, :e + 16]
    ids, w, _ = nemotron_moe.route_topk(fused, torch.zeros(e).cuda(), k, 16)
    assert ids.cpu().tolist() == [[3, 5, 9, 17, 40], [10, 0, 1, 2, 3], [63, 62, 61, 60, 59]]
    assert torch.allclose(w[0].cpu(), torch.full((5,), 0.2))
    bias = torch.zeros(e)
    bias[20] = 10.0  # the bias chooses, the weight stays the plain sigmoid
    ids, w, _ = nemotron_moe.route_topk(fused, bias.cuda(), k, 16)
    assert ids[0, 0].item() == 20
    s = torch.sigmoid(torch.tensor([-1.0, 2.0, 2.0, 2.0, 2.0]))
    assert torch.allclose(w[0].cpu(), s / s.sum(), rtol=1e-6)


def test_padded_rows():
    from hibana_amd.model import nemotron_moe
    e, k, steps = 32, 4, 2
    g = torch.Generator().manual_seed(3)
    fused = torch.randn(6, e + 8, generator=g).cuda()
    bias = torch.zeros(e).cuda()
    slots = torch.tensor([5, 0, 7], dtype=torch.int32).cuda()  # rows 2, 3 are padding
    plain = nemotron_moe.route_topk(fused, bias, k, 8)
    ids, w, lat = nemotron_moe.route_topk(fused, bias, k, 8, slots, steps)
    assert torch.equal(ids[[0, 1, 4, 5]], plain[0][[0, 1, 4, 5]]) and torch.equal(w[[0, 1, 4, 5]], plain[1][[0, 1, 4, 5]])
    assert (ids[2:4] == plain[0][0, 0]).all() and (w[2:4] == 0).all()
    assert torch.equal(lat, plain[2])
    ids, w, _ = nemotron_moe.route_topk(fused, bias, k, 8, slots, steps, repeat=False)
    assert (ids[2:4] == e).all() and (w[2:4] == 0).all()


@pytest.mark.parametrize("m,shared", [(3, True), (48, True), (20, False)])
def test_latent_block_matches_the_oracle(m, shared):
    from hibana_amd.model import nemotron_moe
    from hibana_amd.weights import modelopt
    e, hidden, latent, inter, topk, sh_inter = 16, 512, 256, 384, 4, 640
    ex, (w1, s1, g1, w2, s2, g2) = _experts(e, latent, inter, False, 31, scaling=2.0)
    g = torch.Generator().manual_seed(17)
    router = (torch.randn(e, hidden, generator=g) * 0.05).bfloat16()
    fc1 = (torch.randn(latent, hidden, generator=g) * 0.04).bfloat16()
    fc2 = (torch.randn(hidden, latent, generator=g) * 0.04).bfloat16()
    bias = torch.randn(e, generator=g) * 0.05
    x = torch.randn(m, hidden, generator=g).bfloat16()
    up = down = None
    su = sd = None
    if shared:
        (uw, us, ug), (dw, ds, dg) = _stack(1, sh_inter, hidden, 40), _stack(1, hidden, sh_inter, 41)
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
        one = lambda v: torch.tensor(float(v)).cuda()  # noqa: E731
        up = modelopt.Nvfp4Linear(dev(uw[0]), dev(onv.swizzle_block_scales(us[0])).view(torch.float8_e4m3fn), one(ug[0]), one(1.0), sh_inter, hidden)
        down = modelopt.Nvfp4Linear(dev(dw[0]), dev(onv.swizzle_block_scales(ds[0])).view(torch.float8_e4m3fn), one(dg[0]), one(1.0), hidden, sh_inter)
        su = (onv.unpack_fp4(uw[0], us[0]), np.float32(ug[0]))
        sd = (onv.unpack_fp4(dw[0], ds[0]), np.float32(dg[0]))
    block = nemotron_moe.NemotronMoe(torch.cat([router, fc1]).cuda(), bias.cuda(), fc2.cuda(), ex, topk, up, down)
    got = block(x.cuda())
    assert got.dtype == torch.bfloat16 and got.shape == (m, hidden)

    # the oracle follows the device's routing (checked on its own above) so that a last-bit tie cannot move an expert
    fused = torch.mm(x.cuda(), block.gate_fc1.T, out_dtype=torch.float32)
    ids, w, _ = block.route(fused)
    _check_routing(fused.cpu(), bias, topk, latent, ids, w, _)

    def get(i):
        return onv.unpack_fp4(w1[i], s1[i]), g1[i], onv.unpack_fp4(w2[i], s2[i]), np.float32(g2[i] * np.float32(2.0))

    sh_out = None
    if shared:
        h = layers.nvfp4_dense_ref(x, su[0], su[1], relu2=True)
        sh_out = layers.nvfp4_dense_ref(h, sd[0], sd[1])
    want = layers.latent_moe_ref(x, fc1, fc2, ids.cpu().numpy(), w.cpu(), get, shared=sh_out)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < 2 * NORM_REL, (mx, nr)
