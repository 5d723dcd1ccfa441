"""The small-call latent block (`kernels/nemotron_moe.py`: router / block / w3_block / shared_up / out, at most sixteen
rows) on the GPU: the router's FP32 product against an FP64 one, its routing against the routing op on the same FP32
rows (bit for bit, the reference's claim for its router kernel, hibana/kernels/nemotron_moe.py:3-4), the block against
the oracle's statement of the layer (hibana/model/nemotron/moe.py:508-517) from the router's own ids."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import layers, nvfp4_format as onv
from tests.test_gpu_nvfp4_moe import _experts, _stack
from tests.util import MAX_REL, NORM_REL, errors, random_experts

pytestmark = pytest.mark.gpu


def _linear(n, k, seed):
    """(Nvfp4Linear on the GPU, (oracle's unpacked matrix, its FP32 scale))."""
    from hibana_amd.weights import modelopt
    (w, s, g) = _stack(1, n, k, seed)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    lin = modelopt.Nvfp4Linear(dev(w[0]), dev(onv.swizzle_block_scales(s[0])).view(torch.float8_e4m3fn), torch.tensor(float(g[0])).cuda(),
                               torch.tensor(1.0).cuda(), n, k)
    return lin, (onv.unpack_fp4(w[0], s[0]), np.float32(g[0]))


def _block(e, hidden, latent, inter, topk, sh_inter, seed, w3=False):
    from hibana_amd.model import nemotron_moe
    g = torch.Generator().manual_seed(seed)
    router = (torch.randn(e, hidden, generator=g) * 0.05).bfloat16()
    fc1 = (torch.randn(latent, hidden, generator=g) * 0.04).bfloat16()
    fc2 = (torch.randn(hidden, latent, generator=g) * 0.04).bfloat16()
    bias = torch.randn(e, generator=g) * 0.05
    up = down = su = sd = None
    if sh_inter:
        up, su = _linear(sh_inter, hidden, seed + 1)
        down, sd = _linear(hidden, sh_inter, seed + 2)
    if w3:
        ex, host = random_experts(e, latent, inter, False, seed + 3)
    else:
        ex, host = _experts(e, latent, inter, False, seed + 3, scaling=2.0)
    block = nemotron_moe.NemotronMoe(torch.cat([router, fc1]).cuda(), bias.cuda(), fc2.cuda(), ex, topk, up, down)
    return block, SimpleNamespace(router=router, fc1=fc1, fc2=fc2, bias=bias, su=su, sd=sd, host=host)


GEOMETRIES = {"small": (16, 512, 256, 384, 4, 640), "wide": (64, 1024, 1024, 256, 6, 0), "many": (200, 512, 128, 128, 8, 128)}


@pytest.mark.parametrize("geometry", list(GEOMETRIES))
@pytest.mark.parametrize("m", [1, 3, 16])
def test_router_product_routing_and_plan(geometry, m):
    from hibana_amd.kernels import nemotron_moe as small
    from hibana_amd.model import nemotron_moe
    e, hidden, latent, inter, topk, sh_inter = GEOMETRIES[geometry]
    block, ref = _block(e, hidden, latent, inter, topk, sh_inter, 50 + m)
    x = torch.randn(m, hidden, generator=torch.Generator().manual_seed(m)).bfloat16()
    fused, ids, w, ws, lat = small.router(x.cuda(), block.small_weights(), None, topk, latent=True)
    want = x.double() @ torch.cat([ref.router, ref.fc1]).double().T
    assert fused.dtype == torch.float32 and fused.shape == (m, e + latent)
    assert torch.allclose(fused.cpu().double(), want, rtol=1e-5, atol=2e-5 * float(want.abs().max()))
    # the routing op on the same FP32 rows: the same bits
    ids2, w2, lat2 = nemotron_moe.route_topk(fused, block.bias, topk, latent)
    assert torch.equal(ids, ids2) and torch.equal(w, w2) and torch.equal(lat, lat2)
    # without routing: the product and the latent rows only
    fused3, _, _, ws3, lat3 = small.router(x.cuda(), block.small_weights(), None, topk, route=False, latent=True)
    assert torch.equal(fused3, fused) and torch.equal(lat3, lat)
    # the plan the router left is the plan of these ids: the block from it and the block that plans again agree bit for bit
    a = small.block(x.cuda(), ws, ids, w, block.small_weights())
    b = small.block(x.cuda(), ws3, ids, w, block.small_weights(), plan=True)
    assert torch.equal(a, b)


def test_router_padded_rows_and_a_callers_bias():
    from hibana_amd.kernels import nemotron_moe as small
    from hibana_amd.model import nemotron_moe
    e, hidden, latent, inter, topk, sh_inter = GEOMETRIES["small"]
    block, _ = _block(e, hidden, latent, inter, topk, sh_inter, 9)
    x = torch.randn(6, hidden, generator=torch.Generator().manual_seed(2)).bfloat16().cuda()
    slots = torch.tensor([5, 0, 7], dtype=torch.int32).cuda()  # rows 2, 3 are a graph's padding (two steps a request)
    fused, ids, w, _ = small.router(x, block.small_weights(), None, topk, slots, 2)
    for repeat, pad_id in ((True, -1), (False, e)):
        _, ids, w, _ = small.router(x, block.small_weights(), None, topk, slots, 2, pad_id=pad_id)
        ids2, w2, _ = nemotron_moe.route_topk(fused, block.bias, topk, latent, slots, 2, repeat=repeat)
        assert torch.equal(ids, ids2) and torch.equal(w, w2)
        assert (w[2:4] == 0).all() and (ids[2:4] == (ids[0, 0] if repeat else e)).all()
    _, ids, w, _ = small.router(x, block.small_weights(), None, topk, slots, 2, pad_id=3)
    assert (ids[2:4] == 3).all() and (w[2:4] == 0).all()
    bias = torch.zeros(e)
    bias[11] = 10.0
    _, ids, _, _ = small.router(x, block.small_weights(), bias.cuda(), topk)
    assert (ids[:, 0] == 11).all()
    with pytest.raises(ValueError):
        small.router(torch.zeros(17, hidden, dtype=torch.bfloat16).cuda(), block.small_weights(), None, topk)


def _oracle(ref, x, ids, w, scaling=2.0):
    w1, s1, g1, w2, s2, g2 = ref.host

    def get(i):
        return onv.unpack_fp4(w1[i], s1[i]), g1[i], onv.unpack_fp4(w2[i], s2[i]), np.float32(g2[i] * np.float32(scaling))

    sh_out = None
    if ref.su is not None:
        h = layers.nvfp4_dense_ref(x, ref.su[0], ref.su[1], relu2=True)
        sh_out = layers.nvfp4_dense_ref(h, ref.sd[0], ref.sd[1])
    return layers.latent_moe_ref(x, ref.fc1, ref.fc2, ids.cpu().numpy(), w.cpu(), get, shared=sh_out)


@pytest.mark.parametrize("geometry", list(GEOMETRIES))
@pytest.mark.parametrize("m", [1, 4, 16])
def test_small_block_matches_the_oracle(geometry, m):
    from hibana_amd.kernels import nemotron_moe as small
    e, hidden, latent, inter, topk, sh_inter = GEOMETRIES[geometry]
    block, ref = _block(e, hidden, latent, inter, topk, sh_inter, 70 + m)
    x = torch.randn(m, hidden, generator=torch.Generator().manual_seed(10 + m)).bfloat16()
    got = block(x.cuda())  # at most sixteen rows: the small-call kernels
    again = block.small(x.cuda())
    assert got.dtype == torch.bfloat16 and got.shape == (m, hidden) and torch.equal(got, again)
    # the oracle follows the router's own ids (its routing is checked on its own): a last-bit tie cannot move an expert
    _, ids, w, _ = small.router(x.cuda(), block.small_weights(), None, topk)
    mx, nr = errors(got, _oracle(ref, x, ids, w))
    assert mx < MAX_REL and nr < 2 * NORM_REL, (mx, nr)


@pytest.mark.parametrize("m,mode", [(2, "decode"), (6, "verify")])
def test_small_block_with_a_graphs_padding(m, mode):
    e, hidden, latent, inter, topk, sh_inter = GEOMETRIES["small"]
    block, ref = _block(e, hidden, latent, inter, topk, sh_inter, 21)
    steps = 1 if mode == "decode" else 3
    slots = torch.ones(m // steps, dtype=torch.int32)
    slots[-1] = 0  # the last request is padding
    ctx = SimpleNamespace(mode=mode, slots=slots.cuda(), seq_slots=slots.cuda(), verify_steps=steps)
    x = torch.randn(m, hidden, generator=torch.Generator().manual_seed(m)).bfloat16()
    got = block(x.cuda(), ctx)
    real = m - steps
    assert torch.equal(got[:real], block(x[:real].cuda()))  # the real rows do not see the padding
    # a padded row: its routed weight is zero, so it is the shared expert's output alone
    h = layers.nvfp4_dense_ref(x[real:], ref.su[0], ref.su[1], relu2=True)
    want = layers.nvfp4_dense_ref(h, ref.sd[0], ref.sd[1])
    mx, nr = errors(got[real:], want)
    assert mx < MAX_REL and nr < 2 * NORM_REL, (mx, nr)


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("shared", [True, False])
def test_small_block_around_3_bit_experts(m, shared):
    """`w3_block`: router (latent rows out), the shared expert's up, w3_moe on the latent rows, then out."""
    from hibana_amd.kernels import nemotron_moe as small, w3_moe
    e, hidden, latent, inter, topk = 16, 512, 256, 128, 4
    block, ref = _block(e, hidden, latent, inter, topk, 640 if shared else 0, 33, w3=True)
    assert block.w3 is not None and block.b12x is None
    x = torch.randn(m, hidden, generator=torch.Generator().manual_seed(m)).bfloat16()
    got = block(x.cuda())
    _, ids, w, ws, lat = small.router(x.cuda(), block.small_weights(), None, topk, pad_id=e, latent=True)
    routed = w3_moe.w3_moe(block.w3, lat, ids, w)
    y = routed.cpu().double() @ ref.fc2.double().T
    if shared:
        h = layers.nvfp4_dense_ref(x, ref.su[0], ref.su[1], relu2=True)
        y = y + layers.nvfp4_dense_ref(h, ref.sd[0], ref.sd[1]).double()
    mx, nr = errors(got, y.float().bfloat16())
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    with pytest.raises(ValueError):
        small.block(x.cuda(), ws, ids, w, block.small_weights())  # no NVFP4 experts to run


def test_small_block_at_the_benchmark_geometry():
    """Config 4's block at decode sizes: hidden 4096 -> latent 1024, 512 ReLU^2 experts of intermediate 2688, top-22,
    with a shared expert of intermediate 5376."""
    from hibana_amd import synthetic
    from hibana_amd.kernels import nemotron_moe as small
    from hibana_amd.model import nemotron_moe
    hidden, latent, inter, experts, topk, sh_inter = 4096, 1024, 2688, 512, 22, 5376
    g = torch.Generator().manual_seed(5)
    ex = synthetic.nvfp4_experts(experts, latent, inter, 11, "cuda", keep=True)
    router = (torch.randn(experts, hidden, generator=g) * (1.0 / hidden ** 0.5)).bfloat16()
    fc1 = (torch.randn(latent, hidden, generator=g) * 0.02).bfloat16()
    fc2 = (torch.randn(hidden, latent, generator=g) * 0.02).bfloat16()
    up, su = _linear(sh_inter, hidden, 61)
    down, sd = _linear(hidden, sh_inter, 62)
    block = nemotron_moe.NemotronMoe(torch.cat([router, fc1]).cuda(), torch.zeros(experts).cuda(), fc2.cuda(), ex, topk, up, down)
    for m in (1, 8, 16):
        x = torch.randn(m, hidden, generator=g).bfloat16()
        got = block(x.cuda())
        fused, ids, w, _ = small.router(x.cuda(), block.small_weights(), None, topk)
        ids2, w2, _ = nemotron_moe.route_topk(fused, block.bias, topk, latent)
        assert torch.equal(ids, ids2) and torch.equal(w, w2)

        def get(i):
            s1 = onv.unswizzle_block_scales(ex.s1[i].view(torch.uint8).cpu().numpy(), inter, latent // 16)
            s2 = onv.unswizzle_block_scales(ex.s2[i].view(torch.uint8).cpu().numpy(), latent, inter // 16)
            return (onv.unpack_fp4(ex.w1[i].cpu().numpy(), s1), np.float32(ex.alpha1[i].item()),
                    onv.unpack_fp4(ex.w2[i].cpu().numpy(), s2), np.float32(ex.alpha2[i].item()))

        h = layers.nvfp4_dense_ref(x, su[0], su[1], relu2=True)
        want = layers.latent_moe_ref(x, fc1, fc2, ids.cpu().numpy(), w.cpu(), get, shared=layers.nvfp4_dense_ref(h, sd[0], sd[1]))
        mx, nr = errors(got, want)
        assert mx < MAX_REL and nr < 2 * NORM_REL, (m, mx, nr)
    del block, ex
    torch.cuda.empty_cache()


@pytest.mark.parametrize("m", [1, 7])
def test_small_block_on_an_expert_range(m):
    """Expert parallelism: a rank holds experts lo .. hi - 1 of the E the router scores; pairs of other ranks' experts
    are dropped by its plan and its combine. Without a shared expert the ranks' outputs add up to the whole block's."""
    from hibana_amd.kernels import b12x_moe, nemotron_moe as small
    from hibana_amd.model import nemotron_moe
    e, hidden, latent, inter, topk = 16, 512, 256, 384, 4
    whole, ref = _block(e, hidden, latent, inter, topk, 0, 44)
    w1, s1, g1, w2, s2, g2 = ref.host
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    x = torch.randn(m, hidden, generator=torch.Generator().manual_seed(m)).bfloat16().cuda()
    want = whole(x).float()
    total = torch.zeros_like(want)
    ids_seen = None
    for lo, hi in ((0, 6), (6, 16)):
        part = b12x_moe.B12xExperts(dev(w1[lo:hi]), dev(onv.swizzle_batched(s1[lo:hi])), dev(g1[lo:hi]), 1.0, dev(w2[lo:hi]), dev(onv.swizzle_batched(s2[lo:hi])),
                                    dev(g2[lo:hi]), 1.0, routed_scaling=2.0, base=lo)
        rank = nemotron_moe.NemotronMoe(whole.gate_fc1, whole.bias, whole.fc2, part, topk)
        _, ids, w, ws = small.router(x, rank.small_weights(), None, topk)
        assert ids_seen is None or torch.equal(ids, ids_seen)  # every rank routes over all E experts
        ids_seen = ids
        total += small.block(x, ws, ids, w, rank.small_weights()).float()
    mx, nr = errors(total.bfloat16(), want.bfloat16())
    assert mx < MAX_REL and nr < 2 * NORM_REL, (mx, nr)


@pytest.mark.parametrize("m,mode,w3", [(6, "verify", False), (4, "decode", False), (6, "verify", True), (40, "verify", False)])
def test_block_under_a_budget(m, mode, w3):
    """Decode and verify forwards of a block with a `keep`: the router's launch leaves the routing to the budgeted
    selection, the block plans from its ids (hibana/model/nemotron/moe.py:484-502); past sixteen rows the same routing
    feeds the large-call path. The oracle follows the selection's own ids."""
    from hibana_amd.kernels import nemotron_moe as small
    from hibana_amd.model import nemotron_moe
    e, hidden, latent, inter, topk, sh_inter = GEOMETRIES["many"] if not w3 else (16, 512, 256, 128, 4, 640)
    block, ref = _block(e, hidden, latent, inter, topk, sh_inter, 90, w3=w3)
    block.keep, block.budget, block.per_request = 2, 12, 5
    steps = 1 if mode == "decode" else 2
    slots = torch.ones(m // steps, dtype=torch.int32)
    slots[-1] = 0
    ctx = SimpleNamespace(mode=mode, slots=slots.cuda(), seq_slots=slots.cuda(), verify_steps=steps)
    x = torch.randn(m, hidden, generator=torch.Generator().manual_seed(m)).bfloat16()
    got = block(x.cuda(), ctx)
    if m > block.SMALL_ROWS:
        fused = torch.mm(x.cuda(), block.gate_fc1.T, out_dtype=torch.float32)
    else:
        fused = small.router(x.cuda(), block.small_weights(), None, topk, route=False)[0]
    ids, w, lat = block.route(fused, slots.cuda(), steps, select=True)
    want_ids, want_w, _ = nemotron_moe.route_budget(fused, block.bias, topk, latent, 2, 12, slots.cuda(), steps, per_request=5, repeat=not w3,
                                                    fallback=block.fallback(m, steps))
    assert torch.equal(ids, want_ids) and torch.equal(w, want_w)
    real = m - steps
    used = {int(v) for t in range(real) for v, wt in zip(ids[t].tolist(), w[t].tolist()) if wt > 0}
    assert len(used) <= max(min(12, 5 * (m // steps - 1)), len({int(v) for v in ids[:real, :2].reshape(-1).tolist()}))
    assert not w[real:].any()
    if w3:
        from hibana_amd.kernels import w3_moe
        y = w3_moe.w3_moe(block.w3, lat, ids, w).cpu().double() @ ref.fc2.double().T
        h = layers.nvfp4_dense_ref(x, ref.su[0], ref.su[1], relu2=True)
        want = (y + layers.nvfp4_dense_ref(h, ref.sd[0], ref.sd[1]).double()).float().bfloat16()
    else:
        want = _oracle(ref, x, ids, w)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < 2 * NORM_REL, (mx, nr)
    plain = block(x.cuda(), SimpleNamespace(mode="prefill"))  # prefill routes every token's top k
    assert not torch.equal(plain[:real], got[:real])
