"""NVFP4 routed experts on the GPU (through hb_nvfp4_moe) against the oracle's restatement of the reference's weight-only
latent-MoE mixer (tests/nemotron_reference.py:568-593 of the reference): ReLU^2 experts as Nemotron's, gated SiLU ones
as the 3-bit path's, ragged expert loads, ids outside the local range, unsummed pairs."""
import numpy as np
import pytest
import torch

from oracle import layers, nvfp4_format as onv
from oracle.w3_format import e4m3_bytes
from tests.util import MAX_REL, NORM_REL, errors

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["auto", "tile", "stream", "stream16"], autouse=True)
def kernel_choice(request):
    """Every case runs with the library's own choice between the 128-row tile kernel and the 16-row weight stream, with
    each of them forced, and with the stream's body for slots of at most eight rows switched off (so those slots take the
    sixteen-row body)."""
    from hibana_amd import _lib
    tile, few = {"auto": (0, 0), "tile": (1, 0), "stream": (2, 0), "stream16": (2, 2)}[request.param]
    assert _lib.lib().hb_tune(b"nvfp4_tile", tile) == 0 and _lib.lib().hb_tune(b"nvfp4_few", few) == 0
    yield request.param
    _lib.lib().hb_tune(b"nvfp4_tile", 0)
    _lib.lib().hb_tune(b"nvfp4_few", 0)


def _stack(e, rows, k, seed):
    g = np.random.default_rng(seed)
    packed = g.integers(0, 256, (e, rows, k // 2), dtype=np.uint8)
    scales = e4m3_bytes(np.clip(np.abs(g.normal(0, 1, (e, rows, k // 16))), 2 ** -6, 8.0))
    scale2 = (g.uniform(0.5, 2.0, e) / np.sqrt(k) / 4).astype(np.float32)
    return packed, scales, scale2


def _experts(e, hidden, inter, gated, seed, scaling=1.0, base=0):
    from hibana_amd.kernels import b12x_moe
    n1 = 2 * inter if gated else inter
    w1, s1, g1 = _stack(e, n1, hidden, seed)
    w2, s2, g2 = _stack(e, hidden, inter, seed + 1)
    if gated:  # the kernels read fc1 rows in fc1_order; the oracle takes checkpoint order [up; gate]
        order = layers.fc1_order(inter)
        w1k, s1k = w1[:, order], s1[:, order]
    else:
        w1k, s1k = w1, s1
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    ex = b12x_moe.B12xExperts(dev(w1k), dev(onv.swizzle_batched(s1k)), dev(g1), 1.0, dev(w2), dev(onv.swizzle_batched(s2)), dev(g2), 1.0,
                              routed_scaling=scaling, base=base)
    return ex, (w1, s1, g1, w2, s2, g2)


def _routing(m, topk, e, seed, id_hi=None):
    g = torch.Generator().manual_seed(seed)
    ids = torch.stack([torch.randperm(id_hi or e, generator=g)[:topk] for _ in range(m)]).to(torch.int32)
    w = torch.rand(m, topk, generator=g) + 0.1
    return ids, (w / w.sum(-1, keepdim=True)).contiguous()


@pytest.mark.parametrize("m,topk", [(1, 4), (7, 3), (16, 6), (40, 4), (333, 6)])
def test_relu2_latent_experts_match_the_oracle(m, topk):
    e, hidden, inter = 8, 256, 384
    ex, (w1, s1, g1, w2, s2, g2) = _experts(e, hidden, inter, False, 5, scaling=2.5)
    lat = torch.randn(m, hidden, generator=torch.Generator().manual_seed(m)).bfloat16()
    ids, w = _routing(m, topk, e, 100 + m)

    def get(i):
        return onv.unpack_fp4(w1[i], s1[i]), g1[i], onv.unpack_fp4(w2[i], s2[i]), np.float32(g2[i] * np.float32(2.5))

    want = layers.bf16(layers.latent_experts_ref(lat, ids.numpy(), w, get))
    got = ex(lat.cuda(), ids.cuda(), w.cuda())
    assert got.dtype == torch.bfloat16 and got.shape == (m, hidden)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    again = ex(lat.cuda(), ids.cuda(), w.cuda())
    assert torch.equal(got, again)  # deterministic


def test_skewed_load_and_foreign_ids():
    """Most rows on one expert (several slots for it), some experts idle, ids past the local range dropped."""
    e, hidden, inter, m, topk = 6, 128, 128, 90, 3
    ex, (w1, s1, g1, w2, s2, g2) = _experts(e, hidden, inter, False, 9, base=2)
    lat = torch.randn(m, hidden, generator=torch.Generator().manual_seed(1)).bfloat16()
    g = torch.Generator().manual_seed(2)
    ids = torch.stack([torch.tensor([2, 3 + int(torch.randint(0, 2, (1,), generator=g)), 9 + i % 3]) for i in range(m)]).to(torch.int32)
    ids[::7, 1] = 0  # below the local range
    w = torch.rand(m, topk, generator=g) + 0.1

    def get(i):
        return onv.unpack_fp4(w1[i], s1[i]), g1[i], onv.unpack_fp4(w2[i], s2[i]), g2[i]

    local = ids.numpy() - 2
    keep = (local >= 0) & (local < e)
    want = layers.bf16(layers.latent_experts_ref(lat, np.where(keep, local, 0), torch.where(torch.as_tensor(keep), w, torch.zeros(())), get))
    got = ex(lat.cuda(), ids.cuda(), w.cuda())
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)


@pytest.mark.parametrize("m", [3, 50])
def test_gated_experts_and_pairs(m):
    e, hidden, inter, topk = 4, 256, 128, 2
    ex, (w1, s1, g1, w2, s2, g2) = _experts(e, hidden, inter, True, 21)
    assert ex.gated
    x = torch.randn(m, hidden, generator=torch.Generator().manual_seed(m)).bfloat16()
    ids, w = _routing(m, topk, e, 7)

    def get(i):
        return onv.unpack_fp4(w1[i], s1[i]) * g1[i], onv.unpack_fp4(w2[i], s2[i]) * g2[i]

    pairs = layers.routed_experts_ref(x, ids.numpy(), get, True, 0, e)
    got_pairs = ex(x.cuda(), ids.cuda(), w.cuda(), pairs=True)
    assert got_pairs.dtype == torch.float32
    mx, nr = errors(got_pairs, pairs)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    got = ex(x.cuda(), ids.cuda(), w.cuda())
    mx, nr = errors(got, layers.combine_ref(pairs, ids.numpy(), w, 0, e))
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)


def test_rejects_bad_calls():
    ex, _ = _experts(2, 128, 128, False, 1)
    ids = torch.zeros(2, 1, dtype=torch.int32).cuda()
    w = torch.ones(2, 1).cuda()
    with pytest.raises(ValueError):
        ex(torch.zeros(2, 128).cuda(), ids, w)  # not BF16
    with pytest.raises(ValueError):
        ex(torch.zeros(2, 256).bfloat16().cuda(), ids, w)  # wrong width
    with pytest.raises(RuntimeError):
        ex(torch.zeros(2, 128).bfloat16(), ids.cpu(), w.cpu())  # CPU tensors: no fallback
