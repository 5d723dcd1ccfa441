"""The benchmark configurations at their full geometry on the GPU, against the CPU oracle.

  config 2 / 3   w3 MoE layer, hidden 2048, 512 experts of intermediate 512 + 1 shared, top-10: one token with N(0,1)
                 logits; 32 tokens with Zipf(1.1) routing. Oracle: the C restatement (oracle/c/w3_oracle.c), which
                 unpacks the experts a call names from the checkpoint layout.
  config 1       NVFP4 dense 25600 x 5120 at M = 64 (and 1, 8): (x unpack^T) * s2 (tests/nemotron_reference.py:236-254
                 of the reference), on the weight stream and on the tile kernel.
  config 4       NVFP4 latent-MoE block, 2048 tokens, hidden 4096 -> latent 1024, 512 ReLU^2 experts of intermediate
                 2688, top-22: a token's output depends on its own 22 experts only, so the oracle
                 (tests/nemotron_reference.py:568-593 restated) is evaluated on a seeded sample of token rows; through
                 the tile kernel, the library's own choice and the weight stream.

The 512-expert plan, the slot table at well over a hundred distinct experts, the three-launch plan of 45 056 pairs and
the stream / tile switch-over run here at the sizes they are built for.
"""
import numpy as np
import pytest
import torch

from oracle import c_port, layers, nvfp4_format as onv
from tests.util import MAX_REL, NORM_REL, errors

pytestmark = pytest.mark.gpu

HIDDEN, INTER, EXPERTS, TOPK = 2048, 512, 512, 10


def _host(ex):
    u32 = lambda t: t.view(torch.int32).cpu().numpy().view(np.uint32)  # noqa: E731
    (n1, h), (_, i) = ex.shape13, ex.shape2
    return c_port.HostExperts(u32(ex.planes13), ex.scales13.cpu().numpy(), ex.row13.cpu().numpy(), u32(ex.planes2), ex.scales2.cpu().numpy(),
                              ex.row2.cpu().numpy(), ex.codebook, ex.fc2_codebook, h, i, n1 == 2 * i)


@pytest.fixture(scope="module", params=[7, 8])
def w3_layer(request):
    """(routed experts, shared expert, their host copies) of one seeded config-2/3 layer."""
    from hibana_amd import synthetic
    seed = request.param
    routed = synthetic.w3_experts(EXPERTS, HIDDEN, INTER, True, 300 + seed, "cuda", release=False)
    shared = synthetic.w3_experts(1, HIDDEN, INTER, True, 700 + seed, "cuda", release=False)
    yield seed, routed, shared, _host(routed), _host(shared)
    del routed, shared
    torch.cuda.empty_cache()


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


@pytest.mark.parametrize("m", [1, 4, 8, 16, 32])  # 8 and 16: the launches' shapes for partly filled devices
def test_w3_moe_layer_at_the_benchmark_geometry(w3_layer, m):
    from hibana_amd import synthetic
    from hibana_amd.kernels import ops, w3_moe
    seed, routed, shared, h_routed, h_shared = w3_layer
    if m == 1:
        logits = torch.randn(m, EXPERTS, generator=torch.Generator().manual_seed(seed)).cuda()
    else:
        logits = synthetic.zipf_logits(m, EXPERTS, 1.1, seed, "cuda")
    x = torch.randn(m, HIDDEN, generator=torch.Generator().manual_seed(50 + seed)).bfloat16().cuda()
    gate = (torch.randn(HIDDEN, generator=torch.Generator().manual_seed(60 + seed)) * 0.02).cuda()
    got, ids, weights = w3_moe.moe_layer_logits(routed, x, logits, TOPK, shared=shared, return_routing=True)
    # the routing inside the chain is the routing op's (checked against torch on its own)
    ids2, w2 = ops.route_topk(logits, TOPK)
    assert torch.equal(ids, ids2) and torch.equal(weights, w2)
    ref_ids = torch.topk(torch.softmax(logits.float().cpu(), -1), TOPK).indices
    assert (ids.cpu().long().sort(-1).values == ref_ids.sort(-1).values).float().mean() > 0.99
    distinct = int(torch.unique(ids).numel())
    assert distinct == TOPK if m == 1 else distinct > min(64, 4 * m)
    idn, wn = ids.cpu().numpy(), weights.cpu().numpy()
    want, ran = c_port.moe_layer(h_routed, _bits(x), idn, wn, h_shared)
    assert ran == distinct
    mx, nr = errors(got, _from_bits(want))
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    # from given ids, with the sigmoid gate on the shared expert
    got = w3_moe.moe_layer(routed, x, ids, weights, shared=shared, gate_vec=gate)
    want, _ = c_port.moe_layer(h_routed, _bits(x), idn, wn, h_shared, gate.cpu().numpy())
    mx, nr = errors(got, _from_bits(want))
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    # the routed sum alone
    got = w3_moe.w3_moe(routed, x, ids, weights)
    want, _ = c_port.moe_layer(h_routed, _bits(x), idn, wn)
    mx, nr = errors(got, _from_bits(want))
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)


def test_w3_moe_layer_expert_parallel_halves_at_the_benchmark_geometry(w3_layer):
    """Two ranks' halves of the 512 experts at M = 32: their partial sums, added in FP32, are the whole layer's routed
    sum to within the two BF16 roundings."""
    from dataclasses import replace

    from hibana_amd import synthetic
    from hibana_amd.kernels import ops, w3_moe
    seed, routed, _, h_routed, _ = w3_layer
    logits = synthetic.zipf_logits(32, EXPERTS, 1.1, 90 + seed, "cuda")
    x = torch.randn(32, HIDDEN, generator=torch.Generator().manual_seed(seed)).bfloat16().cuda()
    ids, weights = ops.route_topk(logits, TOPK)
    half = EXPERTS // 2
    cut = lambda t, lo: t[lo:lo + half]  # noqa: E731
    parts = []
    for lo in (0, half):
        rank = replace(routed, planes13=cut(routed.planes13, lo), scales13=cut(routed.scales13, lo), row13=cut(routed.row13, lo),
                       planes2=cut(routed.planes2, lo), scales2=cut(routed.scales2, lo), row2=cut(routed.row2, lo), base=lo, tiled13=None, tiled2=None)
        parts.append(w3_moe.w3_moe(rank, x, ids, weights).float())
    want, _ = c_port.moe_layer(h_routed, _bits(x), ids.cpu().numpy(), weights.cpu().numpy())
    mx, nr = errors(parts[0] + parts[1], _from_bits(want))
    assert mx < MAX_REL and nr < 2 * NORM_REL, (mx, nr)


@pytest.fixture(scope="module")
def nvfp4_dense():
    """Config 1's matrix: codes uniform over the 16 codes, block scales |N(0,1)| clipped to [2^-6, 448], scale 1/448."""
    from hibana_amd.weights import modelopt
    from oracle.w3_format import e4m3_bytes
    n, k = 25600, 5120
    g = np.random.default_rng(1)
    packed = g.integers(0, 256, (n, k // 2), dtype=np.uint8)
    scales = e4m3_bytes(np.clip(np.abs(g.normal(0, 1, (n, k // 16))), 2.0 ** -6, 448.0))
    lin = modelopt.Nvfp4Linear(torch.from_numpy(packed).cuda(), torch.from_numpy(onv.swizzle_block_scales(scales)).cuda().view(torch.float8_e4m3fn),
                               torch.tensor(1.0 / 448.0).cuda(), torch.tensor(1.0).cuda(), n, k).tile()
    unpacked = np.concatenate([onv.unpack_fp4(packed[r0:r0 + 3200], scales[r0:r0 + 3200]) for r0 in range(0, n, 3200)])  # the oracle's unpack, once
    return lin, unpacked


@pytest.mark.parametrize("m,kernel", [(1, 0), (8, 0), (64, 0), (64, 1), (64, 2)])
def test_nvfp4_dense_at_the_benchmark_geometry(nvfp4_dense, m, kernel):
    from hibana_amd import _lib
    from hibana_amd.kernels import ops
    lin, unpacked = nvfp4_dense
    x = torch.randn(m, 5120, generator=torch.Generator().manual_seed(m)).bfloat16()
    assert _lib.lib().hb_tune(b"nvfp4_tile", kernel) == 0
    try:
        got = ops.nvfp4_linear(x.cuda(), lin).cpu()
    finally:
        _lib.lib().hb_tune(b"nvfp4_tile", 0)
    want = torch.empty(m, 25600, dtype=torch.bfloat16)
    for r0 in range(0, 25600, 3200):  # a slice of rows at a time: the FP64 copy of the matrix stays small
        want[:, r0:r0 + 3200] = layers.nvfp4_dense_ref(x, unpacked[r0:r0 + 3200], 1.0 / 448.0)
    assert torch.allclose(got.float(), want.float(), rtol=0.016, atol=0.004)  # the reference's W4A16 bound (tests/gpu/test_bolt_kernels.py:38)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)


def test_nvfp4_dense_partial_tiles_do_not_depend_on_what_the_workspace_held(nvfp4_dense):
    """64 rows at config 1's size share K among four workgroups a tile: whichever finishes last must find the others'
    partial tiles in memory. The workspace is filled with NaN before every call (and its head put back to zero, as the
    library asks of a new workspace); every call gives the first one's bits,
    which are the stream's result to the summation order."""
    from hibana_amd import _lib
    from hibana_amd.kernels import ops
    lin, _ = nvfp4_dense
    n, k, m = 25600, 5120, 64
    lib = _lib.lib()
    x = torch.randn(m, k, generator=torch.Generator().manual_seed(m)).bfloat16().cuda()
    need = lib.hb_nvfp4_gemm_workspace_bytes(m, n, k)
    assert need > 0
    ws = torch.empty(need // 4, dtype=torch.float32, device="cuda")
    y = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    first = None
    for _ in range(12):
        ws.fill_(float("nan"))
        _lib.check(lib.hb_workspace_reset(_lib.ptr(ws), need, _lib.stream()), "reset")  # the head (the tiles' arrival counters) starts at zero
        _lib.check(lib.hb_nvfp4_gemm_ws(_lib.ptr(x), m, _lib.ptr(lin.tiled), lin.global_scale, n, k, 0, _lib.ptr(y), _lib.ptr(ws), need, _lib.stream()), "gemm")
        if first is None:
            first = y.clone()
        assert torch.equal(y, first)
    assert lib.hb_tune(b"nvfp4_tile", 2) == 0
    try:
        stream = ops.nvfp4_linear(x, lin)
    finally:
        lib.hb_tune(b"nvfp4_tile", 0)
    mx, nr = errors(first, stream)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)


@pytest.fixture(scope="module")
def latent_block():
    from hibana_amd import synthetic
    from hibana_amd.model import nemotron_moe
    tokens, hidden, latent, inter, experts, topk = 2048, 4096, 1024, 2688, 512, 22
    g = torch.Generator().manual_seed(5)
    ex = synthetic.nvfp4_experts(experts, latent, inter, 11, "cuda", keep=True)
    router = torch.randn(experts, hidden, generator=g) * (1.0 / hidden ** 0.5)
    fc1 = (torch.randn(latent, hidden, generator=g) * 0.02).bfloat16()
    fc2 = (torch.randn(hidden, latent, generator=g) * 0.02).bfloat16()
    block = nemotron_moe.NemotronMoe(torch.cat([router.bfloat16(), fc1]).cuda(), torch.zeros(experts).cuda(), fc2.cuda(), ex, topk)
    x = torch.randn(tokens, hidden, generator=g).bfloat16()
    yield block, ex, fc1, fc2, x
    del block, ex
    torch.cuda.empty_cache()


@pytest.mark.parametrize("kernel", [0, 1, 2])
def test_latent_moe_block_at_the_benchmark_geometry(latent_block, kernel):
    from hibana_amd import _lib
    block, ex, fc1, fc2, x = latent_block
    latent, inter, topk = 1024, 2688, 22
    assert _lib.lib().hb_tune(b"nvfp4_tile", kernel) == 0
    try:
        got = block(x.cuda())
        again = block(x.cuda())
    finally:
        _lib.lib().hb_tune(b"nvfp4_tile", 0)
    assert torch.equal(got, again)  # deterministic
    fused = torch.mm(x.cuda(), block.gate_fc1.T, out_dtype=torch.float32)
    ids, w, _ = block.route(fused)
    assert int(torch.unique(ids).numel()) == 512 and ids.shape == (2048, topk)
    sample = torch.randperm(2048, generator=torch.Generator().manual_seed(kernel))[:20].sort().values

    def get(i):  # expert i's matrices as the checkpoint holds them, unpacked by the oracle (asked for once an expert)
        s1 = onv.unswizzle_block_scales(ex.s1[i].view(torch.uint8).cpu().numpy(), inter, latent // 16)
        s2 = onv.unswizzle_block_scales(ex.s2[i].view(torch.uint8).cpu().numpy(), latent, inter // 16)
        return (onv.unpack_fp4(ex.w1[i].cpu().numpy(), s1), np.float32(ex.alpha1[i].item()),
                onv.unpack_fp4(ex.w2[i].cpu().numpy(), s2), np.float32(ex.alpha2[i].item()))

    want = layers.latent_moe_ref(x[sample], fc1, fc2, ids[sample.cuda()].cpu().numpy(), w[sample.cuda()].cpu(), get)
    mx, nr = errors(got[sample.cuda()], want)
    assert mx < MAX_REL and nr < 2 * NORM_REL, (mx, nr)
