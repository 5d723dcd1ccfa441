"""NVFP4 kernels on the GPU against the oracle: bit-exact unpack (from row-major and from the 128x4-interleaved block
scales) and the weight-only linear bf16((x Wq^T)_fp32 * s2), as tests/gpu/test_bolt_kernels.py:21-38 of the reference
states it."""
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


def _matrix(n, k, seed, lo=2 ** -6, hi=448.0):
    g = np.random.default_rng(seed)
    packed = g.integers(0, 256, (n, k // 2), dtype=np.uint8)
    scales = e4m3_bytes(np.clip(np.abs(g.normal(0, 1, (n, k // 16))), lo, hi))
    return packed, scales


def _linear(packed, scales, alpha=2.0, inv=0.25):
    from hibana_amd.weights import modelopt
    n, k = packed.shape[0], packed.shape[1] * 2
    sw = torch.from_numpy(onv.swizzle_block_scales(scales)).cuda().view(torch.float8_e4m3fn)
    return modelopt.Nvfp4Linear(torch.from_numpy(packed).cuda(), sw, torch.tensor(alpha).cuda(), torch.tensor(inv).cuda(), n, k)


@pytest.mark.parametrize("n,k", [(64, 128), (128, 256), (192, 640), (1024, 2688)])
def test_unpack_is_bit_exact_from_both_scale_layouts(n, k):
    from hibana_amd.weights import modelopt
    packed, scales = _matrix(n, k, 1)
    want = onv.unpack_fp4(packed, scales)
    got = modelopt.unpack_fp4(torch.from_numpy(packed).cuda(), torch.from_numpy(scales).cuda().view(torch.float8_e4m3fn)).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    lin = _linear(packed, scales)
    deq = lin.dequantize().cpu().numpy()
    ref = onv.linear_dequantize(packed, onv.swizzle_block_scales(scales), 2.0, 0.25, n, k)
    assert np.array_equal(deq.view(np.uint32), ref.view(np.uint32))
    assert lin.bytes == packed.size + onv.swizzle_block_scales(scales).size


def test_every_code_and_signed_zero():
    from hibana_amd.weights import modelopt
    packed = np.tile(np.arange(256, dtype=np.uint8), (64, 1))[:, :64].copy()
    packed[1] = np.arange(192, 256, dtype=np.uint8)
    scales = np.full((64, 8), 0x38, np.uint8)
    got = modelopt.unpack_fp4(torch.from_numpy(packed).cuda(), torch.from_numpy(scales).cuda().view(torch.float8_e4m3fn)).cpu().numpy()
    want = onv.unpack_fp4(packed, scales)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))  # includes -0.0 for code 8


def test_swizzle_helpers_match_the_oracle():
    from hibana_amd.kernels import w3_moe
    from hibana_amd.weights import modelopt
    g = np.random.default_rng(3)
    s = e4m3_bytes(g.uniform(0.01, 1.01, (2, 256, 16)))
    dev = torch.from_numpy(s).cuda().view(torch.float8_e4m3fn)
    sw = modelopt.swizzle_block_scales_batched(dev)
    assert np.array_equal(sw.cpu().numpy(), onv.swizzle_batched(s))
    back = w3_moe.unswizzle_batched(sw, 256, 16)
    assert np.array_equal(back.view(torch.uint8).cpu().numpy(), s)
    odd = e4m3_bytes(g.uniform(0.01, 1.01, (130, 6)))
    one = modelopt.swizzle_block_scales(torch.from_numpy(odd).cuda())
    assert one.shape == (256, 8) and np.array_equal(one.cpu().numpy(), onv.swizzle_block_scales(odd))
    assert np.array_equal(modelopt.unswizzle_block_scales(one, 130, 6).cpu().numpy(), odd)


@pytest.mark.parametrize("m", [1, 8, 17, 64, 65])
@pytest.mark.parametrize("relu2", [False, True])
@pytest.mark.parametrize("n,k", [(128, 512), (320, 2688), (1024, 1024)])
def test_weight_only_linear_matches_the_oracle(m, relu2, n, k):
    from hibana_amd.kernels import ops
    packed, scales = _matrix(n, k, 12, hi=8.0)
    lin = _linear(packed, scales, alpha=0.7, inv=1.0)
    x = torch.randn(m, k, generator=torch.Generator().manual_seed(m)).bfloat16()
    want = layers.nvfp4_dense_ref(x, onv.unpack_fp4(packed, scales), np.float32(0.7), relu2=relu2)
    got = ops.nvfp4_linear(x.cuda(), lin, relu2=relu2)
    assert got.dtype == torch.bfloat16 and got.shape == (m, n)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    torch.testing.assert_close(got.cpu().float(), want.float(), rtol=.016, atol=.004 * float(want.float().abs().max()))
    assert torch.equal(ops.nvfp4_linear(x.cuda(), lin, relu2=relu2), got)
    assert torch.equal(lin(x.cuda()), ops.nvfp4_linear(x.cuda(), lin))


@pytest.mark.parametrize("m", [17, 21, 40, 64, 100, 128, 200])
@pytest.mark.parametrize("ks", [0, 2, 3, 5])
def test_tiles_whose_k_is_shared_among_workgroups(m, ks):
    """A few dozen rows: the workgroups of a tile split K, leave their partial tiles in the workspace and the last one
    to arrive adds them in a fixed order: the oracle's product, the same bits on every call, and (an order of FP32 sums
    aside) the bits of the undivided tile."""
    from hibana_amd import _lib
    from hibana_amd.kernels import ops
    n, k = 320, 2688
    packed, scales = _matrix(n, k, 13, hi=8.0)
    lin = _linear(packed, scales, alpha=0.3, inv=1.0)
    x = torch.randn(m, k, generator=torch.Generator().manual_seed(m)).bfloat16()
    want = layers.nvfp4_dense_ref(x, onv.unpack_fp4(packed, scales), np.float32(0.3), relu2=bool(ks & 1))
    lib = _lib.lib()
    assert lib.hb_tune(b"nvfp4_tile_ks", ks) == 0
    try:
        assert (lib.hb_nvfp4_gemm_workspace_bytes(m, n, k) > 0) == (m > 20)  # up to twenty rows the weight stream serves
        got = [ops.nvfp4_linear(x.cuda(), lin, relu2=bool(ks & 1)) for _ in range(3)]
    finally:
        lib.hb_tune(b"nvfp4_tile_ks", 0)
    assert torch.equal(got[0], got[1]) and torch.equal(got[0], got[2])
    mx, nr = errors(got[0], want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)


def test_up_projection_shape_against_the_dequantized_product():
    """BASELINE config 1 (K = 5120, N = 25600, global scale 1/448), M = 1 and 8: the kernel against
    (x @ unpack^T) * s2 in FP32 on the GPU; the unpack itself is pinned bit-exact on the smaller shapes."""
    from hibana_amd.kernels import ops
    from hibana_amd.weights import modelopt
    torch.manual_seed(0)
    n, k = 25600, 5120
    weight = torch.randint(0, 256, (n, k // 2), device="cuda", dtype=torch.uint8)
    scales = torch.randn(n, k // 16, device="cuda").abs().clamp(2 ** -6, 448).to(torch.float8_e4m3fn)
    lin = modelopt.Nvfp4Linear(weight, modelopt.swizzle_block_scales(scales), torch.tensor(1 / 448.0).cuda(), torch.tensor(1.0).cuda(), n, k)
    assert lin.bytes == 73_728_000
    unscaled = modelopt.unpack_fp4(weight, scales)
    for m in (1, 8):
        x = torch.randn(m, k, device="cuda").bfloat16()
        want = ((x.float() @ unscaled.T) * lin.global_scale).bfloat16()
        got = ops.nvfp4_linear(x, lin)
        mx, nr = errors(got, want)
        assert mx < MAX_REL and nr < NORM_REL, (m, mx, nr)
        assert torch.equal(ops.nvfp4_linear(x * 4, lin), got * 4)  # a power of two commutes with every rounding


def test_w3_copy_serves_the_call_when_enabled():
    from hibana_amd.kernels import ops, w3
    packed, scales = _matrix(128, 256, 5, hi=4.0)
    lin = _linear(packed, scales, alpha=1.0, inv=1.0)
    x = torch.randn(4, 256, generator=torch.Generator().manual_seed(1)).bfloat16().cuda()
    plain = ops.nvfp4_linear(x, lin)
    w3.attach([("lin", lin)], "lloyd")
    assert lin.w3 is not None and lin.bytes == lin.w3.bytes
    assert not ops.w3_decode(lin, 4)
    assert torch.equal(ops.nvfp4_linear(x, lin), plain)
    try:
        w3.set_enabled(True)
        assert ops.w3_decode(lin, 4) and not ops.w3_decode(lin, 200) and not ops.w3_decode(lin, 4, rows=2)
        three = ops.nvfp4_linear(x, lin)
        assert torch.equal(three, w3.w3_linear(x, lin.w3))
        assert errors(three, plain.cpu())[1] < 0.25  # eight levels a group: a coarser copy of the same matrix
    finally:
        w3.set_enabled(None)


@pytest.mark.parametrize("m,pairs", [(3, 0), (40, 0), (5, 64)])
def test_dense_mlp_on_both_paths(m, pairs):
    """`Mlp.__call__` (hibana/model/mlp.py:26-48): NVFP4 gate|up and down against the oracle's dense products around
    silu_and_mul; with 3-bit copies enabled, the decode path - the 3-bit gate|up product, its SiLU product rounded to
    E4M3 per 32-group in one launch, the 3-bit down product on those codes - against the same ops called one by one
    (bit for bit) and against the oracle's rounding of the device's own SiLU product."""
    from hibana_amd.kernels import ops, w3
    from hibana_amd.model.mlp import Mlp
    hidden, inter = 256, 384
    gp, gs = _matrix(2 * inter, hidden, 21, hi=2.0)
    dp, ds = _matrix(hidden, inter, 22, hi=2.0)
    gate_up, down = _linear(gp, gs, alpha=0.05, inv=1.0), _linear(dp, ds, alpha=0.03, inv=1.0)
    gate_up.pairs = pairs
    mlp = Mlp(gate_up, down)
    x = torch.randn(m, hidden, generator=torch.Generator().manual_seed(m)).bfloat16()
    got = mlp(x.cuda())
    h = layers.silu_and_mul(layers.nvfp4_dense_ref(x, onv.unpack_fp4(gp, gs), np.float32(0.05)), pairs)
    want = layers.nvfp4_dense_ref(h, onv.unpack_fp4(dp, ds), np.float32(0.03))
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < 2 * NORM_REL, (mx, nr)  # two products and a BF16 SiLU between them
    with pytest.raises(ValueError):
        mlp(None, prequantized=(x, x))
    if m > w3.MAX_ROWS:
        return
    w3.attach([("gate_up", gate_up), ("down", down)], "lloyd")
    try:
        w3.set_enabled(True)
        three = mlp(x.cuda())
        gu3 = w3.w3_linear(x.cuda(), gate_up.w3)
        q, s = ops.silu_mul_quant_groups(gu3, pairs, torch_chain=True)
        assert torch.equal(three, w3.w3_linear(q, down.w3, s))
        want3 = layers.dense_a8_ref(ops.silu_and_mul(gu3, pairs).cpu(), w3.dequantize(down.w3).cpu().numpy())  # (the unpacking is pinned bit for bit elsewhere)
        mx, nr = errors(three, want3)
        assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    finally:
        w3.set_enabled(None)


def test_bad_calls_raise():
    from hibana_amd.kernels import ops
    from hibana_amd.weights import modelopt
    packed, scales = _matrix(64, 128, 7)
    lin = _linear(packed, scales)
    with pytest.raises(ValueError):
        ops.nvfp4_linear(torch.zeros(2, 64, dtype=torch.bfloat16, device="cuda"), lin)
    with pytest.raises(ValueError):
        ops.nvfp4_linear(torch.zeros(2, 128, device="cuda"), lin)
    with pytest.raises(ValueError):
        modelopt.unpack_fp4(torch.zeros(64, 12, dtype=torch.uint8, device="cuda"), torch.zeros(64, 2, dtype=torch.uint8, device="cuda"))
    with pytest.raises(ValueError):
        modelopt.unswizzle_block_scales(torch.zeros(100), 128, 4)
