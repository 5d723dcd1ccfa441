"""The dense W3 linear on the GPU against the oracle (weight-only: BF16 activations, exact weights, FP32 accumulate)."""
import numpy as np
import pytest
import torch

from oracle import layers, w3_format as ow3
from tests.util import MAX_REL, NORM_REL, errors, random_w3, to_device_w3

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["auto", "tile", "stream", "stream16"], autouse=True)
def kernel_choice(request):
    """Every case runs with the library's own choice between the 128-row MFMA tile kernel and the 16-row weight stream,
    with each of them forced, and with the stream's body for slots of at most four rows switched off (so those slots
    take the sixteen-row body, as they do when the activation matrix is too large for a buffer descriptor)."""
    from hibana_amd import _lib
    tile, few = {"auto": (0, 0), "tile": (1, 0), "stream": (2, 0), "stream16": (2, 2)}[request.param]
    assert _lib.lib().hb_tune(b'w3_tile', tile) == 0 and _lib.lib().hb_tune(b'w3_few', few) == 0
    yield request.param
    _lib.lib().hb_tune(b'w3_tile', 0)
    _lib.lib().hb_tune(b'w3_few', 0)


@pytest.mark.parametrize("m", [1, 2, 4, 5, 16, 17, 33, 64, 128])  # 4 | 5: the last slot the few-row body takes, the first it does not
@pytest.mark.parametrize("n,k,codebook", [(128, 256, "uniform"), (512, 1024, "lloyd"), (1024, 640, "zero8"), (256, 2688, "lloyd"),
                                          (128, 128, "lloyd"), (256, 384, "uniform")])  # one and three chunks: the ring's short tails
def test_w3_linear_matches_the_oracle(m, n, k, codebook):
    from hibana_amd.kernels import w3
    packed, *_ = random_w3(n, k, 7, codebook)
    dev = to_device_w3(packed)
    g = torch.Generator().manual_seed(100 + m)
    x = torch.randn(m, k, generator=g).bfloat16()
    x[:, ::97] *= 30  # outlier channels
    want = layers.dense_ref(x, ow3.dequantize(packed))
    got = w3.w3_linear(x.cuda(), dev)
    assert got.dtype == torch.bfloat16 and got.shape == (m, n)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    again = w3.w3_linear(x.cuda(), dev)
    assert torch.equal(again, got)  # bitwise repeatable


@pytest.mark.parametrize("m", [1, 4, 5, 16, 33, 128])
@pytest.mark.parametrize("n,k", [(256, 384), (512, 2048), (128, 128), (3072, 1024)])  # the last: a draft head's shape (vocabulary rows x hidden)
def test_two_bit_linear_matches_the_oracle(m, n, k, kernel_choice):
    """A four-level codebook (the reference's two-plane variant, its draft head's copy: hibana/proposers/draft_head.py:106)
    through the product at its own density - two-bit tiles, 2.25 bits a weight - on BF16 and on E4M3 activations, and the
    same matrix widened into three-bit tiles gives the same bits."""
    from hibana_amd.kernels import w3
    packed, *_ = random_w3(n, k, 17, "lloyd2")
    dev = to_device_w3(packed)
    g = torch.Generator().manual_seed(300 + m)
    x = torch.randn(m, k, generator=g).bfloat16()
    x[:, ::97] *= 30
    dense = ow3.dequantize(packed)
    want = layers.dense_ref(x, dense)
    got = w3.w3_linear(x.cuda(), dev)
    assert dev.tile_bits == 2 and dev.tiled.numel() == n * k // 4 + n * k // 32
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    assert torch.equal(w3.w3_linear(x.cuda(), dev), got)
    wide = w3.tile(to_device_w3(packed), widen=True)
    assert wide.tile_bits == 3
    if kernel_choice.startswith("stream"):  # the same sums from either layout (the MFMA tile kernel, which serves only three-bit tiles, adds in another order)
        assert torch.equal(w3.w3_linear(x.cuda(), wide), got)
    else:
        mx, nr = errors(w3.w3_linear(x.cuda(), wide), want)
        assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    q, s = w3.quant_groups(x.cuda())
    want8 = layers.dense_a8_ref(x, dense)
    got8 = w3.w3_linear(q, dev, s)
    mx, nr = errors(got8, want8)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    assert torch.equal(w3.w3_linear(q, wide, s), got8)


def test_every_k_split_gives_close_results_and_the_unsplit_bits_repeat():
    from hibana_amd import _lib
    from hibana_amd.kernels import w3
    packed, *_ = random_w3(256, 2048, 8)
    dev = to_device_w3(packed)
    try:
        for m in (3, 16):  # both bodies of the stream; from 16 chunks a wavefront down to 1, even and odd counts
            x = torch.randn(m, 2048, generator=torch.Generator().manual_seed(m)).bfloat16()
            want = layers.dense_ref(x, ow3.dequantize(packed))
            for ks, nbw in ((1, 1), (1, 4), (2, 2), (3, 1), (4, 1), (5, 3), (7, 2), (8, 1), (16, 1), (4, 4), (0, 0)):
                assert _lib.lib().hb_tune(b"w3_ksplit", ks) == 0 and _lib.lib().hb_tune(b"w3_nbw", nbw) == 0
                got = w3.w3_linear(x.cuda(), dev)
                mx, nr = errors(got, want)
                assert mx < MAX_REL and nr < NORM_REL, (m, ks, nbw, mx, nr)
    finally:
        _lib.lib().hb_tune(b"w3_ksplit", 0)
        _lib.lib().hb_tune(b"w3_nbw", 0)


def test_full_size_decode_projection_against_the_dequantized_product():
    """BASELINE config 0 (M = 1, K = N = 5120, uniform codebook, one scale draw per 128): the kernel against
    x @ dequantize(W)^T in FP32 on the GPU; the dequantization itself is pinned bit-exact on the smaller shapes."""
    from hibana_amd.kernels import w3
    torch.manual_seed(0)
    n = k = 5120
    q = torch.randint(0, 8, (n, k), device="cuda", dtype=torch.uint8)
    s = (torch.randn(n, k // 128, device="cuda").abs() * 0.02 + 1e-3).repeat_interleave(4, dim=1)
    row = (s.amax(dim=1) / 448.0).clamp_min(1e-12)
    stored = (s / row[:, None]).to(torch.float8_e4m3fn)
    weight = w3.pack_codes(q, stored, row, "uniform")
    assert weight.bytes == 10_670_080
    x = torch.randn(1, k, device="cuda").bfloat16()
    deq = w3.dequantize(weight)
    levels = torch.tensor(weight.codebook, device="cuda")
    assert torch.equal(deq, levels[q.long()] * (stored.float() * row[:, None]).repeat_interleave(32, dim=1))
    want = (x.float() @ deq.T).bfloat16()
    got = w3.w3_linear(x, weight)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    # linearity in x: f(2x) == 2 f(x) exactly (a power of two commutes with every rounding)
    assert torch.equal(w3.w3_linear(x * 2, weight), got * 2)


def test_unsupported_calls_raise():
    from hibana_amd.kernels import w3
    packed, *_ = random_w3(128, 256, 9)
    dev = to_device_w3(packed)
    with pytest.raises(ValueError):
        w3.w3_linear(torch.zeros(129, 256, dtype=torch.bfloat16, device="cuda"), dev)
    with pytest.raises(ValueError):
        w3.w3_linear(torch.zeros(4, 128, dtype=torch.bfloat16, device="cuda"), dev)
    with pytest.raises(RuntimeError):
        w3.w3_linear(torch.zeros(4, 256, dtype=torch.bfloat16), dev)


@pytest.mark.parametrize("m", [1, 16, 128])
@pytest.mark.parametrize("n,k", [(10240, 5120), (5120, 17408)])
def test_the_references_full_size_shapes(n, k, m):
    """The shapes of the reference's own GPU test of the dense linear (tests/gpu/test_w3_calibration.py:23-45: rows 1 to
    128 on 10240 x 5120 and 5120 x 17408, norm-relative error below 0.004): the kernel against x @ dequantize(W)^T in
    FP32 on the GPU, the dequantization being pinned bit-exact against the oracle on the smaller shapes; bitwise
    repeatable, as that test demands of a graph replay."""
    from hibana_amd.kernels import w3
    g = torch.Generator(device="cuda").manual_seed(n + k + m)
    q = torch.randint(0, 8, (n, k), device="cuda", dtype=torch.uint8, generator=g)
    s = torch.rand(n, k // 32, device="cuda", generator=g) * 0.03 + 1e-3
    row = (s.amax(dim=1) / 448.0).clamp_min(1e-12)
    stored = (s / row[:, None]).to(torch.float8_e4m3fn)
    weight = w3.pack_codes(q, stored, row, "lloyd")
    x = torch.randn(m, k, device="cuda", generator=g).bfloat16()
    want = (x.float() @ w3.dequantize(weight).T).bfloat16()
    got = w3.w3_linear(x, weight)
    mx, nr = errors(got, want)
    assert mx < MAX_REL and nr < NORM_REL, (mx, nr)
    assert torch.equal(w3.w3_linear(x, weight), got)
