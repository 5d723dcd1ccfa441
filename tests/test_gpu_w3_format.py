"""W3 format kernels on the GPU against the oracle: bit-exact packing, repack, unpack and dequantization."""
import numpy as np
import pytest
import torch

from oracle import w3_format as ow3
from tests.util import random_w3, to_device_w3

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,k,codebook", [(128, 128, "uniform"), (256, 384, "lloyd"), (128, 256, "lloyd2"), (640, 1024, "zero8")])
def test_pack_codes_gives_the_oracle_planes(n, k, codebook):
    from hibana_amd.kernels import w3
    packed, q, raw, row = random_w3(n, k, 1, codebook)
    got = w3.pack_codes(torch.from_numpy(q).cuda(), torch.from_numpy(raw).cuda().view(torch.float8_e4m3fn), torch.from_numpy(row).cuda(), codebook)
    assert got.planes.shape == packed["planes"].shape and got.scales.shape == packed["scales"].shape
    assert np.array_equal(got.planes.view(torch.int32).cpu().numpy().view(np.uint32), packed["planes"])
    assert np.array_equal(got.scales.cpu().numpy(), packed["scales"])
    assert got.lut == packed["lut"] and got.bytes == ow3.nbytes(packed)


@pytest.mark.parametrize("n,k,codebook", [(128, 128, "uniform"), (256, 384, "lloyd"), (128, 256, "lloyd2"), (1024, 2048, "lloyd")])
def test_repack_unpack_and_dequantize_are_bit_exact(n, k, codebook):
    from hibana_amd.kernels import w3
    packed, q, raw, row = random_w3(n, k, 2, codebook)
    dev = to_device_w3(packed)
    # the checkpoint layout as stored
    assert np.array_equal(w3.codes(dev).cpu().numpy(), q)
    assert np.array_equal(w3.scale_bytes(dev).view(torch.uint8).cpu().numpy(), raw)
    # the kernels' block layout
    w3.tile(dev)
    bits = 2 if codebook == "lloyd2" else 3  # a two-bit matrix keeps its density: 2.25 bits a weight
    assert dev.tile_bits == bits and dev.tiled.numel() == n * k * bits // 8 + n * k // 32
    assert np.array_equal(w3.codes(dev).cpu().numpy(), q)
    assert np.array_equal(w3.scale_bytes(dev).view(torch.uint8).cpu().numpy(), raw)
    want = ow3.dequantize(packed)
    got = w3.dequantize(dev).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))  # FP32 bit patterns
    assert np.array_equal(w3.group_scales(dev).cpu().numpy().view(np.uint32), ow3.group_scales(packed).view(np.uint32))
    if bits == 2:  # the same matrix widened into three-bit tiles (what the routed experts' kernels read): the same weights
        wide = w3.tile(to_device_w3(packed), widen=True)
        assert wide.tile_bits == 3 and wide.tiled.numel() == n * k * 3 // 8 + n * k // 32
        assert np.array_equal(w3.codes(wide).cpu().numpy(), q)
        assert np.array_equal(w3.dequantize(wide).cpu().numpy().view(np.uint32), want.view(np.uint32))
    w3.tile(dev, release=True)
    assert dev.planes is None and np.array_equal(w3.codes(dev).cpu().numpy(), q)


def test_nearest_level_pack_matches_the_oracle_quantizer():
    from hibana_amd.kernels import w3
    torch.manual_seed(0)
    weight = torch.randn(256, 384) * 0.05
    for codebook, fit in (("uniform", False), ("lloyd", False), ("lloyd2", False)):
        want = ow3.pack(weight.numpy(), codebook, fit_scales=fit)
        got = w3.pack(weight.cuda(), codebook, fit_scales=fit)
        assert np.array_equal(got.planes.view(torch.int32).cpu().numpy().view(np.uint32), want["planes"])
        assert np.array_equal(got.scales.cpu().numpy(), want["scales"])
        assert np.array_equal(got.row_scale.cpu().numpy(), want["row_scale"])
    fitted = w3.pack(weight.cuda(), "lloyd2", fit_scales=True)
    nearest = w3.pack(weight.cuda(), "lloyd2")
    err = lambda p: float((w3.dequantize(p).cpu() - weight).norm() / weight.norm())  # noqa: E731
    assert err(fitted) < 0.36 < err(nearest) < 0.45


def test_interleave_rows_and_validation():
    from hibana_amd.kernels import w3
    torch.manual_seed(3)
    weight = (torch.randn(512, 256) * 0.03).cuda()
    order = w3.pair_order(512, 64)
    moved, packed = w3.interleave_rows(w3.pack(weight), 64), w3.pack(weight[order.cuda()])
    for f in ("planes", "scales", "row_scale"):
        a, b = getattr(moved, f), getattr(packed, f)
        assert torch.equal(a.view(torch.int32) if a.dtype == torch.uint32 else a, b.view(torch.int32) if b.dtype == torch.uint32 else b)
    with pytest.raises(ValueError):
        w3.pack(torch.zeros(128, 160).cuda())
    with pytest.raises(ValueError):
        w3.pack(torch.zeros(96, 256).cuda())
    with pytest.raises(ValueError):
        w3.pack(torch.zeros(128, 128).cuda(), (-3.5, -2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 3.3))
