"""The routed experts' offline quantizer (ratio-grid group scales, nearest level): the oracle pinned against the
nearest-level `pack` and a brute-force search on the CPU; the shipped `w3_moe.quantize` / `calibrate` against the oracle and
the reference's own assertions (tests/unit/test_w3_moe_pack.py:35-47 of the reference) on the GPU."""
import numpy as np
import pytest
import torch

from oracle import nvfp4_format as onv
from oracle import w3_format as ow3


def _weights(n, k, seed):
    g = np.random.default_rng(seed)
    return (g.normal(0, 0.05, (n, k)) * g.uniform(0.2, 3.0, (n, 1))).astype(np.float32)


def test_ratio_one_is_the_nearest_level_pack():
    w = _weights(128, 256, 1)
    raw, row = ow3.fit_scales_ratio(w, "lloyd", ratios=(1.0,))
    packed = ow3.pack(w, "lloyd")
    assert np.array_equal(raw, ow3.scale_bytes(packed)) and np.array_equal(row, packed["row_scale"])
    assert np.array_equal(ow3.quantize_groups(w, raw, row, "lloyd"), ow3.codes(packed))


def test_fitted_scale_is_the_brute_force_minimum():
    w = _weights(128, 128, 2)
    levels = np.asarray(ow3.CODEBOOKS["zero8"], dtype=np.float32)
    ratios = (0.6, 0.8, 1.0)
    raw, row = ow3.fit_scales_ratio(w, "zero8", ratios=ratios)
    base = np.abs(w.reshape(128, 4, 32)).max(-1) / np.float32(3.5)
    for n in range(0, 128, 17):
        for gi in range(4):
            losses, cands = [], []
            for r in ratios:
                byte = ow3.e4m3_bytes(np.float32(base[n, gi] * np.float32(r)) / row[n])
                eff = float(ow3.e4m3_floats(byte)) * float(row[n])
                x = w[n, 32 * gi:32 * gi + 32].astype(np.float64)
                deq = np.array([levels[np.argmin(np.abs(v / max(eff, 1e-30) - levels.astype(np.float64)))] for v in x]) * eff
                losses.append(float(((x - deq) ** 2).sum()))
                cands.append(int(byte))
            assert int(raw[n, gi]) in [c for c, l in zip(cands, losses) if l <= min(losses) * (1 + 1e-5)]
    one, _ = ow3.fit_scales_ratio(w, "zero8", ratios=(1.0,))

    def loss(bytes_):
        q = ow3.quantize_groups(w, bytes_, row, "zero8")
        eff = ow3.e4m3_floats(bytes_) * row[:, None]
        return ((w.reshape(128, 4, 32) - levels[q].reshape(128, 4, 32) * eff[:, :, None]) ** 2).sum(-1)

    assert (loss(raw) <= loss(one) * (1 + 1e-5)).all()


def _nvfp4(e, rows, k, seed):
    g = torch.Generator().manual_seed(seed)
    packed = torch.randint(0, 256, (e, rows, k // 2), generator=g, dtype=torch.uint8)
    scales = (torch.rand(e, rows, k // 16, generator=g) * 0.02 + 0.001).to(torch.float8_e4m3fn)
    return packed, scales


@pytest.mark.gpu
def test_quantize_matches_the_oracle():
    from hibana_amd.kernels import w3_moe
    w = _weights(256, 256, 3)
    codes, scales, row = w3_moe.quantize(torch.from_numpy(w).cuda())
    raw = scales.view(torch.uint8).cpu().numpy()
    want_raw, want_row = ow3.fit_scales_ratio(w, "lloyd")
    assert np.array_equal(row.cpu().numpy(), want_row)
    assert (raw == want_raw).mean() > 0.995  # the device's loss sums may order two near-equal ratios differently
    assert np.array_equal(codes.cpu().numpy(), ow3.quantize_groups(w, raw, want_row, "lloyd"))  # exact under its own scales


@pytest.mark.gpu
def test_calibration_fits_the_nvfp4_experts():
    from hibana_amd.kernels import w3, w3_moe
    e, i, h = 2, 128, 256
    (w13, s13), (w2, s2) = _nvfp4(e, 2 * i, h, 0), _nvfp4(e, h, i, 1)
    g13, g2 = torch.tensor([0.5, 0.25]), torch.tensor([0.125, 2.0])
    dev = lambda *t: [x.cuda() for x in t]  # noqa: E731
    ex, report = w3_moe.calibrate(*dev(w13, s13, g13, w2, s2, g2), chunk=1)
    _, nearest = w3_moe.calibrate(*dev(w13, s13, g13, w2, s2, g2), ratios=(1.0,), chunk=1)
    assert ex.planes13.shape == (e, 2 * i // 32, h // 128, 3, 32, 4) and ex.planes2.shape == (e, h // 32, i // 128, 3, 32, 4)
    inverse = torch.argsort(w3_moe.fc1_order(i)).cuda()
    for k in range(e):  # the report is the error of what the kernel reads, in the checkpoint's row order
        source = torch.from_numpy(onv.unpack_fp4(w13[k].numpy(), s13[k].view(torch.uint8).numpy())).cuda() * g13[k]
        fc1 = w3.dequantize(ex.matrix(k, True))[inverse]
        assert float((fc1 - source).norm() / source.norm()) < 0.25
    assert report["w13"] <= nearest["w13"] and report["w2"] <= nearest["w2"]  # the scale search only helps
    per_weight = 8 * ex.bytes / (e * 3 * i * h)
    assert 3.25 < per_weight < 3.5  # codes and group scales, plus one FP32 multiplier a row
    # and the calibrated experts serve
    x = torch.randn(3, h, generator=torch.Generator().manual_seed(5)).bfloat16().cuda()
    ids = torch.tensor([[0, 1], [1, 0], [0, 1]], dtype=torch.int32).cuda()
    out = w3_moe.w3_moe(ex, x, ids, torch.full((3, 2), 0.5).cuda())
    assert out.shape == (3, h) and bool(torch.isfinite(out.float()).all())
