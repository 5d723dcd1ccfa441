#!/usr/bin/env python3
"""Writes tests/golden/w3_fit_scales.npz: what the reference's fitted-scale quantizers return on small seeded matrices.

Run in the build container only (it imports the reference's CPU functions from /root/reference; nothing of the
reference is copied: the file holds inputs and outputs). The two functions it pins choose, per 32-group, the first of
several candidate scales with the strictly smallest squared error, an FP32 sum whose value near a tie depends on the
summation order - which only running them shows:

    hibana.kernels.w3.pack(weight, codebook, fit_scales=True)            hibana/kernels/w3.py:126-172
    hibana.weights.w3_calibration.fit_scales(weight, ones, levels, ...)  hibana/weights/w3_calibration.py:17-37
    hibana.kernels.w3_moe.quantize(weight, codebook)                     hibana/kernels/w3_moe.py:113-124

Cases: the reference's own seeded test matrix (tests/unit/test_w3_pack.py:36-37), a second Gaussian one, a matrix on a
coarse grid (many exactly equal errors between candidates), and one with groups built to tie: all-zero groups, groups
of one repeated value, groups whose candidates round to the same E4M3 byte (one tiny group next to a huge one in its
row).
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

REFERENCE = "/root/reference"
OUT = Path(__file__).resolve().parent / "w3_fit_scales.npz"


def cases() -> dict[str, torch.Tensor]:
    out = {}
    torch.manual_seed(0)
    out["gauss0"] = torch.randn(256, 384) * 0.05  # the reference's own test matrix
    g = torch.Generator().manual_seed(11)
    out["gauss1"] = torch.randn(128, 256, generator=g) * 0.3
    out["grid"] = torch.randint(-7, 8, (128, 256), generator=g).float() / 8.0
    w = torch.randn(128, 256, generator=g) * 0.1
    w[0:8, 0:64] = 0.0                       # all-zero groups
    w[8:16, 32:64] = 0.125                   # one repeated value
    w[16:24, 0:32] = w[16:24, 0:32] * 1e4    # a huge group: the row's other groups store tiny, coarse E4M3 scales
    w[24:32, :] = 0.0                        # all-zero rows (row scale clamps to 1e-12)
    w[32:40, 64:96] = torch.tensor([3.5, -3.5, 2.25, -2.25, 1.25, -1.25, 0.40625, -0.40625] * 4) * 0.01  # exactly on the levels
    out["ties"] = w
    return out


def main() -> int:
    sys.path.insert(0, REFERENCE)
    from hibana.kernels import w3, w3_moe  # noqa: E402  (the reference, CPU functions only)
    from hibana.weights import w3_calibration  # noqa: E402

    arrays = {}
    for name, weight in cases().items():
        arrays[f"{name}.weight"] = weight.numpy()
        for book in ("lloyd", "uniform", "lloyd2"):
            packed = w3.pack(weight, book, fit_scales=True)
            arrays[f"{name}.{book}.pack.planes"] = packed.planes.view(torch.int32).numpy().view(np.uint32)
            arrays[f"{name}.{book}.pack.scales"] = packed.scales.numpy()
            arrays[f"{name}.{book}.pack.row_scale"] = packed.row_scale.numpy()
            levels = w3._codebook(book)
            sc, rs = w3_calibration.fit_scales(weight, torch.ones(weight.shape[1]), levels, w3_moe.RATIOS)
            arrays[f"{name}.{book}.fit.scales"] = sc.view(torch.uint8).numpy()
            arrays[f"{name}.{book}.fit.row_scale"] = rs.numpy()
            codes, sc2, rs2 = w3_moe.quantize(weight, book)
            assert torch.equal(sc2.view(torch.uint8), sc.view(torch.uint8)) and torch.equal(rs2, rs)
            arrays[f"{name}.{book}.quantize.codes"] = codes.numpy().astype(np.uint8)
    np.savez_compressed(OUT, **arrays)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(arrays)} arrays)")
    return 0


if __name__ == "__main__":
    sys.exit(main())
