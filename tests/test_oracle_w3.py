"""The oracle's W3 format functions against the reference's own known answers and invariants (CPU)."""
import json
import os
import struct

import numpy as np
import pytest
import torch

from oracle import w3_format as w3

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "w3_layout_known_answers.json")))


def _random_matrix(n, k, levels, seed):
    g = np.random.default_rng(seed)
    q = g.integers(0, levels, size=(n, k))
    scale = w3.e4m3_bytes(g.uniform(0.01, 300.0, size=(n, k // 32)))
    row = g.uniform(1e-4, 2e-3, size=n).astype(np.float32)
    return q, scale, row


@pytest.mark.parametrize("entry", GOLDEN["planes"], ids=lambda e: f"bits{e['bits']}-n{e['n']}-k{e['k']}")
def test_single_weight_lands_on_the_hand_derived_bits(entry):
    bits = entry["bits"]
    book = "uniform" if bits == 3 else "lloyd2"
    full = (1 << bits) - 1
    q = np.zeros((entry["N"], entry["K"]), dtype=np.int64)
    q[entry["n"], entry["k"]] = full
    packed = w3.pack_codes(q, np.zeros((entry["N"], entry["K"] // 32), np.uint8), np.ones(entry["N"], np.float32), book)
    expected = np.zeros_like(packed["planes"])
    for nb, kc, i, lane, e, pos in entry["bit"]:
        expected[nb, kc, i, lane, e] |= np.uint32(1 << pos)
    assert np.array_equal(packed["planes"], expected)
    for b in range(bits):  # one bit of the code at a time
        q[entry["n"], entry["k"]] = 1 << b
        one = w3.pack_codes(q, np.zeros((entry["N"], entry["K"] // 32), np.uint8), np.ones(entry["N"], np.float32), book)
        nb, kc, i, lane, e, pos = entry["bit"][b]
        assert one["planes"][nb, kc, i, lane, e] == 1 << pos and np.count_nonzero(one["planes"]) == 1
        assert w3.codes(one)[entry["n"], entry["k"]] == 1 << b


@pytest.mark.parametrize("entry", GOLDEN["scales"], ids=lambda e: f"n{e['n']}-G{e['G']}")
def test_scale_byte_lands_on_the_hand_derived_slot(entry):
    sc = np.zeros((entry["N"], entry["K"] // 32), np.uint8)
    sc[entry["n"], entry["G"]] = 0x38  # 1.0
    packed = w3.pack_codes(np.zeros((entry["N"], entry["K"]), np.int64), sc, np.ones(entry["N"], np.float32), "uniform")
    assert packed["scales"][tuple(entry["at"])] == 0x38 and np.count_nonzero(packed["scales"]) == 1


@pytest.mark.parametrize("codebook", ["uniform", "lloyd2"])
def test_unpack_agrees_with_the_kernel_addressing(codebook):
    """tests/unit/test_w3_pack.py:79-108 of the reference: the word a lane reads (bits*nt + b of its chunk), rotated
    right by rot(s) and masked 0x1111 / 0x2222 / 0x4444, holds the four codes of sub-step s in its nibbles; the scale
    byte (4nt + grp)*2 + i of lane-column t belongs to row 8nt + 2t + i."""
    levels = w3.check_codebook(codebook)
    q, scale, row = _random_matrix(128, 256, len(levels), 1)
    packed = w3.pack_codes(q, scale, row, codebook)
    bits = packed["planes"].shape[2]
    assert np.array_equal(w3.codes(packed), q)
    planes = packed["planes"].astype(np.int64)
    for nb, kc, g, t in [(2, 1, 5, 3), (0, 0, 0, 0), (3, 1, 7, 1)]:
        lane = 4 * g + t
        for nt in range(4):
            words = [int(planes[nb, kc, (bits * nt + b) // 4, lane, (bits * nt + b) % 4]) for b in range(bits)]
            for s in range(8):
                rot = 16 * (s // 4) + (s % 4)
                rotated = [((w >> rot) | (w << (32 - rot))) & 0xFFFFFFFF for w in words]
                q4 = (rotated[0] & 0x1111) | (rotated[1] & 0x2222) | ((rotated[2] & 0x4444) if bits == 3 else 0)
                for j in range(4):
                    assert (q4 >> (4 * j)) & 0xF == q[32 * nb + 8 * nt + g, 128 * kc + 16 * s + 4 * t + j]
        lane_bytes = packed["scales"][nb, kc, t]
        eff = w3.group_scales(packed)
        for nt in range(4):
            for grp in range(4):
                for i in range(2):
                    r = 32 * nb + 8 * nt + 2 * t + i
                    byte = w3.e4m3_floats(lane_bytes[(nt * 4 + grp) * 2 + i:(nt * 4 + grp) * 2 + i + 1])[0]
                    assert np.float32(byte) * row[r] == eff[r, 4 * kc + grp]


def test_shapes_bytes_lut_and_dequantize_definition():
    q, scale, row = _random_matrix(256, 384, 8, 0)
    packed = w3.pack_codes(q, scale, row, "lloyd")
    assert packed["planes"].shape == (8, 3, 3, 32, 4) and packed["planes"].dtype == np.uint32
    assert packed["scales"].shape == (8, 3, 4, 32) and packed["scales"].dtype == np.uint8
    assert w3.nbytes(packed) == 256 * 384 * 3 // 8 + 256 * 12 + 256 * 4
    levels = np.asarray(packed["codebook"], np.float32)
    eff = w3.e4m3_floats(scale) * row[:, None]
    assert np.array_equal(w3.group_scales(packed), eff)
    assert np.array_equal(w3.dequantize(packed), levels[q] * np.repeat(eff, 32, axis=1))
    raw = struct.pack("<q", packed["lut"])
    assert np.array_equal(w3.e4m3_floats(np.frombuffer(raw, np.uint8)), levels)
    assert list(struct.pack("<q", w3.lut_of(w3.CODEBOOKS["uniform"]))) == GOLDEN["lut_uniform_bytes"]
    two = struct.pack("<q", w3.lut_of(w3.CODEBOOKS["lloyd2"]))
    assert np.array_equal(w3.e4m3_floats(np.frombuffer(two[:4], np.uint8)), np.asarray(w3.CODEBOOKS["lloyd2"], np.float32))
    assert not any(two[4:])


@pytest.mark.parametrize("codebook", ["uniform", "lloyd"])
def test_nearest_level_quantizer(codebook):
    """tests/unit/test_w3_pack.py:34-54 of the reference on its own seeded matrix."""
    torch.manual_seed(0)
    weight = (torch.randn(256, 384) * 0.05).numpy()
    packed = w3.pack(weight, codebook)
    deq = w3.dequantize(packed)
    assert np.linalg.norm(deq - weight) / np.linalg.norm(weight) < 0.22
    levels = np.asarray(packed["codebook"], np.float32)
    scale = np.repeat(w3.group_scales(packed), 32, axis=1)
    mids = (levels[1:] + levels[:-1]) / 2
    q = w3.codes(packed)
    assert np.array_equal(q, np.searchsorted(mids, weight / scale, side="left"))
    assert q.min() == 0 and q.max() == 7
    assert np.array_equal(deq, levels[q] * scale)


def test_two_bit_variant_and_fitted_scales():
    """tests/unit/test_w3_pack.py:57-76 of the reference."""
    torch.manual_seed(0)
    weight = (torch.randn(256, 384) * 0.05).numpy()
    nearest, fitted = w3.pack(weight, "lloyd2"), w3.pack(weight, "lloyd2", fit_scales=True)
    err = lambda p: float(np.linalg.norm(w3.dequantize(p) - weight) / np.linalg.norm(weight))  # noqa: E731
    for packed in (nearest, fitted):
        assert packed["planes"].shape == (8, 3, 2, 32, 4)
        assert w3.nbytes(packed) == 256 * 384 * 2 // 8 + 256 * 12 + 256 * 4
        q = w3.codes(packed)
        assert q.min() == 0 and q.max() == 3
    assert err(fitted) < 0.36 < err(nearest) < 0.45
    again = w3.pack_codes(w3.codes(fitted), w3.scale_bytes(fitted), fitted["row_scale"], "lloyd2")
    assert np.array_equal(again["planes"], fitted["planes"]) and np.array_equal(again["scales"], fitted["scales"])
    with pytest.raises(ValueError):
        w3.pack_codes(w3.codes(fitted) + 4, np.zeros((256, 12), np.uint8), fitted["row_scale"], "lloyd2")


def test_validation_errors():
    with pytest.raises(ValueError):
        w3.pack(np.zeros((128, 160), np.float32))
    with pytest.raises(ValueError):
        w3.pack(np.zeros((96, 256), np.float32))
    with pytest.raises(ValueError):
        w3.pack(np.zeros((128, 128), np.float32), (-3.5, -2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 3.3))
    with pytest.raises(ValueError):
        w3.pack_codes(np.zeros((128, 128), np.int64), np.zeros((128, 4), np.uint8), np.zeros(128, np.float32), "lloyd")


def test_interleave_rows_moves_whole_tiles():
    """tests/unit/test_mlp_pairs.py:27-34 of the reference: the moved copy equals the packed interleaved matrix."""
    torch.manual_seed(3)
    weight = (torch.randn(512, 256) * 0.03).numpy()
    order = w3.pair_order(512, 64)
    assert order[:64].tolist() == list(range(64)) and order[64:128].tolist() == list(range(256, 320))
    assert sorted(order.tolist()) == list(range(512))
    moved, packed = w3.interleave_rows(w3.pack(weight), 64), w3.pack(weight[order])
    for f in ("planes", "scales", "row_scale"):
        assert np.array_equal(moved[f], packed[f])
