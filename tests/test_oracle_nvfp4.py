"""The oracle's NVFP4 format functions against the reference's known answers (CPU)."""
import json
import os

import numpy as np

from oracle import nvfp4_format as nv
from oracle.w3_format import e4m3_bytes, e4m3_floats

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "nvfp4_known_answers.json")))


def test_e2m1_table_and_nibble_order():
    packed = np.arange(256, dtype=np.uint8).reshape(32, 8)
    scales = np.full((32, 1), 0x38, np.uint8)  # 1.0
    w = nv.unpack_fp4(packed, scales)
    values = GOLDEN["e2m1_values"]
    for byte in range(256):
        lo, hi = byte & 15, byte >> 4
        r, c = divmod(byte, 8)
        for code, got in ((lo, w[r, 2 * c]), (hi, w[r, 2 * c + 1])):
            want = values[code & 7] * (-1 if code & 8 else 1)
            assert got == want and np.signbit(got) == bool(code & 8)


def test_block_scale_applies_per_sixteen():
    g = np.random.default_rng(0)
    packed = g.integers(0, 256, (4, 32), dtype=np.uint8)
    scales = e4m3_bytes(g.uniform(0.01, 400, (4, 4)))
    w = nv.unpack_fp4(packed, scales)
    ones = nv.unpack_fp4(packed, np.full((4, 4), 0x38, np.uint8))
    assert np.array_equal(w, ones * np.repeat(e4m3_floats(scales), 16, axis=1))


def test_rounding_ties_and_signed_zero():
    assert nv.e2m1_round_codes(np.array(GOLDEN["tie_inputs"], np.float32)).tolist() == GOLDEN["tie_codes"]
    assert nv.e2m1_round_codes(np.array([0.0, -0.0], np.float32)).tolist() == GOLDEN["zero_codes"]
    assert nv.e2m1_round_codes(np.array([7.0, 100.0, -9.0], np.float32)).tolist() == [7, 7, 15]


def test_swizzle_offsets_and_reference_spot_checks():
    for r, c, gp, offset in GOLDEN["swizzle_offsets"]:
        rows = (r // 128 + 1) * 128
        s = np.zeros((rows, gp), np.int64)
        s[r, c] = 7
        sw = nv.swizzle_block_scales(s).reshape(-1)
        assert sw[offset] == 7 and np.count_nonzero(sw) == 1
    # tests/unit/test_modelopt_layout.py:6-22 of the reference
    m, k = 256, 8
    scales = np.arange(m * k, dtype=np.float32).reshape(m, k)
    sw = nv.swizzle_block_scales(scales)
    assert sw.shape == (256, 8) and sorted(sw.ravel().tolist()) == sorted(scales.ravel().tolist())
    assert sw[0, 0] == scales[0, 0]
    assert sw.reshape(2, 4, 32, 2, 4)[0, 0, 0, 0, :].tolist() == scales[0, :4].tolist()
    padded = nv.swizzle_block_scales(np.ones((130, 4), np.float32))
    assert padded.shape == (256, 4) and padded.sum() == 130 * 4


def test_unswizzle_inverts_swizzle_also_per_expert():
    g = np.random.default_rng(3)
    s = e4m3_bytes(g.uniform(0.01, 1.01, (2, 256, 16)))
    back = nv.unswizzle_batched(nv.swizzle_batched(s), 256, 16)
    assert np.array_equal(back, s)
    odd = e4m3_bytes(g.uniform(0.01, 1.01, (130, 6)))
    assert np.array_equal(nv.unswizzle_block_scales(nv.swizzle_block_scales(odd), 130, 6), odd)


def test_linear_dequantize_is_unpack_times_global_scale():
    """tests/unit/test_linear_interface.py:35-38 of the reference."""
    g = np.random.default_rng(0)
    packed = g.integers(0, 256, (128, 32), dtype=np.uint8)
    scales = np.full((128, 4), 0x38, np.uint8)
    got = nv.linear_dequantize(packed, nv.swizzle_block_scales(scales), 2.0, 4.0, 128, 64)
    assert np.array_equal(got, nv.unpack_fp4(packed, scales) * np.float32(8.0))
    e = nv.nvfp4_dequant(packed.reshape(2, 64, 32), scales.reshape(2, 64, 4), np.array([0.5, 0.25], np.float32))
    assert np.array_equal(e[1], nv.unpack_fp4(packed[64:], scales[64:]) * np.float32(0.25))
