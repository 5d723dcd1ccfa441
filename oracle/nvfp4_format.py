"""Oracle restatement of the NVFP4 weight format (test infrastructure, see oracle/__init__.py).

Follows the reference:
  unpack_fp4                 hibana/weights/modelopt.py:150-156   low nibble first, magnitudes [0,.5,1,1.5,2,3,4,6],
                                                                  bit 3 = sign, times the E4M3 block-16 scale (FP32)
  swizzle_block_scales       hibana/weights/modelopt.py:130-139   CUTLASS 128x4 interleave, zero padded
  unswizzle_block_scales     hibana/weights/modelopt.py:142-147
  swizzle_batched            hibana/model/flashnext/moe.py:22-29  the same per expert, viewed as int32
  unswizzle_batched          hibana/kernels/w3_moe.py:97-102
  nvfp4_dequant              hibana/kernels/w3_moe.py:105-110     experts, times a per-expert FP32 global scale
  linear_dequantize          hibana/weights/modelopt.py:73-77     Nvfp4Linear.dequantize: unpack * (alpha * input_scale_inv)
  nvfp4_unscaled_bf16        tests/nemotron_reference.py:180-187  e2m1 * e4m3 without the global scale, exact in BF16

The swizzle is written from the byte-offset form (hibana/kernels/nvfp4_quant.py:10-12):
  offset(r, c) = (r // 128) * 128 * Gp + (c // 4) * 512 + (r % 32) * 16 + ((r // 32) % 4) * 4 + c % 4
not from the reshape/permute chain.

Pinned by (tests/test_oracle_nvfp4.py): the 16-entry E2M1 table (textbook), the spot checks of
tests/unit/test_modelopt_layout.py:6-22 (permutation with padding, first element fixed, row 1 moves to position 32
of the block, padding to 128 rows sums), the inverse property of tests/unit/test_w3_moe_pack.py:49-53, and
Nvfp4Linear.dequantize == unpack_fp4 * (alpha * input_scale_inv) (tests/unit/test_linear_interface.py:35-38).
"""
from __future__ import annotations

import numpy as np

from .w3_format import e4m3_floats

E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)


def fp4_codes(packed: np.ndarray) -> np.ndarray:
    """uint8 [R, K/2] -> 4-bit codes [R, K], element 2i in the low nibble of byte i."""
    packed = np.asarray(packed, dtype=np.uint8)
    out = np.empty((packed.shape[0], packed.shape[1] * 2), dtype=np.int64)
    out[:, 0::2] = packed & 15
    out[:, 1::2] = packed >> 4
    return out


def unpack_fp4(packed: np.ndarray, scale_bytes: np.ndarray) -> np.ndarray:
    """uint8 [R, K/2] + E4M3 bit patterns [R, K/16] -> float32 [R, K] (value * sign * block scale)."""
    packed = np.asarray(packed, dtype=np.uint8)
    scale_bytes = np.asarray(scale_bytes, dtype=np.uint8)
    if packed.ndim != 2 or packed.shape[1] % 8 or scale_bytes.shape != (packed.shape[0], packed.shape[1] // 8):
        raise ValueError("expected packed rows and one scale per sixteen values")
    c = fp4_codes(packed)
    sign = np.where((c & 8) != 0, np.float32(-1), np.float32(1))
    return (E2M1[c & 7] * sign * np.repeat(e4m3_floats(scale_bytes), 16, axis=1)).astype(np.float32)


def _swizzled_offsets(rows: int, groups: int):
    rp, gp = (rows + 127) // 128 * 128, (groups + 3) // 4 * 4
    r = np.arange(rows, dtype=np.int64)[:, None]
    c = np.arange(groups, dtype=np.int64)[None, :]
    off = (r // 128) * 128 * gp + (c // 4) * 512 + (r % 32) * 16 + ((r // 32) % 4) * 4 + c % 4
    return rp, gp, off


def swizzle_block_scales(scales: np.ndarray) -> np.ndarray:
    """[R, G] -> [R_pad128, G_pad4] in the 128x4 interleave, padding zero. Any dtype (bytes or floats)."""
    scales = np.asarray(scales)
    rp, gp, off = _swizzled_offsets(*scales.shape)
    out = np.zeros(rp * gp, dtype=scales.dtype)
    out[off.ravel()] = scales.ravel()
    return out.reshape(rp, gp)


def unswizzle_block_scales(swizzled: np.ndarray, rows: int, groups: int) -> np.ndarray:
    rp, gp, off = _swizzled_offsets(rows, groups)
    flat = np.asarray(swizzled).reshape(-1)
    if flat.size != rp * gp:
        raise ValueError("scale extent does not match padded matrix")
    return flat[off]


def swizzle_batched(scales: np.ndarray) -> np.ndarray:
    """uint8 [E, R, G] -> int32 [E, R_pad, G_pad/4]."""
    parts = [swizzle_block_scales(s) for s in np.asarray(scales, dtype=np.uint8)]
    return np.stack(parts).view(np.int32)


def unswizzle_batched(swizzled: np.ndarray, rows: int, groups: int) -> np.ndarray:
    """int32/uint8 [E, ...] -> uint8 [E, rows, groups]."""
    e = swizzled.shape[0]
    flat = np.ascontiguousarray(swizzled).view(np.uint8).reshape(e, -1)
    return np.stack([unswizzle_block_scales(flat[i], rows, groups) for i in range(e)])


def nvfp4_dequant(packed: np.ndarray, scale_bytes: np.ndarray, scale2: np.ndarray) -> np.ndarray:
    """uint8 [E, R, K/2], E4M3 bytes [E, R, K/16], float32 [E] -> float32 [E, R, K]."""
    e, r, _ = packed.shape
    w = unpack_fp4(packed.reshape(e * r, -1), scale_bytes.reshape(e * r, -1)).reshape(e, r, -1)
    return (w * np.asarray(scale2, dtype=np.float32).reshape(e, 1, 1)).astype(np.float32)


def linear_dequantize(weight, scale_swizzled, alpha, input_scale_inv, out_features, in_features) -> np.ndarray:
    scales = unswizzle_block_scales(np.asarray(scale_swizzled, dtype=np.uint8).reshape(-1), out_features, in_features // 16)
    return (unpack_fp4(weight, scales) * (np.float32(alpha) * np.float32(input_scale_inv))).astype(np.float32)


def e2m1_round_codes(x: np.ndarray) -> np.ndarray:
    """float32 -> E2M1 code (round to nearest, ties to even mantissa, saturating at 6, sign bit 8 kept for -0).
    Pinned by the explicit tie codes of tests/gpu/test_nvfp4_rounding.py:33-37 of the reference:
    [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0] -> [0, 2, 2, 4, 4, 6, 6] and (0.0, -0.0) -> (0, 8)."""
    x = np.asarray(x, dtype=np.float32)
    a = np.abs(x)
    mids = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)
    code = np.searchsorted(mids, a, side="left")  # strictly above the midpoint moves up
    tie = np.zeros_like(code, dtype=bool)
    for i, m in enumerate(mids):  # a tie goes to the even code (even mantissa bit)
        at = a == m
        code = np.where(at, i if i % 2 == 0 else i + 1, code)
        tie |= at
    code = np.minimum(code, 7)
    return (code | np.where(np.signbit(x), 8, 0)).astype(np.int64)
