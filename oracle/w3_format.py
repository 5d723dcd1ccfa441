"""Oracle restatement of the W3 weight format (test infrastructure, see oracle/__init__.py).

Follows hibana/kernels/w3.py of the reference:
  CODEBOOKS, GROUP, CHUNK, FP8_MAX      :52-71
  lut_of                                :105-107   8 E4M3 bytes, entry i in byte i, little-endian signed int64
  check_codebook                        :110-118   4 or 8 ascending levels, each exactly an E4M3 value
  pack_codes / _pack_codes_rows         :175-214   codes + E4M3 group scales + row scales -> fragment-order planes
  codes                                 :217-229   the unpack (bit-exact target)
  group_scales                          :232-236   e4m3(byte).float() * row_scale[n]
  dequantize                            :239-242   levels[code] * group_scale, FP32, in this multiplication order
  pack (nearest level)                  :126-172   amax / max|level| scale, row scale, bucketize against midpoints
  interleave_rows                       :94-102    whole 32-row tiles moved in pair_order
  fit_scales_ratio / quantize_groups    hibana/weights/w3_calibration.py:17-37, hibana/kernels/w3_moe.py:113-124 (ratio-grid group scales)

Everything is written from the closed form of the layout (a weight's bit b sits at bit (4j + b + rot(s)) mod 32 of
word bits*nt + b of lane 4g + t, n = 32nb + 8nt + g, k = 128kc + 16s + 4t + j, rot(s) = 16(s//4) + s%4) with explicit
index arithmetic, not by reshapes, so that a transposed axis in the shipped code cannot hide behind the same mistake
here.

Pinned by (tests/test_oracle_w3.py):
  codes / pack_codes   the kernel-addressing statement of the reference's own test (tests/unit/test_w3_pack.py:79-108:
                       word bits*nt+b of a lane, rotate by rot(s), masks 0x1111/0x2222/0x4444), hand-derived bit
                       positions in tests/golden/w3_layout_known_answers.json, round trip codes(pack_codes(q)) == q
  group_scales         scale byte (4nt+grp)*2+i of lane-column t is row 8nt+2t+i (test_w3_pack.py:101-108)
  dequantize           definition levels[codes] * group_scales (test_w3_pack.py:50)
  lut_of               byte order (test_w3_pack.py:52-54)
  pack                 codes == bucketize(w / scale, mids), extremes used, error < 0.22, byte count
                       (test_w3_pack.py:34-54); 2-bit variant and fitted scales (:57-76)
  interleave_rows      interleave_rows(pack(w)) == pack(w[pair_order]) (tests/unit/test_mlp_pairs.py:27-34)
  fit_scales_ratio     with ratios (1.0,) it must reproduce pack's stored scales and codes exactly; per group the fitted
                       loss is never above the ratio-1.0 loss and is the minimum over a brute-force loop on a tiny matrix;
                       the reference's bounds (tests/unit/test_w3_moe_pack.py:35-47: error < 0.25, fitted <= nearest)
  pack(fit_scales=True), fit_scales_ratio, quantize_groups
                       bit for bit against what the reference's own functions returned on five seeded matrices, among
                       them a coarse-grid one whose candidates' errors differ only in the last bits and one with groups
                       built to tie (tests/golden/w3_fit_scales.npz, written by tests/golden/make_fit_fixtures.py). Both
                       pick, per group, the FIRST candidate whose float32 squared error is strictly the least, and the
                       error is summed in the order torch's CPU reduction takes over 32 contiguous floats (sum32 below):
                       with numpy's pairwise order the coarse-grid fixture fails in one group.
"""
from __future__ import annotations

import struct

import numpy as np
import torch

GROUP = 32
CHUNK = 128
FP8_MAX = 448.0
CODEBOOKS = {
    "uniform": (-3.5, -2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 3.5),
    "lloyd": (-3.5, -2.25, -1.25, -0.40625, 0.40625, 1.25, 2.25, 3.5),
    "lloyd2": (-1.5, -0.4375, 0.4375, 1.5),
    "zero8": (-3.5, -2.5, -1.5, -0.625, 0.0, 0.875, 2.0, 3.5),
}
DEFAULT_CODEBOOK = "lloyd"
FIT_SCALES = tuple(0.55 + 0.05 * i for i in range(10))


def e4m3_bytes(values) -> np.ndarray:
    """float -> E4M3 (OCP e4m3fn, round to nearest even) bit patterns, via torch's cast."""
    t = torch.as_tensor(np.asarray(values, dtype=np.float32))
    return t.to(torch.float8_e4m3fn).view(torch.uint8).numpy().copy()


def e4m3_floats(raw) -> np.ndarray:
    """E4M3 bit patterns -> float32."""
    t = torch.as_tensor(np.array(raw, dtype=np.uint8, copy=True))
    return t.view(torch.float8_e4m3fn).float().numpy().copy()


def check_codebook(codebook) -> tuple[float, ...]:
    codebook = DEFAULT_CODEBOOK if codebook is None else codebook
    levels = CODEBOOKS[codebook] if isinstance(codebook, str) else tuple(float(v) for v in codebook)
    if len(levels) not in (4, 8) or list(levels) != sorted(levels):
        raise ValueError("a codebook is eight (or, two-bit, four) ascending levels")
    if e4m3_floats(e4m3_bytes(levels)).tolist() != list(levels):
        raise ValueError("codebook levels must be exactly representable in E4M3")
    return tuple(levels)


def lut_of(codebook) -> int:
    raw = e4m3_bytes(codebook).tolist()
    return struct.unpack("<q", bytes(raw + [0] * (8 - len(raw))))[0]


def _coords(n: int, k: int):
    """Index arrays over the [n, k] grid: plane word coordinates and the bit rotation of every weight."""
    rows = np.arange(n, dtype=np.int64)[:, None]
    cols = np.arange(k, dtype=np.int64)[None, :]
    nb, nt, g = rows // 32, (rows % 32) // 8, rows % 8
    kc, s, t, j = cols // CHUNK, (cols % CHUNK) // 16, (cols % 16) // 4, cols % 4
    lane = 4 * g + t
    rot = 16 * (s // 4) + (s % 4)
    return nb, nt, kc, lane, rot, j


def pack_codes(q, scale_bytes, row_scale, codebook=None):
    """q int [N, K] in 0..levels-1, scale_bytes uint8 [N, K/32] (E4M3 bit patterns), row_scale float32 [N] ->
    dict(planes uint32 [N/32, K/128, bits, 32, 4], scales uint8 [N/32, K/128, 4, 32], row_scale, codebook, lut,
    out_features, in_features)."""
    q = np.asarray(q)
    scale_bytes = np.asarray(scale_bytes, dtype=np.uint8)
    row_scale = np.asarray(row_scale, dtype=np.float32)
    n, k = q.shape
    levels = check_codebook(codebook)
    if n % 128 or k % CHUNK:
        raise ValueError("N and K must be multiples of 128")
    if q.dtype.kind not in "iu" or q.min() < 0 or q.max() >= len(levels):
        raise ValueError(f"codes must be integers between zero and {len(levels) - 1}")
    sc = e4m3_floats(scale_bytes)
    if scale_bytes.shape != (n, k // GROUP) or row_scale.shape != (n,):
        raise ValueError("calibrated scales do not match the weight shape")
    if not np.isfinite(sc).all() or not np.isfinite(row_scale).all() or (row_scale <= 0).any() or (sc < 0).any():
        raise ValueError("calibrated scales must be finite and nonnegative, with positive row scales")
    bits = 2 if len(levels) == 4 else 3
    nb, nt, kc, lane, rot, j = _coords(n, k)
    chunks = k // CHUNK
    planes = np.zeros((n // 32) * chunks * bits * 32 * 4, dtype=np.float64)  # exact below 2**53
    q64 = q.astype(np.int64)
    for b in range(bits):
        word = bits * nt + b
        dest = (((nb * chunks + kc) * bits + word // 4) * 32 + lane) * 4 + word % 4
        pos = (4 * j + b + rot) % 32
        contribution = (((q64 >> b) & 1) << pos).astype(np.float64)
        planes += np.bincount(np.broadcast_to(dest, q.shape).ravel(), weights=contribution.ravel(), minlength=planes.size)
    planes = planes.astype(np.uint64).astype(np.uint32).reshape(n // 32, chunks, bits, 32, 4)
    # scale byte of row n, 32-group G: scales[nb, G // 4, (n % 8) // 2, (4 * nt + G % 4) * 2 + n % 2]
    rows = np.arange(n, dtype=np.int64)[:, None]
    grp = np.arange(k // GROUP, dtype=np.int64)[None, :]
    snb, snt = rows // 32, (rows % 32) // 8
    dest = ((snb * chunks + grp // 4) * 4 + (rows % 8) // 2) * 32 + (4 * snt + grp % 4) * 2 + rows % 2
    scales = np.zeros((n // 32) * chunks * 4 * 32, dtype=np.uint8)
    scales[np.broadcast_to(dest, scale_bytes.shape).ravel()] = scale_bytes.ravel()
    return {"planes": planes, "scales": scales.reshape(n // 32, chunks, 4, 32), "row_scale": row_scale.copy(),
            "codebook": levels, "lut": lut_of(levels), "out_features": n, "in_features": k}


def codes(w3) -> np.ndarray:
    """The codes of a packed matrix, int64 [N, K]."""
    n, k = w3["out_features"], w3["in_features"]
    planes = w3["planes"].astype(np.int64)
    bits = planes.shape[2]
    nb, nt, kc, lane, rot, j = _coords(n, k)
    out = np.zeros((n, k), dtype=np.int64)
    for b in range(bits):
        word = bits * nt + b
        out |= ((planes[nb, kc, word // 4, lane, word % 4] >> ((4 * j + b + rot) % 32)) & 1) << b
    return out


def scale_bytes(w3) -> np.ndarray:
    """The stored E4M3 group scales in matrix order, uint8 [N, K/32]."""
    n, k = w3["out_features"], w3["in_features"]
    rows = np.arange(n, dtype=np.int64)[:, None]
    grp = np.arange(k // GROUP, dtype=np.int64)[None, :]
    nt = (rows % 32) // 8
    return w3["scales"][rows // 32, grp // 4, (rows % 8) // 2, (4 * nt + grp % 4) * 2 + rows % 2]


def group_scales(w3) -> np.ndarray:
    """Effective per-group scales, float32 [N, K/32]: float(e4m3) * row_scale, one FP32 multiplication."""
    return e4m3_floats(scale_bytes(w3)) * w3["row_scale"].astype(np.float32)[:, None]


def dequantize(w3) -> np.ndarray:
    """FP32 [N, K]: levels[code] * effective scale (FP32 product of FP32 operands)."""
    lv = np.asarray(w3["codebook"], dtype=np.float32)
    return lv[codes(w3)] * np.repeat(group_scales(w3), GROUP, axis=1)


def sum32(err: np.ndarray) -> np.ndarray:
    """float32 sum over a last axis of 32 in the order the reference's `.sum(-1)` takes on the CPU: element i goes into
    partial sum i % 8 (ascending i), then the eight partial sums are added in ascending order. Pinned by the fitted-scale
    fixture: near a tie between two candidate scales the order decides which one wins."""
    v = np.asarray(err, dtype=np.float32).reshape(*err.shape[:-1], 4, 8)
    part = ((v[..., 0, :] + v[..., 1, :]) + v[..., 2, :]) + v[..., 3, :]
    total = part[..., 0]
    for j in range(1, 8):
        total = total + part[..., j]
    return total.astype(np.float32)


def _bucketize(x: np.ndarray, mids: np.ndarray) -> np.ndarray:
    """torch.bucketize(x, mids) with right=False: the number of boundaries strictly below x (a value equal to a
    midpoint takes the lower code)."""
    return np.searchsorted(mids, x, side="left")


def pack(weight, codebook=None, fit_scales: bool = False):
    """Nearest-level quantization of float [N, K] (hibana/kernels/w3.py:126-172)."""
    w = np.asarray(weight, dtype=np.float32)
    n, k = w.shape
    if k % CHUNK or n % 128:
        raise ValueError("N and K must be multiples of 128")
    levels = check_codebook(codebook)
    lv = np.asarray(levels, dtype=np.float32)
    mids = ((lv[1:] + lv[:-1]) / np.float32(2)).astype(np.float32)
    g = w.reshape(n, k // GROUP, GROUP)
    amax = np.abs(g).max(axis=-1)
    scale = (amax / np.float32(max(abs(v) for v in levels))).astype(np.float32)
    if fit_scales:
        best = fitted = None
        for m in FIT_SCALES:
            s = (scale * np.float32(m)).astype(np.float32)
            deq = lv[_bucketize(g / np.maximum(s, np.float32(1e-30))[:, :, None], mids)] * s[:, :, None]
            err = sum32(((deq - g) ** 2).astype(np.float32))
            if best is None:
                best, fitted = err, s
            else:
                better = err < best
                best, fitted = np.where(better, err, best), np.where(better, s, fitted)
        scale = fitted
    row_scale = np.maximum(scale.max(axis=-1) / np.float32(FP8_MAX), np.float32(1e-12)).astype(np.float32)
    raw = e4m3_bytes(np.clip(scale / row_scale[:, None], 0, FP8_MAX))
    eff = (e4m3_floats(raw) * row_scale[:, None]).astype(np.float32)
    normalized = g / np.maximum(eff, np.float32(1e-30))[:, :, None]
    q = _bucketize(normalized.reshape(n, k), mids)
    return pack_codes(q, raw, row_scale, levels)


def nbytes(w3) -> int:
    return w3["planes"].size * 4 + w3["scales"].size + w3["row_scale"].size * 4


def pair_order(rows: int, block: int) -> np.ndarray:
    """hibana/weights/modelopt.py:84-86: [gate; up] rows interleaved in blocks: gate block 0, up block 0, gate 1 ..."""
    half = rows // 2
    out = np.empty(rows, dtype=np.int64)
    for b in range(half // block):
        out[2 * b * block:(2 * b + 1) * block] = np.arange(b * block, (b + 1) * block)
        out[(2 * b + 1) * block:(2 * b + 2) * block] = half + np.arange(b * block, (b + 1) * block)
    return out


def interleave_rows(w3, block: int):
    """hibana/kernels/w3.py:94-102: rows moved in pair_order, planes and scales in whole 32-row tiles."""
    tiles = pair_order(w3["out_features"] // 32, block // 32)
    rows = pair_order(w3["out_features"], block)
    out = dict(w3)
    out["planes"] = np.ascontiguousarray(w3["planes"][tiles])
    out["scales"] = np.ascontiguousarray(w3["scales"][tiles])
    out["row_scale"] = np.ascontiguousarray(w3["row_scale"][rows])
    return out


def fit_scales_ratio(weight, codebook=None, ratios=tuple(round(0.5 + 0.025 * i, 3) for i in range(21))):
    """float32 [N, K] -> (scale bytes uint8 [N, K/32], row scales float32 [N]): per 32-group the stored E4M3 scale among
    e4m3(amax / max|level| * ratio / row scale) over the ratio grid with the smallest squared error at nearest-level codes;
    the first of equal losses stays (hibana/weights/w3_calibration.py:17-37, unit importance; the routed experts'
    quantizer, hibana/kernels/w3_moe.py:113-124). With ratios == (1.0,) this is `pack`'s scale rule. The loss is
    summed by sum32, the order that decides near-ties as the reference does (pinned by tests/golden/w3_fit_scales.npz)."""
    w = np.asarray(weight, dtype=np.float32)
    n, k = w.shape
    levels = check_codebook(codebook)
    lv = np.asarray(levels, dtype=np.float32)
    mids = ((lv[1:] + lv[:-1]) / np.float32(2)).astype(np.float32)
    g = w.reshape(n, k // GROUP, GROUP)
    base = (np.abs(g).max(axis=-1) / np.float32(max(abs(v) for v in levels))).astype(np.float32)
    row_scale = np.maximum(base.max(axis=-1) / np.float32(FP8_MAX), np.float32(1e-12)).astype(np.float32)
    best_loss = np.full(base.shape, np.inf, dtype=np.float32)
    best = np.zeros(base.shape, dtype=np.uint8)
    for ratio in ratios:
        raw = e4m3_bytes(np.clip((base * np.float32(ratio)).astype(np.float32) / row_scale[:, None], 0, FP8_MAX))
        eff = (e4m3_floats(raw) * row_scale[:, None]).astype(np.float32)
        q = _bucketize(g / np.maximum(eff, np.float32(1e-30))[:, :, None], mids)
        err = (g - lv[q] * eff[:, :, None]).astype(np.float32)
        loss = sum32(err * err)
        better = loss < best_loss
        best_loss = np.where(better, loss, best_loss)
        best = np.where(better, raw, best)
    return best.astype(np.uint8), row_scale


def quantize_groups(weight, scale_bytes, row_scale, codebook=None):
    """Nearest-level codes int64 [N, K] of float32 [N, K] under given stored scales (hibana/kernels/w3_moe.py:120-124)."""
    w = np.asarray(weight, dtype=np.float32)
    n, k = w.shape
    levels = check_codebook(codebook)
    lv = np.asarray(levels, dtype=np.float32)
    mids = ((lv[1:] + lv[:-1]) / np.float32(2)).astype(np.float32)
    eff = np.maximum((e4m3_floats(np.asarray(scale_bytes, dtype=np.uint8)) * np.asarray(row_scale, dtype=np.float32)[:, None]).astype(np.float32),
                     np.float32(1e-30))
    return _bucketize(w.reshape(n, k // GROUP, GROUP) / eff[:, :, None], mids).reshape(n, k)

