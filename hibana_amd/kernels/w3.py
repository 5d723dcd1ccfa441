"""Three-bit decode weights on MI355X: the reference's W3 format and op surface (hibana/kernels/w3.py), served by
hand-written gfx950 kernels through the C ABI.

Format (unchanged, it is what checkpoints hold; hibana/kernels/w3.py:75-91 of the reference): per weight a 3-bit
code into an eight-level E4M3 codebook (2-bit with a four-level one), per 32 weights along K an E4M3 scale, per output
row an FP32 multiplier; `planes` / `scales` in the reference's fragment order. At load time `tile()` repacks them into
the 64-row x 128-k block layout the kernels stream (csrc/w3_layout.hpp); the fragment-order tensors can then be
dropped (`release=True`).

Arithmetic: weight-only. Activations stay BF16 (the reference re-quantizes them to E4M3 per 32-group,
hibana/kernels/w3.py:25-28); weights are expanded exactly to BF16 in registers, products accumulate in FP32, the group
scale multiplies each 32-group's FP32 partial sum, the row scale the total.

Every function here that touches packed data runs on the GPU and raises on CPU tensors: there is no fallback path.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, replace

import torch

from hibana_amd import _lib

MAX_ROWS = 128
NARROW_ROWS = 64
GROUP = 32
CHUNK = 128
FP8_MAX = 448.0
CODEBOOKS = {
    "uniform": (-3.5, -2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 3.5),
    "lloyd": (-3.5, -2.25, -1.25, -0.40625, 0.40625, 1.25, 2.25, 3.5),
    "lloyd2": (-1.5, -0.4375, 0.4375, 1.5),
    "zero8": (-3.5, -2.5, -1.5, -0.625, 0.0, 0.875, 2.0, 3.5),
}
FIT_SCALES = tuple(0.55 + 0.05 * i for i in range(10))
DEFAULT_CODEBOOK = "lloyd"

_ENABLED: bool | None = None


def enabled() -> bool:
    """HIBANA_W3_DECODE: serve calls of at most MAX_ROWS rows from the 3-bit copies (hibana/kernels/w3.py:48-51)."""
    if _ENABLED is not None:
        return _ENABLED
    return os.environ.get("HIBANA_W3_DECODE", "0").strip().lower() in ("1", "true", "yes", "on")


def set_enabled(value: bool | None) -> None:
    """Override HIBANA_W3_DECODE for this process (None: read the environment again)."""
    global _ENABLED
    _ENABLED = value


@dataclass
class W3Weight:
    planes: torch.Tensor | None  # [N/32, K/128, bits, 32, 4] uint32, the reference's fragment order (None once released)
    scales: torch.Tensor | None  # [N/32, K/128, 4, 32] uint8 E4M3
    row_scale: torch.Tensor  # [N] float32
    out_features: int
    in_features: int
    codebook: tuple[float, ...]
    lut: int  # the codebook as eight E4M3 bytes, entry i in byte i
    tiled: torch.Tensor | None = None  # uint8, the kernels' block layout (built by tile())
    tile_bits: int = 0  # the bits of `tiled`'s tiles: the codebook's own (a two-bit matrix keeps its density), or 3 when widened

    @property
    def bytes(self) -> int:
        n, k = self.out_features, self.in_features
        return n * k * self.bits // 8 + n * k // GROUP + n * 4

    @property
    def bits(self) -> int:
        return 2 if len(self.codebook) == 4 else 3


def lut_of(codebook: tuple[float, ...]) -> int:
    """The codebook as the kernels take it: level i as an E4M3 byte in byte i of a little-endian signed 64-bit integer,
    a four-level book zero-filled (hibana/kernels/w3.py:105-107)."""
    e4m3 = torch.tensor(codebook, dtype=torch.float32).to(torch.float8_e4m3fn).view(torch.uint8)
    return int.from_bytes(bytes(e4m3.tolist()).ljust(8, b"\0"), "little", signed=True)


def _codebook(codebook) -> tuple[float, ...]:
    """A codebook by name (None: the default) or as a sequence of levels, checked (hibana/kernels/w3.py:110-118)."""
    if codebook is None:
        codebook = DEFAULT_CODEBOOK
    levels = tuple(CODEBOOKS[codebook]) if isinstance(codebook, str) else tuple(map(float, codebook))
    ascending = all(lo <= hi for lo, hi in zip(levels, levels[1:]))
    if len(levels) not in (4, 8) or not ascending:
        raise ValueError("a codebook is eight (or, two-bit, four) ascending levels")
    through_e4m3 = torch.tensor(levels).to(torch.float8_e4m3fn).float()
    if not torch.equal(through_e4m3, torch.tensor(levels)):
        raise ValueError("codebook levels must be exactly representable in E4M3")
    return levels


def tile(w3: W3Weight, release: bool = False, widen: bool = False) -> W3Weight:
    """Build the kernels' block layout from the fragment-order tensors (once). `release` drops the latter. A two-bit
    matrix gets two-bit tiles (2.25 bits a weight, what `w3_linear` streams); `widen`: three-bit tiles whatever the
    codebook (the routed experts' kernels read only those)."""
    want = 3 if widen else w3.bits
    if w3.tiled is not None and w3.tile_bits == 0:
        w3.tile_bits = 3  # a tiled copy handed in as it was loaded: three-bit tiles
    if w3.tiled is None or w3.tile_bits != want:
        if w3.planes is None:
            raise ValueError("W3Weight holds neither planes nor a tiled copy of the tiles asked for")
        _lib.need_gpu(w3.planes, w3.scales)
        n, k = w3.out_features, w3.in_features
        size = _lib.lib().hb_w3_tiled_bytes(n, k, want)
        if size == 0:
            raise ValueError("W3 kernels need N a multiple of 64 and K a multiple of 128")
        tiled = torch.empty(size, dtype=torch.uint8, device=w3.planes.device)
        planes, scales = w3.planes.contiguous(), w3.scales.contiguous()
        _lib.check(_lib.lib().hb_w3_repack(_lib.ptr(planes), _lib.ptr(scales), n, k, w3.bits, want, _lib.ptr(tiled), _lib.stream()), "w3 repack")
        w3.tiled, w3.tile_bits = tiled, want
    if release:
        w3.planes = w3.scales = None
    return w3


def pack_codes(q: torch.Tensor, scale_fp8: torch.Tensor, row_scale: torch.Tensor, codebook=None,
               rows_per_chunk: int = 4096) -> W3Weight:
    """Pack calibrated codes and their exact scales without quantizing again (hibana/kernels/w3.py:198-214)."""
    n, k = q.shape
    if n % 128 or k % CHUNK or rows_per_chunk < 128 or rows_per_chunk % 128:
        raise ValueError("N, K and rows_per_chunk must be multiples of 128")
    levels = _codebook(codebook)
    if q.dtype not in (torch.uint8, torch.int32, torch.int64) or bool(((q < 0) | (q >= len(levels))).any()):
        raise ValueError(f"codes must be integers between zero and {len(levels) - 1}")
    if scale_fp8.shape != (n, k // GROUP) or scale_fp8.dtype != torch.float8_e4m3fn or row_scale.shape != (n,):
        raise ValueError("calibrated scales do not match the weight shape")
    sf = scale_fp8.float()
    if not bool(torch.isfinite(sf).all()) or not bool(torch.isfinite(row_scale).all()) or bool((row_scale <= 0).any()) or bool((sf < 0).any()):
        raise ValueError("calibrated scales must be finite and nonnegative, with positive row scales")
    _lib.need_gpu(q, scale_fp8, row_scale)
    bits = 2 if len(levels) == 4 else 3
    dev = q.device
    codes8 = q.to(torch.uint8).contiguous()
    raw = scale_fp8.contiguous().view(torch.uint8)
    planes = torch.empty((n // 32, k // CHUNK, bits, 32, 4), dtype=torch.uint32, device=dev)
    scales = torch.empty((n // 32, k // CHUNK, 4, 32), dtype=torch.uint8, device=dev)
    _lib.check(_lib.lib().hb_w3_pack_codes(_lib.ptr(codes8), _lib.ptr(raw), n, k, bits, _lib.ptr(planes), _lib.ptr(scales), _lib.stream()),
               "w3 pack_codes")
    return W3Weight(planes, scales, row_scale.float().contiguous(), n, k, levels, lut_of(levels))


def sum32(values: torch.Tensor) -> torch.Tensor:
    """FP32 sum over a last axis of 32 in a FIXED order, the one the reference's CPU `.sum(-1)` takes: element i into
    partial sum i % 8 (ascending i), then the eight partial sums in ascending order. Which candidate scale a group gets
    is decided by strict comparisons of such sums, so the order is part of the format's definition here, not left to
    the device's reduction."""
    lanes = values.unflatten(-1, (4, 8))
    part = ((lanes[..., 0, :] + lanes[..., 1, :]) + lanes[..., 2, :]) + lanes[..., 3, :]
    total = part[..., 0]
    for j in range(1, 8):
        total = total + part[..., j]
    return total


class _Levels:
    """A codebook on a device: its levels, the midpoints that separate them, its largest magnitude."""

    def __init__(self, levels: tuple[float, ...], device):
        self.values = torch.tensor(levels, dtype=torch.float32, device=device)
        self.mids = (self.values[1:] + self.values[:-1]) / 2
        # divisors as tensors: torch divides by a Python scalar on the GPU through its reciprocal, which is off by an ulp
        self.top = torch.tensor(max(abs(v) for v in levels), device=device)
        self.fp8_max = torch.tensor(FP8_MAX, device=device)

    def nearest(self, groups: torch.Tensor, effective: torch.Tensor) -> torch.Tensor:
        """Codes of [N, G, 32] weights under effective group scales [N, G]: a value on a midpoint takes the lower level."""
        return torch.bucketize(groups / effective.clamp_min(1e-30).unsqueeze(-1), self.mids)

    def loss(self, groups: torch.Tensor, effective: torch.Tensor) -> torch.Tensor:
        """Squared error [N, G] of the nearest-level copy under `effective`."""
        copy = self.values[self.nearest(groups, effective)] * effective.unsqueeze(-1)
        return sum32((copy - groups).square())

    def row_scale(self, group_scale: torch.Tensor) -> torch.Tensor:
        return (group_scale.amax(dim=-1) / self.fp8_max).clamp_min(1e-12)

    @staticmethod
    def stored(group_scale: torch.Tensor, row: torch.Tensor) -> torch.Tensor:
        return (group_scale / row.unsqueeze(1)).clamp(0, FP8_MAX).to(torch.float8_e4m3fn)


def first_best(candidates):
    """Of (loss [N, G], payload [N, G]) pairs in order, per group the payload of the FIRST pair whose loss is strictly
    below every earlier one's (the rule of both fitted-scale searches of the reference, hibana/kernels/w3.py:154-164 and
    hibana/weights/w3_calibration.py:28-36)."""
    best_loss = best = None
    for loss, payload in candidates:
        if best is None:
            best_loss, best = loss, payload
            continue
        wins = loss < best_loss
        best_loss = torch.where(wins, loss, best_loss)
        best = torch.where(wins, payload, best)
    return best


def quantize_rows(rows: torch.Tensor, book: _Levels, fit_scales: bool):
    """float [n, K] -> (codes uint8 [n, K], stored scales float8_e4m3fn [n, K/32], row scales [n]) by the nearest-level
    rule of hibana/kernels/w3.py:146-172: group scale = largest magnitude / largest level - or, `fit_scales`, the
    multiple of it among FIT_SCALES with the least squared error -, row scale = largest group scale / 448, the group
    scale stored as the E4M3 of their ratio, codes nearest under the scale as stored."""
    groups = rows.float().unflatten(1, (rows.shape[1] // GROUP, GROUP))
    scale = groups.abs().amax(dim=-1) / book.top
    if fit_scales:
        scale = first_best((book.loss(groups, cand), cand) for cand in (scale * mult for mult in FIT_SCALES))
    row = book.row_scale(scale)
    stored = book.stored(scale, row)
    codes = book.nearest(groups, stored.float() * row.unsqueeze(1)).flatten(1)
    return codes.to(torch.uint8), stored, row


def pack(weight: torch.Tensor, codebook=None, rows_per_chunk: int = 4096, fit_scales: bool = False) -> W3Weight:
    """Nearest-level quantization of a [N, K] float matrix (N, K multiples of 128) into the fragment order,
    hibana/kernels/w3.py:126-143; `rows_per_chunk` rows at a time (the temporaries of the lm_head would not fit
    otherwise). The arithmetic is quantize_rows'."""
    n, k = weight.shape
    if k % CHUNK or n % 128:
        raise ValueError("N and K must be multiples of 128")
    levels = _codebook(codebook)
    book = _Levels(levels, weight.device)
    pieces = [quantize_rows(weight[r0:r0 + rows_per_chunk], book, fit_scales) for r0 in range(0, n, rows_per_chunk)]
    q, stored, row = (torch.cat(column) for column in zip(*pieces))
    return pack_codes(q, stored, row, levels)


def _unpack(w3: W3Weight, want_codes: bool, want_scales: bool):
    n, k = w3.out_features, w3.in_features
    src = w3.tiled if w3.tiled is not None else w3.planes
    _lib.need_gpu(src)
    dev = src.device
    codes8 = torch.empty((n, k), dtype=torch.uint8, device=dev) if want_codes else None
    raw = torch.empty((n, k // GROUP), dtype=torch.uint8, device=dev) if want_scales else None
    if w3.tiled is not None:
        _lib.check(_lib.lib().hb_w3_unpack(_lib.ptr(w3.tiled), n, k, w3.tile_bits or 3, _lib.ptr(codes8), _lib.ptr(raw), _lib.stream()), "w3 unpack")
    else:
        planes, scales = w3.planes.contiguous(), w3.scales.contiguous()
        _lib.check(_lib.lib().hb_w3_unpack_planes(_lib.ptr(planes), _lib.ptr(scales), n, k, w3.bits,
                                                  _lib.ptr(codes8), _lib.ptr(raw), _lib.stream()), "w3 unpack")
    return codes8, raw


def codes(w3: W3Weight) -> torch.Tensor:
    """The codes of a packed matrix, [N, K] int64 (hibana/kernels/w3.py:217-229)."""
    return _unpack(w3, True, False)[0].long()


def scale_bytes(w3: W3Weight) -> torch.Tensor:
    """The stored E4M3 group scales in matrix order, float8_e4m3fn [N, K/32]."""
    return _unpack(w3, False, True)[1].view(torch.float8_e4m3fn)


def group_scales(w3: W3Weight) -> torch.Tensor:
    """Effective per-group scales, [N, K/32] float32 (hibana/kernels/w3.py:232-236)."""
    return scale_bytes(w3).float() * w3.row_scale[:, None]


def dequantize(w3: W3Weight) -> torch.Tensor:
    """FP32 [N, K]: level[code] * (scale * row_scale), the reference's bits (hibana/kernels/w3.py:239-242)."""
    tile(w3)
    n, k = w3.out_features, w3.in_features
    out = torch.empty((n, k), dtype=torch.float32, device=w3.tiled.device)
    _lib.check(_lib.lib().hb_w3_dequant(_lib.ptr(w3.tiled), _lib.ptr(w3.row_scale), w3.lut, n, k, w3.tile_bits, _lib.ptr(out), _lib.stream()), "w3 dequantize")
    return out


def pair_order(rows: int, block: int) -> torch.Tensor:
    """Row order that interleaves [gate; up] in blocks of `block` rows: gate block 0, up block 0, gate block 1, ...
    (hibana/weights/modelopt.py:84-86)."""
    half = rows // 2
    gate = torch.arange(half).reshape(half // block, block)
    return torch.cat((gate, gate + half), dim=1).reshape(-1)


def interleave_rows(weight: W3Weight, block: int) -> W3Weight:
    """`weight`'s rows in pair_order (an MLP's gate|up interleaved in blocks of `block`, a multiple of 32): dim 0 of
    planes and scales counts 32-row tiles, so they move as `block / 32` tiles at a time and the row scales row by row
    (hibana/kernels/w3.py:94-102). The tiled copy, if any, is rebuilt on demand."""
    if weight.planes is None:
        raise ValueError("interleave_rows needs the fragment-order tensors (they were released)")
    if block % 32:
        raise ValueError("rows move in whole 32-row tiles")
    tile_order = pair_order(weight.out_features // 32, block // 32).to(weight.planes.device)
    row_order = pair_order(weight.out_features, block).to(weight.row_scale.device)
    moved = weight.planes.view(torch.int32).index_select(0, tile_order).view(torch.uint32)  # no uint32 gather on the device
    return replace(weight, planes=moved.contiguous(), scales=weight.scales.index_select(0, tile_order).contiguous(),
                   row_scale=weight.row_scale.index_select(0, row_order).contiguous(), tiled=None)


def _quant_check(x: torch.Tensor, multiple: int, name: str) -> None:
    if x.dim() != 2 or x.dtype != torch.bfloat16 or x.shape[1] % multiple:
        raise ValueError(f"{name}: BF16 [M, K] with K a multiple of {multiple}")
    _lib.need_gpu(x)


def quant_rows(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-row E4M3 quantization of a BF16 [M, K] matrix: (x_q float8_e4m3fn [M, K], scale float32 [M]), scale =
    max(amax of the row / 448, 1e-12), x_q = e4m3(x / scale) (hibana/kernels/w3.py:326-330; exact divisions, as
    `quant_groups`). The reference keeps it for comparison (one scale a row loses the small channels next to an outlier)
    and serves `quant_groups`; `w3_linear` takes either."""
    _quant_check(x, 8, "quant_rows")
    m, k = x.shape
    q = torch.empty((m, k), dtype=torch.float8_e4m3fn, device=x.device)
    scale = torch.empty((m,), dtype=torch.float32, device=x.device)
    if m:
        xc = x.contiguous()
        _lib.check(_lib.lib().hb_w3_quant_rows(_lib.ptr(xc), m, k, _lib.ptr(q), _lib.ptr(scale), _lib.stream()), "quant_rows")
    return q, scale


def quant_groups(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-(row, 32-group) E4M3 quantization of a BF16 [M, K] matrix: (x_q float8_e4m3fn [M, K], scale float32
    [M, K/32]), scale = max(amax / 448, 1e-12), x_q = e4m3(x / scale) (hibana/kernels/w3.py:333-337, with the exact
    divisions of its torch statement, hibana/kernels/w3_moe.py:187-190)."""
    _quant_check(x, GROUP, "quant_groups")
    m, k = x.shape
    q = torch.empty((m, k), dtype=torch.float8_e4m3fn, device=x.device)
    scale = torch.empty((m, k // GROUP), dtype=torch.float32, device=x.device)
    if m:
        xc = x.contiguous()
        _lib.check(_lib.lib().hb_w3_quant_groups(_lib.ptr(xc), m, k, _lib.ptr(q), _lib.ptr(scale), _lib.stream()), "quant_groups")
    return q, scale


def w3_linear(x: torch.Tensor, w3: W3Weight, x_scale: torch.Tensor | None = None, splits: int | None = None) -> torch.Tensor:
    """y = x @ W^T for x [M, K], M <= MAX_ROWS; returns BF16 [M, N] (hibana/kernels/w3.py:340-365). BF16 x: the
    weight-only product (x is NOT re-quantized, unlike the reference). E4M3 x with its scale (one per tensor, per row or
    per (row, 32-group), as `quant_groups` makes them): the reference kernel's arithmetic on those codes.
    `splits` is accepted for signature compatibility; the K split is chosen by the library."""
    m, k = x.shape
    if m > MAX_ROWS or k != w3.in_features:
        raise ValueError("w3_linear: unsupported call")
    if x.dtype == torch.float8_e4m3fn:
        if x_scale is None:
            raise ValueError("FP8 activations need their scale")
    elif x.dtype != torch.bfloat16:
        raise ValueError("w3_linear: BF16 activations, or E4M3 ones with their scale")
    _lib.need_gpu(x)
    tile(w3)
    x = x.contiguous()
    y = torch.empty((m, w3.out_features), dtype=torch.bfloat16, device=x.device)
    if m == 0:
        return y
    if x.dtype == torch.float8_e4m3fn:
        groups = k // GROUP
        if x_scale.numel() not in (1, m, m * groups):
            raise ValueError("w3_linear: x_scale must have 1, M or M * K/32 elements")
        scale = x_scale.float().reshape(-1, groups if x_scale.numel() == m * groups else 1).expand(m, groups).contiguous()
        _lib.check(_lib.lib().hb_w3_gemm_e4m3(_lib.ptr(x), _lib.ptr(scale), m, _lib.ptr(w3.tiled), _lib.ptr(w3.row_scale), w3.lut,
                                              w3.out_features, k, w3.tile_bits, _lib.ptr(y), _lib.stream()), "w3_linear")
        return y
    _lib.check(_lib.lib().hb_w3_gemm(_lib.ptr(x), m, _lib.ptr(w3.tiled), _lib.ptr(w3.row_scale), w3.lut, w3.out_features, k, w3.tile_bits,
                                     _lib.ptr(y), _lib.stream()), "w3_linear")
    return y


def _missing(linears):
    return [(name, lin) for name, lin in linears if getattr(lin, "w3", None) is None]


def attach(linears, codebook=DEFAULT_CODEBOOK) -> tuple[int, int]:
    """Nearest-level 3-bit copies for (name, linear) pairs that have none; returns (matrices packed, bytes)
    (hibana/kernels/w3.py:370-378)."""
    todo = _missing(linears)
    for _, lin in todo:
        lin.w3 = tile(pack(lin.dequantize(), codebook))
    return len(todo), sum(lin.w3.bytes for _, lin in todo)


def attach_model(model, log=print, codebook=DEFAULT_CODEBOOK, checkpoint=None, revision: str | None = None) -> dict:
    """3-bit decode copies for every projection `model.linears()` lists (hibana/kernels/w3.py:381-404): calibrated ones
    from a W3 checkpoint when one is given - `checkpoint` a directory or a `CalibratedWeights` (default: the directory
    HIBANA_W3_CHECKPOINT names, for the target at `revision`), which must hold exactly the model's projections -,
    nearest-level copies otherwise. Each copy is tiled for the kernels as it is attached."""
    from hibana_amd.weights.w3_checkpoint import REPLICATED, CalibratedWeights
    source = checkpoint if checkpoint is not None else (os.environ.get("HIBANA_W3_CHECKPOINT") or None)
    if source is not None and not isinstance(source, CalibratedWeights):
        source = CalibratedWeights(source, revision if revision is not None else getattr(model, "revision", None))
    linears = list(model.linears())
    if source is not None and set(source.weights) != {name for name, _ in linears}:
        raise ValueError("calibrated W3 checkpoint must contain every target layer projection")
    todo = _missing(linears)
    if source is None:
        count, total = attach(todo, codebook)
    else:
        wanted = ((name, lin, getattr(lin, "shard", REPLICATED)) for name, lin in todo)
        for (_, lin), copy in zip(todo, source.load_many(wanted)):
            lin.w3 = tile(copy)
        count, total = len(todo), sum(lin.w3.bytes for _, lin in todo)
    torch.cuda.synchronize()
    model.w3_identity = source.identity if source is not None else f"nearest:{codebook}"
    log(f"  w3: packed {count} matrices, {total / 2**30:.2f} GiB of 3-bit decode weights (codebook {codebook})")
    return {"matrices": count, "bytes": total}


def attach_draft(draft, log=print, codebook=DEFAULT_CODEBOOK) -> dict:
    """3-bit copies of a parallel draft model's FP8 matrices, `draft.fp8_weights` name -> linear (hibana/kernels/w3.py:407-412)."""
    count, total = attach(list(draft.fp8_weights.items()), codebook)
    torch.cuda.synchronize()
    log(f"  w3: packed {count} draft matrices, {total / 2**30:.2f} GiB")
    return {"matrices": count, "bytes": total}
