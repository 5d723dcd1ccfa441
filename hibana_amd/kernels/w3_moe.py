"""Three-bit routed experts on MI355X behind the reference's `w3_moe` surface (hibana/kernels/w3_moe.py).

A layer's experts are stacked W3 matrices: fc1 [E, N1, H] (gated: N1 = 2 I with rows in `fc1_order`, every 32-row
block sixteen up rows then their sixteen gate rows; ReLU^2: N1 = I) and fc2 [E, H, I]. `w3_moe` is the routed sum in
selection order; `moe_layer` adds the shared expert and the sigmoid-gated combine of the reference's MoeLayer
(hibana/model/flashnext/moe.py:177-192) in the same chain of launches.

The call is: one planning workgroup (expert-sorted pair list, slots of up to 16 rows), the fc1 stream (epilogue
h = bf16(silu(bf16 gate) * bf16 up) or bf16(relu(bf16 up)^2)), the fc2 stream (FP32 per pair), the combine. Weight-only:
x and h stay BF16. Deterministic (no floating-point atomics), graph-capturable, any number of rows.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import torch

from hibana_amd import _lib
from hibana_amd.kernels import w3

EXPERTS = 512
RATIOS = tuple(round(0.5 + 0.025 * i, 3) for i in range(21))  # group scale = amax / max level * ratio, 0.5 .. 1.0
ORDER_IN_KERNEL = 640  # kept for the reference's callers; the planner here orders any number of pairs on the device
WIDE_ROWS = 1024


@dataclass
class W3Experts:
    planes13: torch.Tensor | None  # [E, N1/32, H/128, 3, 32, 4] uint32, fc1 rows in fc1_order
    scales13: torch.Tensor | None  # [E, N1/32, H/128, 4, 32] uint8 E4M3
    row13: torch.Tensor            # [E, N1] float32
    planes2: torch.Tensor | None   # [E, H/32, I/128, 3, 32, 4]
    scales2: torch.Tensor | None
    row2: torch.Tensor             # [E, H]
    codebook: tuple[float, ...]
    lut: int
    fc2_codebook: tuple[float, ...]
    fc2_lut: int
    base: int = 0
    tiled13: torch.Tensor | None = None  # the kernels' block layout of the stacked fc1 / fc2 (built by tile())
    tiled2: torch.Tensor | None = None
    shape13: tuple[int, int] | None = None  # (N1, H), (H_out, I): kept when the fragment-order tensors are released
    shape2: tuple[int, int] | None = None

    def __post_init__(self):
        if self.shape13 is None:
            self.shape13 = (self.planes13.shape[1] * 32, self.planes13.shape[2] * w3.CHUNK)
            self.shape2 = (self.planes2.shape[1] * 32, self.planes2.shape[2] * w3.CHUNK)

    @property
    def experts(self) -> int:
        return self.row13.shape[0]

    @property
    def bytes(self) -> int:
        (n1, h), (h2, i) = self.shape13, self.shape2
        return self.experts * (n1 * h * 3 // 8 + n1 * h // 32 + n1 * 4 + h2 * i * 3 // 8 + h2 * i // 32 + h2 * 4)

    def _side(self, fc1: bool):
        """(planes, scales, row scales, (rows, k), codebook, lut, tiled) of the fc1 or the fc2 stack."""
        if fc1:
            return self.planes13, self.scales13, self.row13, self.shape13, self.codebook, self.lut, self.tiled13
        return self.planes2, self.scales2, self.row2, self.shape2, self.fc2_codebook, self.fc2_lut, self.tiled2

    def matrix(self, e: int, fc1: bool) -> w3.W3Weight:
        """Expert e's fc1 (rows in fc1_order) or fc2 as a W3Weight (views, no copy)."""
        planes, scales, rows, (n, k), book, lut, tiled = self._side(fc1)
        pick = lambda t: None if t is None else t[e]  # noqa: E731
        return w3.W3Weight(pick(planes), pick(scales), rows[e], n, k, book, lut,
                           tiled=None if tiled is None else tiled.view(self.experts, -1)[e])

    def stacked(self, fc1: bool) -> w3.W3Weight:
        """All experts' fc1 or fc2 as one W3Weight of E * N rows (the checkpoint entry): the expert dim folds into the
        32-row tile dim."""
        planes, scales, rows, (n, k), book, lut, tiled = self._side(fc1)
        fold = lambda t: None if t is None else t.flatten(0, 1)  # noqa: E731
        return w3.W3Weight(fold(planes), fold(scales), rows.flatten(), self.experts * n, k, book, lut, tiled=tiled)

    @classmethod
    def from_stacked(cls, fc1: w3.W3Weight, fc2: w3.W3Weight, experts: int, base: int = 0) -> "W3Experts":
        """The inverse of `stacked`: two matrices of `experts` stacked experts each."""
        fields = []
        for m in (fc1, fc2):
            if m.out_features % experts:
                raise ValueError("a stack's rows must divide among its experts")
            fields += [m.planes.unflatten(0, (experts, -1)), m.scales.unflatten(0, (experts, -1)), m.row_scale.unflatten(0, (experts, -1))]
        return cls(*fields, fc1.codebook, fc1.lut, fc2.codebook, fc2.lut, base)


def gated(experts: W3Experts) -> bool:
    """Gated-SiLU experts (fc1 = [up; gate], 2 I rows) or ReLU^2 ones (fc1 = up, I rows)."""
    return experts.shape13[0] == 2 * experts.shape2[1]


def fc1_order(inter: int, device=None) -> torch.Tensor:
    """Row permutation of w13 = [up; gate] (2 * inter rows): block b of 32 rows is up 16b..16b+15, then gate
    16b..16b+15 (hibana/kernels/w3_moe.py:88-92)."""
    cols = torch.arange(inter, device=device).unflatten(0, (inter // 16, 16))
    return torch.stack((cols, cols + inter), dim=1).reshape(-1)


def tile(experts: W3Experts, release: bool = False) -> W3Experts:
    """Build the kernels' block layout of both stacks (once); `release` drops the fragment-order tensors."""
    for fc1 in (True, False):
        if (experts.tiled13 if fc1 else experts.tiled2) is None:
            stacked = w3.tile(experts.stacked(fc1), widen=True)  # the experts' kernels read three-bit tiles
            if fc1:
                experts.tiled13 = stacked.tiled
            else:
                experts.tiled2 = stacked.tiled
    if release:
        experts.planes13 = experts.scales13 = experts.planes2 = experts.scales2 = None
    return experts


def _struct(experts: W3Experts) -> _lib.HbW3Experts:
    tile(experts)
    (n1, h), (h2, i) = experts.shape13, experts.shape2
    return _lib.HbW3Experts(_lib.ptr(experts.tiled13), _lib.ptr(experts.row13), _lib.ptr(experts.tiled2), _lib.ptr(experts.row2),
                            experts.lut, experts.fc2_lut, experts.experts, experts.base, h, i, h2, int(gated(experts)))


def _check_call(experts: W3Experts, x, ids, weights):
    if x.dtype != torch.bfloat16 or x.ndim != 2 or x.shape[1] != experts.shape13[1]:
        raise ValueError("w3_moe: x must be BF16 [M, hidden]")
    if ids.ndim != 2 or ids.shape[0] != x.shape[0] or weights.shape != ids.shape:
        raise ValueError("w3_moe: ids and weights must be [M, k]")
    _lib.need_gpu(x, ids, weights)


MOE_E4M3 = 16  # hb_w3_moe mode flag: activations through the reference's E4M3 rounding


def w3_moe(experts: W3Experts, x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, pairs: bool = False,
           pairs_bf16: bool = False, e4m3: bool = False) -> torch.Tensor:
    """Routed experts for x [M, H] BF16 with the router's ids [M, k] and weights [M, k] -> BF16 [M, H_out], the
    weighted sum in selection order (no shared expert). An id outside this object's range base .. base + E - 1 (another
    rank's expert, or the "no expert" id 512) adds nothing. With `pairs`, the FP32 (`pairs_bf16`: BF16) output of each
    (row, k) pair [M * k, H_out], unsummed; rows of skipped pairs are unspecified
    (hibana/kernels/w3_moe.py:158-179). `e4m3`: x and h are rounded to E4M3 per (row, 32-group) before their products, as
    the reference kernel does (its torch statement: hibana/kernels/w3_moe.py:193-214); default: weight-only."""
    _check_call(experts, x, ids, weights)
    m, k = ids.shape
    h_out = experts.shape2[0]
    mode = 2 if pairs and pairs_bf16 else int(pairs)
    shape = (m * k, h_out) if pairs else (m, h_out)
    out = torch.empty(shape, dtype=torch.float32 if mode == 1 else torch.bfloat16, device=x.device)
    if m == 0:
        return out
    st = _struct(experts)
    need = _lib.lib().hb_w3_moe_workspace_bytes(m, k, C.byref(st), 0)
    ws = _lib.workspace(x.device, need)
    ids32 = ids.to(torch.int32).contiguous()
    wt = weights.float().contiguous()
    mode |= MOE_E4M3 if e4m3 else 0
    xc = x.contiguous()  # converted operands keep a name until the launch is enqueued
    _lib.check(_lib.lib().hb_w3_moe(C.byref(st), _lib.ptr(xc), _lib.ptr(ids32), _lib.ptr(wt), m, k, mode, _lib.ptr(out),
                                    _lib.ptr(ws), need, _lib.stream()), "w3_moe")
    return out


def moe_layer(experts: W3Experts, x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, shared: W3Experts | None = None,
              gate_vec: torch.Tensor | None = None, e4m3: bool = False) -> torch.Tensor:
    """The MoE layer on 3-bit weights in one chain of launches: routed sum + the shared expert (`shared`: a one-expert
    W3Experts of the same geometry) combined as bf16(bf16(routed) + g * bf16(shared)), g = sigmoid(x . gate_vec) or 1
    (hibana/model/flashnext/moe.py:177-192). `e4m3`: x and h of every expert are rounded to E4M3 per (row, 32-group)
    before their products, as in `w3_moe`."""
    _check_call(experts, x, ids, weights)
    m, k = ids.shape
    out = torch.empty((m, experts.shape2[0]), dtype=torch.bfloat16, device=x.device)
    if m == 0:
        return out
    st = _struct(experts)
    sh = _struct(shared) if shared is not None else None
    need = _lib.lib().hb_w3_moe_workspace_bytes(m, k, C.byref(st), int(shared is not None))
    ws = _lib.workspace(x.device, need)
    ids32 = ids.to(torch.int32).contiguous()
    wt = weights.float().contiguous()
    gv = None if gate_vec is None else gate_vec.float().contiguous()
    entry = _lib.lib().hb_w3_moe_layer_e4m3 if e4m3 else _lib.lib().hb_w3_moe_layer
    xc = x.contiguous()
    _lib.check(entry(C.byref(st), C.byref(sh) if sh is not None else None, _lib.ptr(gv), _lib.ptr(xc),
                     _lib.ptr(ids32), _lib.ptr(wt), m, k, _lib.ptr(out), _lib.ptr(ws), need, _lib.stream()), "moe_layer")
    return out


def moe_layer_logits(experts: W3Experts, x: torch.Tensor, logits: torch.Tensor, topk: int, shared: W3Experts | None = None,
                     gate_vec: torch.Tensor | None = None, return_routing: bool = False, e4m3: bool = False):
    """`moe_layer` from the router's FP32 logits [M, E_total]: softmax top-k routing (ops.route_topk's arithmetic) runs
    in the same chain - several rows: one launch routes and plans, one does fc1 and fc2, one combines; one token: fc1's
    wavefronts route the row themselves and fc2 and the combine are one launch, two in all -
    (hibana/model/flashnext/moe.py:122-144,177-192). With `return_routing`, also the ids and weights it used.
    `e4m3`: the experts' activations are rounded to E4M3 as in `moe_layer`."""
    if x.dtype != torch.bfloat16 or x.ndim != 2 or x.shape[1] != experts.shape13[1]:
        raise ValueError("moe_layer_logits: x must be BF16 [M, hidden]")
    if logits.ndim != 2 or logits.shape[0] != x.shape[0] or logits.dtype != torch.float32:
        raise ValueError("moe_layer_logits: logits must be FP32 [M, experts]")
    _lib.need_gpu(x, logits)
    m, e_total = logits.shape
    out = torch.empty((m, experts.shape2[0]), dtype=torch.bfloat16, device=x.device)
    ids = torch.empty((m, topk), dtype=torch.int32, device=x.device)
    wt = torch.empty((m, topk), dtype=torch.float32, device=x.device)
    if m:
        st = _struct(experts)
        sh = _struct(shared) if shared is not None else None
        need = _lib.lib().hb_w3_moe_workspace_bytes(m, topk, C.byref(st), int(shared is not None))
        ws = _lib.workspace(x.device, need)
        gv = None if gate_vec is None else gate_vec.float().contiguous()
        entry = _lib.lib().hb_w3_moe_layer_logits_e4m3 if e4m3 else _lib.lib().hb_w3_moe_layer_logits
        xc, lg = x.contiguous(), logits.contiguous()
        _lib.check(entry(C.byref(st), C.byref(sh) if sh is not None else None, _lib.ptr(gv), _lib.ptr(xc),
                         _lib.ptr(lg), e_total, m, topk, _lib.ptr(ids), _lib.ptr(wt), _lib.ptr(out),
                         _lib.ptr(ws), need, _lib.stream()), "moe_layer_logits")
    return (out, ids, wt) if return_routing else out


def moe_layer_budget(experts: W3Experts, x: torch.Tensor, logits: torch.Tensor, topk: int, keep: int, budget: int,
                     slots: torch.Tensor | None = None, steps: int = 1, per_request: int = 0, min_cap: int = 0, shared: W3Experts | None = None,
                     gate_vec: torch.Tensor | None = None, return_routing: bool = False):
    """`moe_layer` from the router's BF16 logits [M, E_total] under a budget: `ops.route_budget`'s selection (slots left
    over name no expert) runs in the same chain, its second launch also planning the call
    (hibana/model/flashnext/moe.py:122-135,177-192). The bits of `route_budget` followed by `moe_layer`. With
    `return_routing`, also the ids and weights it used."""
    if x.dtype != torch.bfloat16 or x.ndim != 2 or x.shape[1] != experts.shape13[1]:
        raise ValueError("moe_layer_budget: x must be BF16 [M, hidden]")
    if logits.ndim != 2 or logits.shape[0] != x.shape[0] or logits.dtype != torch.bfloat16:
        raise ValueError("moe_layer_budget: logits must be BF16 [M, experts]")
    m, e_total = logits.shape
    if not (20 <= e_total <= 1024 and 1 <= topk <= 20 and 0 <= keep <= 20) or budget < 0 or steps < 1 or m % steps:
        raise ValueError("moe_layer_budget: 20 <= E <= 1024, topk and keep at most 20, whole requests of `steps` rows")
    if slots is not None and slots.numel() < m // steps:
        raise ValueError("moe_layer_budget: a slot for every request")
    _lib.need_gpu(x, logits, slots)
    out = torch.empty((m, experts.shape2[0]), dtype=torch.bfloat16, device=x.device)
    ids = torch.empty((m, topk), dtype=torch.int32, device=x.device)
    wt = torch.empty((m, topk), dtype=torch.float32, device=x.device)
    if m:
        st = _struct(experts)
        sh = _struct(shared) if shared is not None else None
        need = _lib.lib().hb_w3_moe_workspace_bytes(m, topk, C.byref(st), int(shared is not None))
        ws = _lib.workspace(x.device, need)
        gv = None if gate_vec is None else gate_vec.float().contiguous()
        sl = None if slots is None else slots.to(torch.int32).contiguous()
        xc, lg = x.contiguous(), logits.contiguous()
        _lib.check(_lib.lib().hb_w3_moe_layer_budget(C.byref(st), C.byref(sh) if sh is not None else None, _lib.ptr(gv), _lib.ptr(xc), _lib.ptr(lg),
                                                     e_total, m, topk, keep, budget, _lib.ptr(sl), steps, per_request, min_cap, _lib.ptr(ids),
                                                     _lib.ptr(wt), _lib.ptr(out), _lib.ptr(ws), need, _lib.stream()), "moe_layer_budget")
    return (out, ids, wt) if return_routing else out


# ------------------------------------------------------------------ offline: 3-bit experts from NVFP4 experts

@torch.no_grad()
def fit_scales(weight: torch.Tensor, levels, ratios=RATIOS):
    """float32 [N, K] -> (group scales float8_e4m3fn [N, K/32], row scales float32 [N]): per 32-group the STORED scale,
    among e4m3(amax / max|level| * ratio / row scale) over the ratio grid, with the smallest squared weight error at
    nearest-level codes; the first of equal errors stays (hibana/weights/w3_calibration.py:17-37 with unit importance).
    Unlike `w3.pack(fit_scales=True)` the candidates are compared as they will be stored."""
    book = w3._Levels(tuple(levels), weight.device)
    groups = weight.float().unflatten(1, (weight.shape[1] // w3.GROUP, w3.GROUP))
    base = groups.abs().amax(-1) / book.top
    row = book.row_scale(base)

    def candidates():
        for ratio in ratios:
            stored = book.stored(base * ratio, row).float()
            yield book.loss(groups, stored * row.unsqueeze(1)), stored

    return w3.first_best(candidates()).to(torch.float8_e4m3fn), row


@torch.no_grad()
def quantize(weight: torch.Tensor, codebook="lloyd", ratios=RATIOS):
    """float32 [N, K] -> (codes int32 [N, K], group scales float8_e4m3fn [N, K/32], row scales [N]): `fit_scales`, then
    the nearest level under the fitted scale (hibana/kernels/w3_moe.py:113-124)."""
    levels = w3._codebook(codebook)
    stored, row = fit_scales(weight, levels, ratios)
    book = w3._Levels(levels, weight.device)
    groups = weight.float().unflatten(1, (weight.shape[1] // w3.GROUP, w3.GROUP))
    codes = book.nearest(groups, stored.float() * row.unsqueeze(1))
    return codes.flatten(1).to(torch.int32), stored, row


def nvfp4_dequant(packed: torch.Tensor, scales: torch.Tensor, scale2: torch.Tensor) -> torch.Tensor:
    """NVFP4 experts (uint8 [E, R, K/2], float8_e4m3fn [E, R, K/16], FP32 [E]) -> float32 [E, R, K]: code value x block
    scale, then x the expert's scale (hibana/kernels/w3_moe.py:105-110)."""
    from hibana_amd.weights.modelopt import unpack_fp4
    experts, rows, half = packed.shape
    unscaled = unpack_fp4(packed.flatten(0, 1), scales.flatten(0, 1)).unflatten(0, (experts, rows))
    return unscaled * scale2.float().view(experts, 1, 1)


def _quantized_chunks(packed, scales, scale2, row_order, levels, ratios, chunk):
    """A stack of NVFP4 experts, `chunk` experts at a time -> (their 3-bit W3Weight, squared error, squared norm)."""
    rows = packed.shape[1]
    for lo in range(0, packed.shape[0], chunk):
        piece = slice(lo, lo + chunk)
        source = nvfp4_dequant(packed[piece], scales[piece], scale2[piece])
        if row_order is not None:
            source = source.index_select(1, row_order)
        source = source.flatten(0, 1)
        copy = w3.pack_codes(*quantize(source, levels, ratios), levels, rows_per_chunk=rows)
        delta = w3.dequantize(copy) - source
        yield copy, float(delta.square().sum()), float(source.square().sum())


@torch.no_grad()
def calibrate(w13, s13, scale2_13, w2, s2, scale2_2, codebook="lloyd", ratios=RATIOS, chunk: int = 16):
    """A layer's NVFP4 experts (w13 uint8 [E, 2I, H/2] with rows [up; gate], unswizzled float8 block scales
    [E, 2I, H/16], FP32 scales [E]; w2 likewise) -> (W3Experts with fc1 rows in fc1_order, report {"w13", "w2"}: the
    relative weight error of each stack against the NVFP4 values) (hibana/kernels/w3_moe.py:127-155). Runs on the GPU
    the tensors are on, `chunk` experts at a time."""
    levels = w3._codebook(codebook)
    experts = w13.shape[0]
    stacks = {"w13": (w13, s13, scale2_13, fc1_order(w13.shape[1] // 2, w13.device)), "w2": (w2, s2, scale2_2, None)}
    built, report = {}, {}
    for key, (packed, scales, scale2, row_order) in stacks.items():
        copies, err, norm = [], 0.0, 0.0
        for copy, e2, n2 in _quantized_chunks(packed, scales, scale2, row_order, levels, ratios, chunk):
            copies.append(copy)
            err += e2
            norm += n2
        report[key] = (err / norm) ** 0.5 if norm else 0.0
        planes = torch.cat([c.planes.view(torch.int32) for c in copies]).view(torch.uint32)
        built[key] = w3.W3Weight(planes, torch.cat([c.scales for c in copies]), torch.cat([c.row_scale for c in copies]),
                                 experts * packed.shape[1], packed.shape[2] * 2, levels, w3.lut_of(levels))
    return W3Experts.from_stacked(built["w13"], built["w2"], experts), report


def unswizzle_batched(swizzled: torch.Tensor, rows: int, groups: int) -> torch.Tensor:
    """[E, ...] block scales in the 128x4 interleave -> float8_e4m3fn [E, rows, groups] (hibana/kernels/w3_moe.py:97-102)."""
    from hibana_amd.weights.modelopt import unswizzle_block_scales
    flat = swizzled.reshape(swizzled.shape[0], -1).view(torch.uint8)
    return torch.stack([unswizzle_block_scales(one, rows, groups) for one in flat]).view(torch.float8_e4m3fn)
