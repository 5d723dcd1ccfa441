"""The latent-MoE block of Nemotron-H on MI355X behind the reference's `NemotronMoe` surface
(hibana/model/nemotron/moe.py:343-566): x [M, H] BF16 -> BF16 [M, H],

    fused   = x [router; fc1_latent]^T                 FP32 [M, E + L]   (one GEMM for both readers of x)
    ids, w  = top-k of sigmoid(logits) + bias, weights = the plain sigmoids renormalized
    latent  = bf16(fused[:, E:])
    routed  = sum_k w_k * down_e(relu(up_e latent)^2)  BF16 [M, L]      (NVFP4 or 3-bit experts, scaling in fc2's scale)
    out     = shared_down(relu(shared_up x)^2) + routed fc2_latent^T

Up to sixteen rows (decode, verify) the block runs through the small-call kernels of `kernels/nemotron_moe.py`, four
launches with the two BF16 projections inside them (`small`, :484-502 of the reference). Past that, routing and the
experts run on this package's kernels and the two dense BF16 projections are torch GEMMs (rocBLAS / hipBLASLt), as
they are cuBLAS GEMMs in the reference (`forward`, :508-517).
"""
from __future__ import annotations

import torch

from hibana_amd import _lib
from hibana_amd.kernels import nemotron_moe as small_block, ops
from hibana_amd.kernels.b12x_moe import B12xExperts
from hibana_amd.kernels.w3_moe import W3Experts, w3_moe


def route_topk(fused: torch.Tensor, bias: torch.Tensor, k: int, latent: int, slots: torch.Tensor | None = None, steps: int = 1,
               repeat: bool = True):
    """fused FP32 [M, E + latent] (router logits | fc1 latent) -> (int32 ids [M, k] by descending sigmoid + bias, equal
    scores to the lower id; FP32 renormalized sigmoid weights [M, k], without the routed scaling factor; BF16 latent
    [M, latent]). With `slots`, row r is real iff slots[r // steps] != 0; a padded row takes row 0's top expert at
    weight 0 (without `repeat`: id E, no expert) (hibana/model/nemotron/moe.py:106-121)."""
    if fused.dtype != torch.float32 or fused.ndim != 2 or fused.stride(1) != 1:
        raise ValueError("route_topk: fused must be FP32 [M, E + latent] with contiguous rows")
    _lib.need_gpu(fused, bias)
    m = fused.shape[0]
    e = fused.shape[1] - latent
    dev = fused.device
    ids = torch.empty((m, k), dtype=torch.int32, device=dev)
    w = torch.empty((m, k), dtype=torch.float32, device=dev)
    lat = torch.empty((m, latent), dtype=torch.bfloat16, device=dev)
    if m:
        sl = None if slots is None else slots.to(torch.int32).contiguous()
        bias32 = bias.float().contiguous()
        _lib.check(_lib.lib().hb_route_sigmoid_topk(_lib.ptr(fused), fused.stride(0), _lib.ptr(bias32), m, e, k, latent,
                                                    _lib.ptr(sl), steps, int(repeat), _lib.ptr(ids), _lib.ptr(w), _lib.ptr(lat), _lib.stream()),
                   "route_topk")
    return ids, w, lat


def route_budget(fused: torch.Tensor, bias: torch.Tensor, k: int, latent: int, keep: int, budget: int, slots: torch.Tensor | None = None,
                 steps: int = 1, per_request: int = 0, repeat: bool = True, fallback: int = 0):
    """Budgeted top-k over fused FP32 [R, E + latent] -> (ids [R, k], renormalized weights [R, k], BF16 latent)
    (hibana/model/nemotron/moe.py:266-313): the call reads at most min(budget, per_request x real requests) distinct
    experts (`budget` without `per_request`; 0: the guaranteed experts alone), more only when the rows' guaranteed top
    `keep` exceed it. Each real row takes those of its top k (by sigmoid + bias) that are in the set, in rank order, its
    top `keep` first; its weights are its plain sigmoids renormalized over those. Slots left over (all of a padded
    row's) name the row's top expert (a padded row: row 0's) at weight 0, or without `repeat` no expert (id E).
    `fallback` (< keep): when the guaranteed experts' union exceeds the cap, each real row is guaranteed only its top
    `fallback` and the cap fills by routing weight."""
    if fused.dtype != torch.float32 or fused.ndim != 2 or fused.stride(1) != 1:
        raise ValueError("route_budget: fused must be FP32 [R, E + latent] with contiguous rows")
    r = fused.shape[0]
    e = fused.shape[1] - latent
    if not (1 <= k <= 32 and k <= e <= 1024 and 0 <= fallback <= keep <= k) or budget < 0 or steps < 1 or r % steps:
        raise ValueError("route_budget: k at most 32, E at most 1024, fallback <= keep <= k, whole requests of `steps` rows")
    if slots is not None and slots.numel() < r // steps:
        raise ValueError("route_budget: a slot for every request")
    _lib.need_gpu(fused, bias, slots)
    dev = fused.device
    ids = torch.empty((r, k), dtype=torch.int32, device=dev)
    w = torch.empty((r, k), dtype=torch.float32, device=dev)
    lat = torch.empty((r, latent), dtype=torch.bfloat16, device=dev)
    if r:
        sl = None if slots is None else slots.to(torch.int32).contiguous()
        bias32 = bias.float().contiguous()
        ws = torch.empty((_lib.lib().hb_route_budget_sigmoid_workspace_bytes(r, k),), dtype=torch.uint8, device=dev)
        _lib.check(_lib.lib().hb_route_budget_sigmoid(_lib.ptr(fused), fused.stride(0), _lib.ptr(bias32), r, e, k, latent, keep, budget, _lib.ptr(sl),
                                                      steps, int(repeat), per_request, fallback, _lib.ptr(ws), ws.numel(), _lib.ptr(ids), _lib.ptr(w),
                                                      _lib.ptr(lat), _lib.stream()), "route_budget")
    return ids, w, lat


def relu2_(x: torch.Tensor) -> torch.Tensor:
    """relu(x)^2 in place for BF16 [M, N] (FP32 square, one rounding: torch's relu(x) ** 2)
    (hibana/model/nemotron/moe.py:316-321). The expert kernels and `NemotronMoe.shared` do it in their epilogues; this
    is the standalone form."""
    if x.dtype != torch.bfloat16 or x.ndim != 2 or x.stride(1) != 1 or x.shape[1] % 2 or x.stride(0) % 2:
        raise ValueError("relu2_: BF16 [M, N] with contiguous rows, N and the row stride even")
    _lib.need_gpu(x)
    if x.numel():
        _lib.check(_lib.lib().hb_relu2(_lib.ptr(x), x.shape[0], x.shape[1], x.stride(0), _lib.stream()), "relu2_")
    return x


class NemotronMoe:
    """One block's weights, assembled from tensors already on the device.

    gate_fc1 BF16 [E + L, H] = [router; fc1_latent], bias FP32 [E], fc2 BF16 [H, L], shared_up / shared_down
    `Nvfp4Linear` (or None for a block without a shared expert), `experts` the routed experts carrying the routed
    scaling factor: a `B12xExperts` (NVFP4), a `W3Experts` (3-bit), or any callable
    (latent BF16 [M, L], ids, weights) -> BF16 [M, L]. `keep` / `budget` / `per_request`: budgeted expert selection in
    decode and verify forwards (the reference's HIBANA_MOE_KEEP / _BUDGET / _BUDGET_PER_REQUEST settings, :378-380):
    each token's floor (topk or more, or 0: every token's top k), the cap on the distinct experts a forward reads and
    its share a request."""

    SHARE_MIN = 8  # under a binding cap each token keeps at least its top SHARE_MIN (hibana/model/nemotron/moe.py:350)
    SMALL_ROWS = small_block.MAX_ROWS

    def __init__(self, gate_fc1: torch.Tensor, bias: torch.Tensor, fc2: torch.Tensor, experts, topk: int, shared_up=None, shared_down=None,
                 keep: int = 0, budget: int = 0, per_request: int = 0):
        if keep < 0 or budget < 0 or per_request < 0:
            raise ValueError(f"keep {keep}, budget {budget}, per_request {per_request}: not negative")
        self.gate_fc1, self.bias, self.fc2 = gate_fc1.contiguous(), bias.float().contiguous(), fc2.contiguous()
        self.topk = topk
        self.keep = keep if keep < topk else 0
        self.budget = budget if self.keep else 0
        self.per_request = per_request
        self.shared_up, self.shared_down = shared_up, shared_down
        self.experts = bias.numel()
        self.latent = gate_fc1.shape[0] - self.experts
        self.hidden = gate_fc1.shape[1]
        self.w3 = experts if isinstance(experts, W3Experts) else None
        self.b12x = experts if isinstance(experts, B12xExperts) else None
        self.experts_op = (lambda lat, ids, w: w3_moe(self.w3, lat, ids, w)) if self.w3 is not None else experts
        self._small = None

    def small_weights(self) -> small_block.SmallWeights:
        """What the small-call kernels read (hibana/model/nemotron/moe.py's small_weights), assembled once."""
        if self._small is None:
            self._small = small_block.SmallWeights(self.gate_fc1, self.bias, self.fc2, self.b12x, self.shared_up, self.shared_down)
        return self._small

    @staticmethod
    def _padding(ctx):
        """(slots, steps) of a decode / verify forward whose graph may hold padded requests, else (None, 1)."""
        mode = getattr(ctx, "mode", None)
        if mode == "decode":
            return getattr(ctx, "slots", None), 1
        if mode == "verify":
            return getattr(ctx, "seq_slots", None), int(getattr(ctx, "verify_steps", 1))
        return None, 1

    def selects(self, ctx) -> bool:
        """Whether this forward takes the budgeted selection: decode and verify forwards of a block with a `keep`."""
        return bool(self.keep) and getattr(ctx, "mode", None) in ("decode", "verify")

    def fallback(self, rows: int, steps: int) -> int:
        """The guarantee when the floors' union exceeds the cap: cap / rows within [SHARE_MIN, keep), from the call's
        shape; 0 without a cap or when the rule gives the floor itself (hibana/model/nemotron/moe.py:464-474)."""
        if not self.budget:
            return 0
        cap = min(self.budget, self.per_request * (rows // steps)) if self.per_request else self.budget
        g = max(min(self.SHARE_MIN, self.keep), min(self.keep, cap // rows))
        return g if g < self.keep else 0

    def route(self, fused: torch.Tensor, slots=None, steps: int = 1, repeat: bool | None = None, select: bool = False):
        """FP32 router|fc1 rows -> (ids, renormalized weights, BF16 latent). Padded rows take row 0's first choice at
        weight 0; around 3-bit experts, id E (no expert), which their kernel skips. `select` (a decode or verify
        forward of a block with a `keep`): the budgeted selection (hibana/model/nemotron/moe.py:448-462)."""
        repeat = self.w3 is None if repeat is None else repeat
        if select and self.keep:
            return route_budget(fused, self.bias, self.topk, self.latent, self.keep, self.budget, slots, steps, per_request=self.per_request,
                                repeat=repeat, fallback=self.fallback(fused.shape[0], steps))
        return route_topk(fused, self.bias, self.topk, self.latent, slots, steps, repeat)

    def routed(self, latent: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
        return self.experts_op(latent, ids, weights)

    def shared(self, x: torch.Tensor) -> torch.Tensor:
        """shared_down(relu(shared_up x)^2), the square in FP32 with one rounding (fused into the up projection's epilogue)."""
        return ops.nvfp4_linear(ops.nvfp4_linear(x, self.shared_up, relu2=True), self.shared_down)

    def small(self, x: torch.Tensor, ctx=None) -> torch.Tensor:
        """The block through `kernels/nemotron_moe.py` (at most SMALL_ROWS rows): the router's launch also routes and
        plans as `route` would (hibana/model/nemotron/moe.py:484-502)."""
        w = self.small_weights()
        slots, steps = self._padding(ctx)
        if self.selects(ctx):  # the router's launch leaves the routing to the budgeted selection; the block plans from its ids
            fused, _, _, ws = small_block.router(x, w, None, self.topk, route=False)
            ids, weights, lat = self.route(fused, slots, steps, select=True)
            if self.w3 is not None:
                return small_block.w3_block(x, ws, lat, ids, weights, w, self.w3)
            return small_block.block(x, ws, ids, weights, w, plan=True)
        if self.w3 is not None:  # padded rows name no expert (id E), which w3_moe skips
            _, ids, weights, ws, lat = small_block.router(x, w, None, self.topk, slots, steps, pad_id=self.experts, latent=True)
            return small_block.w3_block(x, ws, lat, ids, weights, w, self.w3)
        _, ids, weights, ws = small_block.router(x, w, None, self.topk, slots, steps)
        return small_block.block(x, ws, ids, weights, w)

    def forward(self, x: torch.Tensor, ctx=None) -> torch.Tensor:
        """Post-norm rows x [M, H] BF16 -> the block's mixer output [M, H] BF16 (hibana/model/nemotron/moe.py:508-517)."""
        x = x.contiguous()
        if 0 < x.shape[0] <= self.SMALL_ROWS and (self.b12x is not None or self.w3 is not None):
            return self.small(x, ctx)
        fused = torch.mm(x, self.gate_fc1.T, out_dtype=torch.float32)  # [M, E + L]
        ids, weights, latent = self.route(fused, *self._padding(ctx), select=self.selects(ctx))
        routed = self.routed(latent, ids, weights)
        if self.shared_up is None:
            return torch.mm(routed, self.fc2.T)
        return torch.addmm(self.shared(x), routed, self.fc2.T)

    __call__ = forward
