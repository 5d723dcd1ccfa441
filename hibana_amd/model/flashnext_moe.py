"""The gated-MoE block of Flash-Next on MI355X behind the reference's `MoeLayer` surface
(hibana/model/flashnext/moe.py:75-192): x [M, H] BF16 -> BF16 [M, H],

    logits  = x router^T                                      BF16 [M, E] (one GEMM), read as FP32 by the routing
    ids, w  = top-k of softmax(logits), renormalized          (padded rows of a graph: id E, weight 0)
    routed  = sum_k w_k * down_e(silu(gate_e x) * up_e x)      3-bit experts
    shared  = shared_down(silu(shared_gate x) * shared_up x)   3-bit, rides in the experts' launches as one more expert
                                                               (calls the reference serves from the NVFP4 linears - more
                                                               than w3.MAX_ROWS rows, or HIBANA_W3_DECODE off - run on them)
    out     = bf16(bf16(routed) + sigmoid(x . shared_gate_vec) * shared)

The block is assembled from tensors already on the device (a loader's job ends there). The routed experts are a
`W3Experts`; the shared expert is either a one-expert `W3Experts` or the pair of linears the reference holds
(`shared_gate_up` with rows [gate; up], `shared_down`), whose 3-bit copies are re-stored once, at construction, in the
experts' row order (`shared_from_linears`). Budgeted expert selection (HIBANA_MOE_KEEP / HIBANA_MOE_BUDGET /
HIBANA_MOE_BUDGET_PER_REQUEST of the reference's configuration) is the constructor's `keep` / `budget` / `per_request`:
decode and verify forwards then read at most a budget of distinct experts (`ops.route_budget`); slots left over name no
expert, which the 3-bit kernels skip.
"""
from __future__ import annotations

import torch

from hibana_amd.kernels import ops, w3, w3_moe


def shared_from_linears(gate_up: w3.W3Weight, down: w3.W3Weight) -> w3_moe.W3Experts:
    """A shared expert held as two 3-bit matrices - gate_up [2 I, H] with rows [gate; up], down [H, I] - as the
    one-expert `W3Experts` the kernels take: fc1 = [up; gate] in `fc1_order` (sixteen up rows, then their sixteen gate
    rows). Rows move in units of sixteen, half a 32-row tile of the fragment order, so the codes are unpacked, reordered
    and packed again (exactly: no requantization)."""
    inter = gate_up.out_features // 2
    if down.in_features != inter or down.out_features != gate_up.in_features:
        raise ValueError("gate_up [2 I, H] and down [H, I] do not describe one expert")
    dev = gate_up.row_scale.device
    rows = torch.cat((torch.arange(inter, 2 * inter), torch.arange(inter)))[w3_moe.fc1_order(inter)].to(dev)  # [up; gate] of [gate; up], then the order
    fc1 = w3.pack_codes(w3.codes(gate_up).index_select(0, rows).to(torch.uint8), w3.scale_bytes(gate_up).view(torch.uint8).index_select(0, rows).view(torch.float8_e4m3fn),
                        gate_up.row_scale.index_select(0, rows), gate_up.codebook)
    if down.planes is None:  # only a tiled copy left: back through the codes
        down = w3.pack_codes(w3.codes(down).to(torch.uint8), w3.scale_bytes(down), down.row_scale, down.codebook)
    return w3_moe.tile(w3_moe.W3Experts.from_stacked(fc1, down, 1))


class MoeLayer:
    MIN_GUARANTEE = 2  # hibana/model/flashnext/moe.py:146-149
    MIN_CAP = 16

    def __init__(self, router: torch.Tensor, shared_gate: torch.Tensor, experts: w3_moe.W3Experts, topk: int, shared: w3_moe.W3Experts | None = None,
                 shared_gate_up=None, shared_down=None, keep: int = 0, budget: int = 0, per_request: int = 0):
        """router BF16 [E, H]; shared_gate [1, H] or [H] (the shared expert's sigmoid gate); `experts` this rank's 3-bit
        experts (a range base .. base + experts - 1 of the E); the shared expert as `shared`, or as the two linears
        `shared_gate_up` / `shared_down` with 3-bit copies attached (`.w3`). `keep` (below topk; topk or more, or 0, is
        the served route): each token's own top experts in decode and verify forwards; with `budget`, the cap on the
        distinct experts such a forward reads, `per_request` its share a request
        (hibana/model/flashnext/moe.py:86-93)."""
        if keep < 0 or budget < 0 or per_request < 0:
            raise ValueError(f"keep {keep}, budget {budget}, per_request {per_request}: not negative")
        self.router = router.contiguous()
        self.experts, self.hidden = router.shape
        self.topk = topk
        self.keep = keep if keep < topk else 0
        self.budget = budget if self.keep else 0
        self.per_request = per_request
        self.shared_gate = shared_gate.float().reshape(1, -1).contiguous()
        self.shared_gate_vec = self.shared_gate.reshape(-1)
        self.w3 = w3_moe.tile(experts)
        if experts.base + experts.experts > self.experts:
            raise ValueError(f"3-bit experts {experts.base}..{experts.base + experts.experts - 1}: the model has {self.experts}")
        if shared is None and shared_gate_up is not None:
            if getattr(shared_gate_up, "w3", None) is None or getattr(shared_down, "w3", None) is None:
                if getattr(shared_gate_up, "weight", None) is None:
                    raise ValueError("the shared expert's linears need their 3-bit copies (w3.attach) or NVFP4 weights to run on")
            else:
                shared = shared_from_linears(shared_gate_up.w3, shared_down.w3)
        self.shared = None if shared is None else w3_moe.tile(shared)
        self.shared_gate_up, self.shared_down = shared_gate_up, shared_down

    @property
    def expert_bytes(self) -> int:
        return self.w3.bytes

    @property
    def bytes(self) -> int:
        return self.expert_bytes + self.router.numel() * 2 + (self.shared.bytes if self.shared is not None else 0)

    @staticmethod
    def _padding(ctx):
        """(slots, steps) of a decode / verify forward whose graph may hold padded requests, else (None, 1)."""
        mode = getattr(ctx, "mode", None)
        if mode == "decode":
            return getattr(ctx, "slots", None), 1
        if mode == "verify":
            return getattr(ctx, "seq_slots", None), int(getattr(ctx, "verify_steps", 1))
        return None, 1

    def guarantee(self, rows: int, steps: int) -> int:
        """Each token's guaranteed top experts under a budget: 2 cap / rows within [MIN_GUARANTEE, keep], the cap that of
        the call's shape (hibana/model/flashnext/moe.py:151-158)."""
        cap = min(self.budget, max(self.MIN_CAP, self.per_request * (rows // steps))) if self.per_request else self.budget
        return max(min(self.MIN_GUARANTEE, self.keep), min(self.keep, 2 * cap // rows))

    def selects(self, ctx) -> bool:
        """Whether this forward takes the budgeted selection: decode and verify forwards of a layer with a `keep`."""
        return bool(self.keep) and getattr(ctx, "mode", None) in ("decode", "verify")

    def route(self, x: torch.Tensor, ctx=None):
        """(ids int32 [M, k], weights FP32 [M, k]); padded rows of a decode / verify graph name no expert
        (hibana/model/flashnext/moe.py:122-144; softmax -> top-k -> renormalize at every size). With a `keep`, decode
        and verify forwards take each token's top `keep` alone (ids [M, keep]) or, under a budget, the selection of
        `ops.route_budget`."""
        logits = torch.mm(x, self.router.T)
        slots, steps = self._padding(ctx)
        if self.selects(ctx):
            if not self.budget:
                return ops.route_topk(logits, self.keep)
            return ops.route_budget(logits, self.topk, self.guarantee(logits.shape[0], steps), self.budget, slots, steps, repeat=False,
                                    per_request=self.per_request, min_cap=self.MIN_CAP)
        return ops.route_topk(logits, self.topk, slots, steps, repeat=False)

    def routed(self, x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
        """The routed experts' weighted sum (this rank's part) for x [M, H] -> BF16 [M, H]."""
        return w3_moe.w3_moe(self.w3, x, ids, weights)

    def shared_on_linears(self, m: int) -> bool:
        """Whether a call of `m` rows runs the shared expert on its own linears: the reference does, and takes their 3-bit
        copies only where `ops.w3_decode` holds - at most w3.MAX_ROWS rows with HIBANA_W3_DECODE on
        (hibana/model/flashnext/moe.py:181-189, hibana/kernels/ops.py:50-53). Linears that hold nothing but a 3-bit
        copy (no NVFP4 weights to run) always ride in the experts' launches."""
        lin = self.shared_gate_up
        if lin is None or self.shared_down is None or getattr(lin, "weight", None) is None or getattr(lin, "in_features", None) is None:
            return False
        return not (ops.w3_decode(lin, m) and ops.w3_decode(self.shared_down, m))

    def __call__(self, x: torch.Tensor, ctx=None) -> torch.Tensor:
        x = x.contiguous()
        if self.shared_on_linears(x.shape[0]):
            # the reference's own chain: the experts' unsummed pair outputs (BF16 from WIDE_ROWS rows), the shared expert
            # on its linears (silu(gate) * up in between), the combine over both
            ids, weights = self.route(x, ctx)
            pairs = w3_moe.w3_moe(self.w3, x, ids, weights, pairs=True, pairs_bf16=x.shape[0] >= w3_moe.WIDE_ROWS)
            shared = ops.nvfp4_linear(ops.silu_and_mul(ops.nvfp4_linear(x, self.shared_gate_up)), self.shared_down)
            return ops.moe_combine_pairs(pairs, ids, weights, shared, x, self.shared_gate_vec, self.w3.base, self.w3.experts)
        slots, _ = self._padding(ctx)
        if slots is None and not self.selects(ctx):  # routing, plan, both streams and the combine as one chain
            logits = torch.mm(x, self.router.T).float()
            return w3_moe.moe_layer_logits(self.w3, x, logits, self.topk, shared=self.shared, gate_vec=self.shared_gate_vec)
        if self.selects(ctx) and self.budget:  # the selection's launches and the experts' as one chain
            logits = torch.mm(x, self.router.T)
            _, steps = self._padding(ctx)
            return w3_moe.moe_layer_budget(self.w3, x, logits, self.topk, self.guarantee(x.shape[0], steps), self.budget, slots, steps,
                                           per_request=self.per_request, min_cap=self.MIN_CAP, shared=self.shared, gate_vec=self.shared_gate_vec)
        ids, weights = self.route(x, ctx)
        return w3_moe.moe_layer(self.w3, x, ids, weights, shared=self.shared, gate_vec=self.shared_gate_vec)
