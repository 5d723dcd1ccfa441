"""The latent-MoE block of a decode / verify call (at most MAX_ROWS rows) behind the reference's small-call surface
(hibana/kernels/nemotron_moe.py:45-68): `router` (the router|fc1_latent product on the matrix cores, then the routing
of every row as `model.nemotron_moe.route_topk` does it from the same FP32 rows, bit for bit, with the call's plan: two
launches), then `block` (routed up beside the shared expert's up, routed down beside its down, the combine,
fc2_latent: four launches), or `w3_block` around 3-bit routed experts.

`weights` is a `SmallWeights` (what the kernels read, the reference's `NemotronMoe.small_weights()` list): assembled
once a block, it holds the device pointers' owners. Activations stay BF16 throughout (weight-only arithmetic: the
reference's small-call kernels round x, the latent and h to NVFP4 for its FP4 tensor cores).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import torch

from hibana_amd import _lib

MAX_ROWS = 16


@dataclass
class SmallWeights:
    """gate_fc1 BF16 [E + L, H] = [router; fc1_latent], bias FP32 [E], fc2 BF16 [H, L], `experts` a `B12xExperts` over
    the latent (or None: the routed experts are 3-bit), shared_up / shared_down `Nvfp4Linear` (or None)."""
    gate_fc1: torch.Tensor
    bias: torch.Tensor
    fc2: torch.Tensor
    experts: object = None
    shared_up: object = None
    shared_down: object = None

    def __post_init__(self):
        if self.gate_fc1.dtype != torch.bfloat16 or self.fc2.dtype != torch.bfloat16:
            raise ValueError("gate_fc1 and fc2 must be BF16")
        self.gate_fc1, self.fc2, self.bias = self.gate_fc1.contiguous(), self.fc2.contiguous(), self.bias.float().contiguous()
        self.experts_total = self.bias.numel()
        self.latent = self.gate_fc1.shape[0] - self.experts_total
        self.hidden = self.gate_fc1.shape[1]
        if self.fc2.shape != (self.hidden, self.latent):
            raise ValueError("fc2 must be [hidden, latent]")
        if (self.shared_up is None) != (self.shared_down is None):
            raise ValueError("a shared expert has both an up and a down projection")
        if self.shared_up is not None:
            self.shared_up.tile()
            self.shared_down.tile()
            if self.shared_up.in_features != self.hidden or (self.shared_down.out_features, self.shared_down.in_features) != (self.hidden, self.shared_up.out_features):
                raise ValueError("shared_up [I, H] and shared_down [H, I] do not describe one expert")
        self._routed = None if self.experts is None else self.experts._struct()

    def struct(self) -> _lib.HbLatentWeights:
        up, down = self.shared_up, self.shared_down
        return _lib.HbLatentWeights(
            _lib.ptr(self.gate_fc1), _lib.ptr(self.bias), _lib.ptr(self.fc2), None if self._routed is None else C.pointer(self._routed),
            None if up is None else _lib.ptr(up.tiled), None if down is None else _lib.ptr(down.tiled),
            0.0 if up is None else up.global_scale, 0.0 if down is None else down.global_scale,
            self.experts_total, self.latent, self.hidden, 0 if up is None else up.out_features)


@dataclass
class Workspace:
    """What `router` leaves for the calls after it: the library's workspace (plan, h, pair outputs, shared expert's
    rows) and the BF16 latent rows."""
    buffer: torch.Tensor
    lat: torch.Tensor
    m: int
    topk: int


def _rows(x: torch.Tensor, weights: SmallWeights) -> int:
    if x.dtype != torch.bfloat16 or x.ndim != 2 or x.shape[1] != weights.hidden:
        raise ValueError("x must be BF16 [M, hidden]")
    if not 0 < x.shape[0] <= MAX_ROWS:
        raise ValueError(f"the small latent block takes 1 .. {MAX_ROWS} rows")
    _lib.need_gpu(x)
    return x.shape[0]


def router(x: torch.Tensor, weights: SmallWeights, bias: torch.Tensor | None, k: int, slots: torch.Tensor | None = None, steps: int = 1,
           route: bool = True, pad_id: int = -1, latent: bool = False):
    """x BF16 [M, H] -> (fused FP32 [M, E + L], ids [M, k], weights [M, k], workspace[, BF16 latent [M, L] with
    `latent`]). With `route`, ids / weights are route_topk's (with `slots`: rows of requests on slot 0 padded: row 0's
    top expert at weight 0, or `pad_id` when >= 0, e.g. E = no expert for the 3-bit experts) and the call is planned;
    else they are unwritten. `bias`: None for the block's own (hibana/kernels/nemotron_moe.py:45-55)."""
    m = _rows(x, weights)
    if bias is not None and bias is not weights.bias:
        if bias.numel() != weights.experts_total:
            raise ValueError("bias must be [E]")
        weights = SmallWeights(weights.gate_fc1, bias, weights.fc2, weights.experts, weights.shared_up, weights.shared_down)
    dev = x.device
    st = weights.struct()
    need = _lib.lib().hb_latent_workspace_bytes(C.byref(st), m, k)
    if need == 0:
        raise ValueError("router: the block's shapes are not ones the kernels take")
    buffer = _lib.workspace(dev, need, "latent")  # the stream's own: a Workspace serves until the next `router` on this stream
    fused = torch.empty((m, weights.experts_total + weights.latent), dtype=torch.float32, device=dev)
    ids = torch.empty((m, k), dtype=torch.int32, device=dev)
    wts = torch.empty((m, k), dtype=torch.float32, device=dev)
    lat = torch.empty((m, weights.latent), dtype=torch.bfloat16, device=dev)
    sl = None if slots is None else slots.to(torch.int32).contiguous()
    xc = x.contiguous()
    _lib.check(_lib.lib().hb_latent_router(C.byref(st), _lib.ptr(xc), m, k, _lib.ptr(sl), steps, int(route), pad_id, _lib.ptr(fused), _lib.ptr(ids),
                                           _lib.ptr(wts), _lib.ptr(lat), _lib.ptr(buffer), need, _lib.stream()), "latent router")
    ws = Workspace(buffer, lat, m, k)
    return (fused, ids, wts, ws, lat) if latent else (fused, ids, wts, ws)


def block(x: torch.Tensor, ws: Workspace, ids: torch.Tensor, wts: torch.Tensor, weights: SmallWeights, plan: bool = False,
          lat: torch.Tensor | None = None) -> torch.Tensor:
    """The rest of the block after `router` -> BF16 [M, H]; `plan` when the caller routed (ids not the router's;
    `lat` then the caller's latent rows, by default the router's) (hibana/kernels/nemotron_moe.py:58-60)."""
    m = _rows(x, weights)
    if weights.experts is None:
        raise ValueError("block: no NVFP4 routed experts (w3_block serves 3-bit ones)")
    if (m, ids.shape[1]) != (ws.m, ws.topk) or ids.shape != wts.shape or ids.shape[0] != m:
        raise ValueError("block: not the call the workspace was made for")
    lat = ws.lat if lat is None else lat.contiguous()
    ids32, wt, xc = ids.to(torch.int32).contiguous(), wts.float().contiguous(), x.contiguous()
    out = torch.empty((m, weights.hidden), dtype=torch.bfloat16, device=x.device)
    st = weights.struct()
    _lib.check(_lib.lib().hb_latent_block(C.byref(st), _lib.ptr(xc), _lib.ptr(lat), _lib.ptr(ids32), _lib.ptr(wt), m, ws.topk, int(plan), _lib.ptr(out),
                                          _lib.ptr(ws.buffer), ws.buffer.numel(), _lib.stream()), "latent block")
    return out


def shared_up(x: torch.Tensor, ws: Workspace, weights: SmallWeights) -> None:
    """relu(shared_up x)^2 into the workspace (nothing without a shared expert)."""
    m = _rows(x, weights)
    if weights.shared_up is None:
        return
    st = weights.struct()
    xc = x.contiguous()
    _lib.check(_lib.lib().hb_latent_shared_up(C.byref(st), _lib.ptr(xc), m, ws.topk, _lib.ptr(ws.buffer), ws.buffer.numel(), _lib.stream()), "latent shared_up")


def out(x: torch.Tensor, ws: Workspace, routed: torch.Tensor, weights: SmallWeights) -> torch.Tensor:
    """bf16(shared_down(what shared_up left) + routed fc2^T) for the routed sum BF16 [M, L] -> BF16 [M, H]."""
    m = _rows(x, weights)
    if routed.dtype != torch.bfloat16 or routed.shape != (m, weights.latent):
        raise ValueError("out: routed must be BF16 [M, latent]")
    res = torch.empty((m, weights.hidden), dtype=torch.bfloat16, device=x.device)
    st = weights.struct()
    rc = routed.contiguous()
    _lib.check(_lib.lib().hb_latent_out(C.byref(st), _lib.ptr(rc), m, ws.topk, _lib.ptr(res), _lib.ptr(ws.buffer), ws.buffer.numel(), _lib.stream()), "latent out")
    return res


def w3_block(x: torch.Tensor, ws: Workspace, lat: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, weights: SmallWeights, experts) -> torch.Tensor:
    """The block after `router` (with `latent`) around 3-bit routed experts (`kernels/w3_moe.py`'s W3Experts): the
    shared expert's up, the routed sum through w3_moe from the router's BF16 latent and ids, then fc2_latent plus the
    shared expert's down -> BF16 [M, H] (hibana/kernels/nemotron_moe.py:63-68)."""
    from hibana_amd.kernels.w3_moe import w3_moe
    shared_up(x, ws, weights)
    return out(x, ws, w3_moe(experts, lat, ids, wts), weights)
