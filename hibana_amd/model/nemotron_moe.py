"""The latent-MoE block of Nemotron-H on MI355X behind the reference's `NemotronMoe` surface
(hibana/model/nemotron/moe.py:343-566): x [M, H] BF16 -> BF16 [M, H],

    fused   = x [router; fc1_latent]^T                 FP32 [M, E + L]   (one GEMM for both readers of x)
    ids, w  = top-k of sigmoid(logits) + bias, weights = the plain sigmoids renormalized
    latent  = bf16(fused[:, E:])
    routed  = sum_k w_k * down_e(relu(up_e latent)^2)  BF16 [M, L]      (NVFP4 or 3-bit experts, scaling in fc2's scale)
    out     = shared_down(relu(shared_up x)^2) + routed fc2_latent^T

Routing and the experts run on this package's kernels for any number of rows (the reference switches to a separate
small-call block at 16 rows; here the same chain serves both); the two dense BF16 projections are torch GEMMs
(rocBLAS / hipBLASLt), as they are cuBLAS GEMMs in the reference (`forward`, :508-517).
"""
from __future__ import annotations

import torch

from hibana_amd import _lib
from hibana_amd.kernels import ops


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


class NemotronMoe:
    """One block's weights, assembled from tensors already on the device.

    gate_fc1 BF16 [E + L, H] = [router; fc1_latent], bias FP32 [E], fc2 BF16 [H, L], shared_up / shared_down
    `Nvfp4Linear` (or None for a block without a shared expert), `experts` a callable
    (latent BF16 [M, L], ids, weights) -> BF16 [M, L] carrying the routed scaling factor: `B12xExperts` for NVFP4
    experts or `lambda l, i, w: w3_moe(w3_experts, l, i, w)` for 3-bit ones."""

    def __init__(self, gate_fc1: torch.Tensor, bias: torch.Tensor, fc2: torch.Tensor, experts, topk: int, shared_up=None, shared_down=None):
        self.gate_fc1, self.bias, self.fc2 = gate_fc1.contiguous(), bias.float().contiguous(), fc2.contiguous()
        self.experts_op, self.topk = experts, topk
        self.shared_up, self.shared_down = shared_up, shared_down
        self.experts = bias.numel()
        self.latent = gate_fc1.shape[0] - self.experts
        self.hidden = gate_fc1.shape[1]

    def route(self, fused: torch.Tensor, slots=None, steps: int = 1, repeat: bool = True):
        return route_topk(fused, self.bias, self.topk, self.latent, slots, steps, repeat)

    def routed(self, latent: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
        return self.experts_op(latent, ids, weights)

    def shared(self, x: torch.Tensor) -> torch.Tensor:
        """shared_down(relu(shared_up x)^2), the square in FP32 with one rounding (fused into the up projection's epilogue)."""
        return ops.nvfp4_linear(ops.nvfp4_linear(x, self.shared_up, relu2=True), self.shared_down)

    def forward(self, x: torch.Tensor, slots=None, steps: int = 1) -> torch.Tensor:
        x = x.contiguous()
        fused = torch.mm(x, self.gate_fc1.T, out_dtype=torch.float32)  # [M, E + L]
        ids, weights, latent = self.route(fused, slots, steps)
        routed = self.routed(latent, ids, weights)
        if self.shared_up is None:
            return torch.mm(routed, self.fc2.T)
        return torch.addmm(self.shared(x), routed, self.fc2.T)

    __call__ = forward
