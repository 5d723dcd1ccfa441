"""NVFP4 routed experts on MI355X behind the reference's `B12xExperts` surface (hibana/kernels/b12x_moe.py:24-68).

The checkpoint's tensors as the reference's model code holds them: packed E2M1 weights w1 [E, N, K/2] and w2
[E, K, N/2], their E4M3 block scales in the 128x4 interleave, one FP32 weight scale per expert matrix. Construction
repacks both stacks once into the block layout the gfx950 stream reads (csrc/nvfp4.hip); the call is the same chain
as the 3-bit experts: plan, fc1 stream (h = bf16(relu(bf16(y))^2), or gated SiLU when w1 has 2 N rows), fc2 stream,
weighted combine in selection order.

Weight-only: activations stay BF16, so the activation input scales `in1` / `in2` of the reference's W4A4 path are
accepted for signature parity and do not enter the arithmetic (there they cancel against the activation quantizer);
fc1's multiplier is g1 and fc2's is g2 x routed_scaling, the form tests/nemotron_reference.py:568-593 states.
"""
from __future__ import annotations

import ctypes as C

import torch

from hibana_amd import _lib


def _tile_stack(weight: torch.Tensor, swizzled: torch.Tensor) -> torch.Tensor:
    """[E, R, K/2] codes + per-expert interleaved block scales -> the stacked block layout, uint8 [E, bytes]."""
    _lib.need_gpu(weight, swizzled)
    e, rows, half = weight.shape
    k = 2 * half
    size = _lib.lib().hb_nvfp4_tiled_bytes(rows, k)
    if size == 0:
        raise ValueError("NVFP4 experts need rows a multiple of 64 and K a multiple of 128")
    rp, gp = (rows + 127) // 128 * 128, (k // 16 + 3) // 4 * 4
    scales = swizzled.contiguous().view(torch.uint8).reshape(e, -1)
    if scales.shape[1] != rp * gp:
        raise ValueError("block-scale extent does not match the padded 128x4 interleave")
    weight = weight.contiguous()
    tiled = torch.empty((e, size), dtype=torch.uint8, device=weight.device)
    for i in range(e):
        _lib.check(_lib.lib().hb_nvfp4_repack(_lib.ptr(weight[i]), _lib.ptr(scales[i]), 1, rows, k, _lib.ptr(tiled[i]), _lib.stream()),
                   "nvfp4 repack")
    return tiled


class B12xExperts:
    def __init__(self, w1: torch.Tensor, s1: torch.Tensor, g1: torch.Tensor, in1, w2: torch.Tensor, s2: torch.Tensor, g2: torch.Tensor,
                 in2, routed_scaling: float = 1.0, base: int = 0, release: bool = False):
        """w1 [E, N, K/2] (gated: [E, 2N, K/2], rows in the 3-bit path's fc1_order), w2 [E, K_out, N/2] uint8; s1, s2
        their interleaved E4M3 block scales; g1, g2 [E] FP32 weight scales; in1, in2 unused (weight-only). `base`: id of
        the first expert held here. `release` drops the references to the checkpoint-layout tensors after the repack."""
        self.experts, n1, self.k = w1.shape[0], w1.shape[1], w1.shape[2] * 2
        self.out_features, self.n = w2.shape[1], w2.shape[2] * 2
        if n1 not in (self.n, 2 * self.n) or w2.shape[0] != self.experts:
            raise ValueError("w1 / w2 shapes do not describe one expert stack")
        self.gated = n1 == 2 * self.n
        self.base = base
        self.tiled1, self.tiled2 = _tile_stack(w1, s1), _tile_stack(w2, s2)
        self.alpha1 = g1.float().reshape(-1).contiguous()
        self.alpha2 = (g2.float().reshape(-1) * routed_scaling).contiguous()
        if self.alpha1.numel() != self.experts or self.alpha2.numel() != self.experts:
            raise ValueError("one weight scale per expert expected")
        self.w1, self.w2, self.s1, self.s2 = (None,) * 4 if release else (w1, w2, s1, s2)

    @property
    def bytes(self) -> int:
        return self.tiled1.numel() + self.tiled2.numel() + 8 * self.experts

    def _struct(self) -> _lib.HbNvfp4Experts:
        return _lib.HbNvfp4Experts(_lib.ptr(self.tiled1), _lib.ptr(self.alpha1), _lib.ptr(self.tiled2), _lib.ptr(self.alpha2),
                                   self.experts, self.base, self.k, self.n, self.out_features, int(self.gated))

    def __call__(self, x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, pairs: bool = False) -> torch.Tensor:
        """BF16 x [M, K], ids / weights [M, k] -> BF16 [M, K_out], the weighted routed sum in selection order
        (hibana/kernels/b12x_moe.py:58-68). With `pairs`, the FP32 outputs per (row, k) pair [M * k, K_out], unsummed."""
        if x.dtype != torch.bfloat16 or x.ndim != 2 or x.shape[1] != self.k:
            raise ValueError("B12xExperts: x must be BF16 [M, K]")
        if ids.ndim != 2 or ids.shape[0] != x.shape[0] or weights.shape != ids.shape:
            raise ValueError("B12xExperts: ids and weights must be [M, k]")
        _lib.need_gpu(x, ids, weights)
        m, topk = ids.shape
        out = torch.empty((m * topk, self.out_features) if pairs else (m, self.out_features),
                          dtype=torch.float32 if pairs else torch.bfloat16, device=x.device)
        if m == 0:
            return out
        st = self._struct()
        need = _lib.lib().hb_nvfp4_moe_workspace_bytes(m, topk, C.byref(st))
        ws = _lib.workspace(x.device, need)
        ids32 = ids.to(torch.int32).contiguous()
        wt = weights.float().contiguous()
        xc = x.contiguous()
        _lib.check(_lib.lib().hb_nvfp4_moe(C.byref(st), _lib.ptr(xc), _lib.ptr(ids32), _lib.ptr(wt), m, topk, int(pairs),
                                           _lib.ptr(out), _lib.ptr(ws), need, _lib.stream()), "nvfp4 experts")
        return out
