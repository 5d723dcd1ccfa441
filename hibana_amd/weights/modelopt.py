"""ModelOpt NVFP4 linears on MI355X (hibana/weights/modelopt.py:57-156 of the reference): E2M1 codes two per byte
(element 2i in the low nibble), one E4M3 scale per 16 weights stored in the CUTLASS 128x4 interleave, an FP32 global
scale alpha * input_scale_inv (= weight_scale_2). `tile()` repacks codes and scales once into the block layout the
gfx950 kernels stream (csrc/nvfp4.hip).

The served op is weight-only (BF16 activations); `input_scale_inv` only takes part in the global scale.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from hibana_amd import _lib

FP8_MAX = 448.0


def _offsets(rows: int, groups: int, device):
    gp = (groups + 3) // 4 * 4
    r = torch.arange(rows, device=device)[:, None]
    c = torch.arange(groups, device=device)[None, :]
    return (r // 128) * (128 * gp) + (c // 4) * 512 + (r % 32) * 16 + ((r // 32) % 4) * 4 + c % 4


def swizzle_block_scales(scales: torch.Tensor) -> torch.Tensor:
    """[R, G] block scales -> the 128-row / four-column interleave [R_pad128, G_pad4], padding zero
    (hibana/weights/modelopt.py:130-139)."""
    rows, groups = scales.shape
    rp, gp = (rows + 127) // 128 * 128, (groups + 3) // 4 * 4
    raw = scales.view(torch.uint8) if scales.dtype == torch.float8_e4m3fn else scales
    out = torch.zeros(rp * gp, dtype=raw.dtype, device=scales.device)
    out[_offsets(rows, groups, scales.device).reshape(-1)] = raw.reshape(-1)
    out = out.reshape(rp, gp)
    return out.view(torch.float8_e4m3fn) if scales.dtype == torch.float8_e4m3fn else out


def unswizzle_block_scales(scales: torch.Tensor, rows: int, groups: int) -> torch.Tensor:
    """Decode the interleave, removing padding (hibana/weights/modelopt.py:142-147)."""
    rp, gp = (rows + 127) // 128 * 128, (groups + 3) // 4 * 4
    if scales.numel() != rp * gp:
        raise ValueError("scale extent does not match padded matrix")
    return scales.reshape(-1)[_offsets(rows, groups, scales.device)]


def swizzle_block_scales_batched(scales: torch.Tensor) -> torch.Tensor:
    """[E, R, G] float8_e4m3fn -> the interleave per expert, viewed as int32 [E, R_pad, G_pad/4]
    (hibana/model/flashnext/moe.py:22-29)."""
    return torch.stack([swizzle_block_scales(s).view(torch.uint8) for s in scales]).view(torch.int32)


def pair_order(rows: int, block: int) -> torch.Tensor:
    from hibana_amd.kernels.w3 import pair_order as order
    return order(rows, block)


@dataclass
class Nvfp4Linear:
    weight: torch.Tensor  # [N, K/2] uint8
    weight_scale_swizzled: torch.Tensor  # [N_pad128, (K/16)_pad4] float8_e4m3fn
    alpha: torch.Tensor  # [] float32 = input_scale * weight_scale_2
    input_scale_inv: torch.Tensor  # [] float32
    out_features: int
    in_features: int
    w3: object = None
    pairs: int = 0
    tiled: torch.Tensor | None = None  # the kernels' block layout (built by tile())
    scale2: float | None = None  # alpha * input_scale_inv as a host float, read from the device ONCE (by tile())

    @property
    def bytes(self) -> int:
        return self.w3.bytes if self.w3 is not None else self.weight.numel() + self.weight_scale_swizzled.numel()

    @property
    def global_scale(self) -> float:
        """The FP32 scale of the matrix as the kernels take it (an argument of the launch). Reading it from the device
        is a synchronization, so it happens once, at load time (`tile()`), never on the call path; assigning new
        `alpha` / `input_scale_inv` tensors needs `scale2 = None` to be read again."""
        if self.scale2 is None:
            self.scale2 = float((self.alpha.float() * self.input_scale_inv.float()).item())
        return self.scale2

    def tile(self) -> "Nvfp4Linear":
        _ = self.global_scale
        if self.tiled is None:
            _lib.need_gpu(self.weight, self.weight_scale_swizzled)
            n, k = self.out_features, self.in_features
            size = _lib.lib().hb_nvfp4_tiled_bytes(n, k)
            if size == 0:
                raise ValueError("NVFP4 kernels need N a multiple of 64 and K a multiple of 128")
            tiled = torch.empty(size, dtype=torch.uint8, device=self.weight.device)
            scales = self.weight_scale_swizzled.contiguous().view(torch.uint8)
            codes = self.weight.contiguous()
            _lib.check(_lib.lib().hb_nvfp4_repack(_lib.ptr(codes), _lib.ptr(scales), 1, n, k, _lib.ptr(tiled), _lib.stream()),
                       "nvfp4 repack")
            self.tiled = tiled
        return self

    def dequantize(self) -> torch.Tensor:
        """FP32 [N, K]: unpack_fp4 times the global scale (hibana/weights/modelopt.py:73-77)."""
        self.tile()
        out = torch.empty((self.out_features, self.in_features), dtype=torch.float32, device=self.weight.device)
        _lib.check(_lib.lib().hb_nvfp4_dequant(_lib.ptr(self.tiled), self.global_scale, self.out_features, self.in_features, _lib.ptr(out),
                                               _lib.stream()), "nvfp4 dequantize")
        return out

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        from hibana_amd.kernels import ops
        return ops.nvfp4_linear(x, self)


def unpack_fp4(packed: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """Dequantize low-nibble-first E2M1 weights with one scale per 16 values -> FP32 [R, K]
    (hibana/weights/modelopt.py:150-156). R a multiple of 64 and K of 128 (the kernels' block)."""
    if packed.ndim != 2 or packed.shape[1] % 8 or scales.shape != (packed.shape[0], packed.shape[1] // 8):
        raise ValueError("expected packed rows and one scale per sixteen values")
    _lib.need_gpu(packed, scales)
    rows, k = packed.shape[0], packed.shape[1] * 2
    size = _lib.lib().hb_nvfp4_tiled_bytes(rows, k)
    if size == 0:
        raise ValueError("NVFP4 kernels need rows a multiple of 64 and K a multiple of 128")
    tiled = torch.empty(size, dtype=torch.uint8, device=packed.device)
    raw = scales.contiguous().view(torch.uint8) if scales.dtype == torch.float8_e4m3fn else scales.contiguous()
    codes = packed.contiguous()
    _lib.check(_lib.lib().hb_nvfp4_repack(_lib.ptr(codes), _lib.ptr(raw), 0, rows, k, _lib.ptr(tiled), _lib.stream()), "nvfp4 repack")
    out = torch.empty((rows, k), dtype=torch.float32, device=packed.device)
    _lib.check(_lib.lib().hb_nvfp4_dequant(_lib.ptr(tiled), 1.0, rows, k, _lib.ptr(out), _lib.stream()), "unpack_fp4")
    return out


def interleave_pairs(lin: Nvfp4Linear, block: int) -> Nvfp4Linear:
    """`lin` (an MLP's gate|up) with its rows interleaved in blocks of `block` (hibana/weights/modelopt.py:89-101)."""
    if lin.w3 is not None or lin.pairs or lin.out_features % (2 * block):
        raise ValueError(f"cannot interleave {lin.out_features} rows in blocks of {block}")
    order = pair_order(lin.out_features, block).to(lin.weight.device)
    scales = unswizzle_block_scales(lin.weight_scale_swizzled.view(torch.uint8).reshape(-1), lin.out_features, lin.in_features // 16)
    lin.weight = lin.weight[order].contiguous()
    lin.weight_scale_swizzled = swizzle_block_scales(scales[order]).view(torch.float8_e4m3fn)
    lin.pairs = block
    lin.tiled = None
    return lin
