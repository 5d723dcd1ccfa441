"""The dense SwiGLU MLP behind the reference's `Mlp.__call__` (hibana/model/mlp.py:26-48): gate|up and down as NVFP4
linears, each with an optional 3-bit decode copy.

    gate_up = nvfp4_linear(x, gate_up)                         (its 3-bit copy at decode sizes, weight-only)
    3-bit decode of `down`:  x_q, s = silu_mul_quant_groups(gate_up, pairs, torch_chain=True);  w3_linear(x_q, down.w3, s)
    otherwise:               nvfp4_linear(silu_and_mul(gate_up, pairs), down)

Assembled from linears already loaded. The reference's NVFP4 activation paths (`prequantized`, the fused prefill
gate/up GEMM that rounds SiLU(gate) * up to NVFP4 in its epilogue) have no counterpart: the NVFP4 kernels here are
weight-only.
"""
from __future__ import annotations

import torch

from hibana_amd.kernels import ops, w3


class Mlp:
    def __init__(self, gate_up, down):
        """gate_up: `Nvfp4Linear` [2 I, H], rows [gate; up] or interleaved in blocks of `gate_up.pairs`; down [H, I]."""
        if gate_up.out_features != 2 * down.in_features or down.out_features != gate_up.in_features:
            raise ValueError("gate_up [2 I, H] and down [H, I] do not describe one MLP")
        self.gate_up, self.down = gate_up, down

    def __call__(self, x: torch.Tensor, prequantized=None) -> torch.Tensor:
        """x [rows, H] BF16 -> BF16 [rows, H]."""
        if prequantized is not None:
            raise ValueError("Mlp: NVFP4 activations are not taken by the weight-only kernels")
        gate_up = ops.nvfp4_linear(x, self.gate_up)
        pairs = self.gate_up.pairs
        if ops.w3_decode(self.down, gate_up.shape[0]):
            # 3-bit decode: the SiLU product in BF16 rounded per 32-group for the 3-bit GEMM, in one launch
            x_q, x_scale = ops.silu_mul_quant_groups(gate_up, pairs, torch_chain=True)
            return w3.w3_linear(x_q, self.down.w3, x_scale)
        return ops.nvfp4_linear(ops.silu_and_mul(gate_up, pairs), self.down)
