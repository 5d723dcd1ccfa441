"""Seeded synthetic weights and routing in the shapes of the benchmark configurations (no checkpoint is read).

W3 matrices: codes uniform in 0..7; one scale draw g = |N(0, 0.02)| + 1e-3 per 128 weights along K, repeated over its
four 32-groups; row_scale = max(g) / 448; stored group scale = e4m3(g / row_scale). Packed with `w3.pack_codes`, the
same entry point calibrated checkpoints load through.
"""
from __future__ import annotations

import torch

from hibana_amd.kernels import w3, w3_moe


def w3_matrix(rows: int, k: int, seed: int, device="cuda", codebook="lloyd", rows_per_piece: int = 65536) -> w3.W3Weight:
    """A random [rows, k] W3 matrix (rows a multiple of 128), generated and packed on `device` in pieces."""
    g = torch.Generator(device=device).manual_seed(seed)
    parts = []
    for r0 in range(0, rows, rows_per_piece):
        n = min(rows_per_piece, rows - r0)
        q = torch.randint(0, len(w3._codebook(codebook)), (n, k), generator=g, device=device, dtype=torch.uint8)  # codes of the book's levels (four: a two-bit matrix)
        s = (torch.randn(n, k // 128, generator=g, device=device).abs() * 0.02 + 1e-3).repeat_interleave(4, dim=1)
        row = (s.amax(dim=1) / torch.tensor(448.0, device=device)).clamp_min(1e-12)
        parts.append(w3.pack_codes(q, (s / row[:, None]).to(torch.float8_e4m3fn), row, codebook))
    if len(parts) == 1:
        return parts[0]
    cat = lambda name: torch.cat([getattr(p, name).view(torch.int32) if getattr(p, name).dtype == torch.uint32 else getattr(p, name) for p in parts])  # noqa: E731
    first = parts[0]
    return w3.W3Weight(cat("planes").view(torch.uint32), cat("scales"), cat("row_scale"), rows, k, first.codebook, first.lut)


def w3_experts(experts: int, hidden: int, inter: int, gated: bool, seed: int, device="cuda", codebook="lloyd",
               release: bool = True) -> w3_moe.W3Experts:
    """`experts` random experts (fc1 rows already in fc1_order: the order is a property of how rows are stored, and
    random rows are random in any order), tiled for the kernels."""
    n1 = 2 * inter if gated else inter
    fc1 = w3_matrix(experts * n1, hidden, 2 * seed, device, codebook)
    fc2 = w3_matrix(experts * hidden, inter, 2 * seed + 1, device, codebook)
    return w3_moe.tile(w3_moe.W3Experts.from_stacked(fc1, fc2, experts), release=release)


def zipf_logits(rows: int, experts: int, s: float, seed: int, device="cuda") -> torch.Tensor:
    """Router logits whose top-k is a draw without replacement from a Zipf(s) popularity over a seeded permutation of
    the experts: log p_e + Gumbel noise, plus a 1e-6 * U(0, 1) jitter that breaks ties by seed."""
    g = torch.Generator().manual_seed(seed)
    rank = torch.randperm(experts, generator=g).double() + 1.0
    logp = -s * rank.log()
    logp = logp - torch.logsumexp(logp, 0)
    u = torch.rand(rows, experts, generator=g, dtype=torch.float64).clamp_min(1e-300)
    gumbel = -(-u.log()).log()
    jitter = 1e-6 * torch.rand(rows, experts, generator=g, dtype=torch.float64)
    return (logp[None, :] + gumbel + jitter).float().to(device)


def nvfp4_experts(experts: int, hidden: int, inter: int, seed: int, device="cuda", global_scale: float = 1.0 / 448.0, routed_scaling: float = 1.0,
                  keep: bool = False):
    """`experts` random ReLU^2 NVFP4 experts (up [inter, hidden], down [hidden, inter]): E2M1 codes uniform over the 16
    codes, one E4M3 scale per 16 drawn as |N(0, 1)| clipped to [2^-6, 448], every matrix's FP32 scale `global_scale`;
    as a `B12xExperts`, block scales handed over in the 128x4 interleave as a checkpoint loader would."""
    from hibana_amd.kernels import b12x_moe
    from hibana_amd.weights.modelopt import swizzle_block_scales
    g = torch.Generator(device=device).manual_seed(seed)

    def stack(rows, k):
        w = torch.randint(0, 256, (experts, rows, k // 2), dtype=torch.uint8, device=device, generator=g)
        sc = torch.randn(experts, rows, k // 16, device=device, generator=g).abs().clamp(2.0 ** -6, 448.0).to(torch.float8_e4m3fn)
        return w, torch.stack([swizzle_block_scales(sc[e]) for e in range(experts)]), torch.full((experts,), global_scale, device=device)

    w1, s1, g1 = stack(inter, hidden)
    w2, s2, g2 = stack(hidden, inter)
    return b12x_moe.B12xExperts(w1, s1, g1, 1.0, w2, s2, g2, 1.0, routed_scaling=routed_scaling, release=not keep)


def nvfp4_linear(out_features: int, in_features: int, seed: int, device="cuda", global_scale: float = 1.0 / 448.0):
    """A random NVFP4 linear as `nvfp4_experts` draws its matrices, tiled: an `Nvfp4Linear` a loader would hand over."""
    from hibana_amd.weights import modelopt
    g = torch.Generator(device=device).manual_seed(seed)
    w = torch.randint(0, 256, (out_features, in_features // 2), dtype=torch.uint8, device=device, generator=g)
    sc = torch.randn(out_features, in_features // 16, device=device, generator=g).abs().clamp(2.0 ** -6, 448.0).to(torch.float8_e4m3fn)
    return modelopt.Nvfp4Linear(w, modelopt.swizzle_block_scales(sc), torch.tensor(global_scale, device=device), torch.tensor(1.0, device=device),
                                out_features, in_features).tile()
