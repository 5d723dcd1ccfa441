"""Shared builders for the parity tests: synthetic W3 / NVFP4 weights made with the ORACLE's packers (numpy), handed
to the shipped code in the reference's checkpoint layout, as a loader would."""
from __future__ import annotations

import numpy as np
import torch

from oracle import w3_format as ow3


def random_w3(n, k, seed, codebook="lloyd", per128=False):
    """Oracle-packed random matrix: returns (oracle dict, q, scale bytes, row scale)."""
    g = np.random.default_rng(seed)
    levels = ow3.check_codebook(codebook)
    q = g.integers(0, len(levels), size=(n, k))
    if per128:  # the benchmark's distribution: one draw per 128 along K, |N(0, 0.02)| + 1e-3
        s = np.abs(g.normal(0, 0.02, size=(n, k // 128))).astype(np.float32) + np.float32(1e-3)
        s = np.repeat(s, 4, axis=1)
    else:
        s = (np.abs(g.normal(0, 0.02, size=(n, k // 32))).astype(np.float32) + np.float32(1e-3))
    row = np.maximum(s.max(axis=1) / np.float32(448.0), np.float32(1e-12)).astype(np.float32)
    raw = ow3.e4m3_bytes(s / row[:, None])
    return ow3.pack_codes(q, raw, row, codebook), q, raw, row


def to_device_w3(packed, device="cuda"):
    """Oracle dict -> shipped W3Weight holding the checkpoint-layout tensors."""
    from hibana_amd.kernels import w3
    planes = torch.from_numpy(packed["planes"].view(np.int32).copy()).view(torch.uint32).to(device)
    scales = torch.from_numpy(packed["scales"].copy()).to(device)
    row = torch.from_numpy(packed["row_scale"].copy()).to(device)
    return w3.W3Weight(planes, scales, row, packed["out_features"], packed["in_features"], packed["codebook"], packed["lut"])


def random_experts(e, hidden, inter, gated, seed, codebook="lloyd", fc2_codebook=None, device="cuda"):
    """E oracle-packed experts -> (shipped W3Experts, list of oracle dicts (fc1, fc2) per expert)."""
    from hibana_amd.kernels import w3_moe
    n1 = 2 * inter if gated else inter
    fc2_codebook = fc2_codebook or codebook
    per = [(random_w3(n1, hidden, seed * 1000 + 2 * i, codebook)[0], random_w3(hidden, inter, seed * 1000 + 2 * i + 1, fc2_codebook)[0]) for i in range(e)]

    def stack(idx, name):
        return np.stack([p[idx][name] for p in per])

    def dev(a, dtype=None):
        t = torch.from_numpy(a.copy())
        return t.to(device)

    ex = w3_moe.W3Experts(dev(stack(0, "planes").view(np.int32)).view(torch.uint32), dev(stack(0, "scales")), dev(stack(0, "row_scale")),
                          dev(stack(1, "planes").view(np.int32)).view(torch.uint32), dev(stack(1, "scales")), dev(stack(1, "row_scale")),
                          per[0][0]["codebook"], per[0][0]["lut"], per[0][1]["codebook"], per[0][1]["lut"])
    return ex, per


def oracle_expert_getter(per, gated, inter):
    """get_expert(e) for oracle.layers: (w13 in checkpoint row order [up; gate], w2), dequantized by the oracle."""
    from oracle import layers
    cache = {}
    inverse = np.argsort(layers.fc1_order(inter)) if gated else None

    def get(e):
        if e not in cache:
            w13 = ow3.dequantize(per[e][0])
            cache[e] = (w13[inverse] if gated else w13, ow3.dequantize(per[e][1]))
        return cache[e]
    return get


def errors(actual: torch.Tensor, expected: torch.Tensor):
    """(scale-relative max error, norm-relative error) of two tensors, in FP64."""
    a, e = actual.double().cpu(), expected.double().cpu()
    scale = e.abs().max().clamp_min(1e-30)
    return float((a - e).abs().max() / scale), float((a - e).norm() / e.norm().clamp_min(1e-30))


MAX_REL = 2e-2   # the build's gate: max |y - ref| / max |ref|
NORM_REL = 4e-3  # the reference's own kernel-vs-torch bound (tests/gpu/test_w3_moe.py:33 of the reference)
