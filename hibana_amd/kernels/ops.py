"""Kernel entry points of the quantized linear / MoE path (hibana/kernels/ops.py:50-92 of the reference, plus the
routing and combine ops of hibana/kernels/flashnext_fused.py that sit either side of the experts)."""
from __future__ import annotations

import torch

from hibana_amd import _lib
from hibana_amd.kernels import w3


def w3_decode(lin, m: int, rows: int | None = None) -> bool:
    """True when this call runs the 3-bit decode copy instead of the NVFP4 weights: at most `rows` rows (None:
    w3.MAX_ROWS) (hibana/kernels/ops.py:50-53)."""
    return lin.w3 is not None and m <= (rows or w3.MAX_ROWS) and w3.enabled()


def nvfp4_linear(x: torch.Tensor, lin, prequantized=None, relu2: bool = False) -> torch.Tensor:
    """BF16 x [M, K] -> BF16 [M, N] on NVFP4 weights, weight-only: bf16((x Wq^T)_fp32 * global scale); the 3-bit copy
    serves the call when one is attached and enabled (hibana/kernels/ops.py:56-83). No host synchronization on the
    call path once `lin.tile()` has run (it caches the global scale as a host float), so the call can be captured."""
    if prequantized is not None:
        raise ValueError("nvfp4_linear: NVFP4 activations are not taken by the weight-only kernels")
    if x.dtype == torch.bfloat16 and w3_decode(lin, x.shape[0]) and not relu2:
        return w3.w3_linear(x, lin.w3)
    if x.dtype != torch.bfloat16 or x.ndim != 2 or x.shape[1] != lin.in_features:
        raise ValueError("nvfp4_linear: x must be BF16 [M, in_features]")
    _lib.need_gpu(x)
    lin.tile()
    m = x.shape[0]
    y = torch.empty((m, lin.out_features), dtype=torch.bfloat16, device=x.device)
    if m:
        xc = x.contiguous()  # held until the launch is enqueued: a temporary's block could be handed out again before that
        need = _lib.lib().hb_nvfp4_gemm_workspace_bytes(m, lin.out_features, lin.in_features)  # a few dozen rows: K shared among workgroups
        ws = _lib.workspace(x.device, need, "gemm") if need else None
        _lib.check(_lib.lib().hb_nvfp4_gemm_ws(_lib.ptr(xc), m, _lib.ptr(lin.tiled), lin.global_scale, lin.out_features, lin.in_features, int(relu2),
                                               _lib.ptr(y), _lib.ptr(ws), need, _lib.stream()), "nvfp4_linear")
    return y


def silu_and_mul(gate_up: torch.Tensor, pairs: int = 0) -> torch.Tensor:
    """silu(gate) * up of BF16 [..., gate | up], or (`pairs`) of gate and up alternating in blocks of `pairs` columns
    (hibana/kernels/ops.py:86-92), on the GPU; the roundings are those of the BF16 tensor expression."""
    if gate_up.dtype != torch.bfloat16 or gate_up.shape[-1] % 4 or (pairs and (pairs % 2 or (gate_up.shape[-1] // 2) % pairs)):
        raise ValueError("silu_and_mul: BF16 [..., 2 * half], half even (and a multiple of an even `pairs`)")
    _lib.need_gpu(gate_up)
    half = gate_up.shape[-1] // 2
    flat = gate_up.reshape(-1, 2 * half).contiguous()
    out = torch.empty((flat.shape[0], half), dtype=torch.bfloat16, device=gate_up.device)
    if flat.shape[0]:
        _lib.check(_lib.lib().hb_silu_and_mul(_lib.ptr(flat), flat.shape[0], half, pairs, _lib.ptr(out), _lib.stream()), "silu_and_mul")
    return out.reshape(*gate_up.shape[:-1], half)


def silu_mul(gate_up: torch.Tensor, pairs: int = 0) -> torch.Tensor:
    """bf16(silu(gate) * up) of BF16 [M, 2 I] from the FP32 product, one rounding (hibana/kernels/flashnext_fused.py:
    624-639); columns as in `silu_and_mul`."""
    if gate_up.dtype != torch.bfloat16 or gate_up.ndim != 2 or gate_up.shape[1] % 4:
        raise ValueError("silu_mul: BF16 [M, 2 I] with I even")
    half = gate_up.shape[1] // 2
    if pairs and (pairs % 2 or half % pairs):
        raise ValueError("silu_mul: pairs must be even and divide I")
    _lib.need_gpu(gate_up)
    gu = gate_up.contiguous()
    out = torch.empty((gu.shape[0], half), dtype=torch.bfloat16, device=gu.device)
    if gu.shape[0]:
        _lib.check(_lib.lib().hb_silu_mul(_lib.ptr(gu), gu.shape[0], half, pairs, _lib.ptr(out), _lib.stream()), "silu_mul")
    return out


def silu_mul_quant_groups(gate_up: torch.Tensor, pairs: int = 0, torch_chain: bool = False):
    """`w3.quant_groups(silu_mul(gate_up))` in one launch, bit for bit: BF16 [M, 2I] -> (E4M3 [M, I], FP32 scales
    [M, I/32]); `pairs`: gate and up interleaved in blocks of that many columns; `torch_chain`: the product as
    `silu_and_mul` rounds it (hibana/kernels/flashnext_fused.py:841-853), the dense MLP's 3-bit decode input
    (hibana/model/mlp.py:36-42)."""
    if gate_up.dtype != torch.bfloat16 or gate_up.ndim != 2 or gate_up.stride(1) != 1 or gate_up.shape[1] % 64:
        raise ValueError("silu_mul_quant_groups: BF16 [M, 2 I] with I a multiple of 32")
    half = gate_up.shape[1] // 2
    if pairs and (pairs % 32 or half % pairs):
        raise ValueError("silu_mul_quant_groups: pairs must be a multiple of 32 dividing I")
    _lib.need_gpu(gate_up)
    gu = gate_up.contiguous()
    m = gu.shape[0]
    q = torch.empty((m, half), dtype=torch.float8_e4m3fn, device=gu.device)
    scales = torch.empty((m, half // 32), dtype=torch.float32, device=gu.device)
    if m:
        _lib.check(_lib.lib().hb_silu_mul_quant_groups(_lib.ptr(gu), m, half, pairs, int(torch_chain), _lib.ptr(q), _lib.ptr(scales), _lib.stream()),
                   "silu_mul_quant_groups")
    return q, scales


def route_topk(logits: torch.Tensor, k: int, slots: torch.Tensor | None = None, steps: int = 1, repeat: bool = False):
    """[M, E] FP32 logits -> (int32 ids [M, k], FP32 renormalized softmax weights [M, k]), largest first. With `slots`,
    row r is real iff slots[r // steps] != 0; a padded row takes expert E at weight 0 (the 3-bit experts skip it) or,
    `repeat`, row 0's first choice at weight 0 (hibana/kernels/flashnext_fused.py:308-319)."""
    _lib.need_gpu(logits, slots)
    m, e = logits.shape
    lg = logits.float().contiguous()
    sl = None if slots is None else slots.to(torch.int32).contiguous()
    ids = torch.empty((m, k), dtype=torch.int32, device=logits.device)
    w = torch.empty((m, k), dtype=torch.float32, device=logits.device)
    if m:
        _lib.check(_lib.lib().hb_route_softmax_topk(_lib.ptr(lg), m, e, k, _lib.ptr(sl), steps, int(repeat), _lib.ptr(ids), _lib.ptr(w),
                                                    _lib.stream()), "route_topk")
    return ids, w


ROUTE_CANDIDATES = 20  # a row takes its experts from its 20 largest logits


def route_budget(logits: torch.Tensor, k: int, keep: int, budget: int, slots: torch.Tensor | None = None, steps: int = 1,
                 repeat: bool = False, per_request: int = 0, min_cap: int = 0):
    """Budgeted top-k (hibana/kernels/flashnext_fused.py:462-502): BF16 [R, E] logits -> (int32 ids [R, k], FP32 weights
    [R, k]). The experts the call reads are chosen for the whole call under a cap: every real row's top `keep`, then the
    experts with the most softmax probability within the real rows' top k until the set holds the cap (`budget`, or
    with `per_request`, min(budget, max(min_cap, per_request x the real requests))); each real row takes its candidates
    (its 20 largest logits, an exact tie to the lower expert) in the set, in rank order, up to k, its weights the
    softmax over E renormalized over them. Slots left over (all of a padded row's: slots[r // steps] == 0) hold id E at
    weight 0, or with `repeat` the row's top 1 (a padded row: row 0's)."""
    if logits.dtype != torch.bfloat16 or logits.ndim != 2:
        raise ValueError("route_budget: BF16 [R, E] logits")
    r, e = logits.shape
    if not (ROUTE_CANDIDATES <= e <= 1024 and 1 <= k <= ROUTE_CANDIDATES and 0 <= keep <= ROUTE_CANDIDATES) or budget < 0 or steps < 1 or r % steps:
        raise ValueError("route_budget: 20 <= E <= 1024, k and keep at most 20, whole requests of `steps` rows")
    if slots is not None and slots.numel() < r // steps:
        raise ValueError("route_budget: a slot for every request")
    _lib.need_gpu(logits, slots)
    lg = logits.contiguous()
    sl = None if slots is None else slots.to(torch.int32).contiguous()
    ids = torch.empty((r, k), dtype=torch.int32, device=logits.device)
    w = torch.empty((r, k), dtype=torch.float32, device=logits.device)
    if r:
        ws = torch.empty((_lib.lib().hb_route_budget_workspace_bytes(r),), dtype=torch.uint8, device=logits.device)
        _lib.check(_lib.lib().hb_route_budget(_lib.ptr(lg), r, e, k, keep, budget, _lib.ptr(sl), steps, int(repeat), per_request, min_cap,
                                              _lib.ptr(ws), ws.numel(), _lib.ptr(ids), _lib.ptr(w), _lib.stream()), "route_budget")
    return ids, w


def moe_combine_pairs(y: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, shared: torch.Tensor | None, x: torch.Tensor | None,
                      gate_w: torch.Tensor | None, e_lo: int = 0, e_n: int = 512) -> torch.Tensor:
    """bf16(bf16(sum_k w_k y_k over this rank's pairs, in slot order) + sigmoid(x . gate_w) * shared) from the unsummed
    pair outputs y [m * topk, H] (FP32 or BF16) (hibana/kernels/flashnext_fused.py:556-571). `shared` None: the
    routed sum alone; `gate_w` None: the shared output is added ungated."""
    _lib.need_gpu(y, ids, weights)
    m, topk = ids.shape
    h = y.shape[1]
    out = torch.empty((m, h), dtype=torch.bfloat16, device=y.device)
    if m == 0:
        return out
    if y.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("moe_combine_pairs: pairs must be FP32 or BF16")
    if y.shape[0] != m * topk or weights.shape != ids.shape or (shared is not None and tuple(shared.shape) != (m, h)):
        raise ValueError("moe_combine_pairs: y [M * k, H], ids / weights [M, k], shared [M, H]")
    if gate_w is not None and shared is not None and (x is None or tuple(x.shape) != (m, h) or gate_w.numel() != h):
        raise ValueError("moe_combine_pairs: the gate takes x [M, H] and gate_w [H] (the layer's input rows)")
    # every converted operand is bound to a name until the launch is enqueued
    yc, ids32, wt = y.contiguous(), ids.to(torch.int32).contiguous(), weights.float().contiguous()
    sh = None if shared is None else shared.to(torch.bfloat16).contiguous()
    xx = None if x is None else x.to(torch.bfloat16).contiguous()
    gw = None if gate_w is None else gate_w.float().reshape(-1).contiguous()
    _lib.check(_lib.lib().hb_moe_combine_pairs(_lib.ptr(yc), int(y.dtype == torch.bfloat16), _lib.ptr(ids32), _lib.ptr(wt), _lib.ptr(sh),
                                               _lib.ptr(xx), _lib.ptr(gw), e_lo, e_n, m, topk, h, _lib.ptr(out), _lib.stream()),
               "moe_combine_pairs")
    return out


def moe_combine(routed: torch.Tensor, shared: torch.Tensor, x: torch.Tensor, gate_w: torch.Tensor) -> torch.Tensor:
    """bf16(routed + sigmoid(x . gate_w) * shared) for BF16 routed / shared [M, H] (hibana/kernels/flashnext_fused.py:
    506-526): the combine kernel on one pair a row at weight 1, whose rounded sum is `routed` itself."""
    if routed.dtype != torch.bfloat16 or routed.ndim != 2 or shared.shape != routed.shape or x.shape != routed.shape or gate_w.numel() != routed.shape[1]:
        raise ValueError("moe_combine: routed, shared and x must be BF16 [M, H] of one shape, gate_w [H]")
    m = routed.shape[0]
    ids = torch.zeros((m, 1), dtype=torch.int32, device=routed.device)
    ones = torch.ones((m, 1), dtype=torch.float32, device=routed.device)
    return moe_combine_pairs(routed, ids, ones, shared, x, gate_w, 0, 1)

