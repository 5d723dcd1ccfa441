"""Oracle restatement of the layer math on the quantized-weight path (test infrastructure, see oracle/__init__.py).

Weight-only numerics: BF16 activations, exactly dequantized weights, FP32 (or wider) accumulation, the rounding
points of the reference kept.

  dense_ref              x.float() @ W_deq.T, one rounding to BF16  (profiling/w3_bench.py:75 `y_exact`;
                         hibana/kernels/w3.py:239-242 for W_deq)
  nvfp4_dense_ref        bf16((x @ Wq^T)_fp32 * s2), Wq = e2m1 * e4m3 exact in BF16
                         (tests/nemotron_reference.py:236-254; tests/gpu/test_bolt_kernels.py:29-32)
  fc1_order              hibana/kernels/w3_moe.py:88-92
  expert_plan            hibana/kernels/csrc/w3_gemm.cu:710-782: ascending distinct local experts, CSR starts, pair
                         indices of each expert in ascending order (a stable sort by expert)
  routed_experts_ref     hibana/kernels/w3_moe.py:193-214 with an identity `quant` (weight-only): h1 = bf16(fc1 x),
                         h = bf16(silu(gate) * up) or bf16(relu(h1)^2) with an FP32 square, y = fc2 h in FP32 per pair
  combine_ref            hibana/kernels/csrc/w3_gemm.cu:1196-1213: v = fma(w_k, y_k, v) over the row's slots in
                         selection order, skipping ids outside the local range, one rounding to BF16
  combine_shared_ref     hibana/kernels/flashnext_fused.py:530-571: bf16(bf16(routed) + sigmoid(x . g) * shared)
  route_softmax_topk     hibana/model/flashnext/moe.py:141-144 (== flashnext_fused.py:278-319): softmax, top-k
                         descending, renormalized
  route_sigmoid_topk     hibana/model/nemotron/moe.py:1-12, tests/nemotron_reference.py:550-565: top-k of
                         sigmoid + bias (ties to the lower id), weights from the plain sigmoid, renormalized, scaled
  route_budget_ref       hibana/kernels/flashnext_fused.py:322-502 (the rank / score / select / pick launches) with the
                         rule as tests/unit/test_moe_selection.py:19-58 writes it out row by row: candidates = the 20
                         largest logits (ties to the lower expert, -0 == +0), core = real rows' top keep, score = sum
                         in row order of the FP32 softmax within the real rows' top k, the set = core + best-scoring
                         others (score > 0, equal scores to the lower expert) up to the cap, rows take their
                         candidates in the set in rank order
  route_budget_sigmoid_ref  hibana/model/nemotron/moe.py:124-313: the same selection (`budget_rule`) on the top k by
                         sigmoid + bias, plain-sigmoid weights over (sum + 1e-20), shares renormalized over the
                         row's k, a `fallback` guarantee when the rows' top keep exceed the cap
  silu_mul               hibana/kernels/flashnext_fused.py:624-639: bf16(silu(gate) * up) from the FP32 product
  latent_moe_ref         tests/nemotron_reference.py:568-593 (ReLU^2 latent experts, BF16 linears, FP32 accumulate)
  silu_and_mul           hibana/kernels/ops.py:86-92
  quant_e4m3_groups      hibana/kernels/w3_moe.py:187-190 (the torch mirror of the activation rounding, the definition
                         to follow; the CUDA quantizer of hibana/kernels/csrc/w3_gemm.cu:291-327 multiplies by an
                         approximate reciprocal instead of dividing, so its bits are PARITY UNPINNED here): per (row,
                         32-group) s = max(amax / 448, 1e-12) in FP32, q = e4m3(clamp(x / s, -448, 448))
  quant_e4m3_rows        hibana/kernels/w3.py:326-330: the same rounding with one scale a row (pinned as quant_e4m3_groups:
                         the brute-force nearest-value search, and a row of one group equals the group form)
  dense_a8_ref           hibana/kernels/w3.py:340-365 with quantized activations (the reference kernel's own math,
                         hibana/kernels/csrc/w3_gemm.cu:105-108,209-210): x is replaced by q * s
  `quant=` of the expert functions: hibana/kernels/w3_moe.py:193-214 with quant = quant_e4m3 (x and h both rounded)

Pinned by (tests/test_oracle_layers.py): special cases that reduce to textbook routines (one token, one expert, weight
one == two dense products; all weights zero == zero; a permutation of slots with equal weights), brute-force
per-pair Python loops on tiny shapes written from the formula in w3_moe.py:205-213, torch.topk/softmax for the
routing, and sortedness/CSR invariants for the plan. quant_e4m3_groups: a brute-force nearest-value search over the
256-entry E4M3 table (ties to the even code) on random and hand-made groups, the group maximum landing on +-448 * s, and
groups that are already E4M3 multiples of their scale coming back unchanged. route_budget_ref: a hand-worked call
whose set and rows follow from the rule by inspection, a cap no smaller than the rows' top-k union == a stable
descending sort's top k with the renormalized softmax of torch, padded requests == the call on the real rows alone, and
the invariants the reference's own unit test states (tests/unit/test_moe_selection.py:66-106).
route_budget_sigmoid_ref: a hand-worked call (bias choosing, plain sigmoids weighing, the fallback guarantee), a cap
that holds every row's top k == route_sigmoid_topk, and the invariants of tests/gpu/test_bolt_kernels.py:188-216.
"""
from __future__ import annotations

import numpy as np
import torch


def bf16(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16)


def dense_ref(x: torch.Tensor, w_deq, wide: bool = True) -> torch.Tensor:
    """x BF16 [M, K], w_deq float32 [N, K] -> BF16 [M, N]; accumulation in FP64 (`wide`) or FP32."""
    w = torch.as_tensor(w_deq)
    if wide:
        return bf16((x.double() @ w.double().T).float())
    return bf16(x.float() @ w.float().T)


def nvfp4_dense_ref(x: torch.Tensor, w_unscaled, scale2: float, relu2: bool = False) -> torch.Tensor:
    """x BF16 [M, K], w_unscaled float32 [N, K] = e2m1 * e4m3 (no global scale) -> BF16 [M, N]."""
    w = torch.as_tensor(w_unscaled)
    y = bf16(((x.double() @ w.double().T).float() * np.float32(scale2)))
    if relu2:
        y = bf16(torch.relu(y.float()).square())
    return y


def quant_e4m3_groups(t: torch.Tensor):
    """t [M, K] (K % 32 == 0) -> (E4M3 bytes uint8 [M, K], scales float32 [M, K/32])."""
    m, k = t.shape
    g = t.float().reshape(m, k // 32, 32)
    s = (g.abs().amax(-1, keepdim=True) / 448.0).clamp_min(1e-12)
    q = (g / s).clamp(-448, 448).to(torch.float8_e4m3fn)
    return q.view(torch.uint8).reshape(m, k), s.reshape(m, k // 32)


def quant_e4m3_rows(t: torch.Tensor):
    """t [M, K] -> (E4M3 bytes uint8 [M, K], scales float32 [M]): one scale a row, s = max(amax of the row / 448, 1e-12),
    q = e4m3(clamp(x / s, -448, 448)) (hibana/kernels/w3.py:326-330; the CUDA kernel, hibana/kernels/csrc/
    w3_gemm.cu:244-288, multiplies by a reciprocal: the divisions here are exact, as in quant_e4m3_groups)."""
    f = t.float()
    s = (f.abs().amax(-1, keepdim=True) / 448.0).clamp_min(1e-12)
    q = (f / s).clamp(-448, 448).to(torch.float8_e4m3fn)
    return q.view(torch.uint8), s.reshape(-1)


def dequant_e4m3_groups(q: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    """float32 [M, K] = e4m3(q) * s, a group's scale over its 32 columns."""
    m, k = q.shape
    return (q.view(torch.float8_e4m3fn).float().reshape(m, k // 32, 32) * s.reshape(m, k // 32, 1)).reshape(m, k)


def rounded_e4m3(t: torch.Tensor) -> torch.Tensor:
    """t through the activation rounding and back: what the E4M3-activation kernels multiply with."""
    return dequant_e4m3_groups(*quant_e4m3_groups(t))


def dense_a8_ref(x: torch.Tensor, w_deq) -> torch.Tensor:
    """x [M, K] rounded to E4M3 per (row, 32-group), times w_deq float32 [N, K], one rounding to BF16."""
    return bf16((rounded_e4m3(x).double() @ torch.as_tensor(w_deq).double().T).float())


def fc1_order(inter: int) -> np.ndarray:
    out = np.empty(2 * inter, dtype=np.int64)
    for b in range(inter // 16):
        out[32 * b:32 * b + 16] = 16 * b + np.arange(16)
        out[32 * b + 16:32 * b + 32] = inter + 16 * b + np.arange(16)
    return out


def expert_plan(ids: np.ndarray, e_lo: int, e_n: int):
    """ids int [M, k] -> (experts ascending local ids [D], starts [D+1], order [sum counts] pair indices q = r*k + slot).
    Pairs whose id is outside [e_lo, e_lo + e_n) are dropped."""
    flat = np.asarray(ids).reshape(-1).astype(np.int64) - e_lo
    valid = (flat >= 0) & (flat < e_n)
    experts = np.unique(flat[valid])
    starts = [0]
    order = []
    for e in experts:
        q = np.nonzero(flat == e)[0]  # ascending
        order.extend(q.tolist())
        starts.append(len(order))
    return experts, np.asarray(starts, dtype=np.int64), np.asarray(order, dtype=np.int64)


def silu_and_mul(gate_up: torch.Tensor, pairs: int = 0) -> torch.Tensor:
    half = gate_up.shape[-1] // 2
    if pairs:
        blocks = gate_up.unflatten(-1, (half // pairs, 2, pairs))
        return (torch.nn.functional.silu(blocks[..., 0, :]) * blocks[..., 1, :]).flatten(-2)
    return torch.nn.functional.silu(gate_up[..., :half]) * gate_up[..., half:]


def expert_pairs_ref(x: torch.Tensor, rows: np.ndarray, w13, w2, gated: bool, quant=None) -> torch.Tensor:
    """One expert on the token rows `rows` of x: w13 float32 [N1, K] with rows in checkpoint order ([up; gate] when
    gated, up alone otherwise), w2 float32 [H, I] -> FP32 [len(rows), H]. `quant` (None: weight-only) rounds x and h
    before their products, as the reference's `quant` argument does."""
    w13, w2 = torch.as_tensor(w13).double(), torch.as_tensor(w2).double()
    xr = x[torch.as_tensor(rows)]
    h1 = bf16(((quant(xr) if quant else xr).double() @ w13.T).float()).float()
    if gated:
        inter = w13.shape[0] // 2
        h = bf16(torch.nn.functional.silu(h1[:, inter:]) * h1[:, :inter])
    else:
        h = bf16(torch.relu(h1).square())
    return ((quant(h) if quant else h).double() @ w2.T).float()


def routed_experts_ref(x: torch.Tensor, ids: np.ndarray, get_expert, gated: bool, e_lo: int = 0, e_n: int = 512, quant=None):
    """FP32 pair outputs [M*k, H] (rows of dropped pairs are zero). get_expert(local id) -> (w13 [N1, K] float32 in
    checkpoint row order, w2 [H, I] float32)."""
    ids = np.asarray(ids)
    m, k = ids.shape
    experts, starts, order = expert_plan(ids, e_lo, e_n)
    pairs = None
    for d, e in enumerate(experts):
        q = order[starts[d]:starts[d + 1]]
        w13, w2 = get_expert(int(e))
        y = expert_pairs_ref(x, q // k, w13, w2, gated, quant)
        if pairs is None:
            pairs = torch.zeros(m * k, y.shape[1], dtype=torch.float32)
        pairs[torch.as_tensor(q)] = y
    return pairs


def combine_ref(pairs: torch.Tensor, ids: np.ndarray, weights: torch.Tensor, e_lo: int = 0, e_n: int = 512) -> torch.Tensor:
    """BF16 [M, H]: the FMA chain over the slots in selection order (an FP32 FMA is one rounding of the exact
    a*b + c, reproduced here in FP64: the product of two FP32 values is exact there)."""
    ids = np.asarray(ids)
    m, k = ids.shape
    v = torch.zeros(m, pairs.shape[1], dtype=torch.float32)
    w = weights.float()
    for slot in range(k):
        local = ids[:, slot] - e_lo
        keep = torch.as_tensor((local >= 0) & (local < e_n))
        y = pairs.view(m, k, -1)[:, slot]
        nxt = (v.double() + w[:, slot, None].double() * y.double()).float()
        v = torch.where(keep[:, None], nxt, v)
    return bf16(v)


def combine_shared_ref(routed: torch.Tensor, shared: torch.Tensor, x: torch.Tensor = None, gate_vec: torch.Tensor = None):
    """bf16(routed + g * shared) with g = sigmoid(x . gate_vec) in FP32, or 1 when no gate vector is given."""
    r, s = routed.float(), shared.float()
    if gate_vec is None:
        return bf16(r + s)
    g = torch.sigmoid((x.double() @ gate_vec.double()).float())[:, None]
    return bf16(r + g * s)


def moe_layer_ref(x, ids, weights, get_expert, gated: bool, shared=None, gate_vec=None, e_lo: int = 0, e_n: int = 512, quant=None):
    """The gated-MoE layer of hibana/model/flashnext/moe.py:177-192 on 3-bit experts: routed sum, plus the shared
    expert (w13, w2 in checkpoint row order) rounded to BF16 on its own, combined as combine_shared_ref. `quant`: the
    activation rounding of the expert functions, for every expert."""
    pairs = routed_experts_ref(x, ids, get_expert, gated, e_lo, e_n, quant)
    if pairs is None:
        width = shared[1].shape[0] if shared is not None else x.shape[1]
        pairs = torch.zeros(np.asarray(ids).size, width)
    routed = combine_ref(pairs, ids, weights, e_lo, e_n)
    if shared is None:
        return routed
    s = bf16(expert_pairs_ref(x, np.arange(x.shape[0]), shared[0], shared[1], gated, quant))
    return combine_shared_ref(routed, s, x, gate_vec)


def route_softmax_topk(logits: torch.Tensor, k: int):
    probs = torch.softmax(logits.float(), dim=-1)
    w, ids = torch.topk(probs, k, dim=-1)
    return ids.to(torch.int32), (w / w.sum(-1, keepdim=True)).contiguous()


def route_sigmoid_topk(logits: torch.Tensor, bias: torch.Tensor, k: int, scaling: float = 1.0):
    s = torch.sigmoid(logits.float())
    choice = s + bias.float()
    # ties to the lower id: a stable descending sort
    ids = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :k]
    w = s.gather(1, ids)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * scaling
    return ids.to(torch.int32), w.contiguous()


ROUTE_CANDIDATES = 20


def budget_rule(cand, prob, share, e: int, k: int, keep: int, cap: int, real, repeat: bool = False, fallback: int = 0, eps: float = 0.0,
                given=None):
    """The selection from the rows' candidate lists (best first): prob[t][c] the weight candidate c of row t carries
    before renormalization, share[t][c] what it adds to its expert's score when within the row's top k. The set: the
    real rows' top `keep` (their top `fallback` when those exceed a cap above 0), then the best-scoring other experts
    (score > 0, equal scores to the lower expert) up to `cap`; a real row takes its candidates in the set, in rank
    order, up to k, at prob / (their sum in rank order + eps). `given`: a set to take instead of the selected one.
    -> (ids int32 [R, k], weights FP32 [R, k], the set, its guaranteed part, the FP32 scores [E])
    (hibana/kernels/flashnext_fused.py:378-456; hibana/model/nemotron/moe.py:166-263)."""
    r = len(cand)
    core = {x for c, live in zip(cand, real) if live for x in c[:keep]}
    if fallback > 0 and cap > 0 and len(core) > cap:
        core = {x for c, live in zip(cand, real) if live for x in c[:fallback]}
    score = np.zeros(e, dtype=np.float32)
    for t, c in enumerate(cand):
        if real[t]:
            for j, x in enumerate(c[:k]):
                score[x] = np.float32(score[x] + np.float32(share[t][j]))
    rest = sorted((x for x in range(e) if x not in core and score[x] > 0), key=lambda x: (-float(score[x]), x))
    chosen = core | set(rest[:max(0, cap - len(core))]) if given is None else set(given)
    ids = np.full((r, k), e, dtype=np.int32)
    w = np.zeros((r, k), dtype=np.float32)
    for t, c in enumerate(cand):
        row = [j for j, x in enumerate(c) if x in chosen][:k] if real[t] else []
        if row:
            total = np.float32(0.0)
            for j in row:
                total = np.float32(total + np.float32(prob[t][j]))
            total = np.float32(total + np.float32(eps))
            ids[t, :len(row)] = [c[j] for j in row]
            w[t, :len(row)] = [np.float32(prob[t][j]) / total for j in row]
        if repeat:
            ids[t, len(row):] = c[0] if real[t] else cand[0][0]
    return torch.from_numpy(ids), torch.from_numpy(w), chosen, core, score


def route_budget_ref(logits: torch.Tensor, k: int, keep: int, budget: int, slots=None, steps: int = 1, repeat: bool = False,
                     per_request: int = 0, min_cap: int = 0, given=None):
    """Flash-Next's form: candidates = a row's 20 largest logits, weights and shares = the FP32 softmax over E; the
    cap is `budget`, or with `per_request`, min(budget, max(min_cap, per_request x the real requests))."""
    lg = logits.float().cpu().numpy().astype(np.float32)
    r, e = lg.shape
    real = [slots is None or int(slots[t // steps]) != 0 for t in range(r)]
    cap = budget
    if per_request > 0:
        cap = min(budget, max(min_cap, per_request * sum(1 for t in range(0, r, steps) if real[t])))
    ex = np.exp(lg - lg.max(-1, keepdims=True), dtype=np.float32)
    p = ex / ex.sum(-1, keepdims=True, dtype=np.float32)
    # a stable ascending sort of the negated logits: the largest first, equal logits (both zeros among them) in id order
    cand = [np.argsort(-(row + np.float32(0.0)), kind="stable")[:ROUTE_CANDIDATES].tolist() for row in lg]
    prob = [p[t, c] for t, c in enumerate(cand)]
    return budget_rule(cand, prob, prob, e, k, keep, cap, real, repeat, given=given)


def route_budget_sigmoid_ref(fused: torch.Tensor, bias: torch.Tensor, k: int, latent: int, keep: int, budget: int, slots=None, steps: int = 1,
                             per_request: int = 0, repeat: bool = True, fallback: int = 0, cand=None, given=None):
    """The latent MoE's form (hibana/model/nemotron/moe.py:124-313): candidates = a row's top k by sigmoid + bias (equal
    scores to the lower expert; `cand`: lists to take instead), weights = the plain sigmoids over (their sum + 1e-20),
    shares = the sigmoids over the sum of the row's k; the cap is `budget`, or with `per_request`,
    min(budget, per_request x the real requests)."""
    e = fused.shape[1] - latent
    r = fused.shape[0]
    real = [slots is None or int(slots[t // steps]) != 0 for t in range(r)]
    cap = budget
    if per_request > 0:
        cap = min(budget, per_request * sum(1 for t in range(0, r, steps) if real[t]))
    s = torch.sigmoid(fused[:, :e].float().cpu())
    if cand is None:
        cand = torch.sort(s + bias.float().cpu(), dim=-1, descending=True, stable=True).indices[:, :k].tolist()
    prob = [s[t, c].numpy() for t, c in enumerate(cand)]
    share = []
    for row in prob:
        total = np.float32(0.0)
        for v in row:
            total = np.float32(total + v)
        share.append(row / np.float32(total + np.float32(1e-20)))
    out = budget_rule(cand, prob, share, e, k, keep, cap, real, repeat, fallback, 1e-20, given)
    return out + (fused[:, e:].cpu().bfloat16(),)


def silu_mul(gate_up: torch.Tensor, pairs: int = 0) -> torch.Tensor:
    half = gate_up.shape[-1] // 2
    if pairs:
        blocks = gate_up.unflatten(-1, (half // pairs, 2, pairs))
        g, u = blocks[..., 0, :].flatten(-2).float(), blocks[..., 1, :].flatten(-2).float()
    else:
        g, u = gate_up[..., :half].float(), gate_up[..., half:].float()
    return (g * torch.sigmoid(g) * u).to(torch.bfloat16)


def latent_experts_ref(lat: torch.Tensor, ids: np.ndarray, weights: torch.Tensor, get_expert):
    """The routed part of the latent MoE: lat BF16 [M, L]; get_expert(e) -> (up_unscaled [I, L] float32, up_s2,
    down_unscaled [L, I] float32, down_s2). Returns the FP32 accumulator [M, L]:
    h = bf16(relu(bf16((lat up^T) s2))^2); acc[tok] += ((h down^T) s2) * w, experts in ascending id order."""
    ids = np.asarray(ids)
    m, k = ids.shape
    acc = torch.zeros(m, lat.shape[1], dtype=torch.float32)
    w = weights.float()
    for e in np.unique(ids):
        tok, slot = np.nonzero(ids == e)
        up, up_s, down, down_s = get_expert(int(e))
        t = torch.as_tensor(tok)
        h = nvfp4_dense_ref(lat[t], up, up_s, relu2=True)
        y = (h.double() @ torch.as_tensor(down).double().T).float() * np.float32(down_s)
        acc.index_add_(0, t, y * w[t, torch.as_tensor(slot), None])
    return acc


def latent_moe_ref(x, fc1, fc2, ids, weights, get_expert, shared=None):
    """x BF16 [M, H], fc1 BF16 [L, H], fc2 BF16 [H, L] -> BF16 [M, H]:
    lat = bf16(x fc1^T); out = bf16(shared + bf16(acc) fc2^T), `shared` the shared expert's BF16 output [M, H] (addmm: one
    rounding of the FP32 sum) or None (hibana/model/nemotron/moe.py:508-517 of the reference)."""
    lat = bf16((x.double() @ fc1.double().T).float())
    acc = latent_experts_ref(lat, ids, weights, get_expert)
    y = bf16(acc).double() @ fc2.double().T
    if shared is not None:
        y = y + shared.double()
    return bf16(y.float())
