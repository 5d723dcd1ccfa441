// Budgeted expert selection as launches of its own: the entry points of the two routing rules (route_budget.hpp has
// the device code).
#include "route_budget.hpp"

namespace hb {

template <int PER, bool IN_ORDER>
__global__ __launch_bounds__(BUDGET_THREADS) void route_pick_kernel(BudgetParams q, int copies_n) {
  extern __shared__ float copies[];  // [copies_n][e]
  budget_pick<PER, IN_ORDER>(q, copies_n, copies);
}

// The sigmoid form's rank launch: the routing kernel on k candidates, its ids as the candidates, its renormalized
// weights as their shares, the plain sigmoids beside them; it also rounds the row's latent columns.
template <int PER>
__global__ __launch_bounds__(64) void route_rank_sigmoid_kernel(RouteParams p) {
  route_row<true, PER>(p, blockIdx.x, threadIdx.x);
}

static void launch_pick(const BudgetParams& q, bool in_order, hipStream_t s) {
  const int copies_n = q.e <= 512 ? BUDGET_WAVES : BUDGET_WAVES / 2;  // 32 KB of LDS either way
  const size_t lds = (size_t)copies_n * q.e * sizeof(float);
  if (q.e <= 512) {
    if (in_order) {
      HB_LAUNCH((route_pick_kernel<8, true>), dim3(1), dim3(BUDGET_THREADS), lds, s, q, copies_n);
    } else {
      HB_LAUNCH((route_pick_kernel<8, false>), dim3(1), dim3(BUDGET_THREADS), lds, s, q, copies_n);
    }
  } else if (in_order) {
    HB_LAUNCH((route_pick_kernel<16, true>), dim3(1), dim3(BUDGET_THREADS), lds, s, q, copies_n);
  } else {
    HB_LAUNCH((route_pick_kernel<16, false>), dim3(1), dim3(BUDGET_THREADS), lds, s, q, copies_n);
  }
}

}  // namespace hb

using namespace hb;

extern "C" int64_t hb_route_budget_workspace_bytes(int r) { return r > 0 ? (int64_t)r * BUDGET_CANDIDATES * 8 : 0; }

extern "C" int hb_route_budget(const void* logits, int r, int e, int k, int keep, int budget, const int32_t* slots, int steps, int repeat,
                               int per_request, int min_cap, void* workspace, int64_t workspace_bytes, int32_t* ids, float* weights,
                               void* stream) {
  if (!logits || !workspace || !ids || !weights) return HB_ENULL;
  if (r <= 0 || e < BUDGET_CANDIDATES || e > BUDGET_THREADS || k <= 0 || k > BUDGET_CANDIDATES || keep < 0 || keep > BUDGET_CANDIDATES ||
      budget < 0 || steps <= 0 || r % steps || per_request < 0 || min_cap < 0)
    return HB_EINVAL;
  if (!aligned(logits, 2) || !aligned(workspace, 4) || !aligned(slots, 4) || !aligned(ids, 4) || !aligned(weights, 4)) return HB_EINVAL;
  if (workspace_bytes < hb_route_budget_workspace_bytes(r)) return HB_EWORKSPACE;
  BudgetParams q{};
  q.logits = static_cast<const uint16_t*>(logits);
  q.slots = slots;
  q.r = r, q.e = e, q.k = k, q.keep = keep, q.budget = budget, q.per_request = per_request, q.min_cap = min_cap, q.steps = steps, q.repeat = repeat;
  q.cands = BUDGET_CANDIDATES;
  q.cand = static_cast<int32_t*>(workspace);
  q.prob = reinterpret_cast<float*>(q.cand + (int64_t)r * BUDGET_CANDIDATES);
  q.share = q.prob;  // a candidate's softmax probability is also what it adds to its expert's score
  q.ids = ids, q.weights = weights;
  hipStream_t s = as_stream(stream);
  if (e <= 512) {
    HB_LAUNCH((route_rank_kernel<8>), dim3((unsigned)r), dim3(64), 0, s, q);
  } else {
    HB_LAUNCH((route_rank_kernel<16>), dim3((unsigned)r), dim3(64), 0, s, q);
  }
  launch_pick(q, false, s);
  return launch_status();
}

extern "C" int64_t hb_route_budget_sigmoid_workspace_bytes(int r, int k) { return r > 0 && k > 0 ? (int64_t)r * k * 12 : 0; }

extern "C" int hb_route_budget_sigmoid(const float* fused, int64_t stride, const float* bias, int r, int e, int k, int latent, int keep, int budget,
                                       const int32_t* slots, int steps, int repeat, int per_request, int fallback, void* workspace,
                                       int64_t workspace_bytes, int32_t* ids, float* weights, void* lat, void* stream) {
  if (!fused || !bias || !workspace || !ids || !weights || (latent > 0 && !lat)) return HB_ENULL;
  if (r <= 0 || e <= 0 || e > BUDGET_THREADS || k <= 0 || k > 32 || k > e || latent < 0 || stride < (int64_t)e + latent || keep < 0 || keep > k ||
      fallback < 0 || fallback > keep || budget < 0 || steps <= 0 || r % steps || per_request < 0)
    return HB_EINVAL;
  if (!aligned(fused, 4) || !aligned(bias, 4) || !aligned(workspace, 4) || !aligned(slots, 4) || !aligned(ids, 4) || !aligned(weights, 4) ||
      !aligned(lat, 2))
    return HB_EINVAL;
  if (workspace_bytes < hb_route_budget_sigmoid_workspace_bytes(r, k)) return HB_EWORKSPACE;
  BudgetParams q{};
  q.slots = slots;
  q.r = r, q.e = e, q.k = k, q.keep = keep, q.budget = budget, q.per_request = per_request, q.min_cap = 0, q.steps = steps, q.repeat = repeat;
  q.cands = k, q.fallback = fallback, q.eps = 1e-20f;
  q.cand = static_cast<int32_t*>(workspace);
  q.prob = reinterpret_cast<float*>(q.cand + (int64_t)r * k);
  float* share = q.prob + (int64_t)r * k;
  q.share = share;
  q.ids = ids, q.weights = weights;
  RouteParams p{};  // every row ranks as a real one: which rows count is the pick launch's business
  p.logits = fused, p.stride = stride, p.bias = bias;
  p.steps = 1, p.e = e, p.k = k, p.per = (e + 63) / 64, p.latent = latent, p.pad_id = e, p.sigmoid = 1;
  p.ids = q.cand, p.weights = share, p.raw = q.prob, p.lat = static_cast<uint16_t*>(lat);
  hipStream_t s = as_stream(stream);
  if (p.per <= 8) {
    HB_LAUNCH((route_rank_sigmoid_kernel<8>), dim3((unsigned)r), dim3(64), 0, s, p);
  } else {
    HB_LAUNCH((route_rank_sigmoid_kernel<16>), dim3((unsigned)r), dim3(64), 0, s, p);
  }
  launch_pick(q, true, s);
  return launch_status();
}
