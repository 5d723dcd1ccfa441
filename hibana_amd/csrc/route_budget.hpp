// Budgeted expert selection (device code shared by the routing launches and the routed layer's chain): a cap on the distinct experts one decode or verify forward reads, chosen for all its rows
// (route_budget, hibana/kernels/flashnext_fused.py:322-502 of the reference; the rule row by row:
// tests/unit/test_moe_selection.py:19-58; the latent MoE's form with its own ranking, hibana/model/nemotron/moe.py:
// 124-313). Two launches, no atomics on floating-point data, no host synchronization:
//   1. rank: a wavefront a row finds the row's candidates, best first, with the weight each would carry: the 20 largest
//      BF16 logits (an exact tie to the lower expert; -0 equals +0) and their softmax probabilities over all experts,
//      or the top k of sigmoid + bias with the plain sigmoids (the routing kernel itself, which also writes each
//      candidate's share of the row's top k: its score contribution);
//   2. pick: one workgroup sums each expert's contributions over the real rows' top k, takes every real row's top
//      `keep` (its top `fallback` when those alone exceed the cap) and then the best-scoring other experts up to the
//      cap, and gives each real row its candidates in that set in rank order, up to k, at weights renormalized over
//      them.
#pragma once

#include "route.hpp"
#include "stream_common.hpp"

namespace hb {


constexpr int BUDGET_CANDIDATES = HB_ROUTE_CANDIDATES;
constexpr int BUDGET_THREADS = 1024, BUDGET_WAVES = BUDGET_THREADS / 64;
constexpr int BUDGET_BATCH = 8;   // rows whose candidates a wavefront requests at once

struct BudgetParams {
  const uint16_t* logits;  // softmax form: BF16 [r, e]
  const int32_t* slots;    // row t is real iff slots[t / steps] != 0 (null: every row)
  int r, e, k, keep, budget, per_request, min_cap, steps, repeat;
  int cands;               // candidates a row (20, or k in the sigmoid form), at most 32
  int fallback;            // or 0: the guarantee when the rows' top `keep` alone exceed the cap
  float eps;               // added to the sum a row's weights are divided by
  int32_t* cand;           // [r, cands]: the row's candidates, best first
  float* prob;             // [r, cands]: the weight each carries before renormalization
  const float* share;      // [r, cands]: what a candidate within the row's top k adds to its expert's score
  int32_t* ids;            // [r, k]
  float* weights;          // [r, k]
};

// A BF16 bit pattern as a 16-bit key that orders like the value (-0 as +0), and back.
__device__ __forceinline__ uint32_t bf16_order(uint32_t h) {
  if (h == 0x8000u) h = 0u;
  return (h & 0x8000u) ? (~h & 0xffffu) : (h | 0x8000u);
}
__device__ __forceinline__ float bf16_order_value(uint32_t o) {
  const uint32_t h = (o & 0x8000u) ? (o & 0x7fffu) : (~o & 0xffffu);
  return __uint_as_float(h << 16);
}

// Lane l holds columns l, l + 64, ... as keys (value order above 65535 - column): distinct, every real one above 0, so
// the wave-wide maximum names the largest logit left and, among equal logits, the lowest expert.
template <int PER>
__global__ __launch_bounds__(64) void route_rank_kernel(BudgetParams q) {
  const int t = blockIdx.x, lane = threadIdx.x, e = q.e;
  const uint16_t* row = q.logits + (int64_t)t * e;
  uint32_t key[PER], raw[PER];
  float val[PER];
#pragma unroll
  for (int j = 0; j < PER; j++) raw[j] = row[min(j * 64 + lane, e - 1)];  // all of the lane's loads before any use
#pragma unroll
  for (int j = 0; j < PER; j++) {
    const int col = j * 64 + lane;
    const uint32_t h = raw[j];
    key[j] = col < e ? (bf16_order(h) << 16) | (uint32_t)(0xffff - col) : 0u;
    val[j] = col < e ? __uint_as_float(h << 16) : -INFINITY;
  }
  // the lane's keys in descending order once: a round is the wave-wide maximum of the heads, and the winner's list
  // moves up by one
#pragma unroll
  for (int pass = 0; pass < PER; pass++) {
#pragma unroll
    for (int j = pass & 1; j + 1 < PER; j += 2) {
      const uint32_t hi = max(key[j], key[j + 1]), lo = min(key[j], key[j + 1]);
      key[j] = hi;
      key[j + 1] = lo;
    }
  }
  float mx = -INFINITY, sum = 0.f, mine_v = 0.f;
  int mine_id = 0;
  for (int c = 0; c < BUDGET_CANDIDATES; c++) {
    const uint32_t top = wave_max_u32(key[0]);
    const int col = 0xffff - (int)(top & 0xffffu);
    const float v = bf16_order_value(top >> 16);
    if (c == 0) {  // the row's maximum: the softmax denominator over all experts
      mx = v;
#pragma unroll
      for (int j = 0; j < PER; j++) sum += j * 64 + lane < e ? expf(val[j] - mx) : 0.f;
      sum = wave_sum(sum);
    }
    if (lane == c) {
      mine_v = v;
      mine_id = col;
    }
    if (lane == (col & 63)) {
#pragma unroll
      for (int j = 0; j + 1 < PER; j++) key[j] = key[j + 1];
      key[PER - 1] = 0u;
    }
  }
  const float mine = expf(mine_v - mx) / sum;
  if (lane < BUDGET_CANDIDATES) {
    q.cand[(int64_t)t * BUDGET_CANDIDATES + lane] = mine_id;
    q.prob[(int64_t)t * BUDGET_CANDIDATES + lane] = mine;
  }
}

// One workgroup (BUDGET_THREADS threads; `copies`: copies_n * e floats of its dynamic LDS). Scores: wavefront w adds the rows t = w (mod copies) into a copy of its own, in row order, and the
// copies are added in wavefront order (the same bits on every run). The set: wavefront 0 holds every expert's key in
// registers (column j * 64 + lane, as above) and finds the need-th largest by bisection on its bits, each step one
// ballot a register. The rows: two a wavefront at a time, one in each half. IN_ORDER: a row's weights are divided by
// the sum of the taken ones added in rank order, as the routing kernel adds a row's top k (a row that keeps all of its
// top k gets that kernel's weights bit for bit); otherwise by a butterfly sum.
template <int PER, bool IN_ORDER>
__device__ __forceinline__ void budget_pick(const BudgetParams& q, int copies_n, float* copies) {
  __shared__ uint32_t keys[BUDGET_THREADS];
  __shared__ uint8_t core[BUDGET_THREADS], core_fallback[BUDGET_THREADS], chosen[BUDGET_THREADS];
  __shared__ int real_requests;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, e = q.e, r = q.r, cands = q.cands;
  // the candidates of the rows this wavefront will write (half a wavefront a row), requested before anything else
  const int half = lane >> 5, hl = lane & 31;
  constexpr int PAIRS = BUDGET_BATCH / 2;
  int cd[PAIRS];
  float pv[PAIRS];
  auto request = [&](int t0) {
#pragma unroll
    for (int b = 0; b < PAIRS; b++) {
      const int t = t0 + 2 * BUDGET_WAVES * b + half;
      const bool live = t < r && hl < cands;
      cd[b] = live ? q.cand[(int64_t)t * cands + hl] : 0;
      pv[b] = live ? q.prob[(int64_t)t * cands + hl] : 0.f;
    }
  };
  request(2 * wave);
  const int first = q.repeat ? q.cand[0] : e;  // a padded row's slots under `repeat`: row 0's first candidate
  for (int i = tid; i < copies_n * e; i += BUDGET_THREADS) copies[i] = 0.f;
  core[tid] = 0;
  core_fallback[tid] = 0;
  if (tid == 0) real_requests = 0;
  __syncthreads();
  if (q.per_request > 0 && q.slots) {  // padded requests do not count towards the cap (an integer sum: any order)
    int mine = 0;
    for (int i = tid; i < r / q.steps; i += BUDGET_THREADS) mine += q.slots[i] != 0;
    if (mine) atomicAdd(&real_requests, mine);
  }
  auto real_row = [&](int t) { return t < r && (!q.slots || q.slots[t / q.steps] != 0); };
  // scores: what the real rows' top k add to their experts; core: the real rows' top `keep` (and top `fallback`)
  if (wave < copies_n) {
    float* mine = copies + wave * e;
    for (int t0 = wave; t0 < r; t0 += copies_n * BUDGET_BATCH) {
      int sc[BUDGET_BATCH];
      float sp[BUDGET_BATCH];
      bool real[BUDGET_BATCH];
#pragma unroll
      for (int b = 0; b < BUDGET_BATCH; b++) {
        const int t = t0 + b * copies_n;
        real[b] = real_row(t) && lane < cands;
        sc[b] = real[b] ? q.cand[(int64_t)t * cands + lane] : 0;
        sp[b] = real[b] ? q.share[(int64_t)t * cands + lane] : 0.f;
      }
#pragma unroll
      for (int b = 0; b < BUDGET_BATCH; b++) {  // a row's candidates are distinct experts: no two lanes meet
        if (real[b] && lane < q.k) mine[sc[b]] += sp[b];
        if (real[b] && lane < q.keep) core[sc[b]] = 1;
        if (real[b] && lane < q.fallback) core_fallback[sc[b]] = 1;
      }
    }
  }
  __syncthreads();
  {
    float score = 0.f;
    if (tid < e)
      for (int w = 0; w < copies_n; w++) score += copies[w * e + tid];
    keys[tid] = tid < e && score > 0.f ? __float_as_uint(score) : 0u;  // positive floats order as their bits
  }
  __syncthreads();
  if (wave == 0) {
    int cap = q.budget;
    if (q.per_request > 0) cap = min(cap, max(q.min_cap, q.per_request * (q.slots ? real_requests : r / q.steps)));
    bool guaranteed[PER];  // columns past e hold no flag and key 0
    int in_core = 0;
#pragma unroll
    for (int j = 0; j < PER; j++) {
      guaranteed[j] = core[j * 64 + lane] != 0;
      in_core += __popcll(__ballot(guaranteed[j]));
    }
    if (q.fallback > 0 && cap > 0 && in_core > cap) {  // the floors overflow the cap: each row's top `fallback` only
      in_core = 0;
#pragma unroll
      for (int j = 0; j < PER; j++) {
        guaranteed[j] = core_fallback[j * 64 + lane] != 0;
        in_core += __popcll(__ballot(guaranteed[j]));
      }
    }
    uint32_t kk[PER];
    int contenders = 0;
#pragma unroll
    for (int j = 0; j < PER; j++) {
      kk[j] = guaranteed[j] ? 0u : keys[j * 64 + lane];
      contenders += __popcll(__ballot(kk[j] != 0u));
    }
    const int need = cap - in_core;
    // the set takes the keys above `at` and, of those equal to it, the `quota` lowest experts
    uint32_t at = 0xffffffffu;
    int quota = 0;
    if (need > 0 && contenders <= need) {
      at = 0u;
    } else if (need > 0) {
      // the need-th largest key: the largest value that `need` keys reach, a bit at a time from the top; a value that
      // exactly `need` keys reach ends the search (the keys at or above it are the answer)
      at = 0u;
      for (int bit = 30; bit >= 0; bit--) {
        const uint32_t trial = at | (1u << bit);
        int n = 0;
#pragma unroll
        for (int j = 0; j < PER; j++) n += __popcll(__ballot(kk[j] >= trial));
        if (n >= need) at = trial;
        if (n == need) break;
      }
      // `at` may now lie below the need-th largest key, between it and the next one: nothing equals it then
      int above = 0;
#pragma unroll
      for (int j = 0; j < PER; j++) above += __popcll(__ballot(kk[j] > at));
      quota = need - above;
    }
    int seen = 0;
#pragma unroll
    for (int j = 0; j < PER; j++) {
      const bool equal = kk[j] == at && kk[j] != 0u;
      const uint64_t mask = __ballot(equal);
      const int before = seen + __popcll(mask & ((1ull << lane) - 1ull));
      chosen[j * 64 + lane] = guaranteed[j] || kk[j] > at || (equal && before < quota);
      seen += __popcll(mask);
    }
  }
  __syncthreads();
  // each real row's candidates in the set, in rank order, up to k; the slots left over name no expert (or repeat one)
  for (int t0 = 2 * wave; t0 < r; t0 += 2 * BUDGET_WAVES * PAIRS) {
    if (t0 != 2 * wave) request(t0);
#pragma unroll
    for (int b = 0; b < PAIRS; b++) {
      const int t = t0 + 2 * BUDGET_WAVES * b + half;
      if (t - half >= r) break;
      const bool real = real_row(t);
      const bool pull = t < r && hl < cands && chosen[cd[b]] != 0;
      const uint32_t mask = (uint32_t)(__ballot(pull) >> (32 * half));
      const int slot = __popc(mask & ((1u << hl) - 1u));
      const bool mine = pull && slot < q.k && real;
      float total = mine ? pv[b] : 0.f;
      if (IN_ORDER) {
        const float part = total;
        float lower = 0.f, upper = 0.f;
#pragma unroll
        for (int i = 0; i < 32; i++)
          if (i < cands) {
            lower += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, part), i));
            upper += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, part), i + 32));
          }
        total = half ? upper : lower;
      } else {
#pragma unroll
        for (int d = 16; d >= 1; d >>= 1) total += __shfl_xor(total, d);  // stays within the half
      }
      total += q.eps;
      const int used = real ? min(__popc(mask), q.k) : 0;
      const int top_a = __builtin_amdgcn_readlane(cd[b], 0), top_b = __builtin_amdgcn_readlane(cd[b], 32);
      if (mine) {
        store_through(&q.ids[(int64_t)t * q.k + slot], cd[b]);  // a plan in this very launch reads them past the L2
        q.weights[(int64_t)t * q.k + slot] = pv[b] / total;
      }
      if (t < r && hl >= used && hl < q.k) {
        store_through(&q.ids[(int64_t)t * q.k + hl], q.repeat ? (real ? (half ? top_b : top_a) : first) : e);
        q.weights[(int64_t)t * q.k + hl] = 0.f;
      }
    }
  }
}

}  // namespace hb
