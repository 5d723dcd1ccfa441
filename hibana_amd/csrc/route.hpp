// Top-k routing of one row by one wavefront (device code shared by the routing launches and by kernels that route for
// themselves).
#pragma once

#include "stream_common.hpp"

namespace hb {

// Top-k routing, one wavefront per row: softmax over all experts, top-k, renormalized
// (hibana/kernels/flashnext_fused.py:278-319 of the reference), or sigmoid scores chosen by score + bias with the plain
// scores as weights (hibana/model/nemotron/moe.py:57-121). Lane l holds experts l * per .. l * per + per - 1 in
// registers as order-preserving 32-bit keys, so a selection round is one wave-wide integer maximum (DPP within rows of
// 16, four scalar reads across them) and a ballot: among equal scores the lowest lane, then the lowest register,
// wins - the lowest expert id. Up to eight registers a lane are sorted once and a round looks at their heads; with
// sixteen a round scans them.
constexpr int ROUTE_PER_LANE = 16;

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t x) {
  x = max(x, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xF, 0xF, false));   // lane ^ 1
  x = max(x, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, false));   // lane ^ 2
  x = max(x, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x141, 0xF, 0xF, false));  // mirror within 8
  x = max(x, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x140, 0xF, 0xF, false));  // mirror within 16
  const uint32_t a = __builtin_amdgcn_readlane((int)x, 0), b = __builtin_amdgcn_readlane((int)x, 16);
  const uint32_t c = __builtin_amdgcn_readlane((int)x, 32), d = __builtin_amdgcn_readlane((int)x, 48);
  return max(max(a, b), max(c, d));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
  return v;
}

// Key of a score: larger score <=> larger key, every real key above 0 (the key of an empty register).
__device__ __forceinline__ uint32_t score_key(float v) {
  const int32_t bits = __builtin_bit_cast(int32_t, v);
  return (uint32_t)(bits ^ ((bits >> 31) & 0x7fffffff)) ^ 0x80000000u;
}

struct RouteParams {
  const float* logits;   // [m, stride]: e logits a row (sigmoid: followed by `latent` FP32 columns)
  int64_t stride;
  const float* bias;     // sigmoid: [e] added to the scores for the choice only
  const int32_t* slots;  // row r is real iff slots[r / steps] != 0 (null: every row)
  int steps, repeat;
  int e, k, per, latent;
  int pad_id;            // the id of a padded row's slots without `repeat` (the callers' default: e, "no expert")
  int sigmoid;           // the rule a kernel that serves both applies (route_any)
  int32_t* ids;
  float* weights;
  uint16_t* lat;         // sigmoid: BF16 [m, latent], the row's latent columns
  float* raw;            // or null: [m, k], the weights before renormalization (a padded row: those of the row it repeats)
};

// THROUGH: the logits were written by other workgroups of the same launch and are read past the compute die's L2.
// Returns, in lane s < k, the id of the row's selection s. `write` = false keeps the row's results in registers only (a
// workgroup that routes for itself a row some other workgroup writes).
template <bool SIGMOID, int PER, bool THROUGH = false>
__device__ __forceinline__ int route_row(const RouteParams& p, int r, int lane, bool write = true, float* weight = nullptr) {
  const int e = p.e, per = p.per, first = lane * per;
  auto logit = [](const float* at) -> float { if constexpr (THROUGH) return load_through(at); else return *at; };
  const bool padded = p.slots && p.slots[r / p.steps] == 0;  // asked for first: the answer picks the row the logits are read from
  if (SIGMOID && p.lat && write) {  // the row's latent columns, rounded: four a lane and sixteen loads in flight where the row allows
    const float* src = p.logits + (int64_t)r * p.stride + e;
    uint16_t* dst = p.lat + (int64_t)r * p.latent;
    if (!THROUGH && !((p.stride | e | p.latent) & 3)) {
      for (int c0 = 4 * lane; c0 < p.latent; c0 += 1024) {
        f32x4_t v[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
          if (c0 + 256 * j < p.latent) v[j] = *reinterpret_cast<const f32x4_t*>(src + c0 + 256 * j);
#pragma unroll
        for (int j = 0; j < 4; j++)
          if (c0 + 256 * j < p.latent) {
            const uint32_t lo = (uint32_t)bf16_of(v[j].x) | ((uint32_t)bf16_of(v[j].y) << 16), hi = (uint32_t)bf16_of(v[j].z) | ((uint32_t)bf16_of(v[j].w) << 16);
            *reinterpret_cast<uint2*>(dst + c0 + 256 * j) = make_uint2(lo, hi);
          }
      }
    } else {
      for (int c = lane; c < p.latent; c += 64) dst[c] = bf16_of(logit(src + c));
    }
  }
  const float* row = p.logits + (int64_t)(padded ? 0 : r) * p.stride;  // a padded row repeats row 0's first choice
  float val[PER];   // the weight an expert would get before renormalization
  uint32_t key[PER];
  float lg[PER];    // the lane's logits: every load is asked for before the first is used
  if (!THROUGH && PER == 8 && per == 8 && e == 512 && !((p.stride | (int64_t)(reinterpret_cast<uintptr_t>(p.logits) >> 2)) & 3)) {
    // the lane's eight logits are 32 consecutive bytes on a 16-byte boundary: two loads instead of eight
    const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(row + first), hi = *reinterpret_cast<const f32x4_t*>(row + first + 4);
    lg[0] = lo.x, lg[1] = lo.y, lg[2] = lo.z, lg[3] = lo.w;
    if constexpr (PER >= 8) lg[4] = hi.x, lg[5] = hi.y, lg[6] = hi.z, lg[7] = hi.w;
  } else {
#pragma unroll
    for (int j = 0; j < PER; j++) lg[j] = logit(row + min(first + j, e - 1));
  }
  if (SIGMOID) {
    float bs[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) bs[j] = p.bias[min(first + j, e - 1)];
#pragma unroll
    for (int j = 0; j < PER; j++) {
      const bool real = j < per && first + j < e;
      val[j] = real ? 1.0f / (1.0f + expf(-lg[j])) : 0.f;
      key[j] = real ? score_key(val[j] + bs[j]) : 0u;
    }
  } else {
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER; j++) {
      val[j] = j < per && first + j < e ? lg[j] : -INFINITY;
      mx = fmaxf(mx, val[j]);
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < PER; j++) {
      val[j] = j < per && first + j < e ? expf(val[j] - mx) : 0.f;
      sum += val[j];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int j = 0; j < PER; j++) {
      val[j] = val[j] / sum;
      key[j] = j < per && first + j < e ? score_key(val[j]) : 0u;
    }
  }
  float total = 0.f, mine = 0.f;
  int mine_id = 0;
  if constexpr (PER == 8) {
    // The lane's registers in descending order once (adjacent exchanges on a strictly larger right neighbour only, so
    // equal keys keep ascending index), their indices as nibbles of one register: a round is then the wave-wide
    // maximum of the heads and the winner's list moving up by one.
    uint32_t at[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) at[j] = j;
#pragma unroll
    for (int pass = 0; pass < PER; pass++) {
#pragma unroll
      for (int j = pass & 1; j + 1 < PER; j += 2) {
        const bool swap = key[j + 1] > key[j];
        const uint32_t ka = key[j], kb = key[j + 1], ia = at[j], ib = at[j + 1];
        key[j] = swap ? kb : ka;
        key[j + 1] = swap ? ka : kb;
        at[j] = swap ? ib : ia;
        at[j + 1] = swap ? ia : ib;
      }
    }
    uint32_t order = 0;
#pragma unroll
    for (int j = 0; j < PER; j++) order |= at[j] << (4 * j);
    uint32_t mine_key = 0;
    for (int s = 0; s < p.k; s++) {
      const uint32_t top = wave_max_u32(key[0]);
      const int winner = __builtin_ctzll(__ballot(key[0] == top));
      const int wj = __builtin_amdgcn_readlane((int)order, winner) & 15;
      if (lane == s) {
        mine_key = top;
        mine_id = winner * per + wj;
      }
      if (lane == winner) {
#pragma unroll
        for (int j = 0; j + 1 < PER; j++) key[j] = key[j + 1];
        key[PER - 1] = 0u;
        order >>= 4;
      }
    }
    if (lane < p.k) {
      if (SIGMOID) {  // the key is score + bias: the plain score is made again from the logit
        mine = 1.0f / (1.0f + expf(-logit(row + mine_id)));
      } else {        // the key is the probability's own bits
        const uint32_t u = mine_key ^ 0x80000000u;
        mine = __builtin_bit_cast(float, u ^ (uint32_t)(((int32_t)u >> 31) & 0x7fffffff));
      }
    }
    for (int s = 0; s < p.k; s++) total += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), s));  // in rank order
  } else {
    for (int s = 0; s < p.k; s++) {
      uint32_t best = 0;
      int at = 0;
      float bv = 0.f;
#pragma unroll
      for (int j = 0; j < PER; j++)
        if (key[j] > best) {  // ascending index within the lane: the first of equals stays
          best = key[j];
          at = j;
          bv = val[j];
        }
      const uint32_t top = wave_max_u32(best);
      const int winner = __builtin_ctzll(__ballot(best == top));
      const int wj = __builtin_amdgcn_readlane(at, winner);
      const float wv = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, bv), winner));
      total += wv;
      if (lane == s) {
        mine = wv;
        mine_id = winner * per + wj;
      }
      if (lane == winner) {
#pragma unroll
        for (int j = 0; j < PER; j++)
          if (j == wj) key[j] = 0u;
      }
    }
  }
  int id = mine_id;
  float w = SIGMOID ? mine / (total + 1e-20f) : mine / total;
  if (padded) {
    id = p.repeat ? __builtin_amdgcn_readfirstlane(mine_id) : p.pad_id;
    w = 0.f;
  }
  if (lane < p.k && write) {
    store_through(&p.ids[(int64_t)r * p.k + lane], id);  // the plan may read it in this very launch, from another workgroup
    p.weights[(int64_t)r * p.k + lane] = w;
    if (p.raw) p.raw[(int64_t)r * p.k + lane] = mine;
  }
  if (weight) *weight = w;
  return id;
}

// Row r by the rule and the register count the parameters name.
__device__ __forceinline__ void route_any(const RouteParams& p, int r, int lane) {
  if (p.sigmoid) {
    if (p.per <= 8) {
      route_row<true, 8>(p, r, lane);
    } else {
      route_row<true, 16>(p, r, lane);
    }
  } else if (p.per <= 8) {
    route_row<false, 8>(p, r, lane);
  } else {
    route_row<false, 16>(p, r, lane);
  }
}

}  // namespace hb
