// The W3 weight stream on gfx950: dense linear and routed-expert grouped GEMMs for decode / verify sized calls.
//
// One wavefront owns a block column of the tile layout: 64 output rows x a range of 128-k chunks, for one "slot" of up
// to 16 activation rows. Per chunk it issues three 128-bit loads of packed codes and one of scales (a contiguous
// 3328-byte block), expands the codes in registers (v_perm_b32 over the 8-byte E4M3 codebook, then the hardware
// FP8 -> BF16 pair conversion: exact), and feeds sixteen v_mfma_f32_16x16x32_bf16 (4 row tiles x 4 scale groups):
// one MFMA is exactly one 32-group, so the group scale is folded into the FP32 accumulator after it
// (acc += part * scale), as the reference kernel does per group (hibana/kernels/csrc/w3_gemm.cu:105-108); the FP32
// row scale is applied in the epilogue (:209-210). Activations are BF16, read straight from global memory (they stay
// in L2) as the MFMA A operand. The wavefronts of a workgroup split K (partials reduced through LDS in a fixed
// order) and/or take neighbouring 64-row blocks. No atomics on floating point anywhere: results are bitwise
// repeatable.
#include <string.h>

#include <vector>

#include "common.hpp"
#include "w3_layout.hpp"

namespace hb {

enum { EPI_DENSE = 0, EPI_FC1_GATED = 1, EPI_FC1_RELU2 = 2, EPI_FC2 = 3 };
constexpr int ROWS_PER_SLOT = 16;
constexpr int PLAN_HEADER = 16;  // plan[0] = slots, plan[1] = distinct experts, plan[2] = routed pairs kept

struct StreamParams {
  const uint8_t* w;       // tile layout, expert 0
  int64_t expert_bytes;   // bytes between experts
  const float* rows;      // row scales, expert 0
  int64_t expert_rows;    // floats between experts
  const uint8_t* w_shared;  // the shared expert (slot expert id < 0), or null
  const float* rows_shared;
  uint32_t lut_lo, lut_hi, lut_lo_shared, lut_hi_shared;
  int n_blocks;           // 64-row blocks per expert matrix
  int chunks;             // K / 128
  const uint16_t* a;      // BF16 activations
  int64_t a_stride;       // elements between rows
  const int32_t* plan;    // grouped calls: slot table
  const int32_t* order;   // grouped calls: sorted position -> pair index
  int m;                  // dense calls: rows
  int topk, pairs;        // grouped calls: pair q < pairs belongs to token q / topk, q >= pairs to token q - pairs
  void* out;
  int64_t out_stride;     // elements between output rows
  int out_bf16;           // EPI_FC2: pair outputs in BF16 instead of FP32
  int ks, nbw;            // wavefronts per workgroup = ks (K splits) * nbw (64-row blocks)
};

struct Chunk {  // the weight side of one 64-row x 128-k block
  u32x4_t w0, w1, w2, sc;
};

struct Rows {  // the activation side: four MFMA A fragments (one per 32-group), read from L2
  u32x4_t a0, a1, a2, a3;
};

__device__ __forceinline__ void load_chunk(Chunk& ch, const uint8_t* blk, int lane, int r16) {
  const u32x4_t* b = reinterpret_cast<const u32x4_t*>(blk);
  ch.w0 = __builtin_nontemporal_load(b + lane);
  ch.w1 = __builtin_nontemporal_load(b + 64 + lane);
  ch.w2 = __builtin_nontemporal_load(b + 128 + lane);
  ch.sc = __builtin_nontemporal_load(b + 192 + r16);
}

__device__ __forceinline__ void load_rows(Rows& ch, const uint16_t* arow) {
  ch.a0 = *reinterpret_cast<const u32x4_t*>(arow);
  ch.a1 = *reinterpret_cast<const u32x4_t*>(arow + 32);
  ch.a2 = *reinterpret_cast<const u32x4_t*>(arow + 64);
  ch.a3 = *reinterpret_cast<const u32x4_t*>(arow + 96);
}

__device__ __forceinline__ bf16x8_t expand8(uint32_t sel_lo, uint32_t sel_hi, uint32_t lut_lo, uint32_t lut_hi) {
  const uint32_t f0 = __builtin_amdgcn_perm(lut_hi, lut_lo, sel_lo);
  const uint32_t f1 = __builtin_amdgcn_perm(lut_hi, lut_lo, sel_hi);
  u32x4_t packed;
  packed.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(f0, 1.0f, false));
  packed.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(f0, 1.0f, true));
  packed.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(f1, 1.0f, false));
  packed.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(f1, 1.0f, true));
  return __builtin_bit_cast(bf16x8_t, packed);
}

// One 16-row tile of a chunk: its three code dwords, its four scale bytes, the four activation fragments.
__device__ __forceinline__ void compute_tile(uint32_t q0, uint32_t q1, uint32_t q2, uint32_t scales, const Rows& ch, f32x4_t& acc,
                                             uint32_t lut_lo, uint32_t lut_hi) {
  uint32_t sel[8];
  w3_selectors(q0, q1, q2, sel);
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
  const f32x4_t p0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ch.a0), expand8(sel[0], sel[1], lut_lo, lut_hi), zero, 0, 0, 0);
  const f32x4_t p1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ch.a1), expand8(sel[2], sel[3], lut_lo, lut_hi), zero, 0, 0, 0);
  const f32x4_t p2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ch.a2), expand8(sel[4], sel[5], lut_lo, lut_hi), zero, 0, 0, 0);
  const f32x4_t p3 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ch.a3), expand8(sel[6], sel[7], lut_lo, lut_hi), zero, 0, 0, 0);
  const float s0 = __builtin_amdgcn_cvt_f32_fp8(scales, 0), s1 = __builtin_amdgcn_cvt_f32_fp8(scales, 1);
  const float s2 = __builtin_amdgcn_cvt_f32_fp8(scales, 2), s3 = __builtin_amdgcn_cvt_f32_fp8(scales, 3);
  acc.x = fmaf(p3.x, s3, fmaf(p2.x, s2, fmaf(p1.x, s1, fmaf(p0.x, s0, acc.x))));
  acc.y = fmaf(p3.y, s3, fmaf(p2.y, s2, fmaf(p1.y, s1, fmaf(p0.y, s0, acc.y))));
  acc.z = fmaf(p3.z, s3, fmaf(p2.z, s2, fmaf(p1.z, s1, fmaf(p0.z, s0, acc.z))));
  acc.w = fmaf(p3.w, s3, fmaf(p2.w, s2, fmaf(p1.w, s1, fmaf(p0.w, s0, acc.w))));
}

__device__ __forceinline__ void compute_chunk(const Chunk& ch, const Rows& rows, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3,
                                              uint32_t lut_lo, uint32_t lut_hi) {
  compute_tile(ch.w0.x, ch.w0.y, ch.w0.z, ch.sc.x, rows, acc0, lut_lo, lut_hi);
  compute_tile(ch.w0.w, ch.w1.x, ch.w1.y, ch.sc.y, rows, acc1, lut_lo, lut_hi);
  compute_tile(ch.w1.z, ch.w1.w, ch.w2.x, ch.sc.z, rows, acc2, lut_lo, lut_hi);
  compute_tile(ch.w2.y, ch.w2.z, ch.w2.w, ch.sc.w, rows, acc3, lut_lo, lut_hi);
}

// The epilogue's roundings use the hardware FP32 -> BF16 conversion (round to nearest even).
__device__ __forceinline__ uint16_t bf16_of(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
__device__ __forceinline__ float through_bf16(float f) { return (float)(__bf16)f; }

// silu with the fast exponential and division: the result is rounded to BF16 right after (8 significant bits).
__device__ __forceinline__ float silu(float g) { return __fdividef(g, 1.0f + __expf(-g)); }

// One output element (or, gated, one up/gate pair) of the 64-row block: row tile `t` (gated: pair index), accumulator
// register r of lane (q, r16); v0 / v1 are the K-complete sums before the row scale.
template <int EPI>
__device__ __forceinline__ void emit(const StreamParams& p, const float* rs, int nb, int p0, int rows, int t, int r, int q, int r16,
                                     float v0, float v1) {
  if (r >= rows) return;    // wave-uniform: this accumulator register holds no row of the slot in any lane
  const int i = 4 * q + r;  // activation row of the slot held by this accumulator register
  if (i >= rows) return;
  const int64_t pos = p0 + i;
  if (EPI == EPI_FC1_GATED) {
    const int n_up = nb * 64 + 32 * t + r16;
    const float up = through_bf16(v0 * rs[n_up]);
    const float gate = through_bf16(v1 * rs[n_up + 16]);
    reinterpret_cast<uint16_t*>(p.out)[pos * p.out_stride + nb * 32 + 16 * t + r16] = bf16_of(silu(gate) * up);
  } else {
    const int n = nb * 64 + 16 * t + r16;
    const float y = v0 * rs[n];
    if (EPI == EPI_FC1_RELU2) {
      const float h = fmaxf(through_bf16(y), 0.f);
      reinterpret_cast<uint16_t*>(p.out)[pos * p.out_stride + n] = bf16_of(h * h);
    } else if (EPI == EPI_DENSE) {
      reinterpret_cast<uint16_t*>(p.out)[pos * p.out_stride + n] = bf16_of(y);
    } else {
      const int64_t pair = p.order[pos];
      if (p.out_bf16) {
        reinterpret_cast<uint16_t*>(p.out)[pair * p.out_stride + n] = bf16_of(y);
      } else {
        reinterpret_cast<float*>(p.out)[pair * p.out_stride + n] = y;
      }
    }
  }
}

// What a workgroup needs to know about its slot (up to 16 activation rows of one expert, or of the dense matrix).
struct Slot {
  int p0, rows;        // first row (sorted position) and number of rows
  const uint8_t* w;    // the expert's tile-layout matrix
  const float* rs;     // its row scales
  uint32_t lut_lo, lut_hi;
};

template <int EPI>
__device__ __forceinline__ Slot slot_of(const StreamParams& p, int slot) {
  Slot s;
  int expert = 0;
  if (EPI == EPI_DENSE) {
    s.p0 = slot * ROWS_PER_SLOT;
    s.rows = min(ROWS_PER_SLOT, p.m - s.p0);
  } else {
    expert = p.plan[PLAN_HEADER + 4 * slot];
    s.p0 = p.plan[PLAN_HEADER + 4 * slot + 1];
    s.rows = p.plan[PLAN_HEADER + 4 * slot + 2];
  }
  s.w = expert < 0 ? p.w_shared : p.w + (int64_t)expert * p.expert_bytes;
  s.rs = expert < 0 ? p.rows_shared : p.rows + (int64_t)expert * p.expert_rows;
  s.lut_lo = expert < 0 ? p.lut_lo_shared : p.lut_lo;
  s.lut_hi = expert < 0 ? p.lut_hi_shared : p.lut_hi;
  return s;
}

// The activation row this lane feeds to the MFMA A operand (row r16 of the slot, columns from 8 q). Lanes past the
// slot's last row read that last row again: their MFMA output rows are never stored.
template <int EPI>
__device__ __forceinline__ const uint16_t* activation_row(const StreamParams& p, const Slot& s, int q, int r16) {
  int64_t arow = s.p0 + min(r16, s.rows - 1);
  if (EPI == EPI_FC1_GATED || EPI == EPI_FC1_RELU2) {
    const int pair = p.order[arow];
    arow = pair < p.pairs ? pair / p.topk : pair - p.pairs;
  }
  return p.a + arow * p.a_stride + 8 * q;
}

// The end of a 64-row block: K-complete sums straight from the registers (ks == 1), or the K split's partial sums
// exchanged through LDS (`partial`: 4 KB per wavefront) and added in split order, then the epilogue. With ks > 1 every
// wavefront of the workgroup must call it (one workgroup barrier).
template <int EPI>
__device__ __forceinline__ void finish_block(const StreamParams& p, const Slot& sl, int nb, bool active, int ks, int nbi, float* partial,
                                             const f32x4_t& acc0, const f32x4_t& acc1, const f32x4_t& acc2, const f32x4_t& acc3) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int q = lane >> 4, r16 = lane & 15;
  const int p0 = sl.p0, rows = sl.rows;
  const float* rs = sl.rs;
  if (p.ks == 1) {
    if (!active) return;
    if (EPI == EPI_FC1_GATED) {
      emit<EPI>(p, rs, nb, p0, rows, 0, 0, q, r16, acc0.x, acc1.x);
      emit<EPI>(p, rs, nb, p0, rows, 0, 1, q, r16, acc0.y, acc1.y);
      emit<EPI>(p, rs, nb, p0, rows, 0, 2, q, r16, acc0.z, acc1.z);
      emit<EPI>(p, rs, nb, p0, rows, 0, 3, q, r16, acc0.w, acc1.w);
      emit<EPI>(p, rs, nb, p0, rows, 1, 0, q, r16, acc2.x, acc3.x);
      emit<EPI>(p, rs, nb, p0, rows, 1, 1, q, r16, acc2.y, acc3.y);
      emit<EPI>(p, rs, nb, p0, rows, 1, 2, q, r16, acc2.z, acc3.z);
      emit<EPI>(p, rs, nb, p0, rows, 1, 3, q, r16, acc2.w, acc3.w);
    } else {
      const f32x4_t all[4] = {acc0, acc1, acc2, acc3};
#pragma unroll
      for (int t = 0; t < 4; t++) {
        emit<EPI>(p, rs, nb, p0, rows, t, 0, q, r16, all[t].x, 0.f);
        emit<EPI>(p, rs, nb, p0, rows, t, 1, q, r16, all[t].y, 0.f);
        emit<EPI>(p, rs, nb, p0, rows, t, 2, q, r16, all[t].z, 0.f);
        emit<EPI>(p, rs, nb, p0, rows, t, 3, q, r16, all[t].w, 0.f);
      }
    }
    return;
  }
  float* mine = partial + (int64_t)wave * 1024;
  {
    const f32x4_t all[4] = {acc0, acc1, acc2, acc3};
#pragma unroll
    for (int t = 0; t < 4; t++) {
      mine[(t * 4 + 0) * 64 + lane] = all[t].x;
      mine[(t * 4 + 1) * 64 + lane] = all[t].y;
      mine[(t * 4 + 2) * 64 + lane] = all[t].z;
      mine[(t * 4 + 3) * 64 + lane] = all[t].w;
    }
  }
  __syncthreads();
  if (!active) return;
  const float* first = partial + (int64_t)nbi * p.ks * 1024;
  if (EPI == EPI_FC1_GATED) {
    for (int idx = ks; idx < 8; idx += p.ks) {
      const int t = idx >> 2, r = idx & 3;
      if (r >= rows) continue;
      float up = 0.f, gate = 0.f;
      for (int s = 0; s < p.ks; s++) {
        up += first[s * 1024 + ((2 * t) * 4 + r) * 64 + lane];
        gate += first[s * 1024 + ((2 * t + 1) * 4 + r) * 64 + lane];
      }
      emit<EPI>(p, rs, nb, p0, rows, t, r, q, r16, up, gate);
    }
  } else {
    for (int idx = ks; idx < 16; idx += p.ks) {
      const int t = idx >> 2, r = idx & 3;
      if (r >= rows) continue;
      float v = 0.f;
      for (int s = 0; s < p.ks; s++) v += first[s * 1024 + (t * 4 + r) * 64 + lane];
      emit<EPI>(p, rs, nb, p0, rows, t, r, q, r16, v, 0.f);
    }
  }
}

// General kernel, any K: one workgroup per (run of p.nbw 64-row blocks, slot), K split p.ks ways across its wavefronts.
// Weights and activations of chunk i + 1 are requested together before chunk i is expanded (two register buffers).
template <int EPI>
__global__ __launch_bounds__(1024) void w3_stream_kernel(StreamParams p) {
  extern __shared__ float partial[];
  if (EPI != EPI_DENSE && (int)blockIdx.y >= p.plan[0]) return;  // a slot the plan did not fill: the whole workgroup leaves
  const Slot sl = slot_of<EPI>(p, blockIdx.y);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int q = lane >> 4, r16 = lane & 15;
  const int ks = wave % p.ks, nbi = wave / p.ks;
  const int nb = blockIdx.x * p.nbw + nbi;
  const bool active = nb < p.n_blocks;
  f32x4_t acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = acc0, acc2 = acc0, acc3 = acc0;
  if (active) {
    const int c0 = (int)((int64_t)ks * p.chunks / p.ks), c1 = (int)((int64_t)(ks + 1) * p.chunks / p.ks);
    const uint8_t* blk = sl.w + ((int64_t)nb * p.chunks + c0) * W3_BLOCK_BYTES;
    if (c0 < c1) {
      Chunk we, wo;
      Rows ae, ao;
      load_chunk(we, blk, lane, r16);
      const uint16_t* aptr = activation_row<EPI>(p, sl, q, r16) + (int64_t)c0 * 128;
      load_rows(ae, aptr);
      int left = c1 - c0 - 1;  // chunks not yet requested
      while (left >= 2) {
        load_chunk(wo, blk + W3_BLOCK_BYTES, lane, r16);
        load_rows(ao, aptr + 128);
        compute_chunk(we, ae, acc0, acc1, acc2, acc3, sl.lut_lo, sl.lut_hi);
        blk += 2 * W3_BLOCK_BYTES;
        aptr += 256;
        load_chunk(we, blk, lane, r16);
        load_rows(ae, aptr);
        compute_chunk(wo, ao, acc0, acc1, acc2, acc3, sl.lut_lo, sl.lut_hi);
        left -= 2;
      }
      if (left == 1) {
        load_chunk(wo, blk + W3_BLOCK_BYTES, lane, r16);
        load_rows(ao, aptr + 128);
        compute_chunk(we, ae, acc0, acc1, acc2, acc3, sl.lut_lo, sl.lut_hi);
        compute_chunk(wo, ao, acc0, acc1, acc2, acc3, sl.lut_lo, sl.lut_hi);
      } else {
        compute_chunk(we, ae, acc0, acc1, acc2, acc3, sl.lut_lo, sl.lut_hi);
      }
    }
  }
  finish_block<EPI>(p, sl, nb, active, ks, nbi, partial, acc0, acc1, acc2, acc3);
}

// ---------------------------------------------------------------------------------------------------- expert plan
//
// The expert-sorted pair list of a routed call (the reference's prep kernel, hibana/kernels/csrc/w3_gemm.cu:710-782):
// distinct local experts in ascending id, each expert's pairs in ascending pair index (a stable sort), cut into slots
// of at most 16 rows. One workgroup; any number of pairs. Integer atomics on LDS counters only (order-independent).
//   plan[0] = slots, plan[1] = distinct experts, plan[2] = kept routed pairs,
//   plan[16 + 4 s ..] = { local expert id (-1: the shared expert), first sorted position, rows, 0 }
//   order[pos] = pair index (row * topk + slot; shared expert rows: pairs + row)
constexpr int PLAN_THREADS = 1024;
constexpr int PLAN_WAVES = PLAN_THREADS / 64;

struct Scan3 {
  int a, b, c;
};

// Exclusive scan of three integers per thread over the workgroup at once; `total` receives the three sums.
__device__ __forceinline__ Scan3 block_exclusive_scan3(Scan3 v, int* scratch /* 3 * (PLAN_WAVES + 1) ints */, Scan3* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  Scan3 inc = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int oa = __shfl_up(inc.a, d), ob = __shfl_up(inc.b, d), oc = __shfl_up(inc.c, d);
    if (lane >= d) {
      inc.a += oa;
      inc.b += ob;
      inc.c += oc;
    }
  }
  __syncthreads();  // scratch may still be read from a previous scan
  if (lane == 63) {
    scratch[wave] = inc.a;
    scratch[PLAN_WAVES + 1 + wave] = inc.b;
    scratch[2 * (PLAN_WAVES + 1) + wave] = inc.c;
  }
  __syncthreads();
  if (threadIdx.x < 3) {
    int* row = scratch + threadIdx.x * (PLAN_WAVES + 1);
    int run = 0;
    for (int wv = 0; wv < PLAN_WAVES; wv++) {
      const int c = row[wv];
      row[wv] = run;
      run += c;
    }
    row[PLAN_WAVES] = run;
  }
  __syncthreads();
  total->a = scratch[PLAN_WAVES];
  total->b = scratch[2 * PLAN_WAVES + 1];
  total->c = scratch[3 * PLAN_WAVES + 2];
  return Scan3{scratch[wave] + inc.a - v.a, scratch[PLAN_WAVES + 1 + wave] + inc.b - v.b, scratch[2 * (PLAN_WAVES + 1) + wave] + inc.c - v.c};
}

__global__ __launch_bounds__(PLAN_THREADS) void moe_plan_kernel(const int32_t* __restrict__ ids, int pairs, int e_lo, int e_n,
                                                                int shared_rows, int32_t* __restrict__ plan, int32_t* __restrict__ order) {
  extern __shared__ int lds[];
  int* seg_count = lds;                         // [PLAN_WAVES][e_n]: pairs of expert e in segment w, then running positions
  int* start = lds + PLAN_WAVES * e_n;          // [e_n]: first sorted position of expert e
  int* scratch = start + e_n;                   // [3 * (PLAN_WAVES + 1)]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < PLAN_WAVES * e_n; i += PLAN_THREADS) seg_count[i] = 0;
  __syncthreads();
  // segment w = pairs [w * seg, (w + 1) * seg), seg a multiple of 64
  const int seg = ((pairs + PLAN_WAVES - 1) / PLAN_WAVES + 63) / 64 * 64;
  const int lo = wave * seg, hi = min(pairs, lo + seg);
  for (int i = lo + lane; i < hi; i += 64) {
    const int e = ids[i] - e_lo;
    if (e >= 0 && e < e_n) atomicAdd(&seg_count[wave * e_n + e], 1);
  }
  __syncthreads();
  // per expert: total count, exclusive positions; slots of 16 rows
  int kept = 0, distinct = 0, slots = 0;
  for (int base = 0; base < e_n; base += PLAN_THREADS) {  // experts in ascending id, PLAN_THREADS at a time
    const int e = base + threadIdx.x;
    int count = 0;
    if (e < e_n)
      for (int wv = 0; wv < PLAN_WAVES; wv++) count += seg_count[wv * e_n + e];
    const int my_slots = (count + ROWS_PER_SLOT - 1) / ROWS_PER_SLOT;
    Scan3 tot;
    const Scan3 at = block_exclusive_scan3(Scan3{count, count > 0 ? 1 : 0, my_slots}, scratch, &tot);
    const int my_start = kept + at.a, my_slot = slots + at.c;
    const int tot_count = tot.a, tot_distinct = tot.b, tot_slots = tot.c;
    if (e < e_n) {
      start[e] = my_start;
      for (int s = 0; s < my_slots; s++) {
        int32_t* entry = plan + PLAN_HEADER + 4 * (my_slot + s);
        entry[0] = e;
        entry[1] = my_start + s * ROWS_PER_SLOT;
        entry[2] = min(ROWS_PER_SLOT, count - s * ROWS_PER_SLOT);
        entry[3] = 0;
      }
      // turn the per-segment counts into the first position of each segment's run
      int run = my_start;
      for (int wv = 0; wv < PLAN_WAVES; wv++) {
        const int c = seg_count[wv * e_n + e];
        seg_count[wv * e_n + e] = run;
        run += c;
      }
    }
    kept += tot_count;
    distinct += tot_distinct;
    slots += tot_slots;
  }
  __syncthreads();
  // the shared expert's rows follow the routed pairs
  const int shared_slots = (shared_rows + ROWS_PER_SLOT - 1) / ROWS_PER_SLOT;
  for (int s = threadIdx.x; s < shared_slots; s += PLAN_THREADS) {
    int32_t* entry = plan + PLAN_HEADER + 4 * (slots + s);
    entry[0] = -1;
    entry[1] = kept + s * ROWS_PER_SLOT;
    entry[2] = min(ROWS_PER_SLOT, shared_rows - s * ROWS_PER_SLOT);
    entry[3] = 0;
  }
  for (int r = threadIdx.x; r < shared_rows; r += PLAN_THREADS) order[kept + r] = pairs + r;
  if (threadIdx.x == 0) {
    plan[0] = slots + shared_slots;
    plan[1] = distinct;
    plan[2] = kept;
  }
  // stable placement: each wavefront walks its segment 64 pairs at a time; a lane's position is its expert's running
  // position in this segment plus the number of lower lanes of the tile with the same expert
  for (int i0 = lo; i0 < hi; i0 += 64) {
    const int i = i0 + lane;
    int e = -1;
    if (i < hi) {
      e = ids[i] - e_lo;
      if (e < 0 || e >= e_n) e = -1;
    }
    uint64_t same = __ballot(e >= 0);
#pragma unroll
    for (int b = 0; b < 20; b++) {
      const uint64_t m = __ballot((e >> b) & 1);
      same &= ((e >> b) & 1) ? m : ~m;
    }
    if (e >= 0) {
      const uint64_t below = same & ((1ull << lane) - 1ull);
      const int base = seg_count[wave * e_n + e];
      order[base + __popcll(below)] = i;
      const bool last = (same >> lane) == 1ull;  // the highest lane of this expert in the tile advances the counter
      if (last) seg_count[wave * e_n + e] = base + __popcll(same);
    }
    // the read of `base` above and the update by `last` are in the same wavefront; LDS operations of one wavefront
    // execute in program order, and the next tile's reads come after this write
  }
}

// ---------------------------------------------------------------------------------------------------- combine
//
// out[r, c] = bf16( bf16(sum over the row's local slots, in selection order, of fma(w, y)) + g * shared ), one
// workgroup per (row, 1024-column span). The reference's combine (hibana/kernels/csrc/w3_gemm.cu:1196-1213) when no
// shared expert is given; with one, its fused form (hibana/kernels/flashnext_fused.py:530-571).
struct CombineParams {
  const void* pairs;      // [m * topk (+ m), h] FP32 or BF16
  int pairs_bf16;
  const int32_t* ids;
  const float* weights;
  const void* shared;     // BF16 [m, h], FP32 [m, h] (shared_f32) or null
  int shared_f32;
  int64_t shared_stride;
  const uint16_t* x;      // BF16 [m, hx] for the gate
  const float* gate_vec;  // [hx] or null
  int hx;
  int e_lo, e_n, m, topk, h;
  uint16_t* out;
};

constexpr int COMBINE_SPAN = 512;  // columns per workgroup (two per thread)
constexpr int COMBINE_MAX_TOPK = 32;

__global__ __launch_bounds__(256) void moe_combine_kernel(CombineParams p) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  float g = 1.0f;
  if (p.gate_vec && p.shared) {
    float dot = 0.f;
    for (int i = threadIdx.x; i < p.hx; i += 256) dot += bf16_bits_to_f32(p.x[(int64_t)r * p.hx + i]) * p.gate_vec[i];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) dot += __shfl_xor(dot, d);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = dot;
    __syncthreads();
    dot = (red[0] + red[1]) + (red[2] + red[3]);
    g = 1.0f / (1.0f + expf(-dot));
  }
  const int c = blockIdx.y * COMBINE_SPAN + 2 * threadIdx.x;  // h is even: a column pair is in or out together
  if (c >= p.h) return;
  float v0 = 0.f, v1 = 0.f;
  // every slot's pair is read (so the loads are all in flight together) and a dropped slot contributes fma(0, 0, v)
  for (int s0 = 0; s0 < p.topk; s0 += 8) {
    float y0[8], y1[8], w[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int s = min(s0 + j, p.topk - 1);
      const int e = p.ids[r * p.topk + s] - p.e_lo;
      const bool keep = s0 + j < p.topk && e >= 0 && e < p.e_n;
      const int64_t at = ((int64_t)r * p.topk + s) * p.h + c;
      float a, b;
      if (p.pairs_bf16) {
        const uint32_t two = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint16_t*>(p.pairs) + at);
        a = __uint_as_float(two << 16);
        b = __uint_as_float(two & 0xffff0000u);
      } else {
        const float2 two = *reinterpret_cast<const float2*>(reinterpret_cast<const float*>(p.pairs) + at);
        a = two.x;
        b = two.y;
      }
      y0[j] = keep ? a : 0.f;
      y1[j] = keep ? b : 0.f;
      w[j] = keep ? p.weights[r * p.topk + s] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
      v0 = fmaf(w[j], y0[j], v0);
      v1 = fmaf(w[j], y1[j], v1);
    }
  }
  if (p.shared) {
    const int64_t at = (int64_t)r * p.shared_stride + c;
    float s0, s1;
    if (p.shared_f32) {
      const float2 two = *reinterpret_cast<const float2*>(reinterpret_cast<const float*>(p.shared) + at);
      s0 = round_bf16(two.x);
      s1 = round_bf16(two.y);
    } else {
      const uint32_t two = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint16_t*>(p.shared) + at);
      s0 = __uint_as_float(two << 16);
      s1 = __uint_as_float(two & 0xffff0000u);
    }
    v0 = round_bf16(v0) + g * s0;
    v1 = round_bf16(v1) + g * s1;
  }
  *reinterpret_cast<uint32_t*>(p.out + (int64_t)r * p.h + c) = (uint32_t)f32_to_bf16_bits(v0) | ((uint32_t)f32_to_bf16_bits(v1) << 16);
}

// ---------------------------------------------------------------------------------------------------- routing
// Softmax top-k (hibana/kernels/flashnext_fused.py:278-319 of the reference): one wavefront per row.
constexpr int ROUTE_PER_LANE = 16;  // up to 1024 experts: lane l holds experts l, l + 64, ...

__global__ __launch_bounds__(64) void route_softmax_topk_kernel(const float* __restrict__ logits, int e, int k, int32_t* __restrict__ ids,
                                                                float* __restrict__ weights) {
  const int r = blockIdx.x, lane = threadIdx.x;
  const float* row = logits + (int64_t)r * e;
  float v[ROUTE_PER_LANE];
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < ROUTE_PER_LANE; j++) {
    const int i = lane + 64 * j;
    v[j] = i < e ? row[i] : -INFINITY;
    mx = fmaxf(mx, v[j]);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d));
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < ROUTE_PER_LANE; j++) {
    v[j] = lane + 64 * j < e ? expf(v[j] - mx) : -1.f;
    sum += fmaxf(v[j], 0.f);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) sum += __shfl_xor(sum, d);
#pragma unroll
  for (int j = 0; j < ROUTE_PER_LANE; j++) v[j] = v[j] >= 0.f ? v[j] / sum : -1.f;
  float total = 0.f, mine = 0.f;
  int mine_id = 0;
  for (int s = 0; s < k; s++) {
    float best = -1.f;
    int at = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < ROUTE_PER_LANE; j++)
      if (v[j] > best) {  // ascending index within the lane: the first of equals stays
        best = v[j];
        at = lane + 64 * j;
      }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
      const float ob = __shfl_xor(best, d);
      const int oa = __shfl_xor(at, d);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    total += best;
    if (lane == s) {
      mine = best;
      mine_id = at;
    }
    if ((at & 63) == lane) {
#pragma unroll
      for (int j = 0; j < ROUTE_PER_LANE; j++)
        if (j == (at >> 6)) v[j] = -1.f;
    }
  }
  if (lane < k) {
    ids[r * k + lane] = mine_id;
    weights[r * k + lane] = mine / total;
  }
}

// ---------------------------------------------------------------------------------------------------- host side
// Measurement hook: events the caller created, recorded around each kernel of the next routed-expert chain.
static std::vector<hipEvent_t> g_events;
static size_t g_event_next = 0;
static inline void mark(hipStream_t stream) {
  if (g_event_next < g_events.size()) (void)hipEventRecord(g_events[g_event_next++], stream);
}

struct Tuning {
  int w3_ksplit = 0, w3_nbw = 0, moe_fc1_ksplit = 0, moe_fc1_nbw = 0, moe_fc2_ksplit = 0, moe_fc2_nbw = 0;
};
static Tuning g_tune;

// Wavefronts per workgroup: K is split until a launch has about `want` wavefronts, keeping at least four chunks per
// wavefront; what is left of a 4-wavefront workgroup takes neighbouring 64-row blocks.
static void pick_shape(int n_blocks, int chunks, int64_t slots, int want, int* ks, int* nbw) {
  int k = 1;
  while (k < 16 && (int64_t)n_blocks * slots * k < want && chunks / (2 * k) >= 4) k *= 2;
  int b = k >= 4 ? 1 : 4 / k;
  while (b > 1 && n_blocks % b) b /= 2;
  *ks = k;
  *nbw = b;
}

// Launch one W3 stream. `busy_slots` is the caller's estimate of the slots that will have rows (the grid covers
// `slots`, the upper bound); K is split until the launch has a few thousand wavefronts.
struct Launch {
  int ks, nbw;  // 0: chosen here
};

template <int EPI>
static int launch_stream(StreamParams& p, int64_t slots, int64_t busy_slots, Launch want, hipStream_t stream) {
  pick_shape(p.n_blocks, p.chunks, busy_slots, 8192, &p.ks, &p.nbw);
  if (want.ks) {
    p.ks = want.ks;
    if (!want.nbw) p.nbw = 1;
  }
  if (want.nbw) p.nbw = want.nbw;
  if (p.ks * p.nbw > 16 || p.ks > p.chunks) return HB_EINVAL;
  const dim3 grid((unsigned)((p.n_blocks + p.nbw - 1) / p.nbw), (unsigned)slots);
  const int waves = p.ks * p.nbw;
  hipLaunchKernelGGL(w3_stream_kernel<EPI>, grid, dim3(64 * waves), p.ks > 1 ? (size_t)waves * 4096 : 0, stream, p);
  return HB_OK;
}

}  // namespace hb

using namespace hb;

extern "C" int hb_tune(const char* key, int value) {
  if (!key) return HB_ENULL;
  struct {
    const char* name;
    int* slot;
  } table[] = {{"w3_ksplit", &g_tune.w3_ksplit},           {"w3_nbw", &g_tune.w3_nbw},
               {"moe_fc1_ksplit", &g_tune.moe_fc1_ksplit}, {"moe_fc1_nbw", &g_tune.moe_fc1_nbw},
               {"moe_fc2_ksplit", &g_tune.moe_fc2_ksplit}, {"moe_fc2_nbw", &g_tune.moe_fc2_nbw}};
  for (auto& t : table)
    if (!strcmp(t.name, key)) {
      if (value < 0 || value > 16 || (value & (value - 1))) return HB_EINVAL;
      *t.slot = value;
      return HB_OK;
    }
  return HB_EINVAL;
}

extern "C" int hb_w3_gemm(const void* x, int m, const void* tiled, const float* row_scale, int64_t lut, int n, int k, void* y, void* stream) {
  if (!x || !tiled || !row_scale || !y) return HB_ENULL;
  if (m <= 0 || n <= 0 || k <= 0 || n % W3_BLOCK_ROWS || k % W3_CHUNK) return HB_EINVAL;
  StreamParams p{};
  p.w = static_cast<const uint8_t*>(tiled);
  p.rows = row_scale;
  p.lut_lo = (uint32_t)((uint64_t)lut & 0xffffffffu);
  p.lut_hi = (uint32_t)((uint64_t)lut >> 32);
  p.n_blocks = n / W3_BLOCK_ROWS;
  p.chunks = k / W3_CHUNK;
  p.a = static_cast<const uint16_t*>(x);
  p.a_stride = k;
  p.m = m;
  p.out = y;
  p.out_stride = n;
  const int64_t slots = (m + ROWS_PER_SLOT - 1) / ROWS_PER_SLOT;
  if (slots > 65535) return HB_EINVAL;
  if (int e = launch_stream<EPI_DENSE>(p, slots, slots, Launch{g_tune.w3_ksplit, g_tune.w3_nbw}, as_stream(stream))) return e;
  return launch_status();
}

// ------------------------------------------------------------------------------------------------ routed experts
namespace {

struct MoeWorkspace {
  int32_t* plan;
  int32_t* order;
  uint16_t* h;   // [(pairs + shared rows), inter] BF16, in sorted order
  float* y;      // [(pairs + shared rows), hidden_out] FP32 (or BF16 pairs), by pair index
  size_t bytes;
};

int64_t max_slots(int64_t pairs, int experts, int shared_rows) {
  const int64_t routed = pairs < pairs / ROWS_PER_SLOT + experts ? pairs : pairs / ROWS_PER_SLOT + experts;
  return routed + (shared_rows + ROWS_PER_SLOT - 1) / ROWS_PER_SLOT;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

MoeWorkspace carve(void* base, int m, int topk, const hb_w3_experts* ex, int shared) {
  const int64_t pairs = (int64_t)m * topk, rows = pairs + (shared ? m : 0);
  MoeWorkspace w{};
  size_t off = 0;
  auto take = [&](size_t bytes) {
    void* ptr = base ? static_cast<char*>(base) + off : nullptr;
    off += align256(bytes);
    return ptr;
  };
  w.plan = static_cast<int32_t*>(take((PLAN_HEADER + 4 * max_slots(pairs, ex->experts, shared ? m : 0)) * sizeof(int32_t)));
  w.order = static_cast<int32_t*>(take(rows * sizeof(int32_t)));
  w.h = static_cast<uint16_t*>(take((size_t)rows * ex->inter * sizeof(uint16_t)));
  w.y = static_cast<float*>(take((size_t)rows * ex->hidden_out * sizeof(float)));
  w.bytes = off;
  return w;
}

int check_experts(const hb_w3_experts* ex) {
  if (!ex) return HB_ENULL;
  if (!ex->fc1 || !ex->fc1_rows || !ex->fc2 || !ex->fc2_rows) return HB_ENULL;
  if (ex->experts <= 0 || ex->hidden <= 0 || ex->inter <= 0 || ex->hidden_out <= 0) return HB_EINVAL;
  const int n1 = ex->gated ? 2 * ex->inter : ex->inter;
  if (ex->hidden % W3_CHUNK || ex->inter % W3_CHUNK || n1 % W3_BLOCK_ROWS || ex->hidden_out % W3_BLOCK_ROWS) return HB_EINVAL;
  return HB_OK;
}

// plan -> fc1 -> fc2 (-> combine): `out_pairs` receives fc2's per-pair outputs (the workspace's y unless the caller
// wants the pairs themselves).
int run_experts(const hb_w3_experts* ex, const hb_w3_experts* shared, const void* x, const int32_t* ids, int m, int topk,
                const MoeWorkspace& ws, void* out_pairs, int pairs_bf16, hipStream_t stream) {
  const int64_t pairs = (int64_t)m * topk;
  const int shared_rows = shared ? m : 0;
  const int64_t slots = max_slots(pairs, ex->experts, shared_rows);
  if (slots > 65535 || pairs > 0x3fffffff) return HB_EINVAL;
  const size_t plan_lds = ((size_t)(PLAN_WAVES + 1) * ex->experts + 3 * (PLAN_WAVES + 1)) * sizeof(int);
  if (plan_lds > 64 * 1024) return HB_EINVAL;
  mark(stream);
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(PLAN_THREADS), plan_lds, stream, ids, (int)pairs, ex->base, ex->experts, shared_rows,
                     ws.plan, ws.order);
  mark(stream);
  const int n1 = ex->gated ? 2 * ex->inter : ex->inter;
  const int64_t est = pairs < 2 * ex->experts ? (pairs + 1) / 2 + (shared_rows + 15) / 16 : slots;  // rough number of busy slots
  StreamParams p{};
  p.w = static_cast<const uint8_t*>(ex->fc1);
  p.expert_bytes = (int64_t)hb_w3_tiled_bytes(n1, ex->hidden);
  p.rows = ex->fc1_rows;
  p.expert_rows = n1;
  p.lut_lo = (uint32_t)((uint64_t)ex->fc1_lut & 0xffffffffu);
  p.lut_hi = (uint32_t)((uint64_t)ex->fc1_lut >> 32);
  if (shared) {
    p.w_shared = static_cast<const uint8_t*>(shared->fc1);
    p.rows_shared = shared->fc1_rows;
    p.lut_lo_shared = (uint32_t)((uint64_t)shared->fc1_lut & 0xffffffffu);
    p.lut_hi_shared = (uint32_t)((uint64_t)shared->fc1_lut >> 32);
  }
  p.n_blocks = n1 / W3_BLOCK_ROWS;
  p.chunks = ex->hidden / W3_CHUNK;
  p.a = static_cast<const uint16_t*>(x);
  p.a_stride = ex->hidden;
  p.plan = ws.plan;
  p.order = ws.order;
  p.topk = topk;
  p.pairs = (int)pairs;
  p.out = ws.h;
  p.out_stride = ex->inter;
  StreamParams f2 = p;
  f2.w = static_cast<const uint8_t*>(ex->fc2);
  f2.expert_bytes = (int64_t)hb_w3_tiled_bytes(ex->hidden_out, ex->inter);
  f2.rows = ex->fc2_rows;
  f2.expert_rows = ex->hidden_out;
  f2.lut_lo = (uint32_t)((uint64_t)ex->fc2_lut & 0xffffffffu);
  f2.lut_hi = (uint32_t)((uint64_t)ex->fc2_lut >> 32);
  if (shared) {
    f2.w_shared = static_cast<const uint8_t*>(shared->fc2);
    f2.rows_shared = shared->fc2_rows;
    f2.lut_lo_shared = (uint32_t)((uint64_t)shared->fc2_lut & 0xffffffffu);
    f2.lut_hi_shared = (uint32_t)((uint64_t)shared->fc2_lut >> 32);
  }
  f2.n_blocks = ex->hidden_out / W3_BLOCK_ROWS;
  f2.chunks = ex->inter / W3_CHUNK;
  f2.a = ws.h;
  f2.a_stride = ex->inter;
  f2.out = out_pairs;
  f2.out_stride = ex->hidden_out;
  f2.out_bf16 = pairs_bf16;
  const Launch l1{g_tune.moe_fc1_ksplit, g_tune.moe_fc1_nbw}, l2{g_tune.moe_fc2_ksplit, g_tune.moe_fc2_nbw};
  if (int e = ex->gated ? launch_stream<EPI_FC1_GATED>(p, slots, est, l1, stream) : launch_stream<EPI_FC1_RELU2>(p, slots, est, l1, stream)) return e;
  mark(stream);
  if (int e = launch_stream<EPI_FC2>(f2, slots, est, l2, stream)) return e;
  mark(stream);
  return launch_status();
}

void launch_combine(const CombineParams& c, hipStream_t stream) {
  hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)c.m, (unsigned)((c.h + COMBINE_SPAN - 1) / COMBINE_SPAN)), dim3(256), 0, stream, c);
  mark(stream);
}

}  // namespace

extern "C" size_t hb_w3_moe_workspace_bytes(int m, int topk, const hb_w3_experts* routed, int shared) {
  if (!routed || m <= 0 || topk <= 0 || check_experts(routed) != HB_OK) return 0;
  return carve(nullptr, m, topk, routed, shared).bytes;
}

extern "C" int hb_w3_moe(const hb_w3_experts* routed, const void* x, const int32_t* ids, const float* weights, int m, int topk, int mode,
                         void* out, void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_experts(routed)) return e;
  if (!x || !ids || !weights || !out || !workspace) return HB_ENULL;
  if (m <= 0 || topk <= 0 || mode < HB_MOE_SUM || mode > HB_MOE_PAIRS_BF16) return HB_EINVAL;
  const MoeWorkspace ws = carve(workspace, m, topk, routed, 0);
  if (workspace_bytes < ws.bytes) return HB_EWORKSPACE;
  void* pairs_out = mode == HB_MOE_SUM ? static_cast<void*>(ws.y) : out;
  if (int e = run_experts(routed, nullptr, x, ids, m, topk, ws, pairs_out, mode == HB_MOE_PAIRS_BF16, as_stream(stream))) return e;
  if (mode == HB_MOE_SUM) {
    CombineParams c{};
    c.pairs = ws.y;
    c.ids = ids;
    c.weights = weights;
    c.e_lo = routed->base;
    c.e_n = routed->experts;
    c.m = m;
    c.topk = topk;
    c.h = routed->hidden_out;
    c.out = static_cast<uint16_t*>(out);
    launch_combine(c, as_stream(stream));
  }
  return launch_status();
}

extern "C" int hb_w3_moe_layer(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                               const int32_t* ids, const float* weights, int m, int topk, void* out, void* workspace,
                               size_t workspace_bytes, void* stream) {
  if (int e = check_experts(routed)) return e;
  if (shared) {
    if (int e = check_experts(shared)) return e;
    if (shared->hidden != routed->hidden || shared->inter != routed->inter || shared->hidden_out != routed->hidden_out ||
        shared->gated != routed->gated)
      return HB_EINVAL;
  }
  if (!x || !ids || !weights || !out || !workspace) return HB_ENULL;
  if (m <= 0 || topk <= 0) return HB_EINVAL;
  const MoeWorkspace ws = carve(workspace, m, topk, routed, shared ? 1 : 0);
  if (workspace_bytes < ws.bytes) return HB_EWORKSPACE;
  if (int e = run_experts(routed, shared, x, ids, m, topk, ws, ws.y, 0, as_stream(stream))) return e;
  CombineParams c{};
  c.pairs = ws.y;
  c.ids = ids;
  c.weights = weights;
  if (shared) {
    c.shared = ws.y + (int64_t)m * topk * routed->hidden_out;
    c.shared_f32 = 1;
    c.shared_stride = routed->hidden_out;
    c.x = static_cast<const uint16_t*>(x);
    c.gate_vec = gate_vec;
    c.hx = routed->hidden;
  }
  c.e_lo = routed->base;
  c.e_n = routed->experts;
  c.m = m;
  c.topk = topk;
  c.h = routed->hidden_out;
  c.out = static_cast<uint16_t*>(out);
  launch_combine(c, as_stream(stream));
  return launch_status();
}

extern "C" int hb_moe_combine_pairs(const void* pairs, int pairs_bf16, const int32_t* ids, const float* weights, const void* shared,
                                    const void* x, const float* gate_vec, int e_lo, int e_n, int m, int topk, int h, void* out,
                                    void* stream) {
  if (!pairs || !ids || !weights || !out) return HB_ENULL;
  if (gate_vec && shared && !x) return HB_ENULL;
  if (m <= 0 || topk <= 0 || h <= 0 || h % 2) return HB_EINVAL;
  CombineParams c{};
  c.pairs = pairs;
  c.pairs_bf16 = pairs_bf16;
  c.ids = ids;
  c.weights = weights;
  c.shared = shared;
  c.shared_stride = h;
  c.x = static_cast<const uint16_t*>(x);
  c.gate_vec = gate_vec;
  c.hx = h;
  c.e_lo = e_lo;
  c.e_n = e_n;
  c.m = m;
  c.topk = topk;
  c.h = h;
  c.out = static_cast<uint16_t*>(out);
  launch_combine(c, as_stream(stream));
  return launch_status();
}

extern "C" int hb_route_softmax_topk(const float* logits, int m, int e, int k, int32_t* ids, float* weights, void* stream) {
  if (!logits || !ids || !weights) return HB_ENULL;
  if (m <= 0 || e <= 0 || k <= 0 || k > e || k > 64 || e > 64 * ROUTE_PER_LANE) return HB_EINVAL;
  hipLaunchKernelGGL(route_softmax_topk_kernel, dim3((unsigned)m), dim3(64), 0, as_stream(stream), logits, e, k, ids, weights);
  return launch_status();
}

extern "C" int hb_debug_events(void* const* events, int count) {
  if (count < 0 || (count > 0 && !events)) return HB_EINVAL;
  g_events.assign(reinterpret_cast<hipEvent_t const*>(events), reinterpret_cast<hipEvent_t const*>(events) + count);
  g_event_next = 0;
  return HB_OK;
}

extern "C" int hb_version(void) { return 1000; }

extern "C" const char* hb_error_string(int code) {
  switch (code) {
    case HB_OK: return "ok";
    case HB_EINVAL: return "unsupported shape, alignment or flag";
    case HB_ENULL: return "a required pointer is null";
    case HB_EWORKSPACE: return "workspace too small";
    case HB_ELAUNCH: return "the HIP runtime refused a launch";
    default: return "unknown error";
  }
}
