// Shared by the W3 and NVFP4 weight streams: launch parameters, the slot table of a routed call, the epilogues
// (row / global scale, the reference's rounding points, SiLU gate or ReLU^2, pair outputs), the K-split exchange through
// LDS, and the host-side helpers of a routed call (workspace, plan launch, combine launch).
#pragma once

#include <hip/hip_ext.h>

#include "common.hpp"

namespace hb {

enum { EPI_DENSE = 0, EPI_FC1_GATED = 1, EPI_FC1_RELU2 = 2, EPI_FC2 = 3, EPI_DENSE_RELU2 = 4 };
constexpr bool epi_dense(int epi) { return epi == EPI_DENSE || epi == EPI_DENSE_RELU2; }
constexpr bool epi_gathers(int epi) { return epi == EPI_FC1_GATED || epi == EPI_FC1_RELU2; }  // activation rows found through `order`
constexpr int ROWS_PER_SLOT = 16;
constexpr int MOE_WIDE_ROWS = 1024;  // rows from which a routed sum keeps its pair outputs in BF16 (the reference's WIDE_ROWS)
constexpr int PLAN_HEADER = 16;  // plan[0] = slots, plan[1] = distinct experts, plan[2] = routed pairs kept, then the two words below
// Two words of a workspace's head that no launch initializes: the caller hands the workspace over zero-filled once, and
// every call leaves them as the next one needs them.
constexpr int PLAN_TICKET = 3;  // the arrival counter of a launch whose last workgroup plans: zero between calls (the last arriver puts it back)
constexpr int PLAN_FAULT = 4;   // sticky: a kernel whose bounded wait gave up ors its HB_FAULT_* bit in; only hb_workspace_reset clears it
constexpr int WAIT_SPINS = 1 << 20;  // polls (about a second) before a wait gives up

struct StreamParams {
  const uint8_t* w;       // tile layout, expert 0
  int64_t expert_bytes;   // bytes between experts
  const float* rows;      // row scales, expert 0
  int64_t expert_rows;    // floats between experts
  const uint8_t* w_shared;  // the shared expert (slot expert id < 0), or null
  const float* rows_shared;
  const float* scalars;   // formats with one FP32 scale per matrix: [experts], or null for `scalar`
  float scalar, scalar_shared;
  uint32_t lut_lo, lut_hi, lut_lo_shared, lut_hi_shared;
  int n_blocks;           // 64-row blocks per expert matrix
  int chunks;             // K / 128
  const uint16_t* a;      // BF16 activations
  int64_t a_stride;       // elements between rows
  const uint8_t* aq;      // E4M3 activation mode: codes [rows, a_stride] ...
  const float* aq_scale;  // ... and their scales [rows, a_stride / 32]
  const uint8_t* a2;      // two-plane form of the BF16 activations (split_row below): [rows, a_stride / 128, 2, 128] E4M3 bytes ...
  const float* a2_scale;  // ... and one FP32 scale a row; slots of at most two rows read these instead of `a`
  const int32_t* plan;    // grouped calls: slot table
  const int32_t* order;   // grouped calls: sorted position -> pair index
  int m;                  // dense calls: rows
  int slot_rows;          // dense calls: rows a slot (0: ROWS_PER_SLOT)
  int topk, pairs;        // grouped calls: pair q < pairs belongs to token q / topk, q >= pairs to token q - pairs
  void* out;
  int64_t out_stride;     // elements between output rows
  uint8_t* oq;            // fc1 in the E4M3 activation mode: h leaves as codes [rows, out_stride] ...
  float* oq_scale;        // ... and scales [rows, out_stride / 32] instead of BF16 in `out`
  int out_bf16;           // EPI_FC2: pair outputs in BF16 instead of FP32
  int ks, nbw;            // wavefronts per workgroup = ks (K splits) * nbw (64-row blocks)
  int ks_inv, chunks_base, chunks_rem;  // set_split(): ceil(65536 / ks), chunks / ks, chunks % ks
  int no_few;             // W3 stream: slots of at most four rows take the sixteen-row body too
  float* partial;         // tile kernel with K shared among workgroups: their partial tiles (see tile_kernel.hpp)
  int tile_ks, tile_mt;   // ... the workgroups a tile (1: none), the 16-row tiles a partial region holds
  uint32_t* tile_tickets; // ... and the tiles' arrival counters (one a tile, in the caller's workspace: zero between calls)
  int64_t* trace;         // measurement hook (hb_debug_trace): a record a workgroup, else null
  int64_t trace_records;  // ... and the records it holds
  int32_t* done;          // fc1 and fc2 in one launch: the slots' arrival counters (plan_done), else null
  int done_need;          // ... and the fc1 workgroups a slot has
  int wait_spins;         // ... and the polls after which a wait for them gives up
  int32_t* fault;         // ... which it records here (the workspace's PLAN_FAULT word)
};

// Device-scope accesses that do not rest in the compute die's own L2: a store that is written through to memory, a
// load that is served from there. A workgroup that has waited for its write-through stores (vmcnt) and then draws a
// ticket has published them to whichever workgroup draws a later ticket and reads with load_through, on any compute
// die, without a cache write-back or invalidate of its own.
__device__ __forceinline__ void store_through(int32_t* at, int32_t v) { __hip_atomic_store(at, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ int32_t load_through(const int32_t* at) { return __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void store_through(float* at, float v) { __hip_atomic_store(at, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float load_through(const float* at) { return __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint16_t load_through(const uint16_t* at) { return __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

__device__ __forceinline__ void store_through(uint16_t* at, uint16_t v) { __hip_atomic_store(at, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// One arrival counter a slot, behind the plan's slot table (`slot_cap`: the table's entries, the launch's upper bound
// on the slots); the plan leaves them zero. A launch that runs fc1 and fc2 together counts there the fc1 workgroups of
// a slot that have finished, and the slot's fc2 workgroups wait for all of them.
// Each counter has a 128-byte line of its own (DONE_PITCH ints apart): the workgroups that poll one slot's counter do
// not stand in the way of another slot's arrivals.
constexpr int DONE_PITCH = 32;
__host__ __device__ inline int32_t* plan_done(int32_t* plan, int64_t slot_cap) { return plan + (PLAN_HEADER + 4 * slot_cap + 31) / 32 * 32; }

// Waits (every lane of the wavefront together) until the counter has reached `need`; false if it has not after `spins`
// polls. The wait is bounded so that every wavefront leaves whatever happens elsewhere; a caller that gets false must
// not use what the count guards (it records the fault and skips its work).
__device__ __forceinline__ bool await_count(const int32_t* at, int need, int spins) {
  bool there = load_through(at) >= need;
  for (int n = 0; !there && n < spins; n++) {
    __builtin_amdgcn_s_sleep(8);
    there = load_through(at) >= need;
  }
  asm volatile("" ::: "memory");  // what the count guards is read after it
  return there;
}

// The epilogue's roundings use the hardware FP32 -> BF16 conversion (round to nearest even).
__device__ __forceinline__ uint16_t bf16_of(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
__device__ __forceinline__ float through_bf16(float f) { return (float)(__bf16)f; }
// Two values rounded to BF16 by one packed conversion (v_cvt_pk_bf16_f32: `lo` in the low half), and the halves of such a
// pair as FP32 again: the same roundings as bf16_of / through_bf16, half the conversions.
typedef __attribute__((ext_vector_type(2))) float f32x2_pair_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_pair_t;
__device__ __forceinline__ uint32_t bf16_pair(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_pair_t{lo, hi}, bf16x2_pair_t));
}
__device__ __forceinline__ float pair_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float pair_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

// silu with the fast exponential and division: the result is rounded to BF16 right after (8 significant bits).
__device__ __forceinline__ float silu(float g) { return __fdividef(g, 1.0f + __expf(-g)); }

// What a workgroup needs to know about its slot (up to 16 activation rows of one expert, or of the dense matrix).
struct Slot {
  int index;           // which slot of the table (or of the dense call)
  int p0, rows;        // first row (sorted position) and number of rows
  const uint8_t* w;    // the expert's tile-layout matrix
  const float* rs;     // its row scales (formats that have them)
  float scalar;        // its FP32 scale (formats with one per matrix)
  uint32_t lut_lo, lut_hi;
};

// The FP32 row scales of a 64-row block at this lane's row-in-tile, one per 16-row tile.
struct RowScales {
  float s[4];
  __device__ __forceinline__ float of(int t) const { return t == 0 ? s[0] : t == 1 ? s[1] : t == 2 ? s[2] : s[3]; }
};

template <bool PER_ROW>
__device__ __forceinline__ RowScales row_scales(const Slot& sl, int nb, int r16) {
  RowScales rs;
#pragma unroll
  for (int t = 0; t < 4; t++) rs.s[t] = PER_ROW ? sl.rs[nb * 64 + 16 * t + r16] : 0.f;
  return rs;
}

// What fc1 hands to fc2 for one element, as the FP32 value of its BF16 rounding: y0 / y1 are the K-complete sums times
// their FP32 scale (gated: the up and the gate row); the roundings are the reference's.
template <int EPI>
__device__ __forceinline__ float fc1_value(float y0, float y1) {
  if (EPI == EPI_FC1_GATED) return through_bf16(silu(through_bf16(y1)) * through_bf16(y0));
  const float h = fmaxf(through_bf16(y0), 0.f);
  return through_bf16(h * h);
}

// Stores one output element (gated: one up/gate pair) of the 64-row block: row tile `t` (gated: pair index), column r16
// of it, slot row i.
template <int EPI>
__device__ __forceinline__ void store_out(const StreamParams& p, const Slot& sl, int nb, int t, int i, int r16, float y0, float y1) {
  const int64_t pos = sl.p0 + i;
  // h goes through to memory: its readers may be workgroups of the same launch on another compute die
  if (EPI == EPI_FC1_GATED) {
    store_through(&reinterpret_cast<uint16_t*>(p.out)[pos * p.out_stride + nb * 32 + 16 * t + r16], bf16_of(fc1_value<EPI>(y0, y1)));
  } else {
    const int n = nb * 64 + 16 * t + r16;
    if (EPI == EPI_FC1_RELU2) {
      store_through(&reinterpret_cast<uint16_t*>(p.out)[pos * p.out_stride + n], bf16_of(fc1_value<EPI_FC1_RELU2>(y0, 0.f)));
    } else if (EPI == EPI_DENSE_RELU2) {
      reinterpret_cast<uint16_t*>(p.out)[pos * p.out_stride + n] = bf16_of(fc1_value<EPI_FC1_RELU2>(y0, 0.f));
    } else if (EPI == EPI_DENSE) {
      reinterpret_cast<uint16_t*>(p.out)[pos * p.out_stride + n] = bf16_of(y0);
    } else {
      const int64_t pair = p.order[pos];
      if (p.out_bf16) {
        reinterpret_cast<uint16_t*>(p.out)[pair * p.out_stride + n] = bf16_of(y0);
      } else {
        reinterpret_cast<float*>(p.out)[pair * p.out_stride + n] = y0;
      }
    }
  }
}

// The largest of a value over the sixteen lanes of a DPP row, in each of them. Lanes that are switched off
// contribute 0 (the values are magnitudes).
__device__ __forceinline__ float row16_max(float x) {
  x = fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, false)));   // lane ^ 1
  x = fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, false)));   // lane ^ 2
  x = fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, false)));  // mirror within 8
  x = fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, false)));  // mirror within 16
  return x;
}

// The activation rounding of one element of h inside fc1's epilogue: `h` = fc1_value of column `col` of sorted row
// `pos`, `amax` the largest magnitude of the column's 32-group. s = max(amax / 448, 1e-12), code = e4m3(h / s), IEEE
// divisions: the arithmetic of the separate quantizer (quant_groups_lane below), value for value.
__device__ __forceinline__ void store_quantized(const StreamParams& p, int64_t pos, int col, float h, float amax, bool first_of_group) {
  const float s = fmaxf(amax / 448.0f, 1e-12f);
  const float v = fminf(fmaxf(h / s, -448.0f), 448.0f);
  p.oq[pos * p.out_stride + col] = (uint8_t)__builtin_amdgcn_cvt_pk_fp8_f32(v, 0.f, 0, false);
  if (first_of_group) p.oq_scale[pos * (p.out_stride >> 5) + (col >> 5)] = s;
}

// One output element (or, gated, one up/gate pair) from accumulator register r of lane (q, r16); v0 / v1 are the
// K-complete sums before the FP32 scale (per output row with PER_ROW, else one per matrix).
template <int EPI, bool PER_ROW>
__device__ __forceinline__ void emit(const StreamParams& p, const Slot& sl, const RowScales& rs, int nb, int t, int r, int q, int r16, float v0,
                                     float v1) {
  if (r >= sl.rows) return;  // wave-uniform: this accumulator register holds no row of the slot in any lane
  const int i = 4 * q + r;   // activation row of the slot held by this accumulator register
  if (i >= sl.rows) return;
  if (EPI == EPI_FC1_GATED) {
    store_out<EPI>(p, sl, nb, t, i, r16, v0 * (PER_ROW ? rs.of(2 * t) : sl.scalar), v1 * (PER_ROW ? rs.of(2 * t + 1) : sl.scalar));
  } else {
    store_out<EPI>(p, sl, nb, t, i, r16, v0 * (PER_ROW ? rs.of(t) : sl.scalar), 0.f);
  }
}

// The E4M3 form of emit for fc1: the four K-complete sums of accumulator register r of lane (q, r16), one per 16-row
// tile, become this slot row's codes of the block's h columns (gated: 32 columns, one group; else 64, two groups). A
// group's columns are the sixteen lanes of this lane's DPP row times two tiles; the row's lanes hold the same slot row,
// so they stay or leave together.
template <int EPI>
__device__ __forceinline__ void quant_emit(const StreamParams& p, const Slot& sl, const RowScales& rs, int nb, int r, int q, int r16, float v0, float v1,
                                           float v2, float v3) {
  if (r >= sl.rows) return;  // wave-uniform
  const int i = 4 * q + r;
  if (i >= sl.rows) return;
  const int64_t pos = sl.p0 + i;
  const float y0 = v0 * rs.of(0), y1 = v1 * rs.of(1), y2 = v2 * rs.of(2), y3 = v3 * rs.of(3);
  if (EPI == EPI_FC1_GATED) {
    const float h0 = fc1_value<EPI>(y0, y1), h1 = fc1_value<EPI>(y2, y3);
    const float amax = row16_max(fmaxf(fabsf(h0), fabsf(h1)));
    store_quantized(p, pos, nb * 32 + r16, h0, amax, r16 == 0);
    store_quantized(p, pos, nb * 32 + 16 + r16, h1, amax, false);
  } else {
    const float h0 = fc1_value<EPI>(y0, 0.f), h1 = fc1_value<EPI>(y1, 0.f), h2 = fc1_value<EPI>(y2, 0.f), h3 = fc1_value<EPI>(y3, 0.f);
    const float lo = row16_max(fmaxf(fabsf(h0), fabsf(h1))), hi = row16_max(fmaxf(fabsf(h2), fabsf(h3)));
    store_quantized(p, pos, nb * 64 + r16, h0, lo, r16 == 0);
    store_quantized(p, pos, nb * 64 + 16 + r16, h1, lo, false);
    store_quantized(p, pos, nb * 64 + 32 + r16, h2, hi, r16 == 0);
    store_quantized(p, pos, nb * 64 + 48 + r16, h3, hi, false);
  }
}

// The slot of rows p0 .. p0 + rows - 1 of `expert` (negative: the shared expert).
__device__ __forceinline__ Slot make_slot(const StreamParams& p, int index, int expert, int p0, int rows) {
  Slot s;
  s.index = index;
  s.p0 = p0;
  s.rows = rows;
  s.w = expert < 0 ? p.w_shared : p.w + (int64_t)expert * p.expert_bytes;
  s.rs = expert < 0 ? p.rows_shared : p.rows + (int64_t)expert * p.expert_rows;
  // an entry without rows names no expert: nothing indexed by it is read
  s.scalar = expert < 0 ? p.scalar_shared : (p.scalars && s.rows > 0) ? p.scalars[expert] : p.scalar;
  s.lut_lo = expert < 0 ? p.lut_lo_shared : p.lut_lo;
  s.lut_hi = expert < 0 ? p.lut_hi_shared : p.lut_hi;
  return s;
}

template <int EPI>
__device__ __forceinline__ Slot slot_of(const StreamParams& p, int slot) {
  if (epi_dense(EPI)) {
    const int per = p.slot_rows ? p.slot_rows : ROWS_PER_SLOT, p0 = slot * per;
    return make_slot(p, slot, 0, p0, min(per, p.m - p0));
  }
  const int32_t* entry = p.plan + PLAN_HEADER + 4 * slot;
  return make_slot(p, slot, entry[0], entry[1], entry[2]);
}

// Which K split (`ks`) and which of the workgroup's blocks (`nbi`) a wavefront is, and the chunks c0 .. c1 - 1 of its
// split (the first chunks % ks splits have one chunk more). No division: wave / ks is a multiply by ceil(65536 / ks),
// exact for the sixteen wavefronts a workgroup can have.
struct WaveShare {
  int ks, nbi, c0, c1;
};
__device__ __forceinline__ WaveShare wave_share(const StreamParams& p, int wave) {
  WaveShare w;
  w.nbi = (wave * p.ks_inv) >> 16;
  w.ks = wave - w.nbi * p.ks;
  w.c0 = w.ks * p.chunks_base + min(w.ks, p.chunks_rem);
  w.c1 = w.c0 + p.chunks_base + (w.ks < p.chunks_rem ? 1 : 0);
  return w;
}
inline void set_split(StreamParams& p) {  // after ks is chosen
  p.ks_inv = (65536 + p.ks - 1) / p.ks;
  p.chunks_base = p.chunks / p.ks;
  p.chunks_rem = p.chunks % p.ks;
}

// The row of the activation matrix that is row r of the slot. Rows past the slot's last read that last row again: their
// MFMA output rows are never stored.
template <int EPI>
__device__ __forceinline__ int64_t activation_row_index(const StreamParams& p, const Slot& s, int r) {
  int64_t arow = s.p0 + min(r, s.rows - 1);
  if (epi_gathers(EPI)) {
    const int pair = p.order[arow];
    arow = pair < p.pairs ? pair / p.topk : pair - p.pairs;
  }
  return arow;
}

// The activation row this lane feeds to the MFMA A operand (row r16 of the slot).
template <int EPI>
__device__ __forceinline__ const uint16_t* activation_row(const StreamParams& p, const Slot& s, int r16) {
  return p.a + activation_row_index<EPI>(p, s, r16) * p.a_stride;
}

// The end of a 64-row block: K-complete sums straight from the registers (ks == 1), or the K split's partial sums
// exchanged through LDS (`partial`: 4 KB at the start of each wavefront's STRIDE floats) and added in split order,
// then the epilogue. With ks > 1 every wavefront of the workgroup must call it (one workgroup barrier). QUANT (fc1 in
// the E4M3 activation mode): the epilogue is quant_emit, a split taking whole accumulator registers (all four tiles
// of slot rows r, r + 4, ...), since a group's maximum needs two tiles.
template <int EPI, bool PER_ROW, int STRIDE = 1024, bool QUANT = false>
__device__ __forceinline__ void finish_block(const StreamParams& p, const Slot& sl, const RowScales& rs, int nb, bool active, int ks, int nbi, float* partial,
                                             const f32x4_t& acc0, const f32x4_t& acc1, const f32x4_t& acc2, const f32x4_t& acc3, int stride_floats = 0) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int q = lane >> 4, r16 = lane & 15;
  const int rows = sl.rows;
  const int stride = stride_floats ? stride_floats : STRIDE;  // floats between the wavefronts' exchange areas (the launch's ring size when it varies)
  if (p.ks == 1) {
    if (!active) return;
    if (QUANT) {
      quant_emit<EPI>(p, sl, rs, nb, 0, q, r16, acc0.x, acc1.x, acc2.x, acc3.x);
      quant_emit<EPI>(p, sl, rs, nb, 1, q, r16, acc0.y, acc1.y, acc2.y, acc3.y);
      quant_emit<EPI>(p, sl, rs, nb, 2, q, r16, acc0.z, acc1.z, acc2.z, acc3.z);
      quant_emit<EPI>(p, sl, rs, nb, 3, q, r16, acc0.w, acc1.w, acc2.w, acc3.w);
    } else if (EPI == EPI_FC1_GATED) {
      emit<EPI, PER_ROW>(p, sl, rs, nb, 0, 0, q, r16, acc0.x, acc1.x);
      emit<EPI, PER_ROW>(p, sl, rs, nb, 0, 1, q, r16, acc0.y, acc1.y);
      emit<EPI, PER_ROW>(p, sl, rs, nb, 0, 2, q, r16, acc0.z, acc1.z);
      emit<EPI, PER_ROW>(p, sl, rs, nb, 0, 3, q, r16, acc0.w, acc1.w);
      emit<EPI, PER_ROW>(p, sl, rs, nb, 1, 0, q, r16, acc2.x, acc3.x);
      emit<EPI, PER_ROW>(p, sl, rs, nb, 1, 1, q, r16, acc2.y, acc3.y);
      emit<EPI, PER_ROW>(p, sl, rs, nb, 1, 2, q, r16, acc2.z, acc3.z);
      emit<EPI, PER_ROW>(p, sl, rs, nb, 1, 3, q, r16, acc2.w, acc3.w);
    } else {
      const f32x4_t all[4] = {acc0, acc1, acc2, acc3};
#pragma unroll
      for (int t = 0; t < 4; t++) {
        emit<EPI, PER_ROW>(p, sl, rs, nb, t, 0, q, r16, all[t].x, 0.f);
        emit<EPI, PER_ROW>(p, sl, rs, nb, t, 1, q, r16, all[t].y, 0.f);
        emit<EPI, PER_ROW>(p, sl, rs, nb, t, 2, q, r16, all[t].z, 0.f);
        emit<EPI, PER_ROW>(p, sl, rs, nb, t, 3, q, r16, all[t].w, 0.f);
      }
    }
    return;
  }
  float* mine = partial + (int64_t)wave * stride;
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
  const float* first = partial + (int64_t)nbi * p.ks * stride;
  if (QUANT) {
    for (int r = ks; r < 4; r += p.ks) {
      if (r >= rows) continue;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      for (int s = 0; s < p.ks; s++) {
#pragma unroll
        for (int t = 0; t < 4; t++) v[t] += first[s * stride + (t * 4 + r) * 64 + lane];
      }
      quant_emit<EPI>(p, sl, rs, nb, r, q, r16, v[0], v[1], v[2], v[3]);
    }
  } else if (EPI == EPI_FC1_GATED) {
    for (int idx = ks; idx < 8; idx += p.ks) {
      const int t = idx >> 2, r = idx & 3;
      if (r >= rows) continue;
      float up = 0.f, gate = 0.f;
      for (int s = 0; s < p.ks; s++) {
        up += first[s * stride + ((2 * t) * 4 + r) * 64 + lane];
        gate += first[s * stride + ((2 * t + 1) * 4 + r) * 64 + lane];
      }
      emit<EPI, PER_ROW>(p, sl, rs, nb, t, r, q, r16, up, gate);
    }
  } else {
    for (int idx = ks; idx < 16; idx += p.ks) {
      const int t = idx >> 2, r = idx & 3;
      if (r >= rows) continue;
      float v = 0.f;
      for (int s = 0; s < p.ks; s++) v += first[s * stride + (t * 4 + r) * 64 + lane];
      emit<EPI, PER_ROW>(p, sl, rs, nb, t, r, q, r16, v, 0.f);
    }
  }
}


// ------------------------------------------------------------------------------------------ activation rounding
//
// BF16 [m, k] -> E4M3 codes [m, k] and one FP32 scale per (row, 32-group): s = max(amax / 448, 1e-12),
// q = e4m3(clamp(x / s, -448, 448)), both quotients IEEE FP32 divisions (the reference's torch statement of its
// quantizer, hibana/kernels/w3_moe.py:187-190; its CUDA kernel, hibana/kernels/csrc/w3_gemm.cu:291-327, multiplies by
// an approximate reciprocal instead). Lane i takes the eight consecutive values from 8 i, four lanes a group; the
// four lanes of a group are neighbours in one wavefront and must all be switched on.
__device__ __forceinline__ void quant_groups_lane(const uint16_t* __restrict__ x, int64_t i, uint8_t* __restrict__ q, float* __restrict__ scales) {
  const u32x4_t raw = *reinterpret_cast<const u32x4_t*>(x + 8 * i);
  float v[8];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    v[2 * j] = __uint_as_float(raw[j] << 16);
    v[2 * j + 1] = __uint_as_float(raw[j] & 0xffff0000u);
  }
  float amax = 0.f;
#pragma unroll
  for (int j = 0; j < 8; j++) amax = fmaxf(amax, fabsf(v[j]));
  amax = fmaxf(amax, __shfl_xor(amax, 1));
  amax = fmaxf(amax, __shfl_xor(amax, 2));
  const float s = fmaxf(amax / 448.0f, 1e-12f);
#pragma unroll
  for (int j = 0; j < 8; j++) v[j] = fminf(fmaxf(v[j] / s, -448.0f), 448.0f);
  int lo = 0, hi = 0;
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], lo, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], lo, true);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(v[4], v[5], hi, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(v[6], v[7], hi, true);
  typedef __attribute__((ext_vector_type(2))) int i32x2_t;
  *reinterpret_cast<i32x2_t*>(q + 8 * i) = i32x2_t{lo, hi};
  if ((i & 3) == 0) scales[i >> 2] = s;
}

// A rounding to run beside a plan: `lanes` = values / 8 (0: none) through quant_groups_lane, or, with split_rows set,
// the rows of x [split_rows, split_k] through split_row (q: the two planes, scales: one a row).
struct QuantJob {
  const uint16_t* x;
  int64_t lanes;
  uint8_t* q;
  float* scales;
  int split_rows, split_k;
};

// BF16 activations as the sum of two E4M3 values under one FP32 scale a row, for the FP8 matrix cores:
//   s = amax of the row / 448 rounded up to a power of two, hi = e4m3(x / s), lo = e4m3(x / s - hi),  x = (hi + lo) * s.
// x / s is exact and has BF16's eight significant bits; hi takes the upper four (rounded to nearest), and what is left is
// a multiple of x's last place below half a step of hi: four significant bits again, so lo holds it EXACTLY as long as
// that last place is not below E4M3's smallest step, 2^-9 - true of every element within a factor 1792 of the row's
// largest; smaller ones are off by at most 2^-10 s, 2^-19 of the largest. Both planes share the scale, so their
// products add in one accumulator, and the sums are those of the BF16 activations up to the order of the additions. Layout: [row][chunk of 128 k]{ 128 hi bytes, 128 lo bytes }. One workgroup (any number of whole
// wavefronts) a row; `red`: LDS, one float a wavefront.
__device__ __forceinline__ void split_row(const uint16_t* __restrict__ x, int k, int64_t row, uint8_t* __restrict__ planes, float* __restrict__ scales,
                                          float* red) {
  const uint16_t* xr = x + row * k;
  const int waves = blockDim.x >> 6;
  float amax = 0.f;
  for (int c = 8 * threadIdx.x; c < k; c += 8 * blockDim.x) {
    const u32x4_t raw = *reinterpret_cast<const u32x4_t*>(xr + c);
#pragma unroll
    for (int j = 0; j < 4; j++) amax = fmaxf(amax, fmaxf(fabsf(__uint_as_float(raw[j] << 16)), fabsf(__uint_as_float(raw[j] & 0xffff0000u))));
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = 0.f;
  for (int w = 0; w < waves; w++) amax = fmaxf(amax, red[w]);
  // up to the next power of two (a zero row: the smallest normal), so that every division below is exact
  const float s = __uint_as_float(max((__float_as_uint(amax / 448.0f) + 0x007fffffu) & 0x7f800000u, 0x00800000u));
  if (threadIdx.x == 0) scales[row] = s;
  uint8_t* out = planes + row * 2 * k;
  for (int c = 8 * threadIdx.x; c < k; c += 8 * blockDim.x) {
    const u32x4_t raw = *reinterpret_cast<const u32x4_t*>(xr + c);
    float v[8];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      v[2 * j] = __uint_as_float(raw[j] << 16);
      v[2 * j + 1] = __uint_as_float(raw[j] & 0xffff0000u);
    }
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = fminf(fmaxf(v[j] / s, -448.0f), 448.0f);
    int h0 = 0, h1 = 0;
    h0 = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], h0, false);
    h0 = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], h0, true);
    h1 = __builtin_amdgcn_cvt_pk_fp8_f32(v[4], v[5], h1, false);
    h1 = __builtin_amdgcn_cvt_pk_fp8_f32(v[6], v[7], h1, true);
    float r[8];
    r[0] = v[0] - __builtin_amdgcn_cvt_f32_fp8(h0, 0);
    r[1] = v[1] - __builtin_amdgcn_cvt_f32_fp8(h0, 1);
    r[2] = v[2] - __builtin_amdgcn_cvt_f32_fp8(h0, 2);
    r[3] = v[3] - __builtin_amdgcn_cvt_f32_fp8(h0, 3);
    r[4] = v[4] - __builtin_amdgcn_cvt_f32_fp8(h1, 0);
    r[5] = v[5] - __builtin_amdgcn_cvt_f32_fp8(h1, 1);
    r[6] = v[6] - __builtin_amdgcn_cvt_f32_fp8(h1, 2);
    r[7] = v[7] - __builtin_amdgcn_cvt_f32_fp8(h1, 3);
    int l0 = 0, l1 = 0;
    l0 = __builtin_amdgcn_cvt_pk_fp8_f32(r[0], r[1], l0, false);
    l0 = __builtin_amdgcn_cvt_pk_fp8_f32(r[2], r[3], l0, true);
    l1 = __builtin_amdgcn_cvt_pk_fp8_f32(r[4], r[5], l1, false);
    l1 = __builtin_amdgcn_cvt_pk_fp8_f32(r[6], r[7], l1, true);
    typedef __attribute__((ext_vector_type(2))) int i32x2_t;
    uint8_t* at = out + (c >> 7) * 256 + (c & 127);
    *reinterpret_cast<i32x2_t*>(at) = i32x2_t{h0, h1};
    *reinterpret_cast<i32x2_t*>(at + 128) = i32x2_t{l0, l1};
  }
}

// One workgroup's share of a QuantJob: `index` counts the job's workgroups from zero.
__device__ __forceinline__ void quant_job_share(const QuantJob& job, int index, float* red) {
  if (job.split_rows) {
    if (index < job.split_rows) split_row(job.x, job.split_k, index, job.q, job.scales, red);
    return;
  }
  const int64_t i = (int64_t)index * blockDim.x + threadIdx.x;
  if (i < job.lanes) quant_groups_lane(job.x, i, job.q, job.scales);  // whole groups: four lanes in or out together
}

// ---------------------------------------------------------------------------------------------------- host side
// Workspace of a routed call, carved from one caller-owned buffer.
struct MoeWorkspace {
  int32_t* plan;
  int32_t* plan_wide;  // [64, experts]: the plan's counts a workgroup when many pairs are shared among several
  int32_t* order;
  uint16_t* h;   // [(pairs + shared rows), inter] BF16, in sorted order
  float* y;      // [(pairs + shared rows), hidden_out] FP32 (or BF16 pairs), by pair index
  uint8_t* xq;   // E4M3 activation mode: codes of x [m, hidden] ...
  float* xs;     // ... and their scales [m, hidden / 32]
  uint8_t* hq;   // the same for h: [(pairs + shared rows), inter], [.., inter / 32]
  float* hs;
  uint8_t* x2;   // the two-plane form of x (split_row): [m, 2 * hidden] ...
  float* x2s;    // ... and its scales [m]
  size_t bytes;
};

int64_t moe_max_slots(int64_t pairs, int experts, int shared_rows, int slot_rows = ROWS_PER_SLOT);
MoeWorkspace moe_carve(void* base, int m, int topk, int experts, int inter, int hidden_out, int shared, int hidden = 0);  // hidden: also the E4M3 activation buffers
// Enqueue the plan kernel; HB_EINVAL if the expert count does not fit its LDS.
// A rounding job rides in the plan's launch (further workgroups beside the one that plans).
int moe_launch_plan(const int32_t* ids, int64_t pairs, int e_lo, int e_n, int shared_rows, const MoeWorkspace& ws, hipStream_t stream,
                    int slot_rows = ROWS_PER_SLOT, const QuantJob* job = nullptr);
void moe_launch_quant_groups(const QuantJob& job, hipStream_t stream);  // the rounding alone
void moe_launch_quant_rows(const uint16_t* x, int64_t m, int k, uint8_t* q, float* scales, hipStream_t stream);  // one scale a row

// Softmax top-k routing of `m` rows of `e` logits into ids / weights [m, topk], then the plan of those ids: one launch
// for up to a few dozen rows, two beyond.
int moe_check_route(int m, int e, int k);  // HB_EINVAL for a row the routing wavefront cannot hold

// A routed call whose experts are chosen under a budget (route_budget.hpp): BF16 logits [m, e] and the rule's settings.
struct BudgetRoute {
  const uint16_t* logits;
  int e, keep, budget, steps, repeat, per_request, min_cap;
  const int32_t* slots;  // or null: every row is real
};
// Rank, then the selection and the plan of its ids in one workgroup's launch (the selection leaves ids / weights in the
// caller's arrays). `scratch`: room for the rows' candidates between the two launches (160 bytes a row).
int moe_launch_budget_plan(const BudgetRoute& b, int m, int topk, int32_t* ids, float* weights, int e_lo, int e_n, int shared_rows,
                           const MoeWorkspace& ws, void* scratch, hipStream_t stream, int slot_rows = ROWS_PER_SLOT);
int moe_launch_route_plan(const float* logits, int m, int e, int topk, int32_t* ids, float* weights, int e_lo, int e_n, int shared_rows,
                          const MoeWorkspace& ws, hipStream_t stream, int slot_rows = ROWS_PER_SLOT, const QuantJob* job = nullptr);

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
void moe_launch_combine(const CombineParams& c, hipStream_t stream);

// The dense ends of a latent block of at most LATENT_MAX_ROWS rows (hibana/kernels/csrc/nemotron_moe.cu of the reference).
// Router: fused FP32 [m, experts + latent] = x [router; fc1_latent]^T and its latent columns as BF16 (one launch);
// with `route`, a second launch: sigmoid + bias top-k routing of the rows (ids, weights; padded rows take `pad_id`, or
// row 0's first choice when it is negative) and, given a workspace, the expert plan of experts e_lo .. e_lo + e_n - 1.
constexpr int LATENT_MAX_ROWS = HB_LATENT_MAX_ROWS;
struct LatentRouter {
  const uint16_t* w;     // BF16 [experts + latent, hidden]
  const float* bias;     // [experts]
  const uint16_t* x;     // BF16 [m, hidden]
  const int32_t* slots;  // or null
  int m, experts, latent, hidden, topk, steps, route, pad_id;
  float* fused;
  int32_t* ids;
  float* weights;
  uint16_t* lat;
  int e_lo, e_n;
  const MoeWorkspace* ws;  // the plan's home, or null: routing only
};
int latent_launch_router(const LatentRouter& r, hipStream_t stream);
// Out: out = bf16(shared + routed fc2^T), routed BF16 [m, latent].
int latent_launch_out(const uint16_t* fc2, const uint16_t* routed, const uint16_t* shared, uint16_t* out, int m, int hidden, int latent, hipStream_t stream);

// The pieces of the combine that every kernel doing it shares, so that each gives the other's bits.
// g = sigmoid(x[r] . gate_vec): 256 threads (t = 0 .. 255, four whole wavefronts) each add their share and leave four
// partial sums in `red` (LDS); after a barrier any thread reads g from them.
__device__ __forceinline__ void combine_gate_partial(const uint16_t* x, const float* gate_vec, int hx, int64_t r, int t, float* red) {
  float dot = 0.f;
  for (int i0 = t; i0 < hx; i0 += 8 * 256) {  // eight of the thread's terms asked for together, added in the order of i
    float xv[8], gv[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int i = min(i0 + 256 * j, hx - 1);
      xv[j] = bf16_bits_to_f32(x[r * hx + i]);
      gv[j] = gate_vec[i];
    }
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (i0 + 256 * j < hx) dot += xv[j] * gv[j];
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) dot += __shfl_xor(dot, d);
  if ((t & 63) == 0) red[t >> 6] = dot;
}
__device__ __forceinline__ float combine_gate_value(const float* red) {
  const float dot = (red[0] + red[1]) + (red[2] + red[3]);
  return 1.0f / (1.0f + expf(-dot));
}
// routed: the FP32 chain over the row's slots; shared: the shared expert's FP32 (or BF16) output
__device__ __forceinline__ float combine_shared(float routed, float g, float shared) { return round_bf16(routed) + g * round_bf16(shared); }

// Measurement hook: the caller's next (start, stop) event pair, if any is armed. A kernel launched through HB_LAUNCH
// then carries the pair: the runtime stamps the two events with that kernel's own begin and end.
bool moe_next_events(hipEvent_t* start, hipEvent_t* stop);
int64_t* moe_trace_buffer(int64_t* records);  // hb_debug_trace's buffer and its capacity in records, or null

#define HB_LAUNCH(kernel, grid, block, lds, stream, ...)                                            \
  do {                                                                                              \
    hipEvent_t hb_e0_, hb_e1_;                                                                      \
    if (hb::moe_next_events(&hb_e0_, &hb_e1_)) {                                                    \
      hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, hb_e0_, hb_e1_, 0, __VA_ARGS__);      \
    } else {                                                                                        \
      hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                            \
    }                                                                                               \
  } while (0)

// Wavefronts per workgroup of a stream launch: K is split until the launch has about `want` wavefronts, keeping at
// least four chunks per wavefront; what is left of a 4-wavefront workgroup takes neighbouring 64-row blocks.
void pick_shape(int n_blocks, int chunks, int64_t slots, int want, int* ks, int* nbw);

// hb_tune keys of the NVFP4 kernels ("nvfp4_tile": 1 forces the tile kernel, 2 the stream, 0 the built-in choice).
int nvfp4_tune(const char* key, int value);
// hb_tune keys of the kernels shared by the routed calls ("route_plan": 2 keeps routing and plan in separate launches).
int moe_tune(const char* key, int value);

}  // namespace hb
