// The W3 weight stream on gfx950: dense linear and routed-expert grouped GEMMs for decode / verify sized calls.
//
// One wavefront owns a block column of the tile layout: 64 output rows x a range of 128-k chunks, for one "slot" of up
// to 16 activation rows. A chunk is a contiguous 3328-byte block (packed codes, then scales); it travels from memory
// into the wavefront's ring in LDS without passing through registers, two chunks ahead of the one being expanded.
// The expansion happens in registers (v_perm_b32 over the 8-byte E4M3 codebook, then the hardware FP8 -> BF16 pair
// conversion: exact) and feeds sixteen v_mfma_f32_16x16x32_bf16 (4 row tiles x 4 scale groups): one MFMA is exactly
// one 32-group, so the group scale is folded into the FP32 accumulator after it (acc += part * scale), as the
// reference kernel does per group (hibana/kernels/csrc/w3_gemm.cu:105-108); the FP32 row scale is applied in the
// epilogue (:209-210). Activations are BF16, read straight from global memory (they stay in L2) as the MFMA A operand.
// Slots of at most four rows (most of a decode or verify step) take a second body that packs the four groups into the
// idle MFMA rows and so folds a quarter of the scales. The wavefronts of a workgroup split K (partials reduced through
// LDS in a fixed order) and/or take neighbouring 64-row blocks. No atomics on floating point anywhere: results are
// bitwise repeatable.
//
// Calls with many rows per weight block (prefill) go to the 128-row MFMA tile kernel of tile_kernel.hpp instead, through
// the TileW3 policy below; the entry points choose (tile_serves_dense for a dense call, pairs per expert for a routed
// one), and hb_tune("w3_tile", 1 | 2) forces one or the other.
#include <string.h>

#include <algorithm>
#include <atomic>
#include <mutex>

#include "ring.hpp"
#include "route.hpp"
#include "stream_common.hpp"
#include "tile_kernel.hpp"
#include "w3_layout.hpp"

namespace hb {

struct Chunk {  // the weight side of one 64-row x 128-k block
  u32x4_t w0, w1, w2, sc;
};

struct Chunk2 {  // the same of a two-bit matrix: eight code dwords a lane
  u32x4_t w0, w1, sc;
};

// The eight selectors of 16-row tile NT of a chunk, and the dword of its four scale bytes.
template <int NT>
__device__ __forceinline__ void chunk_selectors(const Chunk& ch, uint32_t sel[8]) {
  if (NT == 0) w3_selectors(ch.w0.x, ch.w0.y, ch.w0.z, sel);
  if (NT == 1) w3_selectors(ch.w0.w, ch.w1.x, ch.w1.y, sel);
  if (NT == 2) w3_selectors(ch.w1.z, ch.w1.w, ch.w2.x, sel);
  if (NT == 3) w3_selectors(ch.w2.y, ch.w2.z, ch.w2.w, sel);
}
template <int NT>
__device__ __forceinline__ void chunk_selectors(const Chunk2& ch, uint32_t sel[8]) {
  if (NT == 0) w2_selectors(ch.w0.x, ch.w0.y, sel);
  if (NT == 1) w2_selectors(ch.w0.z, ch.w0.w, sel);
  if (NT == 2) w2_selectors(ch.w1.x, ch.w1.y, sel);
  if (NT == 3) w2_selectors(ch.w1.z, ch.w1.w, sel);
}
template <int NT, class C>
__device__ __forceinline__ uint32_t chunk_scales(const C& ch) {
  return NT == 0 ? ch.sc.x : NT == 1 ? ch.sc.y : NT == 2 ? ch.sc.z : ch.sc.w;
}

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

// Half of a 16-row tile of a chunk, sixteen activation rows: 32-groups 0 and 1 (HALF 0: their selectors come from the
// tile's first two code dwords) or 2 and 3 (HALF 1). One MFMA is one group, so the group's scale is folded into the FP32
// accumulator after it, in group order.
template <int HALF, int NT, class C>
__device__ __forceinline__ void compute_half_tile(const C& ch, const u32x4_t& a_lo, const u32x4_t& a_hi, f32x4_t& acc, uint32_t lut_lo, uint32_t lut_hi) {
  const uint32_t scales = chunk_scales<NT>(ch);
  uint32_t sel[8];
  chunk_selectors<NT>(ch, sel);  // the four the half does not use fold away
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
  const f32x4_t p0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a_lo), expand8(sel[4 * HALF], sel[4 * HALF + 1], lut_lo, lut_hi), zero, 0, 0, 0);
  const f32x4_t p1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a_hi), expand8(sel[4 * HALF + 2], sel[4 * HALF + 3], lut_lo, lut_hi), zero, 0, 0, 0);
  const float s0 = HALF ? __builtin_amdgcn_cvt_f32_fp8(scales, 2) : __builtin_amdgcn_cvt_f32_fp8(scales, 0);
  const float s1 = HALF ? __builtin_amdgcn_cvt_f32_fp8(scales, 3) : __builtin_amdgcn_cvt_f32_fp8(scales, 1);
  acc.x = fmaf(p1.x, s1, fmaf(p0.x, s0, acc.x));
  acc.y = fmaf(p1.y, s1, fmaf(p0.y, s0, acc.y));
  acc.z = fmaf(p1.z, s1, fmaf(p0.z, s0, acc.z));
  acc.w = fmaf(p1.w, s1, fmaf(p0.w, s0, acc.w));
}

// The four tiles of a chunk over one half of its groups: once a half is done its two activation fragments are free for
// the next chunk's.
template <int HALF, class C>
__device__ __forceinline__ void compute_half_chunk(const C& ch, const u32x4_t& a_lo, const u32x4_t& a_hi, f32x4_t& acc0, f32x4_t& acc1,
                                                   f32x4_t& acc2, f32x4_t& acc3, uint32_t lut_lo, uint32_t lut_hi) {
  compute_half_tile<HALF, 0>(ch, a_lo, a_hi, acc0, lut_lo, lut_hi);
  compute_half_tile<HALF, 1>(ch, a_lo, a_hi, acc1, lut_lo, lut_hi);
  compute_half_tile<HALF, 2>(ch, a_lo, a_hi, acc2, lut_lo, lut_hi);
  compute_half_tile<HALF, 3>(ch, a_lo, a_hi, acc3, lut_lo, lut_hi);
}

// ------------------------------------------------------------------------------------------------ the weight ring
// (ring.hpp) for W3 blocks: three 16-byte loads a lane of codes, one 4-byte load a lane of scales.
// AUX: the loads' cache policy - 2 (non-temporal) for a call that streams far more than the caches hold, 0 for one
// token's few megabytes, which come in faster as ordinary loads.
template <int AUX, int BITS = 3>
struct W3RingOf;

template <int AUX>
struct W3RingOf<AUX, 3> {
  typedef hb::Chunk Chunk;
  static constexpr int BLOCK_BYTES = W3_BLOCK_BYTES, LOADS = 4;
  // the lane's byte offsets in a block for the 16-byte and the 4-byte loads, and where it reads them back
  static __device__ __forceinline__ void lanes(RingSource& src, int lane, int r16, uint32_t slot0, uint32_t& codes, uint32_t& scales) {
    src.codes = 16u * lane;
    src.scales = 4u * lane;
    codes = slot0 + 16u * lane;
    scales = slot0 + 16u * r16;
  }
  static __device__ __forceinline__ void request(const RingSource& src, int chunk, lds_ptr_t slot) {
    const uint32_t at = (uint32_t)chunk * W3_BLOCK_BYTES;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 16, src.codes, at, 0, AUX);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 16, src.codes, at, 1024, AUX);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 16, src.codes, at, 2048, AUX);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 4, src.scales, at, W3_SCALE_OFFSET, AUX);
    __builtin_amdgcn_sched_barrier(0);  // asked for here, not wherever the scheduler would sink it below the arithmetic
  }
  template <int BEHIND, int SLOT>  // BEHIND: requests that may stay outstanding
  static __device__ __forceinline__ void take(Chunk& ch, uint32_t codes, uint32_t scales) {
    asm volatile(
        "s_waitcnt vmcnt(%6)\n\t"
        "ds_read_b128 %0, %4 offset:%7\n\t"
        "ds_read_b128 %1, %4 offset:%8\n\t"
        "ds_read_b128 %2, %4 offset:%9\n\t"
        "ds_read_b128 %3, %5 offset:%10\n\t"
        "s_waitcnt lgkmcnt(0)"  // the slot is read: it may be given to another chunk
        : "=&v"(ch.w0), "=&v"(ch.w1), "=&v"(ch.w2), "=&v"(ch.sc)
        : "v"(codes), "v"(scales), "n"(BEHIND), "n"(SLOT * W3_BLOCK_BYTES), "n"(SLOT * W3_BLOCK_BYTES + 1024), "n"(SLOT * W3_BLOCK_BYTES + 2048),
          "n"(SLOT * W3_BLOCK_BYTES + W3_SCALE_OFFSET)
        : "memory");
  }
};
// Two-bit blocks: two 16-byte loads a lane of codes, one 4-byte load a lane of scales; the two slots lie in the same
// LDS a wavefront as a three-bit ring's (the launches size it for either).
template <int AUX>
struct W3RingOf<AUX, 2> {
  typedef hb::Chunk2 Chunk;
  static constexpr int BLOCK_BYTES = W2_BLOCK_BYTES, LOADS = 3;
  static __device__ __forceinline__ void lanes(RingSource& src, int lane, int r16, uint32_t slot0, uint32_t& codes, uint32_t& scales) {
    src.codes = 16u * lane;
    src.scales = 4u * lane;
    codes = slot0 + 16u * lane;
    scales = slot0 + 16u * r16;
  }
  static __device__ __forceinline__ void request(const RingSource& src, int chunk, lds_ptr_t slot) {
    const uint32_t at = (uint32_t)chunk * W2_BLOCK_BYTES;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 16, src.codes, at, 0, AUX);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 16, src.codes, at, 1024, AUX);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 4, src.scales, at, W2_SCALE_OFFSET, AUX);
    __builtin_amdgcn_sched_barrier(0);
  }
  template <int BEHIND, int SLOT>
  static __device__ __forceinline__ void take(Chunk& ch, uint32_t codes, uint32_t scales) {
    asm volatile(
        "s_waitcnt vmcnt(%5)\n\t"
        "ds_read_b128 %0, %3 offset:%6\n\t"
        "ds_read_b128 %1, %3 offset:%7\n\t"
        "ds_read_b128 %2, %4 offset:%8\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(ch.w0), "=&v"(ch.w1), "=&v"(ch.sc)
        : "v"(codes), "v"(scales), "n"(BEHIND), "n"(SLOT * W2_BLOCK_BYTES), "n"(SLOT * W2_BLOCK_BYTES + 1024), "n"(SLOT * W2_BLOCK_BYTES + W2_SCALE_OFFSET)
        : "memory");
  }
};
typedef W3RingOf<2> W3Ring;
typedef W3RingOf<0> W3RingCached;
typedef W3RingOf<2, 2> W2Ring;

// A ring that brings in only what the 16-row tiles T0 .. T1 - 1 of a three-bit block need: tile t's three code dwords are
// dwords 3 t .. 3 t + 2 of the lane's twelve, four to a 16-byte load, so the tiles' loads are 3 T0 / 4 .. (3 T1 - 1) / 4 (one
// or two of the three for one tile or a pair of them), and the scales. The Chunk's other registers stay unset and unread.
template <int AUX, int T0, int T1>
struct W3RingPart {
  typedef hb::Chunk Chunk;
  static constexpr int L0 = 3 * T0 / 4, L1 = (3 * T1 - 1) / 4, CODE_LOADS = L1 - L0 + 1;
  static constexpr int BLOCK_BYTES = W3_BLOCK_BYTES, LOADS = CODE_LOADS + 1;
  static_assert(0 <= T0 && T0 < T1 && T1 <= 4 && CODE_LOADS >= 1 && CODE_LOADS <= 2, "a tile or a pair of tiles (the whole block: W3RingOf)");
  static __device__ __forceinline__ void lanes(RingSource& src, int lane, int r16, uint32_t slot0, uint32_t& codes, uint32_t& scales) {
    W3RingOf<AUX>::lanes(src, lane, r16, slot0, codes, scales);
  }
  static __device__ __forceinline__ void request(const RingSource& src, int chunk, lds_ptr_t slot) {
    const uint32_t at = (uint32_t)chunk * W3_BLOCK_BYTES;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 16, src.codes, at, 1024 * L0, AUX);
    if (CODE_LOADS == 2) __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 16, src.codes, at, 1024 * L1, AUX);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 4, src.scales, at, W3_SCALE_OFFSET, AUX);
    __builtin_amdgcn_sched_barrier(0);
  }
  static __device__ __forceinline__ u32x4_t& load_of(Chunk& ch, int l) { return l == 0 ? ch.w0 : l == 1 ? ch.w1 : ch.w2; }
  template <int BEHIND, int SLOT>
  static __device__ __forceinline__ void take(Chunk& ch, uint32_t codes, uint32_t scales) {
    if (CODE_LOADS == 2) {
      asm volatile(
          "s_waitcnt vmcnt(%5)\n\t"
          "ds_read_b128 %0, %3 offset:%6\n\t"
          "ds_read_b128 %1, %3 offset:%7\n\t"
          "ds_read_b128 %2, %4 offset:%8\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=&v"(load_of(ch, L0)), "=&v"(load_of(ch, L1)), "=&v"(ch.sc)
          : "v"(codes), "v"(scales), "n"(BEHIND), "n"(SLOT * W3_BLOCK_BYTES + 1024 * L0), "n"(SLOT * W3_BLOCK_BYTES + 1024 * L1),
            "n"(SLOT * W3_BLOCK_BYTES + W3_SCALE_OFFSET)
          : "memory");
    } else {
      asm volatile(
          "s_waitcnt vmcnt(%4)\n\t"
          "ds_read_b128 %0, %2 offset:%5\n\t"
          "ds_read_b128 %1, %3 offset:%6\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=&v"(load_of(ch, L0)), "=&v"(ch.sc)
          : "v"(codes), "v"(scales), "n"(BEHIND), "n"(SLOT * W3_BLOCK_BYTES + 1024 * L0), "n"(SLOT * W3_BLOCK_BYTES + W3_SCALE_OFFSET)
          : "memory");
    }
  }
};
constexpr int RING_BYTES = ring_bytes<W3Ring>();  // LDS per wavefront; its first 4 KB double as the K-split exchange

// ------------------------------------------------------------------------------------------- slots of one to four rows
//
// Most slots of a decode or verify step hold a handful of rows (an expert a few tokens chose). Twelve of the sixteen
// MFMA output rows are then idle, and they can carry the four 32-groups of a chunk instead: A row 4 j + i holds row i of
// the slot over group j's k range only (zero elsewhere), so the four MFMAs of a tile, one per group, chain into ONE
// accumulator whose rows 4 j .. 4 j + 3 are group j's partial sums. Lane (q, r16) then holds group q's sums for the
// slot's four rows: one scale conversion and four multiply-adds per tile instead of four and sixteen, and sixteen bytes
// of activations per lane and chunk instead of sixty-four. The four groups are added once, after the last chunk, in the
// exchange through LDS that the K splits are added in.
constexpr int FEW_ROWS = 4;

// fc2 stores by pair index, which it reads from the sorted list: asked for ahead of the weights, so that the epilogue
// does not wait on memory once more.
struct FewPairs {
  int pair[FEW_ROWS];
  __device__ __forceinline__ void ask(const StreamParams& p, const Slot& sl, int row0) {
#pragma unroll
    for (int r = 0; r < FEW_ROWS; r++) pair[r] = p.order[sl.p0 + min(row0 + r, sl.rows - 1)];
  }
  __device__ __forceinline__ int of(int r) const { return r == 0 ? pair[0] : r == 1 ? pair[1] : r == 2 ? pair[2] : pair[3]; }
};

__device__ __forceinline__ void store_pair(const StreamParams& p, int64_t pair, int n, float y) {
  if (p.out_bf16) {
    reinterpret_cast<uint16_t*>(p.out)[pair * p.out_stride + n] = bf16_of(y);
  } else {
    reinterpret_cast<float*>(p.out)[pair * p.out_stride + n] = y;
  }
}

template <int NT, class C>
__device__ __forceinline__ void compute_tile_few(const C& w, const Rows& ch, f32x4_t& acc, uint32_t lut_lo, uint32_t lut_hi, uint32_t q8) {
  const uint32_t scales = chunk_scales<NT>(w);
  uint32_t sel[8];
  chunk_selectors<NT>(w, sel);
  f32x4_t part = {0.f, 0.f, 0.f, 0.f};
  part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ch.a0), expand8(sel[0], sel[1], lut_lo, lut_hi), part, 0, 0, 0);
  part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ch.a1), expand8(sel[2], sel[3], lut_lo, lut_hi), part, 0, 0, 0);
  part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ch.a2), expand8(sel[4], sel[5], lut_lo, lut_hi), part, 0, 0, 0);
  part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ch.a3), expand8(sel[6], sel[7], lut_lo, lut_hi), part, 0, 0, 0);
  const float s = __builtin_amdgcn_cvt_f32_fp8(scales >> q8, 0);  // the scale of this lane's group
  acc.x = fmaf(part.x, s, acc.x);
  acc.y = fmaf(part.y, s, acc.y);
  acc.z = fmaf(part.z, s, acc.z);
  acc.w = fmaf(part.w, s, acc.w);
}

// The E4M3-activation form of the four-row body (the arithmetic of the reference kernel, hibana/kernels/csrc/
// w3_gemm.cu:105-108: FP8 x FP8 products, FP32 sums a group, the two group scales folded into the accumulator). The
// codebook's E4M3 bytes are the MFMA operand as they come out of v_perm_b32: no conversion. `a`: the lane's eight
// activation codes of the chunk; xs: the activation scales of the slot's four rows at this lane's group.
__device__ __forceinline__ long fp8x8(uint32_t lo, uint32_t hi) { return (long)(((uint64_t)hi << 32) | lo); }

template <int NT, class C>
__device__ __forceinline__ void compute_tile_few8(const C& w, const long a[4], const f32x4_t& xs, f32x4_t& acc, uint32_t lut_lo, uint32_t lut_hi,
                                                  uint32_t q8) {
  const uint32_t scales = chunk_scales<NT>(w);
  uint32_t sel[8];
  chunk_selectors<NT>(w, sel);
  f32x4_t part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const long b = fp8x8(__builtin_amdgcn_perm(lut_hi, lut_lo, sel[2 * j]), __builtin_amdgcn_perm(lut_hi, lut_lo, sel[2 * j + 1]));
    part = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a[j], b, part, 0, 0, 0);
  }
  const float s = __builtin_amdgcn_cvt_f32_fp8(scales >> q8, 0);  // the weight scale of this lane's group
  acc.x = fmaf(part.x, xs.x * s, acc.x);
  acc.y = fmaf(part.y, xs.y * s, acc.y);
  acc.z = fmaf(part.z, xs.z * s, acc.z);
  acc.w = fmaf(part.w, xs.w * s, acc.w);
}

template <class C>
__device__ __forceinline__ void compute_few8(const C& ch, long a, const f32x4_t& xs, int grp, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2,
                                             f32x4_t& acc3, uint32_t lut_lo, uint32_t lut_hi, uint32_t q8) {
  long rows[4];  // MFMA j's A operand: the lane's codes in its own group, zero in the others
#pragma unroll
  for (int j = 0; j < 4; j++) rows[j] = grp == j ? a : 0L;
  compute_tile_few8<0>(ch, rows, xs, acc0, lut_lo, lut_hi, q8);
  compute_tile_few8<1>(ch, rows, xs, acc1, lut_lo, lut_hi, q8);
  compute_tile_few8<2>(ch, rows, xs, acc2, lut_lo, lut_hi, q8);
  compute_tile_few8<3>(ch, rows, xs, acc3, lut_lo, lut_hi, q8);
}

// `a`: the lane's sixteen activation bytes of the chunk (row r16 % 4 of the slot, the k range of group r16 / 4 that this
// lane owns in the MFMA A operand); grp: that group.
template <class C>
__device__ __forceinline__ void compute_few(const C& ch, const u32x4_t& a, int grp, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2,
                                            f32x4_t& acc3, uint32_t lut_lo, uint32_t lut_hi, uint32_t q8) {
  const u32x4_t none = {0u, 0u, 0u, 0u};
  Rows rows;  // MFMA j's A operand: the lane's bytes in its own group, zero in the others
  rows.a0 = grp == 0 ? a : none;
  rows.a1 = grp == 1 ? a : none;
  rows.a2 = grp == 2 ? a : none;
  rows.a3 = grp == 3 ? a : none;
  compute_tile_few<0>(ch, rows, acc0, lut_lo, lut_hi, q8);
  compute_tile_few<1>(ch, rows, acc1, lut_lo, lut_hi, q8);
  compute_tile_few<2>(ch, rows, acc2, lut_lo, lut_hi, q8);
  compute_tile_few<3>(ch, rows, acc3, lut_lo, lut_hi, q8);
}

// The two bodies of the stream differ in the activations: what registers they keep, when they ask for them, how a
// chunk is computed. `step<ODD, MORE2, MORE1>` computes chunk i (ODD: its parity; MORE2 / MORE1: chunks i + 2 / i + 1
// exist) and asks for the activations whose registers it frees.
struct FewActs {
  static constexpr int LOADS = 1;  // activation loads per chunk
  u32x4_t held[2];                 // the lane's sixteen bytes of the next even and the next odd chunk
  int grp;
  uint32_t q8;
  const uint16_t* at;              // the lane's sixteen bytes of the wavefront's first chunk
  __device__ __forceinline__ u32x4_t load(int i) const { return *reinterpret_cast<const u32x4_t*>(at + (int64_t)i * 128); }
  template <int EPI>
  __device__ __forceinline__ void start(const StreamParams& p, const Slot& sl, int row0, int c0, int n, int lane) {
    const int q = lane >> 4, r16 = lane & 15;
    grp = r16 >> 2;
    at = activation_row<EPI>(p, sl, row0 + (r16 & 3)) + (int64_t)c0 * 128 + 32 * grp + 8 * q;
    q8 = 8 * q;
    held[0] = load(0);
    if (n > 1) held[1] = load(1);
  }
  template <int ODD, bool MORE2, bool MORE1, class C>
  __device__ __forceinline__ void step(const C& ch, int i, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3, const Slot& sl) {
    compute_few(ch, held[ODD], grp, acc0, acc1, acc2, acc3, sl.lut_lo, sl.lut_hi, q8);
    if (MORE2) held[ODD] = load(i + 2);
  }
};

// FewActs over the 16-row tiles T0 .. T1 - 1 of the block only (the other accumulators stay zero).
template <int T0, int T1>
struct FewActsPart : FewActs {
  template <int ODD, bool MORE2, bool MORE1, class C>
  __device__ __forceinline__ void step(const C& ch, int i, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3, const Slot& sl) {
    const u32x4_t none = {0u, 0u, 0u, 0u};
    const u32x4_t a = held[ODD];
    Rows rows;  // as compute_few: the lane's bytes in its own group, zero in the others
    rows.a0 = grp == 0 ? a : none;
    rows.a1 = grp == 1 ? a : none;
    rows.a2 = grp == 2 ? a : none;
    rows.a3 = grp == 3 ? a : none;
    if (T0 <= 0 && 0 < T1) compute_tile_few<0>(ch, rows, acc0, sl.lut_lo, sl.lut_hi, q8);
    if (T0 <= 1 && 1 < T1) compute_tile_few<1>(ch, rows, acc1, sl.lut_lo, sl.lut_hi, q8);
    if (T0 <= 2 && 2 < T1) compute_tile_few<2>(ch, rows, acc2, sl.lut_lo, sl.lut_hi, q8);
    if (T0 <= 3 && 3 < T1) compute_tile_few<3>(ch, rows, acc3, sl.lut_lo, sl.lut_hi, q8);
    if (MORE2) held[ODD] = load(i + 2);
  }
};

struct FewActs8 {  // E4M3 activations: eight codes a lane and chunk, and the scales of the slot's four rows at the lane's output group
  static constexpr int LOADS = 5;
  long held[2];
  f32x4_t scale[2];
  int grp;
  uint32_t q8;
  const uint8_t* at;       // the lane's eight codes of the wavefront's first chunk
  const float* scales;     // the scale matrix
  uint32_t soff[4];        // in it, the scale of slot row row0 + i at group q of that chunk (the launch keeps the matrix under 2^32 scales)
  __device__ __forceinline__ void load(int slot, int i) {
    held[slot] = *reinterpret_cast<const long*>(at + (int64_t)i * 128);
    scale[slot] = f32x4_t{scales[soff[0] + 4 * i], scales[soff[1] + 4 * i], scales[soff[2] + 4 * i], scales[soff[3] + 4 * i]};
  }
  template <int EPI>
  __device__ __forceinline__ void start(const StreamParams& p, const Slot& sl, int row0, int c0, int n, int lane) {
    const int q = lane >> 4, r16 = lane & 15;
    grp = r16 >> 2;
    at = p.aq + activation_row_index<EPI>(p, sl, row0 + (r16 & 3)) * p.a_stride + (int64_t)c0 * 128 + 32 * grp + 8 * q;
    scales = p.aq_scale;
#pragma unroll
    for (int i = 0; i < 4; i++) soff[i] = (uint32_t)(activation_row_index<EPI>(p, sl, row0 + i) * (p.a_stride >> 5)) + 4 * c0 + q;
    q8 = 8 * q;
    load(0, 0);
    if (n > 1) load(1, 1);
  }
  template <int ODD, bool MORE2, bool MORE1, class C>
  __device__ __forceinline__ void step(const C& ch, int i, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3, const Slot& sl) {
    compute_few8(ch, held[ODD], scale[ODD], grp, acc0, acc1, acc2, acc3, sl.lut_lo, sl.lut_hi, q8);
    if (MORE2) load(ODD, i + 2);
  }
};

// Slots of at most TWO rows on the two-plane form of the activations (split_row: x = (hi + lo) * s, both E4M3), on
// v_mfma_f32_16x16x32_fp8_fp8: both planes of both rows ride in the four A rows of a group - A row 4 g + 2 plane + t is
// plane `plane` of slot row t over group g only - so the MFMA count is the BF16 body's (one a group and tile), the
// weights are the codebook's E4M3 bytes as v_perm_b32 delivers them (no conversion: 132 VALU instructions a chunk
// instead of 204) and an A operand is two registers. Both planes are in the same units and their sums add in
// finish_few, where the row's activation scale multiplies the result. Register i of lane (q, r16) of a tile's result is group q's sum for
// plane i / 2 of slot row i % 2 and weight row r16; finish_few adds the planes.
struct FewPlaneActs {
  static constexpr int LOADS = 1;
  long held[2];       // the lane's eight E4M3 bytes (its row, plane and group) of the next even and the next odd chunk
  int grp;
  uint32_t q8;
  const uint8_t* at;  // ... of the wavefront's first chunk
  __device__ __forceinline__ long load(int i) const { return *reinterpret_cast<const long*>(at + (int64_t)i * 256); }
  template <int EPI>
  __device__ __forceinline__ void start(const StreamParams& p, const Slot& sl, int row0, int c0, int n, int lane) {
    const int q = lane >> 4, r16 = lane & 15;
    grp = r16 >> 2;
    q8 = 8 * q;
    at = p.a2 + activation_row_index<EPI>(p, sl, row0 + (r16 & 1)) * (2 * p.a_stride) + (int64_t)c0 * 256 + 64 * (r16 & 2) + 32 * grp + 8 * q;
    held[0] = load(0);
    if (n > 1) held[1] = load(1);
  }
  template <int NT, class C>
  static __device__ __forceinline__ void tile(const C& w, const long a[4], f32x4_t& acc, uint32_t lut_lo, uint32_t lut_hi, uint32_t q8) {
    const uint32_t scales = chunk_scales<NT>(w);
    uint32_t sel[8];
    chunk_selectors<NT>(w, sel);
    f32x4_t part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const long b = fp8x8(__builtin_amdgcn_perm(lut_hi, lut_lo, sel[2 * j]), __builtin_amdgcn_perm(lut_hi, lut_lo, sel[2 * j + 1]));
      part = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a[j], b, part, 0, 0, 0);
    }
    const float s = __builtin_amdgcn_cvt_f32_fp8(scales >> q8, 0);  // the scale of this lane's group
    acc.x = fmaf(part.x, s, acc.x);
    acc.y = fmaf(part.y, s, acc.y);
    acc.z = fmaf(part.z, s, acc.z);
    acc.w = fmaf(part.w, s, acc.w);
  }
  template <int ODD, bool MORE2, bool MORE1, class C>
  __device__ __forceinline__ void step(const C& ch, int i, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3, const Slot& sl) {
    long rows[4];  // MFMA j's A operand: the lane's bytes in its own group, zero in the others
#pragma unroll
    for (int j = 0; j < 4; j++) rows[j] = grp == j ? held[ODD] : 0L;
    tile<0>(ch, rows, acc0, sl.lut_lo, sl.lut_hi, q8);
    tile<1>(ch, rows, acc1, sl.lut_lo, sl.lut_hi, q8);
    tile<2>(ch, rows, acc2, sl.lut_lo, sl.lut_hi, q8);
    tile<3>(ch, rows, acc3, sl.lut_lo, sl.lut_hi, q8);
    if (MORE2) held[ODD] = load(i + 2);
  }
};
constexpr int PLANE_ROWS = 2;

// The activation scales of a slot's (up to) four rows, asked for ahead of the weights like the pair indices.
struct FewScales {
  float s[FEW_ROWS];
  template <int EPI>
  __device__ __forceinline__ void ask(const StreamParams& p, const Slot& sl, int row0) {
#pragma unroll
    for (int r = 0; r < FEW_ROWS; r++) s[r] = p.a2_scale[activation_row_index<EPI>(p, sl, row0 + r)];
  }
  __device__ __forceinline__ float of(int r) const { return r == 0 ? s[0] : r == 1 ? s[1] : r == 2 ? s[2] : s[3]; }
};

struct FullActs {  // up to sixteen rows: lane (q, r16) feeds row r16, k 8 q .. 8 q + 7 of every group
  static constexpr int LOADS = 4;
  Rows held;           // one chunk's fragments; each half is asked for again as soon as its groups are done
  const uint16_t* at;
  template <int EPI>
  __device__ __forceinline__ void start(const StreamParams& p, const Slot& sl, int, int c0, int, int lane) {
    at = activation_row<EPI>(p, sl, lane & 15) + (int64_t)c0 * 128 + 8 * (lane >> 4);
    load_rows(held, at);
  }
  template <int ODD, bool MORE2, bool MORE1, class C>
  __device__ __forceinline__ void step(const C& ch, int i, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3, const Slot& sl) {
    const uint16_t* next = at + (int64_t)(i + 1) * 128;
    compute_half_chunk<0>(ch, held.a0, held.a1, acc0, acc1, acc2, acc3, sl.lut_lo, sl.lut_hi);
    if (MORE1) {
      held.a0 = *reinterpret_cast<const u32x4_t*>(next);
      held.a1 = *reinterpret_cast<const u32x4_t*>(next + 32);
    }
    compute_half_chunk<1>(ch, held.a2, held.a3, acc0, acc1, acc2, acc3, sl.lut_lo, sl.lut_hi);
    if (MORE1) {
      held.a2 = *reinterpret_cast<const u32x4_t*>(next + 64);
      held.a3 = *reinterpret_cast<const u32x4_t*>(next + 96);
    }
  }
};

// The sixteen-row body on E4M3 activations: lane (q, r16) feeds row r16's eight codes of every group (the FP8 MFMA's A
// operand) and folds, per group, the product of the weight scale and the activation scales of the four rows its
// accumulator registers hold (rows 4 q .. 4 q + 3). Both are asked for again by halves, as FullActs does.
struct FullActs8 {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  static constexpr int LOADS = 12;
  long a[4];            // the lane's codes of groups 0..3
  f32x2_t xs_lo[4];     // activation scales of rows 4 q + r at groups 0, 1
  f32x2_t xs_hi[4];     // ... at groups 2, 3
  const uint8_t* at;    // the lane's codes of group 0 of the wavefront's first chunk
  const float* scales;
  uint32_t soff[4];     // the scale of slot row 4 q + r at group 0 of that chunk
  __device__ __forceinline__ void load_half(int half, int i) {
    a[2 * half] = *reinterpret_cast<const long*>(at + (int64_t)i * 128 + 64 * half);
    a[2 * half + 1] = *reinterpret_cast<const long*>(at + (int64_t)i * 128 + 64 * half + 32);
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const f32x2_t v = *reinterpret_cast<const f32x2_t*>(scales + soff[r] + 4 * i + 2 * half);
      if (half) {
        xs_hi[r] = v;
      } else {
        xs_lo[r] = v;
      }
    }
  }
  template <int EPI>
  __device__ __forceinline__ void start(const StreamParams& p, const Slot& sl, int, int c0, int, int lane) {
    const int q = lane >> 4, r16 = lane & 15;
    at = p.aq + activation_row_index<EPI>(p, sl, r16) * p.a_stride + (int64_t)c0 * 128 + 8 * q;
    scales = p.aq_scale;
#pragma unroll
    for (int r = 0; r < 4; r++) soff[r] = (uint32_t)(activation_row_index<EPI>(p, sl, 4 * q + r) * (p.a_stride >> 5)) + 4 * c0;
    load_half(0, 0);
    load_half(1, 0);
  }
  // groups 2 HALF and 2 HALF + 1 of the four tiles
  // groups 2 HALF and 2 HALF + 1 of tile NT
  template <int HALF, int NT, class C>
  __device__ __forceinline__ void half_tile(const C& ch, f32x4_t& acc, uint32_t lut_lo, uint32_t lut_hi) const {
    const uint32_t sc = chunk_scales<NT>(ch);
    uint32_t sel[8];
    chunk_selectors<NT>(ch, sel);  // the four the half does not use fold away
#pragma unroll
    for (int jj = 0; jj < 2; jj++) {
      const int j = 2 * HALF + jj;
      const long b = fp8x8(__builtin_amdgcn_perm(lut_hi, lut_lo, sel[2 * j]), __builtin_amdgcn_perm(lut_hi, lut_lo, sel[2 * j + 1]));
      const f32x4_t part = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a[j], b, f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
      const float ws = j == 0 ? __builtin_amdgcn_cvt_f32_fp8(sc, 0) : j == 1 ? __builtin_amdgcn_cvt_f32_fp8(sc, 1)
                     : j == 2 ? __builtin_amdgcn_cvt_f32_fp8(sc, 2) : __builtin_amdgcn_cvt_f32_fp8(sc, 3);
      const f32x2_t* xs = HALF ? xs_hi : xs_lo;
      acc.x = fmaf(part.x, (jj ? xs[0].y : xs[0].x) * ws, acc.x);
      acc.y = fmaf(part.y, (jj ? xs[1].y : xs[1].x) * ws, acc.y);
      acc.z = fmaf(part.z, (jj ? xs[2].y : xs[2].x) * ws, acc.z);
      acc.w = fmaf(part.w, (jj ? xs[3].y : xs[3].x) * ws, acc.w);
    }
  }
  template <int HALF, class C>
  __device__ __forceinline__ void half_chunk(const C& ch, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3, uint32_t lut_lo,
                                             uint32_t lut_hi) const {
    half_tile<HALF, 0>(ch, acc0, lut_lo, lut_hi);
    half_tile<HALF, 1>(ch, acc1, lut_lo, lut_hi);
    half_tile<HALF, 2>(ch, acc2, lut_lo, lut_hi);
    half_tile<HALF, 3>(ch, acc3, lut_lo, lut_hi);
  }
  template <int ODD, bool MORE2, bool MORE1, class C>
  __device__ __forceinline__ void step(const C& ch, int i, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3, const Slot& sl) {
    half_chunk<0>(ch, acc0, acc1, acc2, acc3, sl.lut_lo, sl.lut_hi);
    if (MORE1) load_half(0, i + 1);
    half_chunk<1>(ch, acc0, acc1, acc2, acc3, sl.lut_lo, sl.lut_hi);
    if (MORE1) load_half(1, i + 1);
  }
};

// The end of a 64-row block for a slot of at most four rows. Lane (g, r16) of each of the block's K splits holds, in
// register r of accumulator t, group g's part of (tile t, slot row r, column r16): sixteen values a lane, each to be
// added over the four groups and the splits. They go to LDS, and the workgroup's 64 x ks lanes share the 16 x 16
// results of the block: lane (q, r16) of split `ks` takes tile q, column r16, of slot rows row0 + ks, row0 + ks + p.ks, ... It
// multiplies by its tile's row scale (`scale`, asked for before the first chunk); a gated pair's gate comes from the
// neighbouring tile's lane. Every wavefront of the workgroup must call it when K is split (one workgroup barrier).
// QUANT (fc1 in the E4M3 activation mode): h leaves as codes and scales; a 32-group is two of the wavefront's DPP rows.
template <int EPI, bool QUANT = false, bool SCALED = false, bool PLANES = false>  // SCALED: the sums are of the two-plane activations and take their row's scale; PLANES: registers 2, 3 hold the lower plane of rows 0, 1
__device__ __forceinline__ void finish_few(const StreamParams& p, const Slot& sl, int row0, float scale, int nb, bool active, int wave, int ks,
                                           int nbi, float* partial, const f32x4_t& acc0, const f32x4_t& acc1, const f32x4_t& acc2,
                                           const f32x4_t& acc3, const FewPairs& pairs = FewPairs{}, const FewScales& xs = FewScales{}) {
  constexpr int STRIDE = RING_BYTES / 4;
  const int lane = threadIdx.x & 63, q = lane >> 4, r16 = lane & 15;
  float* mine = partial + wave * STRIDE;
  const f32x4_t all[4] = {acc0, acc1, acc2, acc3};
#pragma unroll
  for (int t = 0; t < 4; t++) {
    mine[(t * 4 + 0) * 64 + lane] = all[t].x;
    mine[(t * 4 + 1) * 64 + lane] = all[t].y;
    mine[(t * 4 + 2) * 64 + lane] = all[t].z;
    mine[(t * 4 + 3) * 64 + lane] = all[t].w;
  }
  if (p.ks > 1) {
    __syncthreads();
  } else {
    __builtin_amdgcn_wave_barrier();  // the lanes of one wavefront: its LDS operations execute in program order
  }
  if (!active) return;
  const float* first = partial + nbi * p.ks * STRIDE + r16;
  const int rows = min(PLANES ? PLANE_ROWS : FEW_ROWS, sl.rows - row0);
  for (int r = ks; r < rows; r += p.ks) {
    const float* at = first + (q * 4 + r) * 64;
    float v = 0.f;
    for (int s = 0; s < p.ks; s++) {
      v += (at[0] + at[16]) + (at[32] + at[48]);
      if (PLANES) v += (at[128] + at[144]) + (at[160] + at[176]);
      at += STRIDE;
    }
    const float y = SCALED ? v * scale * xs.of(r) : v * scale;
    if (EPI == EPI_FC1_GATED) {
      const float gate = __shfl_xor(y, 16);  // tiles 2 t and 2 t + 1 are a pair's up and gate rows
      if (QUANT) {  // the pairs are in tiles 0 and 2: their two rows of lanes are the group
        const bool pair = (q & 1) == 0;
        const float h = pair ? fc1_value<EPI>(y, gate) : 0.f;
        float amax = row16_max(fabsf(h));
        amax = fmaxf(amax, __shfl_xor(amax, 32));
        if (pair) store_quantized(p, sl.p0 + row0 + r, nb * 32 + 8 * q + r16, h, amax, lane == 0);
      } else if ((q & 1) == 0) {
        store_out<EPI>(p, sl, nb, q >> 1, row0 + r, r16, y, gate);
      }
    } else if (QUANT) {  // tiles 0, 1 and tiles 2, 3 are the block's two groups
      const float h = fc1_value<EPI>(y, 0.f);
      float amax = row16_max(fabsf(h));
      amax = fmaxf(amax, __shfl_xor(amax, 16));
      store_quantized(p, sl.p0 + row0 + r, nb * 64 + 16 * q + r16, h, amax, (lane & 31) == 0);
    } else if (EPI == EPI_FC2) {
      store_pair(p, pairs.of(r), nb * 64 + lane, y);  // lane (q, r16) is column 16 q + r16 of the block
    } else {
      store_out<EPI>(p, sl, nb, q, row0 + r, r16, y, 0.f);
    }
  }
}

// General kernel, any K: one workgroup per (run of p.nbw 64-row blocks, slot), K split p.ks ways across its wavefronts.
// A8: E4M3 activations (p.aq, p.aq_scale), with the two bodies' FP8 forms; fc1 then writes h as E4M3 codes and
// scales (p.oq, p.oq_scale), the activation rounding done in its epilogue.
// SPLIT: slots of at most two rows read the two-plane form of the activations (p.a2) and run on the FP8 matrix cores.
// One workgroup's work: slot `sl` (with rows), the run `bx` of p.nbw 64-row blocks; `rings`: the launch's dynamic LDS.
template <int EPI, bool A8, bool SPLIT, class Ring = W3Ring>
__device__ __forceinline__ void stream_workgroup(const StreamParams& p, const Slot& sl, int bx, uint8_t* rings) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same in every lane: kept in scalars
  const WaveShare share = wave_share(p, wave);
  const int ks = share.ks, nbi = share.nbi, nb = bx * p.nbw + nbi;
  const bool active = nb < p.n_blocks;
  f32x4_t acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = acc0, acc2 = acc0, acc3 = acc0;
  uint8_t* ring = rings + wave * RING_BYTES;
  constexpr bool QUANT = A8 && epi_gathers(EPI);  // fc1 on E4M3 activations hands fc2 E4M3 activations
  if (A8) {
    if (sl.rows <= FEW_ROWS) {  // uniform over the workgroup
      float scale = 0.f;
      FewPairs pairs{};
      if (active) {
        scale = sl.rs[nb * 64 + lane];
        if (EPI == EPI_FC2) pairs.ask(p, sl, 0);
        stream_block<EPI, FewActs8, Ring>(p, sl, 0, nb, share.c0, share.c1, lane, ring, acc0, acc1, acc2, acc3);
      }
      finish_few<EPI, QUANT>(p, sl, 0, scale, nb, active, wave, ks, nbi, reinterpret_cast<float*>(rings), acc0, acc1, acc2, acc3, pairs);
    } else {
      RowScales rs{};
      if (active) {
        stream_block<EPI, FullActs8, Ring>(p, sl, 0, nb, share.c0, share.c1, lane, ring, acc0, acc1, acc2, acc3);
        rs = row_scales<true>(sl, nb, lane & 15);
      }
      finish_block<EPI, true, RING_BYTES / 4, QUANT>(p, sl, rs, nb, active, ks, nbi, reinterpret_cast<float*>(rings), acc0, acc1, acc2, acc3);
    }
  } else if (SPLIT && sl.rows <= PLANE_ROWS) {  // uniform over the workgroup
    float scale = 0.f;
    FewPairs pairs{};
    FewScales xs{};
    if (active) {
      scale = sl.rs[nb * 64 + lane];
      if (EPI == EPI_FC2) pairs.ask(p, sl, 0);
      xs.ask<EPI>(p, sl, 0);
      stream_block<EPI, FewPlaneActs, Ring>(p, sl, 0, nb, share.c0, share.c1, lane, ring, acc0, acc1, acc2, acc3);
    }
    finish_few<EPI, false, true, true>(p, sl, 0, scale, nb, active, wave, ks, nbi, reinterpret_cast<float*>(rings), acc0, acc1, acc2, acc3, pairs, xs);
  } else if (sl.rows <= FEW_ROWS && !p.no_few) {  // uniform over the workgroup
    float scale = 0.f;
    FewPairs pairs{};
    if (active) {
      scale = sl.rs[nb * 64 + lane];  // row 16 q + r16 of the block: asked for ahead of the chunks, there when the epilogue wants it
      if (EPI == EPI_FC2) pairs.ask(p, sl, 0);
      stream_block<EPI, FewActs, Ring>(p, sl, 0, nb, share.c0, share.c1, lane, ring, acc0, acc1, acc2, acc3);  // at least one chunk: ks <= chunks
    }
    finish_few<EPI>(p, sl, 0, scale, nb, active, wave, ks, nbi, reinterpret_cast<float*>(rings), acc0, acc1, acc2, acc3, pairs);
  } else {
    RowScales rs{};
    if (active) {
      stream_block<EPI, FullActs, Ring>(p, sl, 0, nb, share.c0, share.c1, lane, ring, acc0, acc1, acc2, acc3);
      rs = row_scales<true>(sl, nb, lane & 15);
    }
    finish_block<EPI, true, RING_BYTES / 4>(p, sl, rs, nb, active, ks, nbi, reinterpret_cast<float*>(rings), acc0, acc1, acc2, acc3);
  }
}

template <int EPI, bool A8, bool SPLIT = false, int BITS = 3>  // BITS: the tile layout's (two-bit matrices have their own)
__global__ __launch_bounds__(1024) void w3_stream_kernel(StreamParams p) {
  extern __shared__ __align__(16) uint8_t rings[];
  const Slot sl = slot_of<EPI>(p, blockIdx.y);
  if (sl.rows <= 0) return;  // a slot the plan did not fill: the whole workgroup leaves
  stream_workgroup<EPI, A8, SPLIT, W3RingOf<2, BITS>>(p, sl, blockIdx.x, rings);
}

// One token from its router logits: fc1 with the routing inside it, so that the call has no launch for routing and plan.
// Every wavefront of the launch routes the row for itself (about three microseconds in which it could not have known
// its expert anyway; the logits are 2 KB): lane s then holds selection s, slot s is that expert with the token's one
// row, and the slot after the last selection is the shared expert's. The first wavefront of the first workgroup also
// writes what the caller and the next launch read: ids, weights, and the slot table and pair list in the plan's format
// (in selection order: every slot has one row, so no order is better). The activation row is row 0 whatever a slot's
// pair index says: the launch passes a row stride of 0.
template <int EPI>
__global__ __launch_bounds__(1024) void w3_fc1_route_one_kernel(StreamParams p, RouteParams route, int e_lo, int e_n, int shared_slot, int32_t* plan,
                                                                int32_t* order) {
  extern __shared__ __align__(16) uint8_t rings[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool writer = blockIdx.x == 0 && blockIdx.y == 0 && wave == 0;
  const int id = route.per <= 8 ? route_row<false, 8>(route, 0, lane, writer) : route_row<false, 16>(route, 0, lane, writer);
  const int local = id - e_lo;
  const bool here = lane < route.k && local >= 0 && local < e_n;  // an expert of another rank's range has no slot
  if (writer) {
    const int kept = __popcll(__ballot(here));
    if (lane < route.k || lane == shared_slot) {
      int32_t* entry = plan + PLAN_HEADER + 4 * lane;
      entry[0] = lane == shared_slot ? -1 : here ? local : 0;
      entry[1] = lane;
      entry[2] = lane == shared_slot || here ? 1 : 0;
      entry[3] = 0;
      order[lane] = lane;  // a selection's pair index is its own; the shared expert's row follows the pairs
    }
    if (lane == 0) {
      plan[0] = route.k + (shared_slot >= 0 ? 1 : 0);
      plan[1] = plan[2] = kept;
    }
  }
  const int slot = blockIdx.y;
  int expert = -1;
  if (slot != shared_slot) {
    if (!__builtin_amdgcn_readlane((int)here, slot)) return;  // uniform over the workgroup
    expert = __builtin_amdgcn_readlane(local, slot);
  }
  stream_workgroup<EPI, false, false, W3RingCached>(p, make_slot(p, slot, expert, slot, 1), blockIdx.x, rings);
}

// fc1 and fc2 of a routed call in ONE launch, so that fc2's workgroups fill the compute units that fc1's last, partly
// empty round of workgroups leaves idle (and no launch boundary lies between the two). The grid is one-dimensional:
// first every fc1 workgroup (slot-major, the slot table's order), then every fc2 workgroup. A slot's fc2 needs all of
// the slot's h, that is all `groups1` fc1 workgroups of the slot: each of those, once its h is in memory (write-through
// stores, waited for), adds one to the slot's arrival counter (plan_done: zero from the plan), and the slot's fc2
// workgroups wait for the counter before they ask for anything (one wavefront polls with loads that bypass the L2, the
// others stand at a barrier). What fc2 then reads of h it reads with ordinary loads: the lines were written through to
// memory before the count, and this compute die's L2 cannot hold an older copy of them, because every launch starts
// with its L2 invalidated and no workgroup of this launch reads a slot's h before the slot's count is complete (h rows
// are whole 256-byte multiples on 256-byte boundaries, so no line of h is shared with anything read earlier).
// fc2 workgroups cannot starve fc1: the hardware starts a grid's workgroups in index order, so when an fc2 workgroup
// waits, every fc1 workgroup has started, and an fc1 workgroup waits for nothing. HIP does not promise that order;
// should it ever fail to hold, await_count's bound ends the wait, the workgroup records HB_FAULT_WAIT in the
// workspace's fault word (hb_workspace_status reads it) and leaves without storing anything. hb_tune("moe_fused", 2)
// runs the two layers as two launches, which wait for nothing. Same sums in the same order either way: the same bits.
//
// Order of the grid: slot-major, fc2 of a slot `lag` slots behind its fc1 - fc1(0) .. fc1(lag - 1), then fc1(s), fc2(s -
// lag) for s = lag .., then the last `lag` slots' fc2. With `lag` about the slots whose workgroups fill the device once,
// a slot's fc2 workgroups are started when its fc1 workgroups have had a workgroup's lifetime to finish: they rarely
// wait, and fc1 and fc2 workgroups of different lengths run side by side instead of in rounds that start and end
// together. The slots a call does not fill (the table's upper bound is far above them: every pair could name another
// expert) come last in this order, fc1 and fc2 alike, so their workgroups, short as they are, hold nobody back.
template <int EPI1, bool SPLIT>
__global__ __launch_bounds__(1024) void w3_fc12_kernel(StreamParams p1, StreamParams p2, int groups1, int groups2, int slots, int lag) {
  extern __shared__ __align__(16) uint8_t rings[];
  int id = blockIdx.x, slot;
  bool is_fc1;
  const int head = lag * groups1, both = groups1 + groups2, middle = (slots - lag) * both;
  if (id < head) {  // the first slots' fc1
    slot = id / groups1;
    id -= slot * groups1;
    is_fc1 = true;
  } else if (id < head + middle) {  // fc1(s) then fc2(s - lag)
    id -= head;
    const int step = id / both;
    id -= step * both;
    is_fc1 = id < groups1;
    slot = is_fc1 ? lag + step : step;
    if (!is_fc1) id -= groups1;
  } else {  // the last slots' fc2
    id -= head + middle;
    const int step = id / groups2;
    id -= step * groups2;
    slot = slots - lag + step;
    is_fc1 = false;
  }
  const int64_t t0 = p1.trace ? (int64_t)wall_clock64() : 0;
  int64_t t1 = 0;
  int rows = 0;
  if (is_fc1) {
    const Slot sl = slot_of<EPI1>(p1, slot);
    if (sl.rows <= 0) return;
    rows = sl.rows;
    stream_workgroup<EPI1, false, SPLIT>(p1, sl, id, rings);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's part of h has reached memory
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(&p1.done[slot * DONE_PITCH], 1);
  } else {
    const Slot sl = slot_of<EPI_FC2>(p2, slot);
    if (sl.rows <= 0) return;
    rows = sl.rows;
    // one wavefront polls for the workgroup; the others wait at the barrier and learn the outcome through LDS
    int* outcome = reinterpret_cast<int*>(rings);
    if (threadIdx.x < 64) {
      const bool there = await_count(p2.done + slot * DONE_PITCH, p2.done_need, p2.wait_spins);
      if (threadIdx.x == 0) {
        *outcome = there;
        if (!there) atomicOr(p2.fault, HB_FAULT_WAIT);  // the caller reads it with hb_workspace_status
      }
    }
    __syncthreads();
    const bool there = *outcome != 0;
    __syncthreads();  // read by everyone before the rings take the memory
    if (!there) return;  // h is not known to be complete: this workgroup's outputs stay as they were
    if (p1.trace) t1 = (int64_t)wall_clock64();
    stream_workgroup<EPI_FC2, false, false>(p2, sl, id, rings);
  }
  if (p1.trace && threadIdx.x == 0 && (int64_t)blockIdx.x < p1.trace_records) {  // measurement hook: start, end of the wait, end (100 MHz ticks), rows
    int64_t* rec = p1.trace + 4 * (int64_t)blockIdx.x;
    rec[0] = t0;
    rec[1] = t1;
    rec[2] = (int64_t)wall_clock64();
    rec[3] = rows | (is_fc1 ? 1 << 16 : 0);
  }
}

// One token (a decode step): fc2 and the combine in one launch. A workgroup owns a 64-row block of the output; each of
// its first `slots` wavefronts takes one slot of the plan (an expert the token chose, or the shared expert) through all
// of K on the four-row body, adds its groups as finish_few does without a K split, and leaves the slot's 64 outputs in
// LDS under the pair's selection index; with a gate, four more wavefronts meanwhile make its dot product. The first
// wavefront then runs the combine's chain, a column a lane. Every sum is the one the two separate launches make (fc2
// with one K split, then moe_combine_kernel), so the bits are theirs; what goes away is the round trip of the pair
// outputs through memory and a launch.
constexpr int ONE_GATE_WAVES = 4;  // the gate's dot product is laid out over 256 threads
constexpr int ONE_MAX_WAVES = 16;

// One wavefront's product over all of K for the tiles T0 .. T1 - 1 of block row nb (the others' accumulators: zero).
template <int T0, int T1>
__device__ __forceinline__ void one_token_tiles(const StreamParams& p, const Slot& sl, int row0, int nb, int lane, uint8_t* ring, f32x4_t (&acc)[4]) {
  if constexpr (T0 == 0 && T1 == 4) {
    stream_block<EPI_FC2, FewActs, W3RingCached>(p, sl, row0, nb, 0, p.chunks, lane, ring, acc[0], acc[1], acc[2], acc[3]);
  } else {
    stream_block<EPI_FC2, FewActsPart<T0, T1>, W3RingPart<0, T0, T1>>(p, sl, row0, nb, 0, p.chunks, lane, ring, acc[0], acc[1], acc[2], acc[3]);
  }
}

// PARTS: the workgroups a 64-row block (1, 2 or 4), each taking 4 / PARTS of its four 16-row tiles - the same sums a
// column, over more compute units: a workgroup's wavefronts expand only their tiles' codes (a slot's whole K is four
// chunks of 204 VALU instructions a wavefront otherwise, and a workgroup's ten or eleven wavefronts share four SIMDs)
// and ask only for the 16-byte loads those tiles' dwords lie in (one or two of a chunk's three).
template <int PARTS>
__global__ __launch_bounds__(1024) void w3_fc2_combine_one_kernel(StreamParams p, CombineParams c, int slots) {
  extern __shared__ __align__(16) uint8_t rings[];  // a ring a streaming wavefront, then ys [topk + 1][64], then the gate's four partial sums
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nb = blockIdx.x / PARTS, part = blockIdx.x % PARTS, q = lane >> 4, r16 = lane & 15;
  float* ys = reinterpret_cast<float*>(rings + slots * RING_BYTES);
  float* red = ys + (p.topk + 1) * 64;
  // the chain's operands, a selection a lane, asked for now; a pair whose expert is not local has no slot: its place
  // in ys is never written and never read
  float w_mine = 0.f;
  bool keep_mine = false;
  if (wave == 0 && lane < p.topk) {
    const int e = c.ids[lane] - c.e_lo;
    keep_mine = e >= 0 && e < c.e_n;
    w_mine = c.weights[lane];
  }
  if (wave >= slots) {  // only with a gate
    combine_gate_partial(c.x, c.gate_vec, c.hx, 0, (int)threadIdx.x - 64 * slots, red);
  } else {
    const Slot sl = slot_of<EPI_FC2>(p, wave);
    if (sl.rows > 0) {  // uniform over the wavefront
      const float scale = sl.rs[nb * 64 + lane];
      float* mine = reinterpret_cast<float*>(rings + wave * RING_BYTES);
      for (int row0 = 0; row0 < sl.rows; row0 += FEW_ROWS) {  // more than one row: the caller named an expert twice
        f32x4_t acc[4];
#pragma unroll
        for (int t = 0; t < 4; t++) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        FewPairs pairs;
        pairs.ask(p, sl, row0);
        uint8_t* ring = reinterpret_cast<uint8_t*>(mine);
        if (PARTS == 1) {
          one_token_tiles<0, 4>(p, sl, row0, nb, lane, ring, acc);
        } else if (PARTS == 2) {
          if (part == 0) one_token_tiles<0, 2>(p, sl, row0, nb, lane, ring, acc); else one_token_tiles<2, 4>(p, sl, row0, nb, lane, ring, acc);
        } else {
          if (part == 0) one_token_tiles<0, 1>(p, sl, row0, nb, lane, ring, acc);
          else if (part == 1) one_token_tiles<1, 2>(p, sl, row0, nb, lane, ring, acc);
          else if (part == 2) one_token_tiles<2, 3>(p, sl, row0, nb, lane, ring, acc);
          else one_token_tiles<3, 4>(p, sl, row0, nb, lane, ring, acc);
        }
#pragma unroll
        for (int t = 0; t < 4; t++) {
          mine[(t * 4 + 0) * 64 + lane] = acc[t].x;
          mine[(t * 4 + 1) * 64 + lane] = acc[t].y;
          mine[(t * 4 + 2) * 64 + lane] = acc[t].z;
          mine[(t * 4 + 3) * 64 + lane] = acc[t].w;
        }
        __builtin_amdgcn_wave_barrier();  // the lanes of one wavefront: its LDS operations execute in program order
        const int rows = min(FEW_ROWS, sl.rows - row0);
        for (int r = 0; r < rows; r++) {
          const float* at = mine + (q * 4 + r) * 64 + r16;
          float v = 0.f;
          v += (at[0] + at[16]) + (at[32] + at[48]);
          ys[min(pairs.of(r), p.topk) * 64 + lane] = v * scale;  // lane (q, r16) is column 16 q + r16 of the block; the shared expert's row follows the pairs
        }
        __builtin_amdgcn_wave_barrier();  // read before the next pass's blocks land in the ring
      }
    }
  }
  __syncthreads();
  if (wave != 0) return;
  // Every lane runs the chain and only the store is narrowed to this workgroup's tiles: the chain reads its operands
  // from lanes 0 .. topk - 1, and what a lane outside the execution mask holds of a value computed earlier is not
  // defined (the compiler may compute it after the branch that narrowed the mask).
  float v = 0.f;
  for (int s = 0; s < p.topk; s++) {
    const bool keep = __builtin_amdgcn_readlane((int)keep_mine, s) != 0;
    const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, w_mine), s));
    v = fmaf(keep ? w : 0.f, keep ? ys[s * 64 + lane] : 0.f, v);
  }
  if (c.shared) v = combine_shared(v, c.gate_vec ? combine_gate_value(red) : 1.0f, ys[p.topk * 64 + lane]);
  if (PARTS == 1 || q / (4 / PARTS) == part) c.out[nb * 64 + lane] = f32_to_bf16_bits(v);  // lane (q, r16) is column 16 q + r16
}

// ------------------------------------------------------------------------------------ the prefill kernel's W3 format
struct TileW3 {
  typedef hb::Chunk Chunk;
  static constexpr int BLOCK_BYTES = W3_BLOCK_BYTES;
  static constexpr bool SPLIT_A = false, PER_ROW = true;
  static __device__ __forceinline__ void load(Chunk& ch, const uint8_t* blk, int lane, int r16) { load_chunk(ch, blk, lane, r16); }
  // The B operand of 16-row tile nt, 32-group s, scaled by the group's E4M3 scale (a 4-bit level times a 4-bit scale:
  // exact in BF16); the FP32 row scale stays in the epilogue.
  static __device__ __forceinline__ bf16x8_t fragment(const Chunk& ch, int nt, int s, const Slot& sl) {
    typedef __attribute__((ext_vector_type(2))) float f32x2_t;
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_v;
    const uint32_t q0 = nt == 0 ? ch.w0.x : nt == 1 ? ch.w0.w : nt == 2 ? ch.w1.z : ch.w2.y;
    const uint32_t q1 = nt == 0 ? ch.w0.y : nt == 1 ? ch.w1.x : nt == 2 ? ch.w1.w : ch.w2.z;
    const uint32_t q2 = nt == 0 ? ch.w0.z : nt == 1 ? ch.w1.y : nt == 2 ? ch.w2.x : ch.w2.w;
    const uint32_t scales = nt == 0 ? ch.sc.x : nt == 1 ? ch.sc.y : nt == 2 ? ch.sc.z : ch.sc.w;
    uint32_t sel[8];
    w3_selectors(q0, q1, q2, sel);  // the six the step does not use fold away
    const uint32_t f0 = __builtin_amdgcn_perm(sl.lut_hi, sl.lut_lo, sel[2 * s]);
    const uint32_t f1 = __builtin_amdgcn_perm(sl.lut_hi, sl.lut_lo, sel[2 * s + 1]);
    const float g = s == 0 ? __builtin_amdgcn_cvt_f32_fp8(scales, 0) : s == 1 ? __builtin_amdgcn_cvt_f32_fp8(scales, 1)
                  : s == 2 ? __builtin_amdgcn_cvt_f32_fp8(scales, 2) : __builtin_amdgcn_cvt_f32_fp8(scales, 3);
    const f32x2_t a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(f0, 1.0f, false), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(f0, 1.0f, true);
    const f32x2_t c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(f1, 1.0f, false), d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(f1, 1.0f, true);
    u32x4_t packed;
    packed.x = __builtin_bit_cast(uint32_t, bf16x2_v{(__bf16)(a.x * g), (__bf16)(a.y * g)});
    packed.y = __builtin_bit_cast(uint32_t, bf16x2_v{(__bf16)(b.x * g), (__bf16)(b.y * g)});
    packed.z = __builtin_bit_cast(uint32_t, bf16x2_v{(__bf16)(c.x * g), (__bf16)(c.y * g)});
    packed.w = __builtin_bit_cast(uint32_t, bf16x2_v{(__bf16)(d.x * g), (__bf16)(d.y * g)});
    return __builtin_bit_cast(bf16x8_t, packed);
  }
};

// ---------------------------------------------------------------------------------------------------- host side
struct Tuning {  // hb_tune's knobs: relaxed atomics, so a knob set from one thread while another launches is a plain race-free read
  std::atomic<int> w3_tile{0}, w3_few{0}, w3_ksplit{0}, w3_nbw{0}, moe_fc1_ksplit{0}, moe_fc1_nbw{0}, moe_fc2_ksplit{0}, moe_fc2_nbw{0}, moe_one{0}, moe_split{0}, moe_fused{0}, moe_lag{0}, fault_inject{0}, moe_one_parts{0};
};
static Tuning g_tune;

// Launch one W3 stream. `busy_slots` is the caller's estimate of the slots that will have rows (the grid covers
// `slots`, the upper bound); K is split until the launch has a few thousand wavefronts.
struct Launch {
  int ks, nbw;  // 0: chosen here
};

// Chooses the workgroup shape of a launch (p.ks, p.nbw and what follows from them).
static int shape_stream(StreamParams& p, int64_t busy_slots, Launch want) {
  pick_shape(p.n_blocks, p.chunks, busy_slots, 8192, &p.ks, &p.nbw);
  if (want.ks) {
    p.ks = want.ks;
    if (!want.nbw) p.nbw = 1;
  }
  if (want.nbw) p.nbw = want.nbw;
  if (p.ks * p.nbw > 16 || p.ks > p.chunks) return HB_EINVAL;
  set_split(p);
  p.no_few = g_tune.w3_few == 2;  // every slot takes the sixteen-row body
  return HB_OK;
}

template <int EPI>
static int launch_stream(StreamParams& p, int64_t slots, int64_t busy_slots, Launch want, hipStream_t stream, int bits = 3) {
  if (int e = shape_stream(p, busy_slots, want)) return e;
  const dim3 grid((unsigned)((p.n_blocks + p.nbw - 1) / p.nbw), (unsigned)slots);
  const int waves = p.ks * p.nbw;
  const size_t lds = (size_t)waves * RING_BYTES;
  if (bits == 2) {  // dense calls only: the reference's two-plane matrices are dense linears (its draft head)
    if constexpr (epi_dense(EPI)) {
      if (p.aq) {
        HB_LAUNCH((w3_stream_kernel<EPI, true, false, 2>), grid, dim3(64 * waves), lds, stream, p);
      } else {
        HB_LAUNCH((w3_stream_kernel<EPI, false, false, 2>), grid, dim3(64 * waves), lds, stream, p);
      }
      return HB_OK;
    }
    return HB_EINVAL;
  }
  if (p.aq) {
    HB_LAUNCH((w3_stream_kernel<EPI, true>), grid, dim3(64 * waves), lds, stream, p);
  } else if (p.a2 && !p.no_few) {
    HB_LAUNCH((w3_stream_kernel<EPI, false, true>), grid, dim3(64 * waves), lds, stream, p);
  } else {
    HB_LAUNCH((w3_stream_kernel<EPI, false>), grid, dim3(64 * waves), lds, stream, p);
  }
  return HB_OK;
}

}  // namespace hb

using namespace hb;

#ifndef HB_NO_DEBUG_HOOKS
extern "C" int hb_tune(const char* key, int value) {
  if (!key) return HB_ENULL;
  struct {
    const char* name;
    std::atomic<int>* slot;
  } table[] = {{"w3_tile", &g_tune.w3_tile}, {"w3_few", &g_tune.w3_few}, {"w3_ksplit", &g_tune.w3_ksplit},           {"w3_nbw", &g_tune.w3_nbw},
               {"moe_fc1_ksplit", &g_tune.moe_fc1_ksplit}, {"moe_fc1_nbw", &g_tune.moe_fc1_nbw},
               {"moe_fc2_ksplit", &g_tune.moe_fc2_ksplit}, {"moe_fc2_nbw", &g_tune.moe_fc2_nbw}, {"moe_one", &g_tune.moe_one}, {"moe_split", &g_tune.moe_split}, {"moe_fused", &g_tune.moe_fused}, {"moe_lag", &g_tune.moe_lag}, {"fault_inject", &g_tune.fault_inject}, {"moe_one_parts", &g_tune.moe_one_parts}};
  for (auto& t : table)
    if (!strcmp(t.name, key)) {
      if (value < 0 || value > 16) return HB_EINVAL;
      *t.slot = value;
      return HB_OK;
    }
  if (moe_tune(key, value) == HB_OK) return HB_OK;
  return nvfp4_tune(key, value);
}
#endif

extern "C" int hb_w3_gemm(const void* x, int m, const void* tiled, const float* row_scale, int64_t lut, int n, int k, int bits, void* y, void* stream) {
  if (!x || !tiled || !row_scale || !y) return HB_ENULL;
  if (m <= 0 || n <= 0 || k <= 0 || n % W3_BLOCK_ROWS || k % W3_CHUNK || (bits != 2 && bits != 3)) return HB_EINVAL;
  if (!aligned(x, 16) || !aligned(tiled, 16) || !aligned(row_scale, 4) || !aligned(y, 2)) return HB_EINVAL;
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
  // (the MFMA tile kernel reads three-bit tiles; a two-bit matrix is served by the stream at every size)
  if (bits == 3 && tile_takes(m, k) && tile_writes(y, false) && (g_tune.w3_tile == 1 || (g_tune.w3_tile == 0 && tile_serves_dense(m, p.n_blocks)))) {
    if (int e = launch_tile<TileW3, EPI_DENSE>(p, (m + TILE_ROWS - 1) / TILE_ROWS, m, as_stream(stream))) return e;
    return launch_status();
  }
  const int64_t slots = (m + ROWS_PER_SLOT - 1) / ROWS_PER_SLOT;
  if (slots > 65535) return HB_EINVAL;
  if (int e = launch_stream<EPI_DENSE>(p, slots, slots, Launch{g_tune.w3_ksplit, g_tune.w3_nbw}, as_stream(stream), bits)) return e;
  return launch_status();
}

extern "C" int hb_w3_quant_groups(const void* x, int64_t m, int k, void* q, float* scales, void* stream) {
  if (!x || !q || !scales) return HB_ENULL;
  if (m <= 0 || k <= 0 || k % 32) return HB_EINVAL;
  if (!aligned(x, 16) || !aligned(q, 8) || !aligned(scales, 4)) return HB_EINVAL;
  moe_launch_quant_groups(QuantJob{static_cast<const uint16_t*>(x), m * k / 8, static_cast<uint8_t*>(q), scales, 0, 0}, as_stream(stream));
  return launch_status();
}

extern "C" int hb_w3_quant_rows(const void* x, int64_t m, int k, void* q, float* scales, void* stream) {
  if (!x || !q || !scales) return HB_ENULL;
  if (m <= 0 || m > 0x7fffffff || k <= 0 || k % 8) return HB_EINVAL;
  if (!aligned(x, 16) || !aligned(q, 8) || !aligned(scales, 4)) return HB_EINVAL;
  moe_launch_quant_rows(static_cast<const uint16_t*>(x), m, k, static_cast<uint8_t*>(q), scales, as_stream(stream));
  return launch_status();
}

extern "C" int hb_w3_gemm_e4m3(const void* xq, const float* x_scale, int m, const void* tiled, const float* row_scale, int64_t lut, int n, int k,
                               int bits, void* y, void* stream) {
  if (!xq || !x_scale || !tiled || !row_scale || !y) return HB_ENULL;
  if (m <= 0 || n <= 0 || k <= 0 || n % W3_BLOCK_ROWS || k % W3_CHUNK || (int64_t)m * (k / 32) > 0xffffffffll || (bits != 2 && bits != 3)) return HB_EINVAL;
  if (!aligned(xq, 8) || !aligned(x_scale, 8) || !aligned(tiled, 16) || !aligned(row_scale, 4) || !aligned(y, 2)) return HB_EINVAL;
  StreamParams p{};
  p.w = static_cast<const uint8_t*>(tiled);
  p.rows = row_scale;
  p.lut_lo = (uint32_t)((uint64_t)lut & 0xffffffffu);
  p.lut_hi = (uint32_t)((uint64_t)lut >> 32);
  p.n_blocks = n / W3_BLOCK_ROWS;
  p.chunks = k / W3_CHUNK;
  p.aq = static_cast<const uint8_t*>(xq);
  p.aq_scale = x_scale;
  p.a_stride = k;
  p.m = m;
  p.out = y;
  p.out_stride = n;
  const int64_t slots = (m + ROWS_PER_SLOT - 1) / ROWS_PER_SLOT;
  if (slots > 65535) return HB_EINVAL;
  if (int e = launch_stream<EPI_DENSE>(p, slots, slots, Launch{g_tune.w3_ksplit, g_tune.w3_nbw}, as_stream(stream), bits)) return e;
  return launch_status();
}

// ------------------------------------------------------------------------------------------------ routed experts
namespace {

int check_experts(const hb_w3_experts* ex) {
  if (!ex) return HB_ENULL;
  if (!ex->fc1 || !ex->fc1_rows || !ex->fc2 || !ex->fc2_rows) return HB_ENULL;
  if (ex->experts <= 0 || ex->hidden <= 0 || ex->inter <= 0 || ex->hidden_out <= 0) return HB_EINVAL;
  const int n1 = ex->gated ? 2 * ex->inter : ex->inter;
  if (ex->hidden % W3_CHUNK || ex->inter % W3_CHUNK || n1 % W3_BLOCK_ROWS || ex->hidden_out % W3_BLOCK_ROWS) return HB_EINVAL;
  if (!aligned(ex->fc1, 16) || !aligned(ex->fc2, 16) || !aligned(ex->fc1_rows, 4) || !aligned(ex->fc2_rows, 4)) return HB_EINVAL;
  return HB_OK;
}

// plan -> fc1 -> fc2 (-> combine, when `combine` is given): `out_pairs` receives fc2's per-pair outputs (the
// workspace's y unless the caller wants the pairs themselves). One token's fc2 and combine are one launch.
struct Routing {  // set: the chain routes `logits` [m, e] itself into the caller's ids / weights
  const float* logits;
  int e;
  int32_t* ids;
  float* weights;
  const BudgetRoute* budget = nullptr;  // ... under a budget, from BF16 logits (`logits` is then unused)
};

int run_experts(const hb_w3_experts* ex, const hb_w3_experts* shared, const void* x, const int32_t* ids, int m, int topk,
                const MoeWorkspace& ws, void* out_pairs, int pairs_bf16, hipStream_t stream, const Routing* route = nullptr,
                bool e4m3 = false, const CombineParams* combine = nullptr) {
  const int64_t pairs = (int64_t)m * topk;
  const int shared_rows = shared ? m : 0;
  // a dense contraction once an expert sees a few dozen rows: slots of 128 rows on the MFMA tile kernel
  // (E4M3 activations: the stream only)
  const bool dense = !e4m3 && tile_takes(m, ex->hidden) && tile_takes(pairs + shared_rows, ex->inter) && tile_writes(out_pairs, !pairs_bf16) &&
                     (g_tune.w3_tile == 1 || (g_tune.w3_tile == 0 && pairs >= (int64_t)ex->experts * 2 * TILE_DENSE_ROWS));  // the pre-scaled expansion costs more here than the stream's
  const int slot_rows = dense ? TILE_ROWS : ROWS_PER_SLOT;
  const int64_t slots = moe_max_slots(pairs, ex->experts, shared_rows, slot_rows);
  if (slots > 65535) return HB_EINVAL;
  // E4M3 activations: x is rounded by further workgroups of the plan's launch, h in fc1's epilogue
  // weight-only on the stream: x also in its two-plane form, for the slots of at most two rows (fc1 on the FP8 matrix cores)
  const bool split = !e4m3 && !dense && g_tune.moe_split == 1 && g_tune.w3_few != 2;
  const QuantJob xjob = split ? QuantJob{static_cast<const uint16_t*>(x), 0, ws.x2, ws.x2s, m, ex->hidden}
                              : QuantJob{static_cast<const uint16_t*>(x), (int64_t)m * ex->hidden / 8, ws.xq, ws.xs, 0, 0};
  const QuantJob* job = e4m3 || split ? &xjob : nullptr;
  // one token from its logits, a slot a selection, and fc2 + combine as one launch after it: fc1 routes for itself
  const bool route_in_fc1 = route && !route->budget && m == 1 && combine && !e4m3 && !split && !dense && topk <= 63 && slots == topk + shared_rows &&
                            slots + (combine->gate_vec && combine->shared ? ONE_GATE_WAVES : 0) <= ONE_MAX_WAVES && g_tune.moe_one == 0 &&
                            moe_check_route(m, route->e, topk) == HB_OK;
  if (route_in_fc1) {
    // (nothing to launch here)
  } else if (route && route->budget) {
    if (e4m3) return HB_EINVAL;  // weight-only
    if (job) moe_launch_quant_groups(*job, stream);  // the selection's launch carries no rounding job: the two-plane form of x in a launch of its own
    // the rows' candidates rest where the pair outputs will go: the selection has read them before fc2 writes
    if (int e = moe_launch_budget_plan(*route->budget, m, topk, route->ids, route->weights, ex->base, ex->experts, shared_rows, ws, ws.y, stream, slot_rows))
      return e;
  } else if (route) {
    if (int e = moe_launch_route_plan(route->logits, m, route->e, topk, route->ids, route->weights, ex->base, ex->experts, shared_rows, ws, stream,
                                      slot_rows, job))
      return e;
  } else if (int e = moe_launch_plan(ids, pairs, ex->base, ex->experts, shared_rows, ws, stream, slot_rows, job)) {
    return e;
  }
  const int n1 = ex->gated ? 2 * ex->inter : ex->inter;
  const int64_t est = pairs < 2 * ex->experts ? (pairs + 1) / 2 + (shared_rows + 15) / 16 : slots;  // rough number of busy slots
  StreamParams p{};
  p.w = static_cast<const uint8_t*>(ex->fc1);
  p.expert_bytes = (int64_t)hb_w3_tiled_bytes(n1, ex->hidden, 3);
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
  f2.expert_bytes = (int64_t)hb_w3_tiled_bytes(ex->hidden_out, ex->inter, 3);
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
  if (dense) {
    if (int e = ex->gated ? launch_tile<TileW3, EPI_FC1_GATED>(p, slots, m, stream) : launch_tile<TileW3, EPI_FC1_RELU2>(p, slots, m, stream)) return e;
    if (int e = launch_tile<TileW3, EPI_FC2>(f2, slots, pairs + shared_rows, stream)) return e;
    if (combine) moe_launch_combine(*combine, stream);
    return launch_status();
  }
  Launch l1{g_tune.moe_fc1_ksplit, g_tune.moe_fc1_nbw}, l2{g_tune.moe_fc2_ksplit, g_tune.moe_fc2_nbw};
  // Decode batches of a few rows to a couple of dozen leave the device partly empty under the general rule (K split 4,
  // one block a workgroup; fc2: four blocks). Measured on the fused launch at hidden 2048 / intermediate 512: up to
  // about 48 busy slots fc1 with K split 2 on two blocks and fc2 with K split 4 is 3 - 5 % faster a step, from 64 to
  // 128 busy slots both with K split 2 on two blocks 3 %; beyond that the general rule wins.
  const bool unset = !l1.ks && !l1.nbw && !l2.ks && !l2.nbw;
  if (unset && !e4m3 && m > 1 && g_tune.moe_fused != 2 && p.chunks >= 8 && f2.chunks >= 4) {
    if (est <= 48) {
      l1 = Launch{2, 2};
      l2 = Launch{4, 1};
    } else if (est >= 64 && est <= 128) {
      l1 = Launch{2, 2};
      l2 = Launch{2, 2};
    }
  }
  if (e4m3) {  // x and h go through the activation rounding: x_q -> fc1 -> h_q -> fc2
    p.aq = ws.xq;
    p.aq_scale = ws.xs;
    p.oq = ws.hq;
    p.oq_scale = ws.hs;
    f2.aq = ws.hq;
    f2.aq_scale = ws.hs;
  }
  if (split) {
    p.a2 = ws.x2;
    p.a2_scale = ws.x2s;
  }
  // more than one token, weight-only: fc1 and fc2 as one launch when their workgroups have the same shape
  if (!e4m3 && m > 1 && g_tune.moe_fused != 2) {
    StreamParams q1 = p, q2 = f2;
    if (shape_stream(q1, est, l1) == HB_OK && shape_stream(q2, est, l2) == HB_OK && q1.ks * q1.nbw == q2.ks * q2.nbw) {
      const int groups1 = (q1.n_blocks + q1.nbw - 1) / q1.nbw, groups2 = (q2.n_blocks + q2.nbw - 1) / q2.nbw;
      const int64_t total = slots * (groups1 + groups2);
      if (total <= 0x7fffffff) {
        q1.done = q2.done = plan_done(ws.plan, slots);
        q1.trace = moe_trace_buffer(&q1.trace_records);
        q1.done_need = q2.done_need = groups1;
        q2.wait_spins = WAIT_SPINS;
        q2.fault = ws.plan + PLAN_FAULT;
        if (g_tune.fault_inject == 1) {  // a test of the give-up path: a count one above what can arrive, and a wait of a few polls
          q2.done_need = groups1 + 1;
          q2.wait_spins = 8;
        }
        const int waves = q1.ks * q1.nbw;
        // about the slots whose workgroups fill the device once (four workgroups of four wavefronts a compute unit)
        const int lag_tuned = g_tune.moe_lag.load();
        const int lag = (int)std::min<int64_t>(slots, lag_tuned ? 8 * lag_tuned : std::max(8, 2304 / (groups1 + groups2)));
        const bool use_split = q1.a2 && !q1.no_few;
        auto launch = [&](auto kernel) { HB_LAUNCH(kernel, dim3((unsigned)total), dim3(64 * waves), (size_t)waves * RING_BYTES, stream, q1, q2, groups1, groups2, (int)slots, lag); };
        if (ex->gated) {
          use_split ? launch(w3_fc12_kernel<EPI_FC1_GATED, true>) : launch(w3_fc12_kernel<EPI_FC1_GATED, false>);
        } else {
          use_split ? launch(w3_fc12_kernel<EPI_FC1_RELU2, true>) : launch(w3_fc12_kernel<EPI_FC1_RELU2, false>);
        }
        if (combine) moe_launch_combine(*combine, stream);
        return launch_status();
      }
    }
  }
  if (route_in_fc1) {
    StreamParams q = p;
    if (int e = shape_stream(q, est, l1)) return e;
    q.a_stride = 0;  // every slot's row is the token's
    RouteParams rp{};
    rp.logits = route->logits;
    rp.stride = route->e;
    rp.e = route->e;
    rp.k = topk;
    rp.per = (route->e + 63) / 64;
    rp.steps = 1;
    rp.pad_id = route->e;
    rp.ids = route->ids;
    rp.weights = route->weights;
    const dim3 grid((unsigned)((q.n_blocks + q.nbw - 1) / q.nbw), (unsigned)slots);
    const int waves = q.ks * q.nbw;
    auto launch = [&](auto kernel) {
      HB_LAUNCH(kernel, grid, dim3(64 * waves), (size_t)waves * RING_BYTES, stream, q, rp, ex->base, ex->experts, shared ? topk : -1, ws.plan, ws.order);
    };
    ex->gated ? launch(w3_fc1_route_one_kernel<EPI_FC1_GATED>) : launch(w3_fc1_route_one_kernel<EPI_FC1_RELU2>);
  } else if (int e = ex->gated ? launch_stream<EPI_FC1_GATED>(p, slots, est, l1, stream) : launch_stream<EPI_FC1_RELU2>(p, slots, est, l1, stream)) {
    return e;
  }
  int fc2_ks = l2.ks, fc2_nbw;
  if (!fc2_ks) pick_shape(f2.n_blocks, f2.chunks, est, 8192, &fc2_ks, &fc2_nbw);
  // one token, and a separate fc2 would not split K either: the fused launch makes the same sums
  const int one_waves = (int)slots + (combine && combine->gate_vec && combine->shared ? ONE_GATE_WAVES : 0);
  // (its chain hands the selections' weights from lane to lane: at most 64 of them)
  if (combine && m == 1 && topk <= 64 && !e4m3 && one_waves <= ONE_MAX_WAVES && fc2_ks == 1 && g_tune.moe_one != 2) {
    f2.ks = 1;
    f2.nbw = 1;
    set_split(f2);
    // the workgroups a 64-row block: as many as leave the launch within about the device's compute units
    const int parts = g_tune.moe_one_parts ? g_tune.moe_one_parts.load() : f2.n_blocks <= 64 ? 4 : f2.n_blocks <= 128 ? 2 : 1;
    const size_t lds = (size_t)slots * RING_BYTES + (topk + 1) * 256 + 16;
    if (parts == 4) {
      HB_LAUNCH(w3_fc2_combine_one_kernel<4>, dim3(4u * (unsigned)f2.n_blocks), dim3(64 * one_waves), lds, stream, f2, *combine, (int)slots);
    } else if (parts == 2) {
      HB_LAUNCH(w3_fc2_combine_one_kernel<2>, dim3(2u * (unsigned)f2.n_blocks), dim3(64 * one_waves), lds, stream, f2, *combine, (int)slots);
    } else {
      HB_LAUNCH(w3_fc2_combine_one_kernel<1>, dim3((unsigned)f2.n_blocks), dim3(64 * one_waves), lds, stream, f2, *combine, (int)slots);
    }
    return launch_status();
  }
  if (int e = launch_stream<EPI_FC2>(f2, slots, est, l2, stream)) return e;
  if (combine) moe_launch_combine(*combine, stream);
  return launch_status();
}

}  // namespace

extern "C" size_t hb_w3_moe_workspace_bytes(int m, int topk, const hb_w3_experts* routed, int shared) {
  if (!routed || m <= 0 || topk <= 0 || check_experts(routed) != HB_OK) return 0;
  return moe_carve(nullptr, m, topk, routed->experts, routed->inter, routed->hidden_out, shared, routed->hidden).bytes;
}

#ifndef HB_NO_DEBUG_HOOKS
extern "C" int hb_debug_workspace_layout(int m, int topk, const hb_w3_experts* routed, int shared, int64_t* offsets) {
  if (!routed || !offsets) return HB_ENULL;
  if (m <= 0 || topk <= 0 || check_experts(routed) != HB_OK) return HB_EINVAL;
  char* base = reinterpret_cast<char*>(uintptr_t(1) << 20);  // any address: only differences are returned
  const MoeWorkspace ws = moe_carve(base, m, topk, routed->experts, routed->inter, routed->hidden_out, shared, routed->hidden);
  offsets[0] = reinterpret_cast<char*>(ws.plan) - base;
  offsets[1] = reinterpret_cast<char*>(ws.order) - base;
  offsets[2] = reinterpret_cast<char*>(ws.h) - base;
  offsets[3] = reinterpret_cast<char*>(ws.y) - base;
  offsets[4] = reinterpret_cast<char*>(plan_done(ws.plan, moe_max_slots((int64_t)m * topk, routed->experts, shared ? m : 0))) - base;
  offsets[5] = moe_max_slots((int64_t)m * topk, routed->experts, shared ? m : 0);
  return HB_OK;
}
#endif

extern "C" int hb_w3_moe(const hb_w3_experts* routed, const void* x, const int32_t* ids, const float* weights, int m, int topk, int mode,
                         void* out, void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_experts(routed)) return e;
  if (!x || !ids || !weights || !out || !workspace) return HB_ENULL;
  const bool e4m3 = (mode & HB_MOE_E4M3) != 0;
  mode &= ~HB_MOE_E4M3;
  if (m <= 0 || topk <= 0 || mode < HB_MOE_SUM || mode > HB_MOE_PAIRS_BF16) return HB_EINVAL;
  if (!aligned(x, 16) || !aligned(ids, 4) || !aligned(weights, 4) || !aligned(out, 8) || !aligned(workspace, 16)) return HB_EINVAL;
  const MoeWorkspace ws = moe_carve(workspace, m, topk, routed->experts, routed->inter, routed->hidden_out, 0, routed->hidden);
  if (workspace_bytes < ws.bytes) return HB_EWORKSPACE;
  void* pairs_out = mode == HB_MOE_SUM ? static_cast<void*>(ws.y) : out;
  const bool narrow = mode == HB_MOE_SUM && m >= MOE_WIDE_ROWS;  // a summed prefill-sized call: BF16 pair outputs (hibana/model/flashnext/moe.py:186)
  CombineParams c{};
  c.pairs = ws.y;
  c.pairs_bf16 = narrow;
  c.ids = ids;
  c.weights = weights;
  c.e_lo = routed->base;
  c.e_n = routed->experts;
  c.m = m;
  c.topk = topk;
  c.h = routed->hidden_out;
  c.out = static_cast<uint16_t*>(out);
  return run_experts(routed, nullptr, x, ids, m, topk, ws, pairs_out, mode == HB_MOE_PAIRS_BF16 || narrow, as_stream(stream), nullptr, e4m3,
                     mode == HB_MOE_SUM ? &c : nullptr);
}

static int moe_layer(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x, const int32_t* ids,
                     const float* weights, int m, int topk, void* out, void* workspace, size_t workspace_bytes, void* stream,
                     const Routing* route, bool e4m3 = false) {
  if (int e = check_experts(routed)) return e;
  if (shared) {
    if (int e = check_experts(shared)) return e;
    if (shared->hidden != routed->hidden || shared->inter != routed->inter || shared->hidden_out != routed->hidden_out ||
        shared->gated != routed->gated)
      return HB_EINVAL;
  }
  if (!x || !ids || !weights || !out || !workspace) return HB_ENULL;
  if (m <= 0 || topk <= 0) return HB_EINVAL;
  if (!aligned(x, 16) || !aligned(ids, 4) || !aligned(weights, 4) || !aligned(out, 4) || !aligned(workspace, 16) || !aligned(gate_vec, 4)) return HB_EINVAL;
  const MoeWorkspace ws = moe_carve(workspace, m, topk, routed->experts, routed->inter, routed->hidden_out, shared ? 1 : 0, routed->hidden);
  if (workspace_bytes < ws.bytes) return HB_EWORKSPACE;
  // a prefill-sized call keeps its pair outputs (and the shared expert's rows behind them) in BF16, as the reference's
  // layer does from the same size (hibana/model/flashnext/moe.py:186); the shared rows are rounded to BF16 by the combine anyway
  const bool narrow = m >= MOE_WIDE_ROWS;
  CombineParams c{};
  c.pairs = ws.y;
  c.pairs_bf16 = narrow;
  c.ids = ids;
  c.weights = weights;
  if (shared) {
    c.shared = narrow ? static_cast<const void*>(reinterpret_cast<const uint16_t*>(ws.y) + (int64_t)m * topk * routed->hidden_out)
                      : static_cast<const void*>(ws.y + (int64_t)m * topk * routed->hidden_out);
    c.shared_f32 = narrow ? 0 : 1;
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
  return run_experts(routed, shared, x, ids, m, topk, ws, ws.y, narrow, as_stream(stream), route, e4m3, &c);
}

extern "C" int hb_w3_moe_layer(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                               const int32_t* ids, const float* weights, int m, int topk, void* out, void* workspace,
                               size_t workspace_bytes, void* stream) {
  return moe_layer(routed, shared, gate_vec, x, ids, weights, m, topk, out, workspace, workspace_bytes, stream, nullptr);
}

extern "C" int hb_w3_moe_layer_e4m3(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                                    const int32_t* ids, const float* weights, int m, int topk, void* out, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  return moe_layer(routed, shared, gate_vec, x, ids, weights, m, topk, out, workspace, workspace_bytes, stream, nullptr, true);
}

// ------------------------------------------------------------------------------- the entry point that allocates nothing
// hb_w3_moe_layer with its workspace in a device array of this library instead of a caller's buffer, for callers that
// cannot allocate. Every GPU the library runs on holds its own copy of the array at its own address; the array's name
// is a host-side stand-in, so the address is asked for once a device (hipGetSymbolAddress, with that device current)
// and only that pointer is ever handed to a kernel.
static __device__ __align__(256) uint8_t scratch[HB_STATIC_SCRATCH_BYTES];

namespace {
constexpr int SCRATCH_MAX_DEVICES = 64;
std::mutex g_scratch_lock;
void* g_scratch_ptr[SCRATCH_MAX_DEVICES] = {};

// The current device's copy of `scratch`, or null if the runtime will not say where it is.
void* scratch_of_current_device() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= SCRATCH_MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_ptr[device]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    g_scratch_ptr[device] = ptr;
  }
  return g_scratch_ptr[device];
}
}  // namespace

extern "C" int hb_w3_moe_layer_static(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                                      const int32_t* ids, const float* weights, int m, int topk, void* out, void* stream) {
  if (int e = check_experts(routed)) return e;
  if (m <= 0 || topk <= 0) return HB_EINVAL;
  // sized before anything is touched: the same carve as hb_w3_moe_workspace_bytes
  if (moe_carve(nullptr, m, topk, routed->experts, routed->inter, routed->hidden_out, shared ? 1 : 0, routed->hidden).bytes > HB_STATIC_SCRATCH_BYTES)
    return HB_ESCRATCH;
  void* ptr = scratch_of_current_device();
  if (!ptr) return HB_ELAUNCH;
  return moe_layer(routed, shared, gate_vec, x, ids, weights, m, topk, out, ptr, HB_STATIC_SCRATCH_BYTES, stream, nullptr);
}

// ------------------------------------------------------------------------------------- a workspace's head words
__global__ __launch_bounds__(256) void workspace_zero_kernel(uint32_t* at, size_t words) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < words; i += (size_t)gridDim.x * 256) at[i] = 0u;
}

extern "C" int hb_workspace_reset(void* workspace, size_t workspace_bytes, void* stream) {
  if (!workspace) {  // the library's own scratch (hb_w3_moe_layer_static)
    workspace = scratch_of_current_device();
    workspace_bytes = HB_STATIC_SCRATCH_BYTES;
    if (!workspace) return HB_ELAUNCH;
  }
  if (!aligned(workspace, 16) || workspace_bytes < 4) return HB_EINVAL;
  const size_t words = std::min<size_t>(workspace_bytes, HB_WORKSPACE_ZERO_BYTES) / 4;
  hipLaunchKernelGGL(workspace_zero_kernel, dim3((unsigned)std::min<size_t>((words + 255) / 256, 1024)), dim3(256), 0, as_stream(stream),
                     static_cast<uint32_t*>(workspace), words);
  return launch_status();
}

extern "C" int hb_workspace_status(const void* workspace, int32_t* status, int wait, void* stream) {
  if (!status) return HB_ENULL;
  if (!workspace) workspace = scratch_of_current_device();
  if (!workspace) return HB_ELAUNCH;
  if (!aligned(workspace, 16)) return HB_EINVAL;
  if (hipMemcpyAsync(status, static_cast<const int32_t*>(workspace) + PLAN_FAULT, sizeof(int32_t), hipMemcpyDeviceToHost, as_stream(stream)) != hipSuccess)
    return HB_ELAUNCH;
  if (wait && hipStreamSynchronize(as_stream(stream)) != hipSuccess) return HB_ELAUNCH;
  return HB_OK;
}

extern "C" int hb_w3_moe_layer_logits(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                                      const float* logits, int experts_total, int m, int topk, int32_t* ids, float* weights, void* out,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  if (!logits) return HB_ENULL;
  if (!aligned(logits, 4)) return HB_EINVAL;
  const Routing route{logits, experts_total, ids, weights};
  return moe_layer(routed, shared, gate_vec, x, ids, weights, m, topk, out, workspace, workspace_bytes, stream, &route);
}

extern "C" int hb_w3_moe_layer_budget(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                                      const void* logits, int experts_total, int m, int topk, int keep, int budget, const int32_t* slots, int steps,
                                      int per_request, int min_cap, int32_t* ids, float* weights, void* out, void* workspace,
                                      size_t workspace_bytes, void* stream) {
  if (!logits) return HB_ENULL;
  const BudgetRoute b{static_cast<const uint16_t*>(logits), experts_total, keep, budget, steps, 0, per_request, min_cap, slots};
  const Routing route{nullptr, experts_total, ids, weights, &b};
  return moe_layer(routed, shared, gate_vec, x, ids, weights, m, topk, out, workspace, workspace_bytes, stream, &route);
}

extern "C" int hb_w3_moe_layer_logits_e4m3(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                                           const float* logits, int experts_total, int m, int topk, int32_t* ids, float* weights, void* out,
                                           void* workspace, size_t workspace_bytes, void* stream) {
  if (!logits) return HB_ENULL;
  if (!aligned(logits, 4)) return HB_EINVAL;
  const Routing route{logits, experts_total, ids, weights};
  return moe_layer(routed, shared, gate_vec, x, ids, weights, m, topk, out, workspace, workspace_bytes, stream, &route, true);
}
