// NVFP4 (E2M1 codes, E4M3 scale per 16 weights, FP32 global scale) weight-only kernels for gfx950.
//
// Tile layout: blocks of 64 output rows x 128 k, NVFP4_BLOCK_BYTES each, [rows/64][K/128]:
//   bytes    0..4095  codes: four 128-bit loads per lane, load nt of lane l at (nt * 64 + l) * 16. Lane l = 16 q + r owns,
//                     for the 16-row tile nt, the weights  row 64 nb + 16 nt + r,  k = 128 c + 16 b + 4 q + i
//                     (b = 0..7 the 16-blocks of the chunk, i = 0..3): dword b / 2 of the load, its low half for even b,
//                     high half for odd b, nibble i. That is the B operand of v_mfma_f32_16x16x16_bf16, one MFMA per
//                     16-block, so the block scale multiplies the MFMA's FP32 result.
//   bytes 4096..4607  scales: 32 B per row-in-tile r at 4096 + 32 r: byte 8 nt + b is the E4M3 scale of row
//                     64 nb + 16 nt + r, block 8 c + b.
// Codes expand with v_cvt_scalef32_pk_bf16_fp4 (two weights per instruction, exact).
#include <string.h>

#include <atomic>

#include "ring.hpp"
#include "stream_common.hpp"
#include "tile_kernel.hpp"

namespace hb {

constexpr int NVFP4_BLOCK_BYTES = 4608;
constexpr int NVFP4_SCALE_OFFSET = 4096;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

__host__ __device__ inline int64_t swizzled_scale_offset(int64_t r, int c, int groups_pad) {
  return (r / 128) * 128 * groups_pad + (c / 4) * 512 + (r % 32) * 16 + ((r / 32) % 4) * 4 + c % 4;
}

// One thread per (block, tile, lane): the lane's four code dwords of one 16-row tile.
__global__ __launch_bounds__(256) void nvfp4_repack_codes_kernel(const uint8_t* __restrict__ weight, int64_t blocks, int chunks,
                                                                 uint8_t* __restrict__ tiled) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= blocks * 256) return;
  const int64_t blk = id >> 8;
  const int nt = (int)(id >> 6) & 3, lane = (int)(id & 63), q = lane >> 4, r = lane & 15;
  const int64_t nb = blk / chunks;
  const int c = (int)(blk % chunks);
  const int64_t n = nb * 64 + nt * 16 + r;
  const uint8_t* src = weight + n * (chunks * 64) + c * 64;  // 64 bytes per chunk per row
  uint32_t d[4];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    // blocks 2e and 2e+1: bytes at k/2 = 8 b + 2 q, two bytes each (four nibbles)
    const uint32_t lo = src[16 * e + 2 * q] | ((uint32_t)src[16 * e + 2 * q + 1] << 8);
    const uint32_t hi = src[16 * e + 8 + 2 * q] | ((uint32_t)src[16 * e + 8 + 2 * q + 1] << 8);
    d[e] = lo | (hi << 16);
  }
  *reinterpret_cast<u32x4_t*>(tiled + blk * NVFP4_BLOCK_BYTES + (nt * 64 + lane) * 16) = u32x4_t{d[0], d[1], d[2], d[3]};
}

// One thread per scale byte.
__global__ __launch_bounds__(256) void nvfp4_repack_scales_kernel(const uint8_t* __restrict__ scales, int swizzled, int64_t blocks,
                                                                  int chunks, uint8_t* __restrict__ tiled) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= blocks * 512) return;
  const int64_t blk = id >> 9;
  const int within = (int)(id & 511), r = within >> 5, nt = (within >> 3) & 3, b = within & 7;
  const int64_t nb = blk / chunks;
  const int c = (int)(blk % chunks);
  const int64_t n = nb * 64 + nt * 16 + r;
  const int groups = chunks * 8, g = 8 * c + b;
  const uint8_t v = swizzled ? scales[swizzled_scale_offset(n, g, (groups + 3) / 4 * 4)] : scales[n * groups + g];
  tiled[blk * NVFP4_BLOCK_BYTES + NVFP4_SCALE_OFFSET + 32 * r + 8 * nt + b] = v;
}

__device__ __forceinline__ float e2m1_to_f32(uint32_t code) {
  const uint32_t a = code & 7u;
  const float mag = a < 4u ? 0.5f * (float)a : a == 4u ? 2.0f : a == 5u ? 3.0f : a == 6u ? 4.0f : 6.0f;
  return (code & 8u) ? -mag : mag;
}

// One thread per (block, tile, lane): 32 dequantized weights, e2m1 * float(scale) then * global (two roundings).
__global__ __launch_bounds__(256) void nvfp4_dequant_kernel(const uint8_t* __restrict__ tiled, float global_scale, int64_t blocks, int chunks,
                                                            float* __restrict__ out) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= blocks * 256) return;
  const int64_t blk = id >> 8;
  const int nt = (int)(id >> 6) & 3, lane = (int)(id & 63), q = lane >> 4, r = lane & 15;
  const int64_t nb = blk / chunks;
  const int c = (int)(blk % chunks);
  const int k = chunks * 128;
  const uint8_t* base = tiled + blk * NVFP4_BLOCK_BYTES;
  const int64_t n = nb * 64 + nt * 16 + r;
  const u32x4_t d = *reinterpret_cast<const u32x4_t*>(base + (nt * 64 + lane) * 16);
  const uint32_t dw[4] = {d.x, d.y, d.z, d.w};
  for (int b = 0; b < 8; b++) {
    const float s = e4m3_to_f32(base[NVFP4_SCALE_OFFSET + 32 * r + 8 * nt + b]);
    const uint32_t half = (dw[b >> 1] >> (16 * (b & 1))) & 0xffffu;
    float* o = out + n * k + c * 128 + 16 * b + 4 * q;
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = __fmul_rn(__fmul_rn(e2m1_to_f32((half >> (4 * i)) & 15u), s), global_scale);
  }
}

struct Fp4Chunk {  // the weight side of a chunk: four 16-row tiles of codes, their block scales
  u32x4_t w0, w1, w2, w3, s0, s1;
};

struct Fp4Rows {  // the activation side: eight MFMA A fragments (one per 16-block), read from L2
  u32x2_t a0, a1, a2, a3, a4, a5, a6, a7;
};

__device__ __forceinline__ void load_fp4_chunk(Fp4Chunk& ch, const uint8_t* blk, int lane, int r16) {
  const u32x4_t* b = reinterpret_cast<const u32x4_t*>(blk);
  ch.w0 = __builtin_nontemporal_load(b + lane);
  ch.w1 = __builtin_nontemporal_load(b + 64 + lane);
  ch.w2 = __builtin_nontemporal_load(b + 128 + lane);
  ch.w3 = __builtin_nontemporal_load(b + 192 + lane);
  ch.s0 = __builtin_nontemporal_load(b + 256 + 2 * r16);
  ch.s1 = __builtin_nontemporal_load(b + 257 + 2 * r16);
}

// One 16-block: two conversions, one MFMA, the block scale folded into the accumulator.
#define HB_FP4_BLOCK(codes, BYTE0, a_frag, scale_dword, SBYTE, acc)                                                                   \
  {                                                                                                                                   \
    u32x2_t packed;                                                                                                                   \
    packed.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, 1.0f, BYTE0));                           \
    packed.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, 1.0f, BYTE0 + 1));                       \
    const f32x4_t part = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(bf16x4_t_s, a_frag), __builtin_bit_cast(bf16x4_t_s, packed), \
                                                                   f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);                           \
    const float s = __builtin_amdgcn_cvt_f32_fp8(scale_dword, SBYTE);                                                                 \
    acc.x = fmaf(part.x, s, acc.x);                                                                                                   \
    acc.y = fmaf(part.y, s, acc.y);                                                                                                   \
    acc.z = fmaf(part.z, s, acc.z);                                                                                                   \
    acc.w = fmaf(part.w, s, acc.w);                                                                                                   \
  }

typedef __attribute__((ext_vector_type(4))) short bf16x4_t_s;  // the 16x16x16 builtin takes its BF16 operands as 4 x i16

// Half of a 16-row tile of a chunk: 16-blocks 0 .. 3 (two code dwords, one scale dword, four activation fragments) or
// 4 .. 7; the blocks of a chunk fold into the accumulator in ascending order either way.
__device__ __forceinline__ void fp4_half_tile(uint32_t c01, uint32_t c23, uint32_t sc, const u32x2_t& a0, const u32x2_t& a1, const u32x2_t& a2,
                                              const u32x2_t& a3, f32x4_t& acc) {
  HB_FP4_BLOCK(c01, 0, a0, sc, 0, acc)
  HB_FP4_BLOCK(c01, 2, a1, sc, 1, acc)
  HB_FP4_BLOCK(c23, 0, a2, sc, 2, acc)
  HB_FP4_BLOCK(c23, 2, a3, sc, 3, acc)
}

// ------------------------------------------------------------------------------------------------ the weight ring
// (ring.hpp) for NVFP4 blocks: four 16-byte loads a lane of codes, two 4-byte loads a lane of scales.
struct Fp4Ring {
  typedef Fp4Chunk Chunk;
  static constexpr int BLOCK_BYTES = NVFP4_BLOCK_BYTES, LOADS = 6;
  static __device__ __forceinline__ void lanes(RingSource& src, int lane, int r16, uint32_t slot0, uint32_t& codes, uint32_t& scales) {
    src.codes = 16u * lane;
    src.scales = 4u * lane;
    codes = slot0 + 16u * lane;
    scales = slot0 + 32u * r16;
  }
  static __device__ __forceinline__ void request(const RingSource& src, int chunk, lds_ptr_t slot) {
    const uint32_t at = (uint32_t)chunk * NVFP4_BLOCK_BYTES;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 16, src.codes, at, 0, 2);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 16, src.codes, at, 1024, 2);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 16, src.codes, at, 2048, 2);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot, 16, src.codes, at, 3072, 2);
    // the instruction's offset field (which moves both ends) stops at 4095: the scales' place is given by hand
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot + NVFP4_SCALE_OFFSET, 4, src.scales, at + NVFP4_SCALE_OFFSET, 0, 2);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src.row, slot + NVFP4_SCALE_OFFSET, 4, src.scales, at + NVFP4_SCALE_OFFSET, 256, 2);
    __builtin_amdgcn_sched_barrier(0);  // asked for here, not wherever the scheduler would sink it below the arithmetic
  }
  template <int BEHIND, int SLOT>
  static __device__ __forceinline__ void take(Chunk& ch, uint32_t codes, uint32_t scales) {
    asm volatile(
        "s_waitcnt vmcnt(%8)\n\t"
        "ds_read_b128 %0, %6 offset:%9\n\t"
        "ds_read_b128 %1, %6 offset:%10\n\t"
        "ds_read_b128 %2, %6 offset:%11\n\t"
        "ds_read_b128 %3, %6 offset:%12\n\t"
        "ds_read_b128 %4, %7 offset:%13\n\t"
        "ds_read_b128 %5, %7 offset:%14\n\t"
        "s_waitcnt lgkmcnt(0)"  // the slot is read: it may be given to another chunk
        : "=&v"(ch.w0), "=&v"(ch.w1), "=&v"(ch.w2), "=&v"(ch.w3), "=&v"(ch.s0), "=&v"(ch.s1)
        : "v"(codes), "v"(scales), "n"(BEHIND), "n"(SLOT * NVFP4_BLOCK_BYTES), "n"(SLOT * NVFP4_BLOCK_BYTES + 1024),
          "n"(SLOT * NVFP4_BLOCK_BYTES + 2048), "n"(SLOT * NVFP4_BLOCK_BYTES + 3072), "n"(SLOT * NVFP4_BLOCK_BYTES + NVFP4_SCALE_OFFSET),
          "n"(SLOT * NVFP4_BLOCK_BYTES + NVFP4_SCALE_OFFSET + 16)
        : "memory");
  }
};
constexpr int FP4_RING_BYTES = ring_bytes<Fp4Ring>();  // LDS per wavefront; its first 4 KB double as the K-split exchange

// The stream's activations: lane (q, r16) feeds row r16, k 4 q .. 4 q + 3 of every 16-block. One chunk's fragments are
// held; each half is asked for again (for the next chunk) as soon as its blocks are done.
struct Fp4Acts {
  static constexpr int LOADS = 8;
  Fp4Rows held;
  const uint16_t* at;
  __device__ __forceinline__ void load_lo(const uint16_t* from) {
    held.a0 = *reinterpret_cast<const u32x2_t*>(from);
    held.a1 = *reinterpret_cast<const u32x2_t*>(from + 16);
    held.a2 = *reinterpret_cast<const u32x2_t*>(from + 32);
    held.a3 = *reinterpret_cast<const u32x2_t*>(from + 48);
  }
  __device__ __forceinline__ void load_hi(const uint16_t* from) {
    held.a4 = *reinterpret_cast<const u32x2_t*>(from + 64);
    held.a5 = *reinterpret_cast<const u32x2_t*>(from + 80);
    held.a6 = *reinterpret_cast<const u32x2_t*>(from + 96);
    held.a7 = *reinterpret_cast<const u32x2_t*>(from + 112);
  }
  template <int EPI>
  __device__ __forceinline__ void start(const StreamParams& p, const Slot& sl, int, int c0, int, int lane) {
    at = activation_row<EPI>(p, sl, lane & 15) + (int64_t)c0 * 128 + 4 * (lane >> 4);
    load_lo(at);
    load_hi(at);
  }
  template <int ODD, bool MORE2, bool MORE1>
  __device__ __forceinline__ void step(const Fp4Chunk& ch, int i, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3, const Slot&) {
    const uint16_t* next = at + (int64_t)(i + 1) * 128;
    fp4_half_tile(ch.w0.x, ch.w0.y, ch.s0.x, held.a0, held.a1, held.a2, held.a3, acc0);
    fp4_half_tile(ch.w1.x, ch.w1.y, ch.s0.z, held.a0, held.a1, held.a2, held.a3, acc1);
    fp4_half_tile(ch.w2.x, ch.w2.y, ch.s1.x, held.a0, held.a1, held.a2, held.a3, acc2);
    fp4_half_tile(ch.w3.x, ch.w3.y, ch.s1.z, held.a0, held.a1, held.a2, held.a3, acc3);
    if (MORE1) load_lo(next);
    fp4_half_tile(ch.w0.z, ch.w0.w, ch.s0.y, held.a4, held.a5, held.a6, held.a7, acc0);
    fp4_half_tile(ch.w1.z, ch.w1.w, ch.s0.w, held.a4, held.a5, held.a6, held.a7, acc1);
    fp4_half_tile(ch.w2.z, ch.w2.w, ch.s1.y, held.a4, held.a5, held.a6, held.a7, acc2);
    fp4_half_tile(ch.w3.z, ch.w3.w, ch.s1.w, held.a4, held.a5, held.a6, held.a7, acc3);
    if (MORE1) load_hi(next);
  }
};

// ---------------------------------------------------------------------------------------- slots of one to eight rows
//
// With at most eight rows in the slot the sixteen MFMA rows carry two 16-blocks at once: A row 8 p + i holds row i of
// the slot over the k of block 2 j + p only (zero over the other block's), so one v_mfma_f32_16x16x32_bf16 does the
// blocks 2 j and 2 j + 1 of a tile (one code dword: four conversions) and leaves block 2 j + p's partial sums in its
// output rows 8 p .. 8 p + 7. Half the MFMAs, scale conversions and folds of the sixteen-row body, and four 8-byte
// activation loads a chunk instead of eight. Lane (q, r16) ends up with block parity q / 2 of slot rows 4 (q % 2) ..
// + 3: the two parities are added across the lanes after the last chunk, which leaves the sixteen-row layout.
constexpr int FP4_FEW_ROWS = 8;

struct Fp4Pieces {  // the lane's four 8-byte pieces of a chunk, one per block pair
  u32x2_t p0, p1, p2, p3;
};

struct Fp4FewActs {
  static constexpr int LOADS = 4;
  Fp4Pieces even, odd;  // of the next even and the next odd chunk
  bool upper;           // this lane's A row belongs to the odd blocks (p = 1)
  uint32_t shift;       // 8 * (q / 2): where this lane's OUTPUT rows find their block's scale in a scale dword
  const uint16_t* at;   // the lane's piece of block pair 0 of the wavefront's first chunk
  __device__ __forceinline__ void load(Fp4Pieces& to, int i) const {
    const uint16_t* from = at + (int64_t)i * 128;
    to.p0 = *reinterpret_cast<const u32x2_t*>(from);
    to.p1 = *reinterpret_cast<const u32x2_t*>(from + 32);
    to.p2 = *reinterpret_cast<const u32x2_t*>(from + 64);
    to.p3 = *reinterpret_cast<const u32x2_t*>(from + 96);
  }
  template <int EPI>
  __device__ __forceinline__ void start(const StreamParams& p, const Slot& sl, int, int c0, int n, int lane) {
    const int q = lane >> 4, r16 = lane & 15;
    upper = r16 >= 8;
    shift = 8 * (q >> 1);
    at = activation_row<EPI>(p, sl, r16 & 7) + (int64_t)c0 * 128 + (upper ? 16 : 0) + 4 * q;
    load(even, 0);
    if (n > 1) load(odd, 1);
  }
  // MFMA j's A operand: the lane's piece in its own block's half, zero in the other
  __device__ __forceinline__ u32x4_t operand(const u32x2_t& piece) const {
    u32x4_t a;  // word by word: a select between two vectors built from the same piece is compiled through memory
    a.x = upper ? 0u : piece.x;
    a.y = upper ? 0u : piece.y;
    a.z = upper ? piece.x : 0u;
    a.w = upper ? piece.y : 0u;
    return a;
  }
  // One tile over one block pair: the pair's code dword, the scale dword holding its two scales in bytes BYTE, BYTE + 1.
  template <int BYTE>
  __device__ __forceinline__ void pair(uint32_t codes, uint32_t sc, const u32x4_t& a, f32x4_t& acc) const {
    u32x4_t b;
    b.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, 1.0f, 0));
    b.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, 1.0f, 1));
    b.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, 1.0f, 2));
    b.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, 1.0f, 3));
    const f32x4_t part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                                 f32x4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    const float s = __builtin_amdgcn_cvt_f32_fp8(sc >> shift, BYTE);  // the scale of block BYTE + q / 2 of the dword
    acc.x = fmaf(part.x, s, acc.x);
    acc.y = fmaf(part.y, s, acc.y);
    acc.z = fmaf(part.z, s, acc.z);
    acc.w = fmaf(part.w, s, acc.w);
  }
  __device__ __forceinline__ void tile(const u32x4_t& w, uint32_t sc_lo, uint32_t sc_hi, const u32x4_t& a0, const u32x4_t& a1, const u32x4_t& a2,
                                       const u32x4_t& a3, f32x4_t& acc) const {
    pair<0>(w.x, sc_lo, a0, acc);
    pair<2>(w.y, sc_lo, a1, acc);
    pair<0>(w.z, sc_hi, a2, acc);
    pair<2>(w.w, sc_hi, a3, acc);
  }
  template <int ODD, bool MORE2, bool MORE1>
  __device__ __forceinline__ void step(const Fp4Chunk& ch, int i, f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3, const Slot&) {
    Fp4Pieces& held = ODD ? odd : even;
    const u32x4_t a0 = operand(held.p0), a1 = operand(held.p1), a2 = operand(held.p2), a3 = operand(held.p3);
    tile(ch.w0, ch.s0.x, ch.s0.y, a0, a1, a2, a3, acc0);
    __builtin_amdgcn_sched_barrier(0);  // a tile at a time: interleaving the four costs more registers than there are
    tile(ch.w1, ch.s0.z, ch.s0.w, a0, a1, a2, a3, acc1);
    __builtin_amdgcn_sched_barrier(0);
    tile(ch.w2, ch.s1.x, ch.s1.y, a0, a1, a2, a3, acc2);
    __builtin_amdgcn_sched_barrier(0);
    tile(ch.w3, ch.s1.z, ch.s1.w, a0, a1, a2, a3, acc3);
    if (MORE2) load(held, i + 2);
  }
};

__device__ __forceinline__ void add_parities(f32x4_t& acc) {
  acc.x += __shfl_xor(acc.x, 32);
  acc.y += __shfl_xor(acc.y, 32);
  acc.z += __shfl_xor(acc.z, 32);
  acc.w += __shfl_xor(acc.w, 32);
}

// y = x Wq^T, dense or grouped by the expert plan: one wavefront per (64-row block, K range, slot of 16 activation rows),
// the same launch shape, slot table, weight ring, K-split exchange and epilogues as the W3 stream.
template <int EPI>
__device__ __forceinline__ void nvfp4_workgroup(const StreamParams& p, int slot, int bx, uint8_t* rings) {
  const Slot sl = slot_of<EPI>(p, slot);
  if (sl.rows <= 0) return;  // a slot the plan did not fill: the whole workgroup leaves
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same in every lane: kept in scalars
  if (wave >= p.ks * p.nbw) return;  // a launch shared with a matrix that takes more wavefronts a workgroup
  const WaveShare share = wave_share(p, wave);
  const int ks = share.ks, nbi = share.nbi, nb = bx * p.nbw + nbi;
  const bool active = nb < p.n_blocks;
  f32x4_t acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = acc0, acc2 = acc0, acc3 = acc0;
  if (active) {  // at least one chunk: the launch keeps ks <= chunks
    uint8_t* ring = rings + wave * FP4_RING_BYTES;
    if (sl.rows <= FP4_FEW_ROWS && !p.no_few) {  // uniform over the workgroup
      stream_block<EPI, Fp4FewActs, Fp4Ring>(p, sl, 0, nb, share.c0, share.c1, lane, ring, acc0, acc1, acc2, acc3);
      add_parities(acc0);  // lanes q = 0, 1 now hold slot rows 0 .. 7 as the epilogue expects them; q = 2, 3 stand for rows past the slot's end
      add_parities(acc1);
      add_parities(acc2);
      add_parities(acc3);
    } else {
      stream_block<EPI, Fp4Acts, Fp4Ring>(p, sl, 0, nb, share.c0, share.c1, lane, ring, acc0, acc1, acc2, acc3);
    }
  }
  finish_block<EPI, false, FP4_RING_BYTES / 4>(p, sl, RowScales{}, nb, active, ks, nbi, reinterpret_cast<float*>(rings), acc0, acc1, acc2, acc3);
}

template <int EPI>
__global__ __launch_bounds__(1024) void nvfp4_stream_kernel(StreamParams p) {
  extern __shared__ __align__(16) uint8_t rings[];
  nvfp4_workgroup<EPI>(p, blockIdx.y, blockIdx.x, rings);
}

// Two matrices of different geometry in one launch (the routed experts' layer beside the shared expert's, which reads
// other activations): the first `first` workgroups are (slot, block group) of the dense `b`, slot-major - every one of
// them has a whole K range to stream, so they start first - the rest of the planned `a`. Should the two shapes differ
// in wavefronts a workgroup, the smaller one's workgroups retire the wavefronts they do not use.
template <int EPI_A, int EPI_B>
__global__ __launch_bounds__(1024) void nvfp4_twin_kernel(StreamParams a, StreamParams b, int groups_a, int groups_b, int first) {
  extern __shared__ __align__(16) uint8_t rings[];
  int id = blockIdx.x;
  if (id < first) {
    const int slot = id / groups_b;
    nvfp4_workgroup<EPI_B>(b, slot, id - slot * groups_b, rings);
  } else {
    id -= first;
    const int slot = id / groups_a;
    nvfp4_workgroup<EPI_A>(a, slot, id - slot * groups_a, rings);
  }
}

// experiments (hb_tune): the stream's workgroup shape ("nvfp4_ksplit", "nvfp4_nbw"); "nvfp4_tile": 1 forces the tile kernel, 2 the stream
static std::atomic<int> g_nvfp4_ksplit{0}, g_nvfp4_nbw{0}, g_nvfp4_tile{0}, g_nvfp4_few{0}, g_nvfp4_tile_ks{0};  // "nvfp4_few": 2 switches off the body for slots of at most eight rows; "nvfp4_tile_ks": the workgroups that share a tile's K

static int shape_nvfp4(StreamParams& p, int64_t busy_slots) {
  pick_shape(p.n_blocks, p.chunks, busy_slots, 4096, &p.ks, &p.nbw);
  if (g_nvfp4_ksplit) {
    p.ks = g_nvfp4_ksplit;
    p.nbw = g_nvfp4_nbw ? g_nvfp4_nbw.load() : 1;
  }
  if (p.ks * p.nbw > 16 || p.ks > p.chunks || (p.ks & (p.ks - 1))) return HB_EINVAL;
  set_split(p);
  p.no_few = g_nvfp4_few == 2;
  return HB_OK;
}

template <int EPI>
static int launch_nvfp4(StreamParams& p, int64_t slots, int64_t busy_slots, hipStream_t stream) {
  if (int e = shape_nvfp4(p, busy_slots)) return e;
  const dim3 grid((unsigned)((p.n_blocks + p.nbw - 1) / p.nbw), (unsigned)slots);
  const int waves = p.ks * p.nbw;
  HB_LAUNCH(nvfp4_stream_kernel<EPI>, grid, dim3(64 * waves), (size_t)waves * FP4_RING_BYTES, stream, p);
  return HB_OK;
}

// `a` over its plan's slots beside the dense `b` in one launch (nvfp4_twin_kernel).
template <int EPI_A, int EPI_B>
static int launch_twin(StreamParams& a, int64_t slots_a, int64_t busy_a, StreamParams& b, int64_t slots_b, hipStream_t stream) {
  if (int e = shape_nvfp4(a, busy_a)) return e;
  if (int e = shape_nvfp4(b, slots_b)) return e;
  if (b.ks * b.nbw != a.ks * a.nbw) {  // one workgroup size (and LDS a workgroup) for both: the plan's matrix sets it
    const int waves = a.ks * a.nbw;
    b.ks = std::min(b.ks, waves);
    b.nbw = waves / b.ks;
    set_split(b);
  }
  const int groups_a = (a.n_blocks + a.nbw - 1) / a.nbw, groups_b = (b.n_blocks + b.nbw - 1) / b.nbw;
  const int64_t first = slots_b * groups_b, all = first + slots_a * groups_a;
  if (all > 0x7fffffff) return HB_EINVAL;
  const int waves = std::max(a.ks * a.nbw, b.ks * b.nbw);
  HB_LAUNCH((nvfp4_twin_kernel<EPI_A, EPI_B>), dim3((unsigned)all), dim3(64 * waves), (size_t)waves * FP4_RING_BYTES, stream, a, b, groups_a, groups_b, (int)first);
  return HB_OK;
}

// ------------------------------------------------------------------------------ the prefill kernel's NVFP4 format
__device__ __forceinline__ uint32_t scaled_pair(uint32_t codes, int byte, float scale) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  f32x2_t w;
  switch (byte) {  // the byte selector is an immediate of the instruction
    case 0: w = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes, 1.0f, 0); break;
    case 1: w = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes, 1.0f, 1); break;
    case 2: w = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes, 1.0f, 2); break;
    default: w = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(codes, 1.0f, 3); break;
  }
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_v;
  const bf16x2_v packed = {(__bf16)(w.x * scale), (__bf16)(w.y * scale)};
  return __builtin_bit_cast(uint32_t, packed);
}

struct TileNvfp4 {
  typedef Fp4Chunk Chunk;
  static constexpr int BLOCK_BYTES = NVFP4_BLOCK_BYTES;
  static constexpr bool SPLIT_A = true, PER_ROW = false;
  static __device__ __forceinline__ void load(Chunk& ch, const uint8_t* blk, int lane, int r16) { load_fp4_chunk(ch, blk, lane, r16); }
  // k-step s = blocks 2 s, 2 s + 1: dword s of the tile's codes (low half the even block), scale bytes 2 s, 2 s + 1 of
  // the tile's eight
  static __device__ __forceinline__ bf16x8_t fragment(const Chunk& ch, int nt, int s, const Slot&) {
    const u32x4_t w = nt == 0 ? ch.w0 : nt == 1 ? ch.w1 : nt == 2 ? ch.w2 : ch.w3;
    const u32x4_t sc4 = nt < 2 ? ch.s0 : ch.s1;
    const uint32_t sd = (nt & 1) ? (s < 2 ? sc4.z : sc4.w) : (s < 2 ? sc4.x : sc4.y);
    const float s_even = (s & 1) ? __builtin_amdgcn_cvt_f32_fp8(sd, 2) : __builtin_amdgcn_cvt_f32_fp8(sd, 0);
    const float s_odd = (s & 1) ? __builtin_amdgcn_cvt_f32_fp8(sd, 3) : __builtin_amdgcn_cvt_f32_fp8(sd, 1);
    const uint32_t codes = w[s];
    u32x4_t packed;
    packed.x = scaled_pair(codes, 0, s_even);
    packed.y = scaled_pair(codes, 1, s_even);
    packed.z = scaled_pair(codes, 2, s_odd);
    packed.w = scaled_pair(codes, 3, s_odd);
    return __builtin_bit_cast(bf16x8_t, packed);
  }
};

static inline unsigned grid_for(int64_t threads) { return (unsigned)((threads + 255) / 256); }

}  // namespace hb

using namespace hb;

static StreamParams dense_params(const void* tiled, float scale, int n, int k, const void* x, int m, void* y) {
  StreamParams p{};
  p.w = static_cast<const uint8_t*>(tiled);
  p.scalar = scale;
  p.n_blocks = n / 64;
  p.chunks = k / 128;
  p.a = static_cast<const uint16_t*>(x);
  p.a_stride = k;
  p.m = m;
  p.out = y;
  p.out_stride = n;
  return p;
}

extern "C" size_t hb_nvfp4_tiled_bytes(int64_t rows, int k) {
  if (rows <= 0 || k <= 0 || rows % 64 || k % 128) return 0;
  return (size_t)(rows / 64) * (size_t)(k / 128) * NVFP4_BLOCK_BYTES;
}

extern "C" int hb_nvfp4_repack(const uint8_t* weight, const uint8_t* scales, int swizzled, int64_t rows, int k, void* tiled, void* stream) {
  if (!weight || !scales || !tiled) return HB_ENULL;
  if (rows <= 0 || k <= 0 || rows % 64 || k % 128) return HB_EINVAL;
  const int chunks = k / 128;
  const int64_t blocks = rows / 64 * chunks;
  hipLaunchKernelGGL(nvfp4_repack_codes_kernel, dim3(grid_for(blocks * 256)), dim3(256), 0, as_stream(stream), weight, blocks, chunks,
                     static_cast<uint8_t*>(tiled));
  hipLaunchKernelGGL(nvfp4_repack_scales_kernel, dim3(grid_for(blocks * 512)), dim3(256), 0, as_stream(stream), scales, swizzled, blocks, chunks,
                     static_cast<uint8_t*>(tiled));
  return launch_status();
}

extern "C" int hb_nvfp4_dequant(const void* tiled, float global_scale, int64_t rows, int k, float* out, void* stream) {
  if (!tiled || !out) return HB_ENULL;
  if (rows <= 0 || k <= 0 || rows % 64 || k % 128) return HB_EINVAL;
  const int chunks = k / 128;
  const int64_t blocks = rows / 64 * chunks;
  hipLaunchKernelGGL(nvfp4_dequant_kernel, dim3(grid_for(blocks * 256)), dim3(256), 0, as_stream(stream), static_cast<const uint8_t*>(tiled),
                     global_scale, blocks, chunks, out);
  return launch_status();
}

// `workspace`: room for partial tiles (hb_nvfp4_gemm_workspace_bytes), or null: no call shares K among workgroups.
static int nvfp4_gemm(const void* x, int m, const void* tiled, float global_scale, int n, int k, int relu2, void* y, void* workspace, size_t workspace_bytes,
                      hipStream_t stream) {
  if (!x || !tiled || !y) return HB_ENULL;
  if (m <= 0 || n <= 0 || k <= 0 || n % 64 || k % 128) return HB_EINVAL;
  if (!aligned(x, 16) || !aligned(tiled, 16) || !aligned(y, 2) || !aligned(workspace, 16)) return HB_EINVAL;
  StreamParams p = dense_params(tiled, global_scale, n, k, x, m, y);
  // between the weight stream's sixteen rows a pass and a call that fills the device with 128-row tiles: tiles whose K
  // is shared among workgroups
  int ks = workspace && m > TILE_SPLIT_ROWS ? tile_split(m, p.n_blocks, p.chunks) : 1;
  if (g_nvfp4_tile_ks && workspace) ks = std::min(g_nvfp4_tile_ks.load(), p.chunks);
  if (tile_partial_bytes(m, p.n_blocks, ks) > workspace_bytes || tile_ticket_bytes(m, p.n_blocks) > HB_WORKSPACE_ZERO_BYTES) ks = 1;
  if (tile_takes(m, k) && tile_writes(y, false) && (g_nvfp4_tile == 1 || (g_nvfp4_tile == 0 && (ks > 1 || tile_serves_dense(m, p.n_blocks))))) {
    const int64_t tile_slots = (m + TILE_ROWS - 1) / TILE_ROWS;
    if (ks > 1) {
      p.tile_ks = ks;
      p.tile_mt = tile_partial_mt(m);
      p.tile_tickets = static_cast<uint32_t*>(workspace) + PLAN_HEADER;
      p.partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + tile_ticket_bytes(m, p.n_blocks));
    }
    if (int e = relu2 ? launch_tile<TileNvfp4, EPI_DENSE_RELU2>(p, tile_slots, m, stream) : launch_tile<TileNvfp4, EPI_DENSE>(p, tile_slots, m, stream)) return e;
    return launch_status();
  }
  const int64_t slots = (m + ROWS_PER_SLOT - 1) / ROWS_PER_SLOT;
  if (slots > 65535) return HB_EINVAL;
  if (int e = relu2 ? launch_nvfp4<EPI_DENSE_RELU2>(p, slots, slots, stream) : launch_nvfp4<EPI_DENSE>(p, slots, slots, stream)) return e;
  return launch_status();
}

extern "C" int hb_nvfp4_gemm(const void* x, int m, const void* tiled, float global_scale, int n, int k, int relu2, void* y, void* stream) {
  return nvfp4_gemm(x, m, tiled, global_scale, n, k, relu2, y, nullptr, 0, as_stream(stream));
}

extern "C" size_t hb_nvfp4_gemm_workspace_bytes(int m, int n, int k) {
  if (m <= TILE_SPLIT_ROWS || n <= 0 || k <= 0 || n % 64 || k % 128) return 0;
  const int want = g_nvfp4_tile_ks ? std::min(g_nvfp4_tile_ks.load(), k / 128) : tile_split(m, n / 64, k / 128);
  return tile_partial_bytes(m, n / 64, want);
}

extern "C" int hb_nvfp4_gemm_ws(const void* x, int m, const void* tiled, float global_scale, int n, int k, int relu2, void* y, void* workspace,
                                size_t workspace_bytes, void* stream) {
  return nvfp4_gemm(x, m, tiled, global_scale, n, k, relu2, y, workspace_bytes ? workspace : nullptr, workspace_bytes, as_stream(stream));
}

// ------------------------------------------------------------------------------------------------ routed experts
namespace {


int check_experts(const hb_nvfp4_experts* ex) {
  if (!ex) return HB_ENULL;
  if (!ex->fc1 || !ex->fc1_scale2 || !ex->fc2 || !ex->fc2_scale2) return HB_ENULL;
  if (ex->experts <= 0 || ex->hidden <= 0 || ex->inter <= 0 || ex->hidden_out <= 0) return HB_EINVAL;
  const int n1 = ex->gated ? 2 * ex->inter : ex->inter;
  if (ex->hidden % 128 || ex->inter % 128 || n1 % 64 || ex->hidden_out % 64) return HB_EINVAL;
  if (!aligned(ex->fc1, 16) || !aligned(ex->fc2, 16) || !aligned(ex->fc1_scale2, 4) || !aligned(ex->fc2_scale2, 4)) return HB_EINVAL;
  return HB_OK;
}

// The two launches' parameters of a routed call over a filled plan: fc1 from x into ws.h, fc2 from there into `out_pairs`.
void expert_params(const hb_nvfp4_experts* ex, const void* x, int m, int topk, const MoeWorkspace& ws, void* out_pairs, int pairs_bf16, StreamParams& p,
                   StreamParams& f2) {
  const int64_t pairs = (int64_t)m * topk;
  const int n1 = ex->gated ? 2 * ex->inter : ex->inter;
  p = StreamParams{};
  p.w = static_cast<const uint8_t*>(ex->fc1);
  p.expert_bytes = (int64_t)hb_nvfp4_tiled_bytes(n1, ex->hidden);
  p.scalars = ex->fc1_scale2;
  p.n_blocks = n1 / 64;
  p.chunks = ex->hidden / 128;
  p.a = static_cast<const uint16_t*>(x);
  p.a_stride = ex->hidden;
  p.plan = ws.plan;
  p.order = ws.order;
  p.topk = topk;
  p.pairs = (int)pairs;
  p.out = ws.h;
  p.out_stride = ex->inter;
  f2 = p;
  f2.w = static_cast<const uint8_t*>(ex->fc2);
  f2.expert_bytes = (int64_t)hb_nvfp4_tiled_bytes(ex->hidden_out, ex->inter);
  f2.scalars = ex->fc2_scale2;
  f2.n_blocks = ex->hidden_out / 64;
  f2.chunks = ex->inter / 128;
  f2.a = ws.h;
  f2.a_stride = ex->inter;
  f2.out = out_pairs;
  f2.out_stride = ex->hidden_out;
  f2.out_bf16 = pairs_bf16;
}

// the slots the stream's shape is chosen for: a call of few pairs fills about one slot a distinct expert
int64_t busy_slots(int64_t pairs, int experts, int64_t slots) { return pairs < 2 * experts ? (pairs + 1) / 2 : slots; }

// plan -> fc1 -> fc2: `out_pairs` receives fc2's per-pair outputs.
int run_experts(const hb_nvfp4_experts* ex, const void* x, const int32_t* ids, int m, int topk, const MoeWorkspace& ws, void* out_pairs,
                int pairs_bf16, hipStream_t stream) {
  const int64_t pairs = (int64_t)m * topk;
  // a dense contraction once an expert sees a few dozen rows: slots of 128 rows on the MFMA tile kernel; below that the
  // 16-row slots of the weight stream
  const bool dense = tile_takes(m, ex->hidden) && tile_takes(pairs, ex->inter) && tile_writes(out_pairs, !pairs_bf16) &&
                     (g_nvfp4_tile == 1 || (g_nvfp4_tile == 0 && pairs >= (int64_t)ex->experts * TILE_DENSE_ROWS));
  const int slot_rows = dense ? TILE_ROWS : ROWS_PER_SLOT;
  const int64_t slots = moe_max_slots(pairs, ex->experts, 0, slot_rows);
  if (slots > 65535) return HB_EINVAL;
  if (int e = moe_launch_plan(ids, pairs, ex->base, ex->experts, 0, ws, stream, slot_rows)) return e;
  const int64_t est = busy_slots(pairs, ex->experts, slots);
  StreamParams p, f2;
  expert_params(ex, x, m, topk, ws, out_pairs, pairs_bf16, p, f2);
  if (dense) {
    if (int e = ex->gated ? launch_tile<TileNvfp4, EPI_FC1_GATED>(p, slots, m, stream) : launch_tile<TileNvfp4, EPI_FC1_RELU2>(p, slots, m, stream)) return e;
    if (int e = launch_tile<TileNvfp4, EPI_FC2>(f2, slots, pairs, stream)) return e;
    return launch_status();
  }
  if (int e = ex->gated ? launch_nvfp4<EPI_FC1_GATED>(p, slots, est, stream) : launch_nvfp4<EPI_FC1_RELU2>(p, slots, est, stream)) return e;
  if (int e = launch_nvfp4<EPI_FC2>(f2, slots, est, stream)) return e;
  return launch_status();
}

// ------------------------------------------------------------------------------------- the small latent block
struct LatentWorkspace {
  MoeWorkspace moe;    // the routed experts' (absent without NVFP4 experts)
  uint16_t* routed;    // BF16 [m, latent]: the routed sum
  uint16_t* shared_h;  // BF16 [m, shared_inter]
  uint16_t* shared_y;  // BF16 [m, hidden]
  size_t bytes;
};

LatentWorkspace latent_carve(const hb_latent_weights* w, void* base, int m, int topk) {
  LatentWorkspace l{};
  size_t off = 0;
  if (w->routed) {
    l.moe = moe_carve(base, m, topk, w->routed->experts, w->routed->inter, w->routed->hidden_out, 0);
    off = l.moe.bytes;
  }
  auto take = [&](size_t bytes) {
    void* ptr = base ? static_cast<char*>(base) + off : nullptr;
    off += (bytes + 255) & ~(size_t)255;
    return static_cast<uint16_t*>(ptr);
  };
  l.routed = take((size_t)m * w->latent * 2);
  l.shared_h = take((size_t)m * w->shared_inter * 2);
  l.shared_y = take((size_t)m * w->hidden * 2);
  l.bytes = off;
  return l;
}

int check_latent(const hb_latent_weights* w, int m, int topk) {
  if (!w) return HB_ENULL;
  if (!w->gate_fc1 || !w->bias || !w->fc2) return HB_ENULL;
  if (m <= 0 || m > LATENT_MAX_ROWS || topk <= 0) return HB_EINVAL;
  if (w->experts_total <= 0 || w->latent <= 0 || w->hidden <= 0 || w->latent % 128 || w->hidden % 512) return HB_EINVAL;
  if (!aligned(w->gate_fc1, 16) || !aligned(w->fc2, 16) || !aligned(w->bias, 4)) return HB_EINVAL;
  if (w->routed) {
    if (int e = check_experts(w->routed)) return e;
    if (w->routed->hidden != w->latent || w->routed->hidden_out != w->latent || w->routed->base + w->routed->experts > w->experts_total) return HB_EINVAL;
  }
  if ((w->shared_up != nullptr) != (w->shared_down != nullptr)) return HB_ENULL;
  if (w->shared_up && (w->shared_inter <= 0 || w->shared_inter % 128 || w->hidden % 128 || !aligned(w->shared_up, 16) || !aligned(w->shared_down, 16)))
    return HB_EINVAL;
  return HB_OK;
}

}  // namespace

int hb::nvfp4_tune(const char* key, int value) {
  std::atomic<int>* slot = !strcmp(key, "nvfp4_tile") ? &g_nvfp4_tile : !strcmp(key, "nvfp4_ksplit") ? &g_nvfp4_ksplit : !strcmp(key, "nvfp4_nbw") ? &g_nvfp4_nbw
              : !strcmp(key, "nvfp4_few") ? &g_nvfp4_few : !strcmp(key, "nvfp4_tile_ks") ? &g_nvfp4_tile_ks : nullptr;
  if (!slot || value < 0 || value > 16) return HB_EINVAL;
  *slot = value;
  return HB_OK;
}

extern "C" size_t hb_nvfp4_moe_workspace_bytes(int m, int topk, const hb_nvfp4_experts* routed) {
  if (!routed || m <= 0 || topk <= 0 || check_experts(routed) != HB_OK) return 0;
  return moe_carve(nullptr, m, topk, routed->experts, routed->inter, routed->hidden_out, 0).bytes;
}

extern "C" int hb_nvfp4_moe(const hb_nvfp4_experts* routed, const void* x, const int32_t* ids, const float* weights, int m, int topk, int mode,
                            void* out, void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_experts(routed)) return e;
  if (!x || !ids || !weights || !out || !workspace) return HB_ENULL;
  if (m <= 0 || topk <= 0 || mode < HB_MOE_SUM || mode > HB_MOE_PAIRS_BF16) return HB_EINVAL;
  if (!aligned(x, 16) || !aligned(ids, 4) || !aligned(weights, 4) || !aligned(out, 8) || !aligned(workspace, 16)) return HB_EINVAL;
  const MoeWorkspace ws = moe_carve(workspace, m, topk, routed->experts, routed->inter, routed->hidden_out, 0);
  if (workspace_bytes < ws.bytes) return HB_EWORKSPACE;
  const bool sum = mode == HB_MOE_SUM;
  void* pairs_out = sum ? static_cast<void*>(ws.y) : out;
  // a summed prefill-sized call keeps its pair outputs in BF16: half the traffic of its widest tensor, as the reference's
  // layer does from the same size (hibana/model/flashnext/moe.py:186)
  const bool narrow = sum && m >= MOE_WIDE_ROWS;
  if (int e = run_experts(routed, x, ids, m, topk, ws, pairs_out, mode == HB_MOE_PAIRS_BF16 || narrow, as_stream(stream))) return e;
  if (sum) {
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
    moe_launch_combine(c, as_stream(stream));
  }
  return launch_status();
}

extern "C" size_t hb_latent_workspace_bytes(const hb_latent_weights* w, int m, int topk) {
  if (check_latent(w, m, topk) != HB_OK) return 0;
  return latent_carve(w, nullptr, m, topk).bytes;
}

extern "C" int hb_latent_router(const hb_latent_weights* w, const void* x, int m, int topk, const int32_t* slots, int steps, int route, int pad_id,
                                float* fused, int32_t* ids, float* weights, void* lat, void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_latent(w, m, topk)) return e;
  if (!x || !fused || !lat || !workspace || (route && (!ids || !weights))) return HB_ENULL;
  if (!aligned(x, 16) || !aligned(fused, 4) || !aligned(ids, 4) || !aligned(weights, 4) || !aligned(lat, 2) || !aligned(slots, 4) || !aligned(workspace, 16))
    return HB_EINVAL;
  if (pad_id > w->experts_total) return HB_EINVAL;
  const LatentWorkspace l = latent_carve(w, workspace, m, topk);
  if (workspace_bytes < l.bytes) return HB_EWORKSPACE;
  LatentRouter r{};
  r.w = static_cast<const uint16_t*>(w->gate_fc1);
  r.bias = w->bias;
  r.x = static_cast<const uint16_t*>(x);
  r.slots = slots;
  r.m = m;
  r.experts = w->experts_total;
  r.latent = w->latent;
  r.hidden = w->hidden;
  r.topk = topk;
  r.steps = steps;
  r.route = route != 0;
  r.pad_id = pad_id;
  r.fused = fused;
  r.ids = ids;
  r.weights = weights;
  r.lat = static_cast<uint16_t*>(lat);
  if (w->routed) {
    r.e_lo = w->routed->base;
    r.e_n = w->routed->experts;
    r.ws = &l.moe;
  }
  if (int e = latent_launch_router(r, as_stream(stream))) return e;
  return launch_status();
}

extern "C" int hb_latent_shared_up(const hb_latent_weights* w, const void* x, int m, int topk, void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_latent(w, m, topk)) return e;
  if (!x || !workspace || !w->shared_up) return HB_ENULL;
  if (!aligned(x, 16) || !aligned(workspace, 16)) return HB_EINVAL;
  const LatentWorkspace l = latent_carve(w, workspace, m, topk);
  if (workspace_bytes < l.bytes) return HB_EWORKSPACE;
  StreamParams up = dense_params(w->shared_up, w->shared_up_scale, w->shared_inter, w->hidden, x, m, l.shared_h);
  if (int e = launch_nvfp4<EPI_DENSE_RELU2>(up, 1, 1, as_stream(stream))) return e;
  return launch_status();
}

extern "C" int hb_latent_out(const hb_latent_weights* w, const void* routed, int m, int topk, void* out, void* workspace, size_t workspace_bytes,
                             void* stream) {
  if (int e = check_latent(w, m, topk)) return e;
  if (!routed || !out || !workspace) return HB_ENULL;
  if (!aligned(routed, 16) || !aligned(out, 2) || !aligned(workspace, 16)) return HB_EINVAL;
  const LatentWorkspace l = latent_carve(w, workspace, m, topk);
  if (workspace_bytes < l.bytes) return HB_EWORKSPACE;
  if (w->shared_up) {  // the shared expert's down projection of what hb_latent_shared_up left
    StreamParams down = dense_params(w->shared_down, w->shared_down_scale, w->hidden, w->shared_inter, l.shared_h, m, l.shared_y);
    if (int e = launch_nvfp4<EPI_DENSE>(down, 1, 1, as_stream(stream))) return e;
  }
  if (int e = latent_launch_out(static_cast<const uint16_t*>(w->fc2), static_cast<const uint16_t*>(routed), w->shared_up ? l.shared_y : nullptr,
                                static_cast<uint16_t*>(out), m, w->hidden, w->latent, as_stream(stream)))
    return e;
  return launch_status();
}

extern "C" int hb_latent_block(const hb_latent_weights* w, const void* x, const void* lat, const int32_t* ids, const float* weights, int m, int topk,
                               int plan, void* out, void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_latent(w, m, topk)) return e;
  if (!w->routed) return HB_ENULL;
  if (!x || !lat || !ids || !weights || !out || !workspace) return HB_ENULL;
  if (!aligned(x, 16) || !aligned(lat, 16) || !aligned(ids, 4) || !aligned(weights, 4) || !aligned(out, 2) || !aligned(workspace, 16)) return HB_EINVAL;
  const LatentWorkspace l = latent_carve(w, workspace, m, topk);
  if (workspace_bytes < l.bytes) return HB_EWORKSPACE;
  const hb_nvfp4_experts* ex = w->routed;
  hipStream_t s = as_stream(stream);
  const int64_t pairs = (int64_t)m * topk, slots = moe_max_slots(pairs, ex->experts, 0, ROWS_PER_SLOT), est = busy_slots(pairs, ex->experts, slots);
  if (plan)
    if (int e = moe_launch_plan(ids, pairs, ex->base, ex->experts, 0, l.moe, s)) return e;
  StreamParams fc1, fc2;
  expert_params(ex, lat, m, topk, l.moe, l.moe.y, 0, fc1, fc2);
  if (w->shared_up) {
    StreamParams up = dense_params(w->shared_up, w->shared_up_scale, w->shared_inter, w->hidden, x, m, l.shared_h);
    StreamParams down = dense_params(w->shared_down, w->shared_down_scale, w->hidden, w->shared_inter, l.shared_h, m, l.shared_y);
    if (int e = ex->gated ? launch_twin<EPI_FC1_GATED, EPI_DENSE_RELU2>(fc1, slots, est, up, 1, s) : launch_twin<EPI_FC1_RELU2, EPI_DENSE_RELU2>(fc1, slots, est, up, 1, s))
      return e;
    if (int e = launch_twin<EPI_FC2, EPI_DENSE>(fc2, slots, est, down, 1, s)) return e;
  } else {
    if (int e = ex->gated ? launch_nvfp4<EPI_FC1_GATED>(fc1, slots, est, s) : launch_nvfp4<EPI_FC1_RELU2>(fc1, slots, est, s)) return e;
    if (int e = launch_nvfp4<EPI_FC2>(fc2, slots, est, s)) return e;
  }
  CombineParams c{};
  c.pairs = l.moe.y;
  c.ids = ids;
  c.weights = weights;
  c.e_lo = ex->base;
  c.e_n = ex->experts;
  c.m = m;
  c.topk = topk;
  c.h = w->latent;
  c.out = l.routed;
  moe_launch_combine(c, s);
  if (int e = latent_launch_out(static_cast<const uint16_t*>(w->fc2), l.routed, w->shared_up ? l.shared_y : nullptr, static_cast<uint16_t*>(out), m, w->hidden,
                                w->latent, s))
    return e;
  return launch_status();
}
