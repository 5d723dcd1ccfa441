// W3 tile layout for gfx950: the unit a wavefront streams is a block of 64 output rows x 128 k.
//
//   block (nb, c) of a [rows, K] matrix starts at byte ((nb * K/128 + c) * W3_BLOCK_BYTES), nb = row / 64, c = k / 128.
//   bytes    0..3071  codes: three 128-bit loads per lane, load v of lane l at (v * 64 + l) * 16. Lane l = 16 q + r
//                     owns, for each of the four 16-row tiles nt of the block, the 32 weights
//                         row 64 nb + 16 nt + r,   k = 128 c + 32 j + 8 q + i   (j = 0..3, i = 0..7),
//                     which is exactly the B operand of four v_mfma_f32_16x16x32_bf16 (one per 32-group j).
//                     The lane's twelve dwords D[4 v + e] hold tile nt in Q0 = D[3 nt], Q1 = D[3 nt + 1], Q2 = D[3 nt + 2].
//                     "Selector" s = 2 j + i / 4 is a dword whose byte i % 4 is the code of weight (j, i):
//                         s0 = Q0 & 0x07070707        s1 = (Q0 >> 3) & 0x07070707
//                         s2 = Q1 & 0x07070707        s3 = (Q1 >> 3) & 0x07070707
//                         s4 = Q2 & 0x07070707        s5 = (Q2 >> 3) & 0x07070707
//                         s6 = ((Q0 >> 6) & 0x03030303) | ((Q2 >> 4) & 0x04040404)
//                         s7 = ((Q1 >> 6) & 0x03030303) | ((Q2 >> 5) & 0x04040404)
//                     so a selector feeds v_perm_b32 over the 8-byte E4M3 codebook directly.
//   bytes 3072..3327  scales: 16 B per row-in-tile r at 3072 + 16 r: byte 4 nt + j is the E4M3 scale of row
//                     64 nb + 16 nt + r, 32-group 4 c + j.
//
// The same density as the reference layout (3 bits + 1/4 bit per weight); the FP32 row scales stay a separate array.
//
// Two-bit matrices (four-level codebooks: the reference's two-plane variant, hibana/kernels/w3.py:12-19,89-91) have a
// tile layout of their own at their own density (2 + 1/4 bits a weight): blocks of 2304 bytes,
//   bytes    0..2047  codes: two 128-bit loads per lane; the lane's eight dwords hold tile nt in Q0 = D[2 nt],
//                     Q1 = D[2 nt + 1], four 2-bit codes a byte: selector s = 2 j + i / 4 (byte i % 4 = weight (j, i)) is
//                         s0 = Q0 & 0x03030303, s1 = (Q0 >> 2) & 0x03030303, s2 = (Q0 >> 4) & .., s3 = (Q0 >> 6) & ..,
//                         s4 .. s7 the same of Q1;
//   bytes 2048..2303  scales, as above.
// The kernels that take either layout are told the `bits` of the tiles (3 or 2).
#pragma once

#include <stdint.h>

namespace hb {

constexpr int W3_BLOCK_ROWS = 64;
constexpr int W3_CHUNK = 128;
constexpr int W3_BLOCK_BYTES = 3328;
constexpr int W3_SCALE_OFFSET = 3072;

constexpr int W2_BLOCK_BYTES = 2304;
constexpr int W2_SCALE_OFFSET = 2048;
__host__ __device__ constexpr int w3_block_bytes(int bits) { return bits == 2 ? W2_BLOCK_BYTES : W3_BLOCK_BYTES; }
__host__ __device__ constexpr int w3_scale_base(int bits) { return bits == 2 ? W2_SCALE_OFFSET : W3_SCALE_OFFSET; }

// Two-bit tiles: where bit b (0..1) of weight (tile nt, group j, element i) of a lane sits among the lane's eight dwords.
__host__ __device__ inline void w2_bit_slot(int nt, int j, int i, int b, int* dword, int* pos) {
  const int s = 2 * j + (i >> 2), byte = i & 3;
  *dword = 2 * nt + (s >> 2);
  *pos = 8 * byte + 2 * (s & 3) + b;
}

// The eight selectors of one two-bit tile from its two dwords.
__host__ __device__ inline void w2_selectors(uint32_t q0, uint32_t q1, uint32_t sel[8]) {
  sel[0] = q0 & 0x03030303u;
  sel[1] = (q0 >> 2) & 0x03030303u;
  sel[2] = (q0 >> 4) & 0x03030303u;
  sel[3] = (q0 >> 6) & 0x03030303u;
  sel[4] = q1 & 0x03030303u;
  sel[5] = (q1 >> 2) & 0x03030303u;
  sel[6] = (q1 >> 4) & 0x03030303u;
  sel[7] = (q1 >> 6) & 0x03030303u;
}

// Where the three bits of weight (tile nt, group j, element i) of a lane sit among the lane's twelve dwords.
// Returns for bit b (0..2) the dword index and the bit position.
__host__ __device__ inline void w3_bit_slot(int nt, int j, int i, int b, int* dword, int* pos) {
  const int s = 2 * j + (i >> 2), byte = i & 3;
  if (s < 6) {
    *dword = 3 * nt + (s >> 1);
    *pos = 8 * byte + 3 * (s & 1) + b;
  } else if (b < 2) {
    *dword = 3 * nt + (s - 6);  // s6 -> Q0, s7 -> Q1
    *pos = 8 * byte + 6 + b;
  } else {
    *dword = 3 * nt + 2;
    *pos = 8 * byte + 6 + (s - 6);
  }
}

// Byte offset of dword d of lane l inside a block.
__host__ __device__ inline int w3_dword_offset(int lane, int d) { return ((d >> 2) * 64 + lane) * 16 + (d & 3) * 4; }

// Byte offset of the scale of (tile nt, row-in-tile r, group j) inside a block.
__host__ __device__ inline int w3_scale_offset(int nt, int r, int j) { return W3_SCALE_OFFSET + 16 * r + 4 * nt + j; }

// The eight selectors of one tile from its three dwords.
__host__ __device__ inline void w3_selectors(uint32_t q0, uint32_t q1, uint32_t q2, uint32_t sel[8]) {
  sel[0] = q0 & 0x07070707u;
  sel[1] = (q0 >> 3) & 0x07070707u;
  sel[2] = q1 & 0x07070707u;
  sel[3] = (q1 >> 3) & 0x07070707u;
  sel[4] = q2 & 0x07070707u;
  sel[5] = (q2 >> 3) & 0x07070707u;
  sel[6] = ((q0 >> 6) & 0x03030303u) | ((q2 >> 4) & 0x04040404u);
  sel[7] = ((q1 >> 6) & 0x03030303u) | ((q2 >> 5) & 0x04040404u);
}

// Reference (checkpoint) layout: bit b of code[n, k] (hibana/kernels/w3.py:12-19,178-191 of the reference).
// Returns the flat uint32 index into planes [rows/32, K/128, bits, 32, 4] and the bit position.
__host__ __device__ inline void w3_ref_bit_slot(int64_t n, int k, int b, int bits, int chunks, int64_t* word, int* pos) {
  const int64_t nb = n >> 5;
  const int nt = (int)(n & 31) >> 3, g = (int)(n & 7);
  const int kc = k >> 7, s = (k & 127) >> 4, t = (k & 15) >> 2, j = k & 3;
  const int w = bits * nt + b;
  *word = (((nb * chunks + kc) * bits + (w >> 2)) * 32 + (4 * g + t)) * 4 + (w & 3);
  *pos = (4 * j + b + 16 * (s >> 2) + (s & 3)) & 31;
}

// Reference layout: flat byte index of the scale of row n, 32-group grp into scales [rows/32, K/128, 4, 32].
__host__ __device__ inline int64_t w3_ref_scale_slot(int64_t n, int grp, int chunks) {
  const int64_t nb = n >> 5;
  const int nt = (int)(n & 31) >> 3;
  return ((nb * chunks + (grp >> 2)) * 4 + ((n & 7) >> 1)) * 32 + (4 * nt + (grp & 3)) * 2 + (n & 1);
}

}  // namespace hb
