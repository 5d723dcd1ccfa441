// The prefill-size kernel of the routed experts and the dense linears, shared by the weight formats.
//
// When an expert (or a dense call) has many activation rows the product is a dense contraction and belongs on the MFMA
// pipe: one workgroup of four wavefronts takes a slot of up to 128 activation rows and four neighbouring 64-row weight
// blocks (one a wavefront), all of K. Per 128-k chunk
//   - the slot's activation tile (128 rows x 128 k BF16, 32 KB) is brought into LDS by LDS-direct loads
//     (global_load_lds_dwordx4: no registers in between), double buffered, the sixteen 16-byte pieces of a row
//     XOR-swizzled by the row so that the A fragment reads of sixteen rows hit sixteen different bank groups;
//   - each wavefront expands its block's codes ONCE to scaled BF16 (code value x block / group scale: exact in BF16 for
//     both formats) and reuses the four B fragments for every 16-row tile of the slot: v_mfma_f32_16x16x32_bf16,
//     accumulators for 8 x 4 tiles in registers; the FP32 matrix / row scale is applied in the epilogue.
//
// A format provides: Chunk (the registers of one 64-row x 128-k block), BLOCK_BYTES, load(), fragment() (the scaled B
// operand of 16-row tile nt and 32-k step s), SPLIT_A (how the lane's eight k of a step lie: NVFP4's tile layout gives
// lane q the k 4q..4q+3 of both 16-blocks of the step, so its A fragment is two 8-byte reads; W3's gives it 8q..8q+7),
// and PER_ROW (FP32 scale per output row, else one per matrix).
#pragma once

#include <algorithm>
#include <atomic>

#include "stream_common.hpp"

namespace hb {

constexpr int TILE_ROWS = 128;
constexpr int TILE_MT = TILE_ROWS / 16;
// A 16-row tile of an activation buffer is 4 KB and 16 bytes of padding: with the tiles a multiple of 512 bytes apart
// the compiler pairs the 8-byte reads of neighbouring tiles into one instruction and then moves registers to put a
// fragment's two halves side by side (a quarter of the loop's VALU instructions); off that grid every half is its own
// read, straight into its place.
constexpr int TILE_PITCH = 16 * 256 + 16;
constexpr int TILE_BUF = TILE_MT * TILE_PITCH;  // bytes of one activation buffer
constexpr int TILE_DENSE_ROWS = 24;        // average rows an expert from which the tile kernel serves a routed call
typedef __attribute__((ext_vector_type(2))) uint32_t tile_u32x2_t;

// Brings chunk `chunk` of the slot's activation tile into `buf`: a wavefront takes rows wave * 32 .. + 31 in eight
// instructions of four rows each; lane l lands at byte 16 l of the instruction's kilobyte, i.e. row (l >> 4), slot
// (l & 15) of it, and therefore fetches piece slot ^ (row & 15) of its row. `piece[j]`: that piece's byte offset from
// the activation matrix's start for chunk 0 (32 bits: the launch refuses matrices of 4 GiB and more); the chunk moves
// the scalar base, so a chunk's staging is eight loads and no arithmetic.
__device__ __forceinline__ void stage_tile(const StreamParams& p, const uint32_t (&piece)[8], uint8_t* buf, int chunk, int tiles, int wave) {
  const uint8_t* base = reinterpret_cast<const uint8_t*>(p.a) + (int64_t)chunk * 256;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    if (wave * 32 + j * 4 < tiles * 16) {  // wave-uniform: whole 16-row tiles past the slot's rows are never read
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base + piece[j]),
                                       (__attribute__((address_space(3))) void*)(buf + (wave * 2 + (j >> 2)) * TILE_PITCH + (j & 3) * 1024), 16, 0, 0);
    }
  }
}

// ST: the slot's number of 16-row tiles when it is a compile-time constant (no test around a tile's MFMAs, so every
// accumulator stays in place from chunk to chunk), or 0 for any count.
//
// K shared among workgroups (p.tile_ks > 1, dense calls of a few dozen rows, which alone would fill too few compute
// units): workgroup z of a tile takes chunks c0 .. c1 - 1, leaves its unscaled FP32 accumulators in `p.partial`
// (stores written through to memory and waited for: a release at device scope, which writes back the whole L2, costs
// each workgroup tens of microseconds here), counts itself on the tile's arrival counter, and the one that arrives
// last (an acquire, then ordinary loads) adds all the partial tiles in the order of z - the same sum whichever it is -
// and runs the epilogue. The counters (p.tile_tickets, one a tile) lie at the head of the caller's workspace, ahead of
// the partial tiles: zero when the caller hands the workspace over, put back to zero by every last arriver, so calls in
// flight together on workspaces of their own share nothing.

__device__ __forceinline__ void store_through16(f32x4_t* at, const f32x4_t& v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(at), "v"(v) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_but(void) { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

template <class Fmt, int EPI, int ST>
__device__ __forceinline__ void tile_slot(const StreamParams& p, const Slot& sl, uint8_t* tile_lds, int c0, int c1, int z) {
  constexpr bool FULL = ST > 0;
  constexpr int MT = FULL ? ST : TILE_MT;
  constexpr int BUFS = 2, BUF = TILE_BUF;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same in every lane: kept in scalars
  const int q = lane >> 4, r16 = lane & 15;
  const int nb = blockIdx.x * 4 + wave;
  const bool active = nb < p.n_blocks;
  const int tiles = FULL ? ST : (sl.rows + 15) >> 4;
  int32_t* rowtab = reinterpret_cast<int32_t*>(tile_lds + BUFS * BUF);
  if (threadIdx.x < TILE_ROWS) {  // the source row of each slot row (rows past the last repeat it)
    int64_t arow = sl.p0 + min((int)threadIdx.x, sl.rows - 1);
    if (epi_gathers(EPI)) {
      const int pair = p.order[arow];
      arow = pair < p.pairs ? pair / p.topk : pair - p.pairs;
    }
    rowtab[threadIdx.x] = (int)arow;
  }
  __syncthreads();
  uint32_t piece[8];
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const int row = wave * 32 + j * 4 + (lane >> 4);
    piece[j] = (uint32_t)rowtab[row] * (uint32_t)(p.a_stride * 2) + (uint32_t)((((lane & 15) ^ (row & 15))) << 4);
  }
  f32x4_t acc[MT][4];
#pragma unroll
  for (int t = 0; t < MT; t++)
#pragma unroll
    for (int nt = 0; nt < 4; nt++) acc[t][nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const uint8_t* blk = sl.w + (int64_t)(active ? nb : 0) * p.chunks * Fmt::BLOCK_BYTES;
  // One chunk: the products of the chunk's four 32-k steps from its weights `w` and its activation buffer.
  auto multiply = [&](const typename Fmt::Chunk& w, const uint8_t* buf) {
#pragma unroll
    for (int s = 0; s < 4; s++) {  // 32-k steps of the chunk
      bf16x8_t b[4];
#pragma unroll
      for (int nt = 0; nt < 4; nt++) b[nt] = Fmt::fragment(w, nt, s, sl);
      // lane (q, r16) of tile t: row 16 t + r16; its eight k of the step as the format's tile layout owns them
      const int half = (q & 1) << 3;
      const int slot_lo = ((4 * s + (q >> 1)) ^ r16) << 4, slot_hi = ((4 * s + 2 + (q >> 1)) ^ r16) << 4;
      const int slot_one = ((4 * s + q) ^ r16) << 4;
#pragma unroll
      for (int t = 0; t < MT; t++) {
        if (FULL || t < tiles) {
          const uint8_t* row = buf + t * TILE_PITCH + r16 * 256;
          u32x4_t a;
          if (Fmt::SPLIT_A) {
            const tile_u32x2_t lo = *reinterpret_cast<const tile_u32x2_t*>(row + half + slot_lo);
            const tile_u32x2_t hi = *reinterpret_cast<const tile_u32x2_t*>(row + half + slot_hi);
            a = u32x4_t{lo.x, lo.y, hi.x, hi.y};
          } else {
            a = *reinterpret_cast<const u32x4_t*>(row + slot_one);
          }
          const bf16x8_t af = __builtin_bit_cast(bf16x8_t, a);
#pragma unroll
          for (int nt = 0; nt < 4; nt++) acc[t][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[nt], af, acc[t][nt], 0, 0, 0);
        }
      }
    }
  };
  auto request = [&](typename Fmt::Chunk& w, uint8_t* buf, int c) {  // a chunk's weights and this wavefront's share of its activation rows
    Fmt::load(w, blk + (int64_t)c * Fmt::BLOCK_BYTES, lane, r16);
    stage_tile(p, piece, buf, c, tiles, wave);
  };
  typename Fmt::Chunk cur, nxt;
  request(cur, tile_lds, c0);
  wait_but<0>();
  __syncthreads();
  for (int c = c0; c < c1; c++) {
    uint8_t* buf = tile_lds + ((c - c0) & 1) * BUF;
    if (c + 1 < c1) request(nxt, tile_lds + ((c - c0 + 1) & 1) * BUF, c + 1);
    multiply(cur, buf);
    cur = nxt;
    wait_but<0>();    // this wavefront's LDS-direct loads have landed before it signals
    __syncthreads();  // the next buffer is complete and this one is free to refill
  }
  if (p.tile_ks > 1) {
    const int64_t region = (int64_t)p.tile_mt * 4 * 64;  // f32x4 a wavefront
    const int64_t tile = (int64_t)blockIdx.y * gridDim.x + blockIdx.x;
    f32x4_t* mine = reinterpret_cast<f32x4_t*>(p.partial) + ((tile * p.tile_ks + z) * 4 + wave) * region + lane;
    if (active) {
#pragma unroll
      for (int t = 0; t < MT; t++)
        if (FULL || t < tiles)
#pragma unroll
          for (int nt = 0; nt < 4; nt++) store_through16(mine + (t * 4 + nt) * 64, acc[t][nt]);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the partial tile is in memory before the count
    __syncthreads();
    int* last = reinterpret_cast<int*>(rowtab);  // the row table has served
    if (threadIdx.x == 0) {
      unsigned int* ticket = p.tile_tickets + tile;
      const unsigned drawn = atomicAdd(ticket, 1u);
      *last = drawn == (unsigned)p.tile_ks - 1u;
      if (*last) *ticket = 0u;
    }
    __syncthreads();
    if (!*last || !active) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");  // drop what this compute die's L2 holds of the others' regions
    const f32x4_t* all = reinterpret_cast<const f32x4_t*>(p.partial) + (tile * p.tile_ks * 4 + wave) * region + lane;
#pragma unroll
    for (int t = 0; t < MT; t++)
      if (FULL || t < tiles)
#pragma unroll
        for (int nt = 0; nt < 4; nt++) {
          f32x4_t sum = all[(t * 4 + nt) * 64];
          for (int k = 1; k < p.tile_ks; k++) sum += all[(int64_t)k * 4 * region + (t * 4 + nt) * 64];
          acc[t][nt] = sum;
        }
  }
  if (!active) return;
  // The weights are the MFMA's A operand and the activations its B: accumulator register r of lane (q, r16) of tile
  // (t, nt) is slot row 16 t + r16, weight row nb * 64 + 16 nt + 4 q + r - four neighbouring output columns a lane, one
  // store of 8 (BF16) or 16 bytes (FP32) for them.
  const int i16 = r16;
#pragma unroll
  for (int t = 0; t < MT; t++) {
    if (FULL || t < tiles) {
      const int i = 16 * t + i16;
      if (i < sl.rows) {
        const int64_t pos = sl.p0 + i;
        if (EPI == EPI_FC1_GATED) {
#pragma unroll
          for (int g = 0; g < 2; g++) {
            float h[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
              const float su = Fmt::PER_ROW ? sl.rs[nb * 64 + 32 * g + 4 * q + r] : sl.scalar, sg = Fmt::PER_ROW ? sl.rs[nb * 64 + 32 * g + 16 + 4 * q + r] : sl.scalar;
              const uint32_t ug = bf16_pair(acc[t][2 * g][r] * su, acc[t][2 * g + 1][r] * sg);  // up and gate rounded to BF16 ...
              h[r] = silu(pair_hi(ug)) * pair_lo(ug);                                          // ... and their product, rounded below
            }
            *reinterpret_cast<tile_u32x2_t*>(reinterpret_cast<uint16_t*>(p.out) + pos * p.out_stride + nb * 32 + 16 * g + 4 * q) =
                tile_u32x2_t{bf16_pair(h[0], h[1]), bf16_pair(h[2], h[3])};
          }
        } else {
          const int64_t at = (EPI == EPI_FC2 ? (int64_t)p.order[pos] : pos) * p.out_stride + nb * 64 + 4 * q;
#pragma unroll
          for (int nt = 0; nt < 4; nt++) {
            float y[4];
#pragma unroll
            for (int r = 0; r < 4; r++) y[r] = acc[t][nt][r] * (Fmt::PER_ROW ? sl.rs[nb * 64 + 16 * nt + 4 * q + r] : sl.scalar);
            if (EPI == EPI_FC1_RELU2 || EPI == EPI_DENSE_RELU2) {  // bf16(relu(bf16(y))^2), two values a conversion
              const uint32_t u01 = bf16_pair(y[0], y[1]), u23 = bf16_pair(y[2], y[3]);
              // relu on the bits: a negative value (and -0) is a negative integer; a NaN stays one, as torch's relu leaves it
              const float h0 = __int_as_float(max((int)(u01 << 16), 0)), h1 = __int_as_float(max((int)(u01 & 0xffff0000u), 0));
              const float h2 = __int_as_float(max((int)(u23 << 16), 0)), h3 = __int_as_float(max((int)(u23 & 0xffff0000u), 0));
              y[0] = h0 * h0;
              y[1] = h1 * h1;
              y[2] = h2 * h2;
              y[3] = h3 * h3;
            }
            if (EPI == EPI_FC1_RELU2 || EPI == EPI_DENSE_RELU2 || EPI == EPI_DENSE || p.out_bf16) {
              *reinterpret_cast<tile_u32x2_t*>(reinterpret_cast<uint16_t*>(p.out) + at + 16 * nt) = tile_u32x2_t{bf16_pair(y[0], y[1]), bf16_pair(y[2], y[3])};
            } else {
              *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(p.out) + at + 16 * nt) = f32x4_t{y[0], y[1], y[2], y[3]};
            }
          }
        }
      }
    }
  }
}

template <class Fmt, int EPI>
__global__ __launch_bounds__(256, 2) void tile_kernel(StreamParams p) {
  extern __shared__ __align__(16) uint8_t tile_lds[];  // two activation buffers, then the row table
  const Slot sl = slot_of<EPI>(p, blockIdx.y);
  if (sl.rows <= 0) return;  // a slot the plan did not fill: the whole workgroup leaves
  // uniform over the workgroup; more compile-time counts than the full slot were tried: with a third body the
  // compiler spills and every one of them gets slower
  // blockIdx.z shares K: the first chunks % tile_ks of them take one chunk more
  const int ks = p.tile_ks > 1 ? p.tile_ks : 1, z = blockIdx.z, base = p.chunks / ks, rem = p.chunks - base * ks;
  const int c0 = z * base + min(z, rem), c1 = c0 + base + (z < rem ? 1 : 0);
  if (sl.rows > TILE_ROWS - 16) {
    tile_slot<Fmt, EPI, TILE_MT>(p, sl, tile_lds, c0, c1, z);
  } else {
    tile_slot<Fmt, EPI, 0>(p, sl, tile_lds, c0, c1, z);
  }
}

// A dense call goes to the tile kernel when that is the faster of the two by a model fitted to measurements (both
// costs are proportional to K): the weight stream takes about 23 us per 16 activation rows and 25600 output rows at
// K = 5120; the tile kernel (no K split: one workgroup per 256 output rows and 128 activation rows, 512 resident) about
// 130 us per round of workgroups.
inline bool tile_serves_dense(int m, int n_blocks) {
  const int64_t groups = (int64_t)((n_blocks + 3) / 4) * ((m + TILE_ROWS - 1) / TILE_ROWS), rounds = (groups + 511) / 512;
  return m > 2 * ROWS_PER_SLOT && (int64_t)n_blocks * 64 * m > 2300000 * rounds;
}

// Whether an activation matrix of `rows` rows is one the tile kernel takes: it addresses the matrix with 32-bit byte
// offsets ...
inline bool tile_takes(int64_t rows, int64_t a_stride) { return rows * a_stride * 2 <= 0xffffffffll; }
// ... and writes four neighbouring output columns with one store: 8 bytes of BF16, 16 of FP32.
inline bool tile_writes(const void* out, bool f32) { return aligned(out, f32 ? 16 : 8); }

// `slots`: the grid's second dimension (routed: the plan's upper bound; dense: ceil(m / TILE_ROWS)); `a_rows`: rows of
// the activation matrix.
// Workgroups a tile for a dense call of m rows (K shared among them), given room for their partial tiles: about four
// hundred workgroups in all (measured at 25600 x 5120: the best count from 24 to 128 rows), each with at least four
// chunks. 1: the call has two hundred tiles or more and fills the device alone.
inline int tile_split(int m, int n_blocks, int chunks) {
  const int64_t tiles = (int64_t)((n_blocks + 3) / 4) * ((m + TILE_ROWS - 1) / TILE_ROWS);
  if (tiles >= 200) return 1;
  return (int)std::max<int64_t>(1, std::min<int64_t>(chunks / 4, 400 / tiles));
}
constexpr int TILE_SPLIT_ROWS = 20;  // up to here two passes of the weight stream are the faster
inline int tile_partial_mt(int m) { return (std::min(m, TILE_ROWS) + 15) / 16; }
inline int64_t tile_count(int m, int n_blocks) { return (int64_t)((n_blocks + 3) / 4) * ((m + TILE_ROWS - 1) / TILE_ROWS); }
// The workspace of a call whose tiles share K: the tiles' arrival counters (a multiple of 256 bytes), then the partial tiles.
// (behind the PLAN_HEADER words every workspace begins with, so that the fault word means the same in all of them)
inline size_t tile_ticket_bytes(int m, int n_blocks) { return ((size_t)(PLAN_HEADER + tile_count(m, n_blocks)) * sizeof(uint32_t) + 255) & ~(size_t)255; }
inline size_t tile_partial_bytes(int m, int n_blocks, int ks) {
  return ks > 1 ? tile_ticket_bytes(m, n_blocks) + (size_t)tile_count(m, n_blocks) * ks * 4 * tile_partial_mt(m) * 4 * 64 * sizeof(f32x4_t) : 0;
}

template <class Fmt, int EPI>
static int launch_tile(StreamParams& p, int64_t slots, int64_t a_rows, hipStream_t stream) {
  if (!tile_takes(a_rows, p.a_stride)) return HB_EINVAL;
  p.slot_rows = TILE_ROWS;
  const unsigned groups = (unsigned)((p.n_blocks + 3) / 4);
  const int ks = p.tile_ks > 1 ? p.tile_ks : 1;
  if (ks > 1) {
    if (!p.partial || !p.tile_tickets || ks > p.chunks) return HB_EINVAL;
  }
  const dim3 grid(groups, (unsigned)slots, (unsigned)ks);
  HB_LAUNCH((tile_kernel<Fmt, EPI>), grid, dim3(256), 2 * TILE_BUF + TILE_ROWS * sizeof(int32_t), stream, p);
  return HB_OK;
}

}  // namespace hb
