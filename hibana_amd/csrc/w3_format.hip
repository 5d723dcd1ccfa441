// W3 format kernels: reference layout <-> tile layout, codes <-> planes, bit-exact dequantization.
// These run at load time or in tests; the streaming GEMMs are in w3_stream.hip.
#include "common.hpp"
#include "w3_layout.hpp"

namespace hb {

// One thread per (block, lane): builds the lane's code dwords (twelve of a three-bit tile, eight of a two-bit one) from
// the reference planes; two-bit codes into three-bit tiles leave the third bit zero.
__global__ __launch_bounds__(256) void w3_repack_codes_kernel(const uint32_t* __restrict__ planes, int64_t blocks, int chunks,
                                                              int bits, int tile_bits, uint8_t* __restrict__ tiled) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= blocks * 64) return;
  const int64_t blk = id >> 6;
  const int lane = (int)(id & 63), q = lane >> 4, r = lane & 15;
  const int64_t nb = blk / chunks;
  const int c = (int)(blk % chunks);
  uint32_t d[12];
#pragma unroll
  for (int i = 0; i < 12; i++) d[i] = 0;
  for (int nt = 0; nt < 4; nt++) {
    const int64_t n = nb * 64 + nt * 16 + r;
    for (int j = 0; j < 4; j++)
      for (int i = 0; i < 8; i++) {
        const int k = c * 128 + j * 32 + q * 8 + i;
        for (int b = 0; b < bits; b++) {
          int64_t word;
          int pos, dw, dpos;
          w3_ref_bit_slot(n, k, b, bits, chunks, &word, &pos);
          const uint32_t bit = (planes[word] >> pos) & 1u;
          if (tile_bits == 2) {
            w2_bit_slot(nt, j, i, b, &dw, &dpos);
          } else {
            w3_bit_slot(nt, j, i, b, &dw, &dpos);
          }
          d[dw] |= bit << dpos;
        }
      }
  }
  uint8_t* base = tiled + blk * w3_block_bytes(tile_bits);
#pragma unroll
  for (int i = 0; i < 12; i++)
    if (i < 4 * tile_bits) *reinterpret_cast<uint32_t*>(base + w3_dword_offset(lane, i)) = d[i];
}

// One thread per scale byte of the tile layout.
__global__ __launch_bounds__(256) void w3_repack_scales_kernel(const uint8_t* __restrict__ scales, int64_t blocks, int chunks,
                                                               int tile_bits, uint8_t* __restrict__ tiled) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= blocks * 256) return;
  const int64_t blk = id >> 8;
  const int within = (int)(id & 255), r = within >> 4, nt = (within >> 2) & 3, j = within & 3;
  const int64_t nb = blk / chunks;
  const int c = (int)(blk % chunks);
  const int64_t n = nb * 64 + nt * 16 + r;
  tiled[blk * w3_block_bytes(tile_bits) + w3_scale_base(tile_bits) + 16 * r + 4 * nt + j] = scales[w3_ref_scale_slot(n, 4 * c + j, chunks)];
}

// One thread per plane word of the reference layout.
__global__ __launch_bounds__(256) void w3_pack_planes_kernel(const uint8_t* __restrict__ codes, int64_t rows, int k, int bits,
                                                             uint32_t* __restrict__ planes) {
  const int chunks = k >> 7;
  const int64_t total = (rows >> 5) * chunks * bits * 128;
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= total) return;
  const int e = (int)(id & 3), lane = (int)((id >> 2) & 31);
  int64_t rest = id >> 7;
  const int i = (int)(rest % bits);
  rest /= bits;
  const int kc = (int)(rest % chunks);
  const int64_t nb = rest / chunks;
  const int w = 4 * i + e, nt = w / bits, b = w % bits, g = lane >> 2, t = lane & 3;
  const int64_t n = nb * 32 + nt * 8 + g;
  uint32_t word = 0;
  for (int s = 0; s < 8; s++)
    for (int j = 0; j < 4; j++) {
      const int kk = kc * 128 + s * 16 + t * 4 + j;
      const uint32_t bit = (codes[n * k + kk] >> b) & 1u;
      word |= bit << ((4 * j + b + 16 * (s >> 2) + (s & 3)) & 31);
    }
  planes[id] = word;
}

__global__ __launch_bounds__(256) void w3_pack_scales_kernel(const uint8_t* __restrict__ scale_bytes, int64_t rows, int k,
                                                             uint8_t* __restrict__ scales) {
  const int groups = k >> 5, chunks = k >> 7;
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= rows * groups) return;
  const int64_t n = id / groups;
  const int grp = (int)(id % groups);
  scales[w3_ref_scale_slot(n, grp, chunks)] = scale_bytes[id];
}

// One thread per (block, tile, lane): the lane's 32 codes of one 16-row tile.
// The eight selectors of tile nt of a lane, from either tile layout.
__device__ __forceinline__ void tile_selectors(const uint8_t* base, int lane, int nt, int bits, uint32_t sel[8]) {
  if (bits == 2) {
    w2_selectors(*reinterpret_cast<const uint32_t*>(base + w3_dword_offset(lane, 2 * nt)),
                 *reinterpret_cast<const uint32_t*>(base + w3_dword_offset(lane, 2 * nt + 1)), sel);
  } else {
    w3_selectors(*reinterpret_cast<const uint32_t*>(base + w3_dword_offset(lane, 3 * nt)),
                 *reinterpret_cast<const uint32_t*>(base + w3_dword_offset(lane, 3 * nt + 1)),
                 *reinterpret_cast<const uint32_t*>(base + w3_dword_offset(lane, 3 * nt + 2)), sel);
  }
}

__global__ __launch_bounds__(256) void w3_unpack_kernel(const uint8_t* __restrict__ tiled, int64_t blocks, int chunks, int bits,
                                                        uint8_t* __restrict__ codes, uint8_t* __restrict__ scale_bytes) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= blocks * 256) return;
  const int64_t blk = id >> 8;
  const int nt = (int)(id >> 6) & 3, lane = (int)(id & 63), q = lane >> 4, r = lane & 15;
  const int64_t nb = blk / chunks;
  const int c = (int)(blk % chunks);
  const int k = chunks * 128;
  const uint8_t* base = tiled + blk * w3_block_bytes(bits);
  const int64_t n = nb * 64 + nt * 16 + r;
  if (codes) {
    uint32_t sel[8];
    tile_selectors(base, lane, nt, bits, sel);
    for (int j = 0; j < 4; j++) {
      uint8_t* out = codes + n * k + c * 128 + j * 32 + q * 8;
      *reinterpret_cast<uint32_t*>(out) = sel[2 * j];
      *reinterpret_cast<uint32_t*>(out + 4) = sel[2 * j + 1];
    }
  }
  if (scale_bytes && q == 0) {
    for (int j = 0; j < 4; j++) scale_bytes[n * (k >> 5) + 4 * c + j] = base[w3_scale_base(bits) + 16 * r + 4 * nt + j];
  }
}

// One thread per (row, 128-chunk) of the reference layout.
__global__ __launch_bounds__(256) void w3_unpack_planes_kernel(const uint32_t* __restrict__ planes, const uint8_t* __restrict__ scales,
                                                               int64_t rows, int k, int bits, uint8_t* __restrict__ codes,
                                                               uint8_t* __restrict__ scale_bytes) {
  const int chunks = k >> 7;
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= rows * chunks) return;
  const int64_t n = id / chunks;
  const int kc = (int)(id % chunks);
  if (codes) {
    for (int kk = kc * 128; kk < kc * 128 + 128; kk++) {
      uint32_t code = 0;
      for (int b = 0; b < bits; b++) {
        int64_t word;
        int pos;
        w3_ref_bit_slot(n, kk, b, bits, chunks, &word, &pos);
        code |= ((planes[word] >> pos) & 1u) << b;
      }
      codes[n * k + kk] = (uint8_t)code;
    }
  }
  if (scale_bytes)
    for (int j = 0; j < 4; j++) scale_bytes[n * (k >> 5) + 4 * kc + j] = scales[w3_ref_scale_slot(n, 4 * kc + j, chunks)];
}

// One thread per (block, tile, lane): 32 dequantized weights. Two FP32 products, each rounded:
// effective = float(scale byte) * row_scale[row]; weight = level * effective.
__global__ __launch_bounds__(256) void w3_dequant_kernel(const uint8_t* __restrict__ tiled, const float* __restrict__ row_scale,
                                                         uint64_t lut, int64_t blocks, int chunks, int bits, float* __restrict__ out) {
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= blocks * 256) return;
  const int64_t blk = id >> 8;
  const int nt = (int)(id >> 6) & 3, lane = (int)(id & 63), q = lane >> 4, r = lane & 15;
  const int64_t nb = blk / chunks;
  const int c = (int)(blk % chunks);
  const int k = chunks * 128;
  const uint8_t* base = tiled + blk * w3_block_bytes(bits);
  const int64_t n = nb * 64 + nt * 16 + r;
  float level[8];
#pragma unroll
  for (int i = 0; i < 8; i++) level[i] = e4m3_to_f32((uint32_t)(lut >> (8 * i)) & 0xffu);
  uint32_t sel[8];
  tile_selectors(base, lane, nt, bits, sel);
  const float row = row_scale[n];
  for (int j = 0; j < 4; j++) {
    const float eff = __fmul_rn(e4m3_to_f32(base[w3_scale_base(bits) + 16 * r + 4 * nt + j]), row);
    float* o = out + n * k + c * 128 + j * 32 + q * 8;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const uint32_t code = (sel[2 * j + (i >> 2)] >> (8 * (i & 3))) & 7u;
      float lv = level[0];
#pragma unroll
      for (int t = 1; t < 8; t++) lv = code == (uint32_t)t ? level[t] : lv;
      o[i] = __fmul_rn(lv, eff);
    }
  }
}

static inline unsigned grid_for(int64_t threads) { return (unsigned)((threads + 255) / 256); }

}  // namespace hb

using namespace hb;

extern "C" size_t hb_w3_tiled_bytes(int64_t rows, int k, int bits) {
  if (rows <= 0 || k <= 0 || rows % W3_BLOCK_ROWS || k % W3_CHUNK || (bits != 2 && bits != 3)) return 0;
  return (size_t)(rows / W3_BLOCK_ROWS) * (size_t)(k / W3_CHUNK) * w3_block_bytes(bits);
}

static int check_shape(int64_t rows, int k, int bits) {
  if (rows <= 0 || k <= 0 || rows % W3_BLOCK_ROWS || k % W3_CHUNK || (bits != 2 && bits != 3)) return HB_EINVAL;
  if ((rows / W3_BLOCK_ROWS) * (int64_t)(k / W3_CHUNK) * 256 > (int64_t)0x7fffffff * 256) return HB_EINVAL;
  return HB_OK;
}

extern "C" int hb_w3_repack(const uint32_t* planes, const uint8_t* scales, int64_t rows, int k, int bits, int tile_bits, void* tiled, void* stream) {
  if (!planes || !scales || !tiled) return HB_ENULL;
  if (int e = check_shape(rows, k, bits)) return e;
  if (tile_bits != 3 && tile_bits != bits) return HB_EINVAL;  // codes are widened, never narrowed
  const int chunks = k / W3_CHUNK;
  const int64_t blocks = rows / W3_BLOCK_ROWS * chunks;
  hipLaunchKernelGGL(w3_repack_codes_kernel, dim3(grid_for(blocks * 64)), dim3(256), 0, as_stream(stream), planes, blocks, chunks, bits, tile_bits,
                     static_cast<uint8_t*>(tiled));
  hipLaunchKernelGGL(w3_repack_scales_kernel, dim3(grid_for(blocks * 256)), dim3(256), 0, as_stream(stream), scales, blocks, chunks, tile_bits,
                     static_cast<uint8_t*>(tiled));
  return launch_status();
}

extern "C" int hb_w3_pack_codes(const uint8_t* codes, const uint8_t* scale_bytes, int64_t rows, int k, int bits, uint32_t* planes,
                                uint8_t* scales, void* stream) {
  if (!codes || !scale_bytes || !planes || !scales) return HB_ENULL;
  if (int e = check_shape(rows, k, bits)) return e;
  const int64_t words = rows / 32 * (k / 128) * bits * 128;
  hipLaunchKernelGGL(w3_pack_planes_kernel, dim3(grid_for(words)), dim3(256), 0, as_stream(stream), codes, rows, k, bits, planes);
  hipLaunchKernelGGL(w3_pack_scales_kernel, dim3(grid_for(rows * (k / 32))), dim3(256), 0, as_stream(stream), scale_bytes, rows, k, scales);
  return launch_status();
}

extern "C" int hb_w3_unpack(const void* tiled, int64_t rows, int k, int bits, uint8_t* codes, uint8_t* scale_bytes, void* stream) {
  if (!tiled) return HB_ENULL;
  if (int e = check_shape(rows, k, bits)) return e;
  const int chunks = k / W3_CHUNK;
  const int64_t blocks = rows / W3_BLOCK_ROWS * chunks;
  hipLaunchKernelGGL(w3_unpack_kernel, dim3(grid_for(blocks * 256)), dim3(256), 0, as_stream(stream), static_cast<const uint8_t*>(tiled),
                     blocks, chunks, bits, codes, scale_bytes);
  return launch_status();
}

extern "C" int hb_w3_unpack_planes(const uint32_t* planes, const uint8_t* scales, int64_t rows, int k, int bits, uint8_t* codes,
                                   uint8_t* scale_bytes, void* stream) {
  if (!planes || !scales) return HB_ENULL;
  if (int e = check_shape(rows, k, bits)) return e;
  hipLaunchKernelGGL(w3_unpack_planes_kernel, dim3(grid_for(rows * (k / 128))), dim3(256), 0, as_stream(stream), planes, scales, rows, k,
                     bits, codes, scale_bytes);
  return launch_status();
}

extern "C" int hb_w3_dequant(const void* tiled, const float* row_scale, int64_t lut, int64_t rows, int k, int bits, float* out, void* stream) {
  if (!tiled || !row_scale || !out) return HB_ENULL;
  if (int e = check_shape(rows, k, bits)) return e;
  const int chunks = k / W3_CHUNK;
  const int64_t blocks = rows / W3_BLOCK_ROWS * chunks;
  hipLaunchKernelGGL(w3_dequant_kernel, dim3(grid_for(blocks * 256)), dim3(256), 0, as_stream(stream), static_cast<const uint8_t*>(tiled),
                     row_scale, (uint64_t)lut, blocks, chunks, bits, out);
  return launch_status();
}

// Measurement hook: a plain streaming read of `bytes` (a multiple of 16 KB), the yardstick a weight stream is held
// against. Each wavefront reads 16 KB in sixteen 128-bit loads a lane, all in flight together, and folds them into
// one word a workgroup (so that nothing is optimized away).
__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4_t* __restrict__ src, int64_t pieces, uint32_t* __restrict__ sink) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // one 16 KB piece a wavefront
  uint32_t fold = 0;
  if (wave < pieces) {
    const u32x4_t* at = src + wave * 1024 + lane;
    u32x4_t v[16];
#pragma unroll
    for (int j = 0; j < 16; j++) v[j] = __builtin_nontemporal_load(at + 64 * j);
#pragma unroll
    for (int j = 0; j < 16; j++) fold ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
  }
  if (fold == 0x9e3779b9u) sink[blockIdx.x] = fold;  // (practically never: the loads stay, the store does not cost)
}

#ifndef HB_NO_DEBUG_HOOKS
extern "C" int hb_debug_stream_read(const void* src, size_t bytes, void* sink, void* stream) {
  if (!src || !sink) return HB_ENULL;
  if (bytes == 0 || bytes % 16384 || !aligned(src, 16) || !aligned(sink, 4)) return HB_EINVAL;
  const int64_t pieces = (int64_t)(bytes / 16384);
  hipLaunchKernelGGL(stream_read_kernel, dim3((unsigned)((pieces + 3) / 4)), dim3(256), 0, as_stream(stream), static_cast<const u32x4_t*>(src), pieces,
                     static_cast<uint32_t*>(sink));
  return launch_status();
}
#endif

// Measurement hook: the weight stream's traffic without its arithmetic - what its request structure alone gets from
// this device. A workgroup of four wavefronts reads one 64-row block of sixteen 3328-byte chunks (53 248 bytes, at
// place table[group] of `src`: a dependent read first, as the stream reads its plan entry), each wavefront four of
// the chunks through a two-slot LDS ring (LDS-direct loads, read back with ds_read_b128, the next chunk but one asked
// for after each read-back), with sixteen bytes of activations a lane and chunk beside them; then the K split's
// exchange (sixteen floats a lane to LDS, a barrier, four partial sums back) and one store a lane. LDS a workgroup as
// the stream's (four workgroups a compute unit).
constexpr int SKELETON_CHUNK = W3_BLOCK_BYTES, SKELETON_PIECE = 4 * SKELETON_CHUNK, SKELETON_LDS = 40000;
__global__ __launch_bounds__(256) void ring_skeleton_kernel(const uint8_t* __restrict__ src, const int32_t* __restrict__ table, int places,
                                                            const u32x4_t* __restrict__ acts, float* __restrict__ out, uint32_t* __restrict__ sink) {
  extern __shared__ __align__(16) uint8_t rings[];
  typedef __attribute__((address_space(3))) uint8_t* lds_t;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t mine = (int64_t)blockIdx.x * 4 + wv;
  const int64_t wave = (int64_t)min(max(table[blockIdx.x], 0), places - 1) * 4 + wv;
  const lds_t slot0 = (lds_t)(rings + wv * 2 * SKELETON_CHUNK), slot1 = slot0 + SKELETON_CHUNK;
  const __amdgpu_buffer_rsrc_t row = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(src + wave * SKELETON_PIECE), 0, SKELETON_PIECE, 0x00020000);
  auto ask = [&](lds_t slot, int c) {
    const uint32_t at = (uint32_t)c * SKELETON_CHUNK;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(row, slot, 16, 16u * lane, at, 0, 2);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(row, slot, 16, 16u * lane, at, 1024, 2);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(row, slot, 16, 16u * lane, at, 2048, 2);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(row, slot, 4, 4u * lane, at, 3072, 2);
  };
  const u32x4_t* arow = acts + ((wave * 7) & 31) * 256 + (wv * 4) * 16 + (lane >> 2);  // one of 32 rows of 4 KB, this wavefront's K quarter
  u32x4_t held[2];
  ask(slot0, 0);
  held[0] = arow[0];
  ask(slot1, 1);
  held[1] = arow[16];
  uint32_t fold = 0;
  const uint32_t base = (uint32_t)(uintptr_t)slot0 + 16u * lane;
#pragma unroll
  for (int c = 0; c < 4; c++) {
    u32x4_t a, b, d;
    if (c < 3) {  // the next chunk's four loads and activation load may stay outstanding
      asm volatile("s_waitcnt vmcnt(5)\n\tds_read_b128 %0, %3 offset:%4\n\tds_read_b128 %1, %3 offset:%5\n\tds_read_b128 %2, %3 offset:%6\n\ts_waitcnt lgkmcnt(0)"
                   : "=&v"(a), "=&v"(b), "=&v"(d)
                   : "v"(base), "n"((c & 1) * SKELETON_CHUNK), "n"((c & 1) * SKELETON_CHUNK + 1024), "n"((c & 1) * SKELETON_CHUNK + 2048)
                   : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)\n\tds_read_b128 %0, %3 offset:%4\n\tds_read_b128 %1, %3 offset:%5\n\tds_read_b128 %2, %3 offset:%6\n\ts_waitcnt lgkmcnt(0)"
                   : "=&v"(a), "=&v"(b), "=&v"(d)
                   : "v"(base), "n"((c & 1) * SKELETON_CHUNK), "n"((c & 1) * SKELETON_CHUNK + 1024), "n"((c & 1) * SKELETON_CHUNK + 2048)
                   : "memory");
    }
    if (c + 2 < 4) ask((c & 1) ? slot1 : slot0, c + 2);
    fold ^= a.x ^ b.y ^ d.z ^ held[c & 1].x ^ held[c & 1].w;
    if (c + 2 < 4) held[c & 1] = arow[16 * (c + 2)];
  }
  float* part = reinterpret_cast<float*>(rings) + wv * (2 * SKELETON_CHUNK / 4);
#pragma unroll
  for (int j = 0; j < 16; j++) part[j * 64 + lane] = __uint_as_float((fold + j) & 0x3fffffffu);
  __syncthreads();
  float v = 0.f;
#pragma unroll
  for (int k = 0; k < 4; k++) v += reinterpret_cast<const float*>(rings)[k * (2 * SKELETON_CHUNK / 4) + wv * 64 + lane];
  out[mine * 64 + lane] = v;
  if (fold == 0x9e3779b9u) sink[blockIdx.x] = fold;  // (practically never)
}

#ifndef HB_NO_DEBUG_HOOKS
extern "C" int hb_debug_ring_skeleton(const void* src, size_t src_bytes, const int32_t* table, int groups, const void* acts, size_t acts_bytes, float* out,
                                      size_t out_bytes, void* sink, size_t sink_bytes, void* stream) {
  if (!src || !table || !acts || !out || !sink) return HB_ENULL;
  const int64_t places = (int64_t)(src_bytes / (4 * SKELETON_PIECE));
  if (groups <= 0 || places <= 0 || places > 0x7fffffff || !aligned(src, 16) || !aligned(table, 4) || !aligned(acts, 16) || !aligned(out, 4) || !aligned(sink, 4))
    return HB_EINVAL;
  // what the kernel touches: 32 activation rows of 4 KB, 256 floats of output and one sink word a workgroup
  if (acts_bytes < 32 * 4096 || out_bytes < (size_t)groups * 256 * sizeof(float) || sink_bytes < (size_t)groups * sizeof(uint32_t)) return HB_EINVAL;
  hipLaunchKernelGGL(ring_skeleton_kernel, dim3((unsigned)groups), dim3(256), SKELETON_LDS, as_stream(stream), static_cast<const uint8_t*>(src), table,
                     (int)places, static_cast<const u32x4_t*>(acts), out, static_cast<uint32_t*>(sink));
  return launch_status();
}
#endif

// Measurement hook: the rate this device's matrix cores give a kernel that does nothing else, the yardstick an expert
// GEMM is held against. Every wavefront runs `iters` rounds of eight independent v_mfma_f32_16x16x32_bf16 (16 384
// FLOP each) on registers; eight wavefronts a workgroup, two a SIMD.
__global__ __launch_bounds__(512) void mfma_rate_kernel(int iters, float* __restrict__ sink) {
  const int lane = threadIdx.x & 63;
  bf16x8_t a, b;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    a[j] = (__bf16)(0.001f * (float)(lane + j));
    b[j] = (__bf16)(0.002f * (float)(lane ^ j));
  }
  f32x4_t acc[8];
#pragma unroll
  for (int c = 0; c < 8; c++) acc[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int i = 0; i < iters; i++) {
#pragma unroll
    for (int c = 0; c < 8; c++) acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[c], 0, 0, 0);
  }
  float fold = 0.f;
#pragma unroll
  for (int c = 0; c < 8; c++) fold += acc[c].x + acc[c].y + acc[c].z + acc[c].w;
  if (fold == 12345.678f) sink[blockIdx.x] = fold;  // (practically never: the products stay, the store does not cost)
}

#ifndef HB_NO_DEBUG_HOOKS
extern "C" int64_t hb_debug_mfma_rate(int blocks, int iters, void* sink, void* stream) {
  if (!sink) return HB_ENULL;  // the HB_E* codes are negative themselves
  if (blocks <= 0 || blocks > 65536 || iters <= 0 || iters > (1 << 20) || !aligned(sink, 4)) return HB_EINVAL;
  hipLaunchKernelGGL(mfma_rate_kernel, dim3((unsigned)blocks), dim3(512), 0, as_stream(stream), iters, static_cast<float*>(sink));
  if (launch_status() != HB_OK) return HB_ELAUNCH;
  return (int64_t)blocks * 8 * iters * 8 * 16384;  // the launch's FLOP
}
#endif
