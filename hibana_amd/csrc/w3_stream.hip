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

#include "stream_common.hpp"
#include "tile_kernel.hpp"
#include "w3_layout.hpp"

namespace hb {

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

// General kernel, any K: one workgroup per (run of p.nbw 64-row blocks, slot), K split p.ks ways across its wavefronts.
// Weights and activations of chunk i + 1 are requested together before chunk i is expanded (two register buffers).
template <int EPI>
__global__ __launch_bounds__(1024) void w3_stream_kernel(StreamParams p) {
  extern __shared__ float partial[];
  const Slot sl = slot_of<EPI>(p, blockIdx.y);
  if (sl.rows <= 0) return;  // a slot the plan did not fill: the whole workgroup leaves
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
      const uint16_t* aptr = activation_row<EPI>(p, sl, r16) + 8 * q + (int64_t)c0 * 128;
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
  finish_block<EPI, true>(p, sl, nb, active, ks, nbi, partial, acc0, acc1, acc2, acc3);
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
struct Tuning {
  int w3_tile = 0, w3_ksplit = 0, w3_nbw = 0, moe_fc1_ksplit = 0, moe_fc1_nbw = 0, moe_fc2_ksplit = 0, moe_fc2_nbw = 0;
};
static Tuning g_tune;

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
  HB_LAUNCH(w3_stream_kernel<EPI>, grid, dim3(64 * waves), p.ks > 1 ? (size_t)waves * 4096 : 0, stream, p);
  return HB_OK;
}

}  // namespace hb

using namespace hb;

extern "C" int hb_tune(const char* key, int value) {
  if (!key) return HB_ENULL;
  struct {
    const char* name;
    int* slot;
  } table[] = {{"w3_tile", &g_tune.w3_tile}, {"w3_ksplit", &g_tune.w3_ksplit},           {"w3_nbw", &g_tune.w3_nbw},
               {"moe_fc1_ksplit", &g_tune.moe_fc1_ksplit}, {"moe_fc1_nbw", &g_tune.moe_fc1_nbw},
               {"moe_fc2_ksplit", &g_tune.moe_fc2_ksplit}, {"moe_fc2_nbw", &g_tune.moe_fc2_nbw}};
  for (auto& t : table)
    if (!strcmp(t.name, key)) {
      if (value < 0 || value > 16 || (value & (value - 1))) return HB_EINVAL;
      *t.slot = value;
      return HB_OK;
    }
  return nvfp4_tune(key, value);
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
  if (g_tune.w3_tile == 1 || (g_tune.w3_tile == 0 && tile_serves_dense(m, p.n_blocks))) {
    if (int e = launch_tile<TileW3, EPI_DENSE>(p, (m + TILE_ROWS - 1) / TILE_ROWS, as_stream(stream))) return e;
    return launch_status();
  }
  const int64_t slots = (m + ROWS_PER_SLOT - 1) / ROWS_PER_SLOT;
  if (slots > 65535) return HB_EINVAL;
  if (int e = launch_stream<EPI_DENSE>(p, slots, slots, Launch{g_tune.w3_ksplit, g_tune.w3_nbw}, as_stream(stream))) return e;
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
  return HB_OK;
}

// plan -> fc1 -> fc2 (-> combine): `out_pairs` receives fc2's per-pair outputs (the workspace's y unless the caller
// wants the pairs themselves).
struct Routing {  // set: the chain routes `logits` [m, e] itself into the caller's ids / weights
  const float* logits;
  int e;
  int32_t* ids;
  float* weights;
};

int run_experts(const hb_w3_experts* ex, const hb_w3_experts* shared, const void* x, const int32_t* ids, int m, int topk,
                const MoeWorkspace& ws, void* out_pairs, int pairs_bf16, hipStream_t stream, const Routing* route = nullptr) {
  const int64_t pairs = (int64_t)m * topk;
  const int shared_rows = shared ? m : 0;
  // a dense contraction once an expert sees a few dozen rows: slots of 128 rows on the MFMA tile kernel
  const bool dense = g_tune.w3_tile == 1 || (g_tune.w3_tile == 0 && pairs >= (int64_t)ex->experts * 2 * TILE_DENSE_ROWS);  // the pre-scaled expansion costs more here than the stream's
  const int slot_rows = dense ? TILE_ROWS : ROWS_PER_SLOT;
  const int64_t slots = moe_max_slots(pairs, ex->experts, shared_rows, slot_rows);
  if (slots > 65535) return HB_EINVAL;
  if (route) {
    if (int e = moe_launch_route_plan(route->logits, m, route->e, topk, route->ids, route->weights, ex->base, ex->experts, shared_rows, ws, stream,
                                      slot_rows))
      return e;
  } else if (int e = moe_launch_plan(ids, pairs, ex->base, ex->experts, shared_rows, ws, stream, slot_rows)) {
    return e;
  }
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
  if (dense) {
    if (int e = ex->gated ? launch_tile<TileW3, EPI_FC1_GATED>(p, slots, stream) : launch_tile<TileW3, EPI_FC1_RELU2>(p, slots, stream)) return e;
    if (int e = launch_tile<TileW3, EPI_FC2>(f2, slots, stream)) return e;
    return launch_status();
  }
  const Launch l1{g_tune.moe_fc1_ksplit, g_tune.moe_fc1_nbw}, l2{g_tune.moe_fc2_ksplit, g_tune.moe_fc2_nbw};
  if (int e = ex->gated ? launch_stream<EPI_FC1_GATED>(p, slots, est, l1, stream) : launch_stream<EPI_FC1_RELU2>(p, slots, est, l1, stream)) return e;
  if (int e = launch_stream<EPI_FC2>(f2, slots, est, l2, stream)) return e;
  return launch_status();
}

}  // namespace

extern "C" size_t hb_w3_moe_workspace_bytes(int m, int topk, const hb_w3_experts* routed, int shared) {
  if (!routed || m <= 0 || topk <= 0 || check_experts(routed) != HB_OK) return 0;
  return moe_carve(nullptr, m, topk, routed->experts, routed->inter, routed->hidden_out, shared).bytes;
}

extern "C" int hb_w3_moe(const hb_w3_experts* routed, const void* x, const int32_t* ids, const float* weights, int m, int topk, int mode,
                         void* out, void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_experts(routed)) return e;
  if (!x || !ids || !weights || !out || !workspace) return HB_ENULL;
  if (m <= 0 || topk <= 0 || mode < HB_MOE_SUM || mode > HB_MOE_PAIRS_BF16) return HB_EINVAL;
  const MoeWorkspace ws = moe_carve(workspace, m, topk, routed->experts, routed->inter, routed->hidden_out, 0);
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
    moe_launch_combine(c, as_stream(stream));
  }
  return launch_status();
}

static int moe_layer(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x, const int32_t* ids,
                     const float* weights, int m, int topk, void* out, void* workspace, size_t workspace_bytes, void* stream,
                     const Routing* route) {
  if (int e = check_experts(routed)) return e;
  if (shared) {
    if (int e = check_experts(shared)) return e;
    if (shared->hidden != routed->hidden || shared->inter != routed->inter || shared->hidden_out != routed->hidden_out ||
        shared->gated != routed->gated)
      return HB_EINVAL;
  }
  if (!x || !ids || !weights || !out || !workspace) return HB_ENULL;
  if (m <= 0 || topk <= 0) return HB_EINVAL;
  const MoeWorkspace ws = moe_carve(workspace, m, topk, routed->experts, routed->inter, routed->hidden_out, shared ? 1 : 0);
  if (workspace_bytes < ws.bytes) return HB_EWORKSPACE;
  if (int e = run_experts(routed, shared, x, ids, m, topk, ws, ws.y, 0, as_stream(stream), route)) return e;
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
  moe_launch_combine(c, as_stream(stream));
  return launch_status();
}

extern "C" int hb_w3_moe_layer(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                               const int32_t* ids, const float* weights, int m, int topk, void* out, void* workspace,
                               size_t workspace_bytes, void* stream) {
  return moe_layer(routed, shared, gate_vec, x, ids, weights, m, topk, out, workspace, workspace_bytes, stream, nullptr);
}

extern "C" int hb_w3_moe_layer_logits(const hb_w3_experts* routed, const hb_w3_experts* shared, const float* gate_vec, const void* x,
                                      const float* logits, int experts_total, int m, int topk, int32_t* ids, float* weights, void* out,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  if (!logits) return HB_ENULL;
  const Routing route{logits, experts_total, ids, weights};
  return moe_layer(routed, shared, gate_vec, x, ids, weights, m, topk, out, workspace, workspace_bytes, stream, &route);
}
