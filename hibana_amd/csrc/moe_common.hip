// Kernels and host helpers shared by every routed-expert call: the expert plan, the combine, softmax top-k routing.
#include <string.h>

#include <atomic>
#include <mutex>
#include <vector>

#include "route.hpp"
#include "route_budget.hpp"
#include "stream_common.hpp"

namespace hb {

// ---------------------------------------------------------------------------------------------------- routing
// (route.hpp: a row a wavefront)
template <bool SIGMOID, int PER>
__global__ __launch_bounds__(64) void route_topk_kernel(RouteParams p) {
  route_row<SIGMOID, PER>(p, blockIdx.x, threadIdx.x);
}

template <bool SIGMOID>
static void launch_route(const RouteParams& p, int m, hipStream_t stream) {
  if (p.per <= 8) {
    HB_LAUNCH((route_topk_kernel<SIGMOID, 8>), dim3((unsigned)m), dim3(64), 0, stream, p);
  } else {
    HB_LAUNCH((route_topk_kernel<SIGMOID, 16>), dim3((unsigned)m), dim3(64), 0, stream, p);
  }
}

// ---------------------------------------------------------------------------------------------------- expert plan
//
// The expert-sorted pair list of a routed call (the reference's prep kernel, hibana/kernels/csrc/w3_gemm.cu:710-782):
// distinct local experts in ascending id, each expert's pairs in ascending pair index (a stable sort), cut into slots
// of at most 16 rows. One workgroup; any number of pairs. Integer atomics on LDS counters only (order-independent).
//   plan[0] = slots, plan[1] = distinct experts, plan[2] = kept routed pairs,
//   plan[16 + 4 s ..] = { local expert id (-1: the shared expert), first sorted position, rows, 0 }: the shared
//                        expert's slots first, then the routed experts' (the heavily loaded ones before the others)
//   order[pos] = pair index (row * topk + slot; shared expert rows: pairs + row)
constexpr int PLAN_THREADS = 1024;
constexpr int PLAN_WAVES = PLAN_THREADS / 64;
constexpr int PLAN_BATCH = 8;  // tiles of 64 pairs whose ids a wavefront requests at once
constexpr int PLAN_WIDE_PAIRS = 8192;   // from this many pairs the plan is shared among workgroups (three launches)
constexpr int PLAN_WIDE_GROUPS = 64;
// Up to this many rows the plan workgroup routes them itself (one a wavefront): a row's selection is some 700 dependent
// VALU instructions, so on ONE compute unit more than four rows take longer than a launch of their own over the device
// (measured, whole layer: 22.1 against 22.5 us at one row, even at four, 50.7 against 46.8 us at sixteen).
constexpr int ROUTE_FUSED_ROWS = 4;

struct Scan3 {
  int a, b, c;
};

// Inclusive prefix sum over the wavefront's lanes without LDS: shifts within rows of sixteen lanes, then the rows' last
// lanes broadcast to the rows after them (DPP).
__device__ __forceinline__ int wave_inclusive_sum(int x) {
  x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, false);  // row_shr:1
  x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xF, 0xF, false);  // row_shr:2
  x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xF, 0xF, false);  // row_shr:4
  x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xF, 0xF, false);  // row_shr:8
  x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1 and 3
  x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2 and 3
  return x;
}

// Exclusive scan over the workgroup of two words a thread whose four 16-bit halves are sums of their own (none reaches
// 65536, so no carry crosses a half): one DPP scan a word in each wavefront, the wavefronts' totals through LDS, one
// barrier. `total` receives the two sums. scratch: 2 * PLAN_WAVES ints, not in use by anyone before the call's barrier.
struct Scan2 {
  int lo, hi;
};
__device__ __forceinline__ Scan2 block_exclusive_scan2(Scan2 v, int* scratch, Scan2* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const int lo = wave_inclusive_sum(v.lo), hi = wave_inclusive_sum(v.hi);
  if (lane == 63) {
    scratch[wave] = lo;
    scratch[PLAN_WAVES + wave] = hi;
  }
  __syncthreads();
  int before_lo = 0, before_hi = 0, all_lo = 0, all_hi = 0;
  for (int w = 0; w < waves; w++) {  // the same address in every lane: broadcast reads
    const int a = scratch[w], b = scratch[PLAN_WAVES + w];
    before_lo += w < wave ? a : 0;
    before_hi += w < wave ? b : 0;
    all_lo += a;
    all_hi += b;
  }
  total->lo = all_lo;
  total->hi = all_hi;
  return Scan2{before_lo + lo - v.lo, before_hi + hi - v.hi};
}

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

// The plan of at most 64 pairs (a decode step), by one wavefront, a pair a lane: no counters per expert, no scan over
// the experts. Lanes with the same expert find each other by ballots over the id's bits; what precedes an expert in
// either order (sorted positions: ascending id; slot table: shared, heavily loaded, the rest) is summed in a loop over
// the lanes. Writes exactly what the general form writes.
__device__ __forceinline__ void plan_few_pairs(const int32_t* ids, int pairs, int e_lo, int e_n, int shared_rows, int32_t* __restrict__ plan,
                                               int32_t* __restrict__ order, int slot_rows, int slot_cap) {
  const int lane = threadIdx.x & 63;
  int e = lane < pairs ? load_through(&ids[lane]) - e_lo : -1;
  if (e < 0 || e >= e_n) e = -1;
  int id_bits = 1;
  while ((1 << id_bits) < e_n) id_bits++;
  uint64_t same = __ballot(e >= 0);
  const int kept = __popcll(same);
  for (int b = 0; b < id_bits; b++) {
    const uint64_t m = __ballot((e >> b) & 1);
    same &= ((e >> b) & 1) ? m : ~m;
  }
  const int rank = __popcll(same & ((1ull << lane) - 1ull)), count = e >= 0 ? __popcll(same) : 0;
  const bool first = e >= 0 && rank == 0;
  const int my_slots = (count + slot_rows - 1) / slot_rows;
  const bool heavy = 4 * count > slot_rows;
  int start = 0, heavy_before = 0, light_before = 0, heavy_total = 0, light_total = 0, distinct = 0;
  for (int j = 0; j < pairs; j++) {  // uniform: lane j's expert, if lane j is the first of it
    const int ej = __builtin_amdgcn_readlane(first ? e : -1, j);
    if (ej < 0) continue;
    const int cj = __builtin_amdgcn_readlane(count, j), sj = __builtin_amdgcn_readlane(my_slots, j);
    const bool hj = 4 * cj > slot_rows;
    distinct++;
    heavy_total += hj ? sj : 0;
    light_total += hj ? 0 : sj;
    if (ej < e) {
      start += cj;
      heavy_before += hj ? sj : 0;
      light_before += hj ? 0 : sj;
    }
  }
  const int shared_slots = (shared_rows + slot_rows - 1) / slot_rows;
  const int slots = shared_slots + heavy_total + light_total;
  if (e >= 0) order[start + rank] = lane;
  if (first) {
    const int my_slot = shared_slots + (heavy ? heavy_before : heavy_total + light_before);
    for (int s = 0; s < my_slots; s++) {
      int32_t* entry = plan + PLAN_HEADER + 4 * (my_slot + s);
      entry[0] = e;
      entry[1] = start + s * slot_rows;
      entry[2] = min(slot_rows, count - s * slot_rows);
      entry[3] = 0;
    }
  }
  for (int s = lane; s < shared_slots; s += 64) {
    int32_t* entry = plan + PLAN_HEADER + 4 * s;
    entry[0] = -1;
    entry[1] = kept + s * slot_rows;
    entry[2] = min(slot_rows, shared_rows - s * slot_rows);
    entry[3] = 0;
  }
  for (int r = lane; r < shared_rows; r += 64) order[kept + r] = pairs + r;
  for (int s = slots + lane; s < slot_cap; s += 64) {
    int32_t* entry = plan + PLAN_HEADER + 4 * s;
    entry[0] = entry[1] = entry[2] = entry[3] = 0;
  }
  for (int s = lane; s < slot_cap; s += 64) plan_done(plan, slot_cap)[s * DONE_PITCH] = 0;
  if (lane == 0) {
    plan[0] = slots;
    plan[1] = distinct;
    plan[2] = kept;
  }
}

// What every form of the plan writes behind the experts' slots: the shared expert's slots and rows, "no rows" in the
// entries the launches' grids reach beyond the last slot (a workgroup learns that it has nothing to do from its own
// entry, without a second dependent read of the count), the slots' arrival counters at zero, the header.
__device__ __forceinline__ void plan_tail(int32_t* __restrict__ plan, int32_t* __restrict__ order, int pairs, int shared_rows, int slot_rows, int slot_cap,
                                          int slots, int distinct, int kept, bool counters = true) {
  const int shared_slots = (shared_rows + slot_rows - 1) / slot_rows;
  for (int s = threadIdx.x; s < shared_slots; s += blockDim.x) {
    int32_t* entry = plan + PLAN_HEADER + 4 * s;
    entry[0] = -1;
    entry[1] = kept + s * slot_rows;
    entry[2] = min(slot_rows, shared_rows - s * slot_rows);
    entry[3] = 0;
  }
  for (int r = threadIdx.x; r < shared_rows; r += blockDim.x) order[kept + r] = pairs + r;
  for (int s = slots + threadIdx.x; s < slot_cap; s += blockDim.x) {
    int32_t* entry = plan + PLAN_HEADER + 4 * s;
    entry[0] = entry[1] = entry[2] = entry[3] = 0;
  }
  if (counters)
    for (int s = threadIdx.x; s < slot_cap; s += blockDim.x) plan_done(plan, slot_cap)[s * DONE_PITCH] = 0;
  if (threadIdx.x == 0) {
    plan[0] = slots;
    plan[1] = distinct;
    plan[2] = kept;
  }
}

// The plan of a call of at most PLAN_ROWS_MAX rows in which no row names an expert twice (the library's own routing
// of a decode or verify call), by one workgroup of PLAN_THREADS: an expert's rows are one bit each of a 64-bit word in
// LDS (integer ORs: their order does not matter), its pair count is the word's population, and a pair's place among
// its expert's is the population below its row's bit - ascending pair index, as the general form places them. One
// trip to memory for the ids (every thread's loads asked for together), one scan, no per-tile matching. Writes
// exactly what plan_work writes.
constexpr int PLAN_ROWS_MAX = 64;
constexpr int PLAN_ROWS_PER_THREAD = 4;  // 64 rows of at most 64 selections over 1024 threads
__device__ __forceinline__ void plan_by_rows(const int32_t* ids, int rows, int topk, int e_lo, int e_n, int shared_rows, int32_t* __restrict__ plan,
                                             int32_t* __restrict__ order, int slot_rows, int slot_cap, int* lds, bool cleared = false) {
  uint32_t* occ_lo = reinterpret_cast<uint32_t*>(lds);  // [e_n] rows 0 .. 31 that name expert e
  uint32_t* occ_hi = occ_lo + e_n;                      // [e_n] rows 32 .. 63
  int* start = lds + 2 * e_n;                           // [e_n] first sorted position of expert e
  int* scratch = start + e_n;                           // [2 * PLAN_WAVES]
  const int pairs = rows * topk;
  int mine[PLAN_ROWS_PER_THREAD], row_of[PLAN_ROWS_PER_THREAD];
#pragma unroll
  for (int j = 0; j < PLAN_ROWS_PER_THREAD; j++) {  // asked for before anything else is done
    const int q = threadIdx.x + j * PLAN_THREADS;
    mine[j] = q < pairs ? load_through(&ids[q]) - e_lo : -1;
  }
  for (int e = threadIdx.x; e < 2 * e_n; e += PLAN_THREADS) occ_lo[e] = 0u;
#pragma unroll
  for (int j = 0; j < PLAN_ROWS_PER_THREAD; j++) row_of[j] = (threadIdx.x + j * PLAN_THREADS) / topk;
  __syncthreads();
#pragma unroll
  for (int j = 0; j < PLAN_ROWS_PER_THREAD; j++) {
    if (mine[j] < 0 || mine[j] >= e_n) mine[j] = -1;
    if (mine[j] >= 0) atomicOr(row_of[j] < 32 ? &occ_lo[mine[j]] : &occ_hi[mine[j]], 1u << (row_of[j] & 31));
  }
  __syncthreads();
  const int e = threadIdx.x;  // one thread an expert: the launch keeps e_n <= PLAN_THREADS
  const int count = e < e_n ? __popc(occ_lo[e]) + __popc(occ_hi[e]) : 0;  // at most 64
  const int my_slots = (count + slot_rows - 1) / slot_rows;
  const bool heavy = 4 * count > slot_rows;
  // four sums in two words: rows (at most 4096) and light slots; heavy slots and distinct experts (at most 1024 each)
  Scan2 tot;
  const Scan2 at = block_exclusive_scan2(Scan2{count | (heavy ? 0 : my_slots) << 16, (heavy ? my_slots : 0) | (count > 0 ? 1 << 16 : 0)}, scratch, &tot);
  const int shared_slots = (shared_rows + slot_rows - 1) / slot_rows;
  const int kept = tot.lo & 0xffff, distinct = tot.hi >> 16, heavy_slots = tot.hi & 0xffff;
  const int slots = shared_slots + heavy_slots + (tot.lo >> 16);
  if (e < e_n) {
    const int my_start = at.lo & 0xffff;
    start[e] = my_start;
    const int my_slot = shared_slots + (heavy ? (at.hi & 0xffff) : heavy_slots + (at.lo >> 16));
    for (int s = 0; s < my_slots; s++) {
      int32_t* entry = plan + PLAN_HEADER + 4 * (my_slot + s);
      entry[0] = e;
      entry[1] = my_start + s * slot_rows;
      entry[2] = min(slot_rows, count - s * slot_rows);
      entry[3] = 0;
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < PLAN_ROWS_PER_THREAD; j++) {
    if (mine[j] < 0) continue;
    const int r = row_of[j];
    const uint32_t lo = occ_lo[mine[j]], hi = occ_hi[mine[j]];
    const int below = r < 32 ? __popc(lo & ((1u << r) - 1u)) : __popc(lo) + __popc(hi & ((1u << (r - 32)) - 1u));
    order[start[mine[j]] + below] = threadIdx.x + j * PLAN_THREADS;
  }
  // `cleared`: the launch's other workgroups have already put "no rows" into every entry and zeroed the arrival counters
  plan_tail(plan, order, pairs, shared_rows, slot_rows, cleared ? slots : slot_cap, slots, distinct, kept, !cleared);
}

// The plan itself, by one workgroup of PLAN_THREADS (`group` of `groups` when many pairs are shared): `lds` is the
// launch's dynamic LDS.
template <bool WIDE>  // false: one workgroup (phase 0) and nothing of the shared form compiled in
__device__ __forceinline__ void plan_work(const int32_t* ids, int pairs, int e_lo, int e_n, int shared_rows, int32_t* __restrict__ plan,
                                          int32_t* __restrict__ order, int slot_rows, int slot_cap, int32_t* __restrict__ wide, int groups_, int phase_,
                                          int group_, int* lds) {
  const int groups = WIDE ? groups_ : 1, phase = WIDE ? phase_ : 0;
  if (!WIDE && pairs <= 64) {  // a decode step: one wavefront plans it
    if (threadIdx.x < 64) plan_few_pairs(ids, pairs, e_lo, e_n, shared_rows, plan, order, slot_rows, slot_cap);
    return;
  }
  int* seg_count = lds;                         // [PLAN_WAVES][e_n]: pairs of expert e in segment w, then running positions
  int* start = lds + PLAN_WAVES * e_n;          // [e_n]: first sorted position of expert e
  int* scratch = start + e_n;                   // [3 * (PLAN_WAVES + 1)]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, group = WIDE ? group_ : 0;
  // segment (group, w) = pairs [(group * PLAN_WAVES + w) * seg, ... + seg), seg a multiple of 64
  const int seg = (((pairs + groups - 1) / groups + PLAN_WAVES - 1) / PLAN_WAVES + 63) / 64 * 64;
  const int lo = min(pairs, (group * PLAN_WAVES + wave) * seg), hi = min(pairs, lo + seg);
  const int batch = seg > 64 ? PLAN_BATCH : 1;  // long segments: the ids of a batch of tiles are requested together
  const int nseg = WIDE ? PLAN_WAVES : min(PLAN_WAVES, (pairs + seg - 1) / seg);  // segments that hold pairs: the others' counters are neither cleared nor read
  const int e = threadIdx.x;  // one thread an expert: the launch keeps e_n <= PLAN_THREADS
  if (phase != 2) {
    for (int i = threadIdx.x; i < nseg * e_n; i += PLAN_THREADS) seg_count[i] = 0;
    __syncthreads();
  }
  int only = -1;  // seg == 64: the local expert of this lane's one pair, kept for the placement (no second read of the ids)
  for (int i0 = lo + lane; phase != 2 && i0 < hi; i0 += 64 * batch) {
    if (batch == 1) {
      const int e = load_through(&ids[i0]) - e_lo;
      if (e >= 0 && e < e_n) {
        atomicAdd(&seg_count[wave * e_n + e], 1);
        only = e;
      }
      continue;
    }
    int e[PLAN_BATCH];
#pragma unroll
    for (int j = 0; j < PLAN_BATCH; j++) e[j] = i0 + 64 * j < hi ? load_through(&ids[i0 + 64 * j]) - e_lo : -1;
#pragma unroll
    for (int j = 0; j < PLAN_BATCH; j++)
      if (e[j] >= 0 && e[j] < e_n) atomicAdd(&seg_count[wave * e_n + e[j]], 1);
  }
  __syncthreads();
  if (phase == 1) {  // this group's pairs of each expert
    if (e < e_n) {
      int count = 0;
      for (int wv = 0; wv < PLAN_WAVES; wv++) count += seg_count[wv * e_n + e];
      wide[group * e_n + e] = count;
    }
    return;
  }
  if (phase == 3) {  // the first position of each of this group's segments' runs, from the group's own
    if (e < e_n) {
      int run = wide[group * e_n + e];
      for (int wv = 0; wv < PLAN_WAVES; wv++) {
        const int c = seg_count[wv * e_n + e];
        seg_count[wv * e_n + e] = run;
        run += c;
      }
    }
    __syncthreads();
  } else {
  // Slot order is the order the hardware starts a launch's workgroups in, so the long-running slots go first: the
  // shared expert's (full slots), then the experts with more than a quarter slot of rows, then the rest, each class in
  // ascending expert id. Sorted positions are another matter: ascending expert id, the shared rows after the routed
  // pairs.
  const int shared_slots = (shared_rows + slot_rows - 1) / slot_rows;
  int count = 0;
  int of_group[PLAN_WIDE_GROUPS];  // phase 2: the groups' counts of this thread's expert, all asked for at once
  if (e < e_n) {
    if (phase == 0) {
      for (int wv = 0; wv < nseg; wv++) count += seg_count[wv * e_n + e];
    } else {
#pragma unroll
      for (int g = 0; g < PLAN_WIDE_GROUPS; g++) of_group[g] = g < groups ? wide[g * e_n + e] : 0;
#pragma unroll
      for (int g = 0; g < PLAN_WIDE_GROUPS; g++) count += of_group[g];
    }
  }
  const int my_slots = (count + slot_rows - 1) / slot_rows;
  const bool heavy = 4 * count > slot_rows;
  Scan3 tot;  // a: rows; b: heavy slots, and distinct experts in the upper half (neither sum reaches 65536); c: light slots
  const Scan3 at = block_exclusive_scan3(Scan3{count, (heavy ? my_slots : 0) | (count > 0 ? 1 << 16 : 0), heavy ? 0 : my_slots}, scratch, &tot);
  const int kept = tot.a, distinct = tot.b >> 16, heavy_slots = tot.b & 0xffff;
  const int slots = shared_slots + heavy_slots + tot.c;
  if (e < e_n) {
    const int my_start = at.a, my_slot = shared_slots + (heavy ? (at.b & 0xffff) : heavy_slots + at.c);
    start[e] = my_start;
    for (int s = 0; s < my_slots; s++) {
      int32_t* entry = plan + PLAN_HEADER + 4 * (my_slot + s);
      entry[0] = e;
      entry[1] = my_start + s * slot_rows;
      entry[2] = min(slot_rows, count - s * slot_rows);
      entry[3] = 0;
    }
    // turn the per-segment (phase 2: per-group) counts into the first position of each segment's (group's) run
    int run = my_start;
    if (phase == 0) {
      for (int wv = 0; wv < nseg; wv++) {
        const int c = seg_count[wv * e_n + e];
        seg_count[wv * e_n + e] = run;
        run += c;
      }
    } else {
#pragma unroll
      for (int g = 0; g < PLAN_WIDE_GROUPS; g++) {
        if (g < groups) wide[g * e_n + e] = run;
        run += of_group[g];
      }
    }
  }
  __syncthreads();
  plan_tail(plan, order, pairs, shared_rows, slot_rows, slot_cap, slots, distinct, kept);
  if (phase == 2) return;
  }
  // stable placement: each wavefront walks its segment 64 pairs at a time; a lane's position is its expert's running
  // position in this segment plus the number of lower lanes of the tile with the same expert
  int id_bits = 1;
  while ((1 << id_bits) < e_n) id_bits++;
  for (int i0 = lo; i0 < hi; i0 += 64 * batch) {
    int eb[PLAN_BATCH];
#pragma unroll
    for (int j = 0; j < PLAN_BATCH; j++) {
      const int i = i0 + 64 * j + lane;
      int e;
      if (seg == 64) {  // uniform: one tile a wavefront, read when it was counted
        e = j == 0 ? only : -1;
      } else {
        e = j < batch && i < hi ? load_through(&ids[i]) - e_lo : -1;
        if (e < 0 || e >= e_n) e = -1;
      }
      eb[j] = e;
    }
#pragma unroll
    for (int j = 0; j < PLAN_BATCH; j++) {
      if (j < batch && i0 + 64 * j < hi) {  // wave-uniform: some pair of the segment is in this tile
        const int i = i0 + 64 * j + lane, e = eb[j];
        uint64_t same = __ballot(e >= 0);
        for (int b = 0; b < id_bits; b++) {
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
      }
    }
    // the read of `base` above and the update by `last` are in the same wavefront; LDS operations of one wavefront
    // execute in program order, and the next tile's reads come after this write
  }
}

// With `route.logits` set the workgroup first routes the route_rows rows itself (softmax top-k, a row a wavefront at a
// time) into route.ids / route.weights, which `ids` then names.
//
// With `job.lanes` set the launch has further workgroups, which round the job's activations to E4M3 and plan nothing.
//
// Many pairs (a prefill chunk) are shared among `groups` workgroups in three launches of this kernel, `wide` [groups, e_n]
// between them: phase 1, each group counts its share of the pairs per expert; phase 2, one workgroup adds the groups'
// counts, writes the slot table and turns `wide` into the first sorted position of each group's run of each expert;
// phase 3, each group places its share. Phase 0 is all of it in one workgroup.
template <bool WIDE>
__global__ __launch_bounds__(PLAN_THREADS) void moe_plan_kernel(const int32_t* ids, int pairs, int e_lo, int e_n, int shared_rows,
                                                                int32_t* __restrict__ plan, int32_t* __restrict__ order, RouteParams route,
                                                                int route_rows, int slot_rows, int slot_cap, int32_t* __restrict__ wide, int groups,
                                                                int phase, QuantJob job) {
  extern __shared__ int lds[];
  if (!WIDE && blockIdx.x > 0) {  // the workgroups beside the plan's: the activation rounding
    quant_job_share(job, blockIdx.x - 1, reinterpret_cast<float*>(lds));
    return;
  }
  if (route.logits) {
    for (int r = threadIdx.x >> 6; r < route_rows; r += PLAN_WAVES) {
      route_any(route, r, threadIdx.x & 63);
    }
    __syncthreads();
  }
  plan_work<WIDE>(ids, pairs, e_lo, e_n, shared_rows, plan, order, slot_rows, slot_cap, wide, groups, phase, blockIdx.x, lds);
}

// Routing and plan of a verify-sized call in ONE launch: `route_groups` workgroups route ROUTE_GROUP_ROWS rows each (a
// row a wavefront, spread over the device, as the routing launch does), and the one that finishes last plans - it
// learns that it is the last from an arrival counter in the call's own workspace (plan[PLAN_TICKET]: zero when the
// caller hands the workspace over, put back to zero by every last arriver, as the split-K counters of the reference's
// dense kernel are, hibana/kernels/csrc/w3_gemm.cu:230-240), so calls in flight together, each on a workspace of its
// own, share nothing. A workgroup's ids are written through to memory and waited for before its ticket is drawn, and
// the plan reads ids past its own L2 (store_through / load_through): no cache write-back, no invalidate. Nobody
// waits: a workgroup that is not the last leaves. `by_rows`: the rows name no expert twice and are at most
// PLAN_ROWS_MAX (plan_by_rows). Workgroups past the routing ones round the job's activations, as in moe_plan_kernel.
constexpr int ROUTE_GROUP_ROWS = 1;

__global__ __launch_bounds__(PLAN_THREADS) void moe_route_plan_kernel(const int32_t* ids, int pairs, int e_lo, int e_n, int shared_rows,
                                                                      int32_t* __restrict__ plan, int32_t* __restrict__ order, RouteParams route,
                                                                      int route_rows, int route_groups, int by_rows, int slot_rows, int slot_cap,
                                                                      QuantJob job) {
  extern __shared__ int lds[];
  __shared__ int last;
  if ((int)blockIdx.x >= route_groups) {
    quant_job_share(job, blockIdx.x - route_groups, reinterpret_cast<float*>(lds));
    return;
  }
  const int wave = threadIdx.x >> 6, r = blockIdx.x * ROUTE_GROUP_ROWS + wave;
  if (wave < ROUTE_GROUP_ROWS && r < route_rows) {
    route_any(route, r, threadIdx.x & 63);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this row's ids (write-through stores) have reached memory before the ticket is drawn
  } else if (by_rows && wave >= ROUTE_GROUP_ROWS) {
    // Meanwhile the wavefronts that route nothing put "no rows" into every entry of the slot table and zero the slots'
    // arrival counters, a word a thread over the launch's routing workgroups - with stores that go through to memory
    // and are waited for, so the words are there, and in no L2 as modified lines, before anyone's ticket: the planner's
    // own stores to the entries it fills come after its ticket and are the only modified copies.
    constexpr int IDLE = PLAN_THREADS - 64 * ROUTE_GROUP_ROWS;
    int32_t* done = plan_done(plan, slot_cap);
    for (int i = blockIdx.x * IDLE + (int)threadIdx.x - 64 * ROUTE_GROUP_ROWS; i < 5 * slot_cap; i += route_groups * IDLE)
      store_through(i < 4 * slot_cap ? plan + PLAN_HEADER + i : done + (i - 4 * slot_cap) * DONE_PITCH, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned* ticket = reinterpret_cast<unsigned*>(plan + PLAN_TICKET);
    const unsigned drawn = atomicAdd(ticket, 1u);
    last = drawn == (unsigned)route_groups - 1u;
    if (last) store_through(plan + PLAN_TICKET, 0);  // every other workgroup of this launch has drawn: the counter is zero for the next call
  }
  __syncthreads();
  if (!last) return;  // the last arriver: every row's ids are in memory, and the plan reads them from there (load_through)
  if (by_rows) {
    plan_by_rows(ids, route_rows, route.k, e_lo, e_n, shared_rows, plan, order, slot_rows, slot_cap, lds, true);
  } else {
    plan_work<false>(ids, pairs, e_lo, e_n, shared_rows, plan, order, slot_rows, slot_cap, nullptr, 1, 0, 0, lds);
  }
}

// Budgeted selection and the plan of its ids in one launch: the selection is one workgroup's work already, and so is
// the plan of a decode or verify call; the ids go through to memory and are waited for before the plan reads them back
// past the L2, as in the routing launch above. `PLAN`: false leaves the plan to launches of its own (a call of more
// pairs than one workgroup plans).
template <int PER, bool PLAN>
__global__ __launch_bounds__(PLAN_THREADS) void moe_budget_plan_kernel(BudgetParams q, int copies_n, int e_lo, int e_n, int shared_rows,
                                                                       int32_t* __restrict__ plan, int32_t* __restrict__ order, int slot_rows,
                                                                       int slot_cap) {
  extern __shared__ int lds[];
  budget_pick<PER, false>(q, copies_n, reinterpret_cast<float*>(lds));
  if (!PLAN) return;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's ids have reached memory
  __syncthreads();                                    // ... and everyone's; the selection's use of the LDS is over
  plan_work<false>(q.ids, q.r * q.k, e_lo, e_n, shared_rows, plan, order, slot_rows, slot_cap, nullptr, 1, 0, 0, lds);
}

// ---------------------------------------------------------------------------------------------------- combine
//
// out[r, c] = bf16( bf16(sum over the row's local slots, in selection order, of fma(w, y)) + g * shared ), one
// workgroup per (row, 512-column span). The reference's combine (hibana/kernels/csrc/w3_gemm.cu:1196-1213) when no
// shared expert is given; with one, its fused form (hibana/kernels/flashnext_fused.py:530-571).
constexpr int COMBINE_SPAN = 512;  // columns per workgroup (two per thread)

// A row's weighted sum of its pairs at columns c, c + 1, in selection order (FP32 fma chain). The pairs of B slots are
// read together (so the loads are all in flight at once) and a dropped slot contributes fma(0, 0, v).
template <int B, bool BF16>
struct CombineBatch {
  int e[B];
  float w[B];
  uint32_t half[B];
  float2 full[B];
  // every load of the batch is asked for before any is used: ids and weights (the same for the whole workgroup), then
  // the pairs - also a dropped slot's, whose values are then set aside (a pair's address does not depend on its id)
  __device__ __forceinline__ void load(const CombineParams& p, int r, int c, int s0) {
#pragma unroll
    for (int j = 0; j < B; j++) {
      const int s = min(s0 + j, p.topk - 1);
      e[j] = p.ids[r * p.topk + s];
      w[j] = p.weights[r * p.topk + s];
    }
#pragma unroll
    for (int j = 0; j < B; j++) {
      const int s = min(s0 + j, p.topk - 1);
      const int64_t at = ((int64_t)r * p.topk + s) * p.h + c;
      if (BF16) {
        half[j] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint16_t*>(p.pairs) + at);
      } else {
        full[j] = *reinterpret_cast<const float2*>(reinterpret_cast<const float*>(p.pairs) + at);
      }
    }
  }
  __device__ __forceinline__ void add(const CombineParams& p, int s0, float& v0, float& v1) {
    float y0[B], y1[B];
#pragma unroll
    for (int j = 0; j < B; j++) {
      const int local = e[j] - p.e_lo;
      const bool keep = s0 + j < p.topk && local >= 0 && local < p.e_n;
      const float a = BF16 ? __uint_as_float(half[j] << 16) : full[j].x, b = BF16 ? __uint_as_float(half[j] & 0xffff0000u) : full[j].y;
      y0[j] = keep ? a : 0.f;
      y1[j] = keep ? b : 0.f;
      w[j] = keep ? w[j] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < B; j++) {
      v0 = fmaf(w[j], y0[j], v0);
      v1 = fmaf(w[j], y1[j], v1);
    }
  }
};

struct CombineShared {  // the shared expert's two columns, FP32 or BF16
  float2 f32 = {0.f, 0.f};
  uint32_t bf16 = 0;
  __device__ __forceinline__ void load(const CombineParams& p, int r, int c) {
    const int64_t at = (int64_t)r * p.shared_stride + c;
    if (p.shared_f32) {
      f32 = *reinterpret_cast<const float2*>(reinterpret_cast<const float*>(p.shared) + at);
    } else {
      bf16 = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint16_t*>(p.shared) + at);
    }
  }
};

// One (row, 512-column span) a workgroup. The first batch of pairs and the shared expert's columns are asked for AHEAD
// of the gate's dot product, whose barrier would otherwise stand between two trips to memory: the gate's own loads
// follow them, and everything is on its way together.
template <int B, bool BF16>
__device__ __forceinline__ void combine_span(const CombineParams& p, float* red) {
  const int r = blockIdx.x;
  const int c = blockIdx.y * COMBINE_SPAN + 2 * threadIdx.x;  // h is even: a column pair is in or out together
  const bool in = c < p.h;                                    // a thread past the row's end reads column 0 and stores nothing: it is needed at the barrier
  const int cl = in ? c : 0;
  CombineBatch<B, BF16> batch;
  CombineShared sh;
  batch.load(p, r, cl, 0);
  if (p.shared) sh.load(p, r, cl);
  float g = 1.0f;
  if (p.gate_vec && p.shared) {  // uniform over the launch
    combine_gate_partial(p.x, p.gate_vec, p.hx, r, threadIdx.x, red);
    __syncthreads();
    g = combine_gate_value(red);
  }
  float v0 = 0.f, v1 = 0.f;
  batch.add(p, 0, v0, v1);
  for (int s0 = B; s0 < p.topk; s0 += B) {
    batch.load(p, r, cl, s0);
    batch.add(p, s0, v0, v1);
  }
  if (p.shared) {
    const float s0 = p.shared_f32 ? sh.f32.x : __uint_as_float(sh.bf16 << 16);
    const float s1 = p.shared_f32 ? sh.f32.y : __uint_as_float(sh.bf16 & 0xffff0000u);
    v0 = combine_shared(v0, g, s0);
    v1 = combine_shared(v1, g, s1);
  }
  if (in) *reinterpret_cast<uint32_t*>(p.out + (int64_t)r * p.h + c) = (uint32_t)f32_to_bf16_bits(v0) | ((uint32_t)f32_to_bf16_bits(v1) << 16);
}
// B: the slots read together - 8 or 12 where the call is long or top-k small, 24 for a short call of many slots
// (one wait on memory instead of three); a kernel of its own each, so that the longer batches' registers are theirs alone.
template <int B>
__global__ __launch_bounds__(256) void moe_combine_kernel(CombineParams p) {
  __shared__ float red[4];
  if (p.pairs_bf16) {
    combine_span<B, true>(p, red);
  } else {
    combine_span<B, false>(p, red);
  }
}

// ------------------------------------------------------------------ the latent block's BF16 projections (M <= 16)
//
// y[i, n] = sum_k x[i, k] w[n, k] for at most sixteen rows of x, on the BF16 matrix cores with nothing staged: a
// wavefront takes sixteen weight rows over `steps` K steps of 32 from k0; lane (q, r16) holds k = 32 s + 8 q .. + 7 of
// weight row n0 + r16 (the B operand) and of activation row r16 (A; rows past m read row m - 1 and are never stored).
// Register i of lane (q, r16) of the result is y[4 q + i][n0 + r16]. Up to eight steps are in flight at a time.
struct GemvFrags {
  u32x4_t v[8];
};
__device__ __forceinline__ void gemv16_load(GemvFrags& f, const uint16_t* __restrict__ base, int64_t ld, int row, int k0, int steps, int lane) {
  const uint16_t* at = base + row * ld + k0 + 8 * (lane >> 4);
#pragma unroll
  for (int j = 0; j < 8; j++)
    if (j < steps) f.v[j] = *reinterpret_cast<const u32x4_t*>(at + 32 * j);
}
__device__ __forceinline__ void gemv16_mfma(f32x4_t& acc, const GemvFrags& a, const GemvFrags& b, int steps) {
#pragma unroll
  for (int j = 0; j < 8; j++)
    if (j < steps) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a.v[j]), __builtin_bit_cast(bf16x8_t, b.v[j]), acc, 0, 0, 0);
}
__device__ __forceinline__ f32x4_t gemv16_wave(const uint16_t* __restrict__ w, int64_t ldw, int n0, int n, const uint16_t* __restrict__ x, int64_t ldx, int m,
                                               int k0, int steps, int lane) {
  const int r16 = lane & 15, wrow = min(n0 + r16, n - 1), xrow = min(r16, m - 1);
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < steps; s0 += 8) {
    GemvFrags a, b;
    gemv16_load(b, w, ldw, wrow, k0 + 32 * s0, steps - s0, lane);
    gemv16_load(a, x, ldx, xrow, k0 + 32 * s0, steps - s0, lane);
    gemv16_mfma(acc, a, b, steps - s0);
  }
  return acc;
}
// The K splits' partial tiles, one per wavefront, added in wavefront order: thread t < 256 returns y[t / 16][n0 + t % 16].
__device__ __forceinline__ float gemv16_reduce(const f32x4_t& acc, float* part, int waves) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  *reinterpret_cast<f32x4_t*>(part + wave * 256 + lane * 4) = acc;
  __syncthreads();
  float sum = 0.f;
  if (threadIdx.x < 256) {
    const int row = threadIdx.x >> 4, at = ((row >> 2) * 16 + (threadIdx.x & 15)) * 4 + (row & 3);
    for (int w = 0; w < waves; w++) sum += part[w * 256 + at];
  }
  return sum;
}

// The router's product of a small latent block (hibana/kernels/csrc/nemotron_moe.cu:496-558 of the reference):
// fused[m, n] = x [router; fc1_latent]^T in FP32, sixteen output columns a workgroup, K split over its sixteen
// wavefronts; the latent columns (e .. n - 1) are also left rounded to BF16.
struct RouterGemv {
  const uint16_t* w;  // BF16 [n, k]
  const uint16_t* x;  // BF16 [m, k]
  float* fused;       // FP32 [m, n]
  uint16_t* lat;      // BF16 [m, n - e]
  int n, k, m, e;
};
__global__ __launch_bounds__(1024) void latent_router_kernel(RouterGemv g) {
  __shared__ __align__(16) float part[16 * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n0 = blockIdx.x * 16, per_wave = g.k / 16;
  const f32x4_t acc = gemv16_wave(g.w, g.k, n0, g.n, g.x, g.k, g.m, wave * per_wave, per_wave / 32, lane);
  const float sum = gemv16_reduce(acc, part, 16);
  if (threadIdx.x < 256) {
    const int row = threadIdx.x >> 4, n = n0 + (threadIdx.x & 15);
    if (row < g.m && n < g.n) {
      g.fused[(int64_t)row * g.n + n] = sum;
      if (n >= g.e) g.lat[(int64_t)row * (g.n - g.e) + n - g.e] = bf16_of(sum);
    }
  }
}

// The last launch of a small latent block (nemotron_moe.cu's out kernel): out = bf16(shared + routed fc2^T) with
// routed BF16 [m, latent]; sixteen output columns a workgroup, K split over its wavefronts (at most eight steps each).
struct OutGemv {
  const uint16_t* w;       // fc2 BF16 [n, k]
  const uint16_t* routed;  // BF16 [m, k]
  const uint16_t* shared;  // BF16 [m, n] or null
  uint16_t* out;           // BF16 [m, n]
  int n, k, m, waves;
};
__global__ __launch_bounds__(1024) void latent_out_kernel(OutGemv g) {
  __shared__ __align__(16) float part[16 * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n0 = blockIdx.x * 16;
  const int per_wave = g.k / g.waves;
  const int out_row = threadIdx.x >> 4, out_n = n0 + (threadIdx.x & 15);
  const bool stores = threadIdx.x < 256 && out_row < g.m && out_n < g.n;  // a workgroup has at least these 256 threads
  const float base = stores && g.shared ? bf16_bits_to_f32(g.shared[(int64_t)out_row * g.n + out_n]) : 0.f;
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  if (wave < g.waves) acc = gemv16_wave(g.w, g.k, n0, g.n, g.routed, g.k, g.m, wave * per_wave, per_wave / 32, lane);
  const float sum = gemv16_reduce(acc, part, g.waves);
  if (stores) g.out[(int64_t)out_row * g.n + out_n] = f32_to_bf16_bits(base + sum);
}

// ---------------------------------------------------------------------------------------------------- host side
// The measurement hook's state: `g_events_armed` is all a launch reads while no events are armed (one relaxed load); the
// list itself is only touched under its lock.
static std::atomic<bool> g_events_armed{false};
static std::mutex g_events_lock;
static std::vector<hipEvent_t> g_events;
static size_t g_event_next = 0;
bool moe_next_events(hipEvent_t* start, hipEvent_t* stop) {
  if (!g_events_armed.load(std::memory_order_relaxed)) return false;
  std::lock_guard<std::mutex> hold(g_events_lock);
  if (g_event_next + 1 >= g_events.size()) return false;
  *start = g_events[g_event_next];
  *stop = g_events[g_event_next + 1];
  g_event_next += 2;
  return true;
}

void pick_shape(int n_blocks, int chunks, int64_t slots, int want, int* ks, int* nbw) {
  int k = 1;
  while (k < 16 && (int64_t)n_blocks * slots * k < want && chunks / (2 * k) >= 4) k *= 2;
  int b = k >= 4 ? 1 : 4 / k;
  while (b > 1 && n_blocks % b) b /= 2;
  *ks = k;
  *nbw = b;
}

int64_t moe_max_slots(int64_t pairs, int experts, int shared_rows, int slot_rows) {
  const int64_t routed = pairs < pairs / slot_rows + experts ? pairs : pairs / slot_rows + experts;
  return routed + (shared_rows + slot_rows - 1) / slot_rows;
}

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

MoeWorkspace moe_carve(void* base, int m, int topk, int experts, int inter, int hidden_out, int shared, int hidden) {
  const int64_t pairs = (int64_t)m * topk, rows = pairs + (shared ? m : 0);
  MoeWorkspace w{};
  size_t off = 0;
  auto take = [&](size_t bytes) {
    void* ptr = base ? static_cast<char*>(base) + off : nullptr;
    off += align256(bytes);
    return ptr;
  };
  w.plan = static_cast<int32_t*>(take((PLAN_HEADER + (4 + DONE_PITCH) * moe_max_slots(pairs, experts, shared ? m : 0, ROWS_PER_SLOT) + 32) * sizeof(int32_t)));  // entries, then plan_done
  w.plan_wide = static_cast<int32_t*>(take((size_t)PLAN_WIDE_GROUPS * experts * sizeof(int32_t)));
  w.order = static_cast<int32_t*>(take(rows * sizeof(int32_t)));
  w.h = static_cast<uint16_t*>(take((size_t)rows * inter * sizeof(uint16_t)));
  w.y = static_cast<float*>(take((size_t)rows * hidden_out * sizeof(float)));
  if (hidden) {
    w.xq = static_cast<uint8_t*>(take((size_t)m * hidden));
    w.xs = static_cast<float*>(take((size_t)m * (hidden / 32) * sizeof(float)));
    w.hq = static_cast<uint8_t*>(take((size_t)rows * inter));
    w.hs = static_cast<float*>(take((size_t)rows * (inter / 32) * sizeof(float)));
    w.x2 = static_cast<uint8_t*>(take((size_t)m * 2 * hidden));
    w.x2s = static_cast<float*>(take((size_t)m * sizeof(float)));
  }
  w.bytes = off;
  return w;
}

__global__ __launch_bounds__(256) void quant_groups_kernel(QuantJob job) {
  __shared__ float red[4];
  quant_job_share(job, blockIdx.x, red);
}

// BF16 [m, k] (k % 8 == 0) -> E4M3 codes [m, k] and ONE FP32 scale a row: s = max(amax / 448, 1e-12),
// q = e4m3(clamp(x / s, -448, 448)), IEEE divisions as in quant_groups_lane (the reference's per-row quantizer,
// hibana/kernels/csrc/w3_gemm.cu:244-288, which multiplies by a reciprocal). One workgroup a row: the row's largest
// magnitude over the four wavefronts through LDS, then every lane rounds its runs of eight values.
__global__ __launch_bounds__(256) void quant_rows_kernel(const uint16_t* __restrict__ x, int k, uint8_t* __restrict__ q, float* __restrict__ scales) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const uint16_t* xr = x + row * k;
  float amax = 0.f;
  for (int c = 8 * threadIdx.x; c < k; c += 8 * 256) {
    const u32x4_t raw = *reinterpret_cast<const u32x4_t*>(xr + c);
#pragma unroll
    for (int j = 0; j < 4; j++) amax = fmaxf(amax, fmaxf(fabsf(__uint_as_float(raw[j] << 16)), fabsf(__uint_as_float(raw[j] & 0xffff0000u))));
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = fmaxf(amax / 448.0f, 1e-12f);
  if (threadIdx.x == 0) scales[row] = s;
  for (int c = 8 * threadIdx.x; c < k; c += 8 * 256) {
    const u32x4_t raw = *reinterpret_cast<const u32x4_t*>(xr + c);
    float v[8];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      v[2 * j] = __uint_as_float(raw[j] << 16);
      v[2 * j + 1] = __uint_as_float(raw[j] & 0xffff0000u);
    }
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = fminf(fmaxf(v[j] / s, -448.0f), 448.0f);
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(v[4], v[5], hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(v[6], v[7], hi, true);
    typedef __attribute__((ext_vector_type(2))) int i32x2_t;
    *reinterpret_cast<i32x2_t*>(q + row * k + c) = i32x2_t{lo, hi};
  }
}

void moe_launch_quant_rows(const uint16_t* x, int64_t m, int k, uint8_t* q, float* scales, hipStream_t stream) {
  HB_LAUNCH(quant_rows_kernel, dim3((unsigned)m), dim3(256), 0, stream, x, k, q, scales);
}

void moe_launch_quant_groups(const QuantJob& job, hipStream_t stream) {
  const unsigned groups = job.split_rows ? (unsigned)job.split_rows : (unsigned)((job.lanes + 255) / 256);
  HB_LAUNCH(quant_groups_kernel, dim3(groups), dim3(256), 0, stream, job);
}

static std::atomic<int> g_route_plan_fused{0};  // hb_tune("route_plan", 2): routing and plan as two launches; 1: the general plan also where plan_by_rows serves
int moe_tune(const char* key, int value) {
  if (strcmp(key, "route_plan") || value < 0 || value > 2) return HB_EINVAL;
  g_route_plan_fused.store(value, std::memory_order_relaxed);
  return HB_OK;
}

static unsigned plan_groups(const QuantJob* job) {
  if (!job) return 1u;
  return 1u + (job->split_rows ? (unsigned)job->split_rows : (unsigned)((job->lanes + PLAN_THREADS - 1) / PLAN_THREADS));
}

int moe_launch_plan(const int32_t* ids, int64_t pairs, int e_lo, int e_n, int shared_rows, const MoeWorkspace& ws, hipStream_t stream, int slot_rows,
                    const QuantJob* job) {
  const size_t plan_lds = ((size_t)(PLAN_WAVES + 1) * e_n + 3 * (PLAN_WAVES + 1)) * sizeof(int);
  if (plan_lds > 64 * 1024 || e_n > PLAN_THREADS || pairs > 0x3fffffff) return HB_EINVAL;
  const int slot_cap = (int)moe_max_slots(pairs, e_n, shared_rows, slot_rows);
  if (pairs >= PLAN_WIDE_PAIRS) {  // a share of about a thousand pairs a workgroup
    const int groups = (int)std::min<int64_t>(PLAN_WIDE_GROUPS, pairs / 1024);
    if (job) moe_launch_quant_groups(*job, stream);
    for (int phase = 1; phase <= 3; phase++)
      HB_LAUNCH(moe_plan_kernel<true>, dim3(phase == 2 ? 1 : groups), dim3(PLAN_THREADS), plan_lds, stream, ids, (int)pairs, e_lo, e_n, shared_rows, ws.plan,
                ws.order, RouteParams{}, 0, slot_rows, slot_cap, ws.plan_wide, groups, phase, QuantJob{});
    return HB_OK;
  }
  HB_LAUNCH(moe_plan_kernel<false>, dim3(plan_groups(job)), dim3(PLAN_THREADS), plan_lds, stream, ids, (int)pairs, e_lo, e_n, shared_rows, ws.plan, ws.order,
            RouteParams{}, 0, slot_rows, slot_cap, ws.plan_wide, 1, 0, job ? *job : QuantJob{});
  return HB_OK;
}

int moe_check_route(int m, int e, int k) { return m <= 0 || e <= 0 || k <= 0 || k > e || k > 64 || e > 64 * ROUTE_PER_LANE ? HB_EINVAL : HB_OK; }

// Routing by `rp` (either rule) and the plan of its ids, in as few launches as the size allows.
static int launch_route_plan(const RouteParams& rp, int m, int e_lo, int e_n, int shared_rows, const MoeWorkspace& ws, hipStream_t stream, int slot_rows,
                             const QuantJob* job) {
  const int64_t pairs = (int64_t)m * rp.k;
  const size_t plan_lds = ((size_t)(PLAN_WAVES + 1) * e_n + 3 * (PLAN_WAVES + 1)) * sizeof(int);
  if (plan_lds > 64 * 1024 || e_n > PLAN_THREADS || pairs > 0x3fffffff) return HB_EINVAL;
  if (m > ROUTE_FUSED_ROWS && pairs < PLAN_WIDE_PAIRS && g_route_plan_fused.load(std::memory_order_relaxed) != 2) {
    // a verify-sized call: the routing spread over the device, the plan by the workgroup that finishes last
    const int groups = (m + ROUTE_GROUP_ROWS - 1) / ROUTE_GROUP_ROWS;
    // rows that name no expert twice: every row is real (a padded row repeats one id over its slots)
    const int by_rows = !rp.slots && m <= PLAN_ROWS_MAX && rp.k <= 64 && g_route_plan_fused.load(std::memory_order_relaxed) != 1;
    HB_LAUNCH(moe_route_plan_kernel, dim3((unsigned)groups + plan_groups(job) - 1u), dim3(PLAN_THREADS), plan_lds, stream, rp.ids, (int)pairs, e_lo, e_n,
              shared_rows, ws.plan, ws.order, rp, m, groups, by_rows, slot_rows, (int)moe_max_slots(pairs, e_n, shared_rows, slot_rows),
              job ? *job : QuantJob{});
    return HB_OK;
  }
  if (m > ROUTE_FUSED_ROWS) {  // a prefill-sized call: a wavefront a row over the whole device, then the plan's launches
    if (rp.sigmoid) {
      launch_route<true>(rp, m, stream);
    } else {
      launch_route<false>(rp, m, stream);
    }
    return moe_launch_plan(rp.ids, pairs, e_lo, e_n, shared_rows, ws, stream, slot_rows, job);
  }
  HB_LAUNCH(moe_plan_kernel<false>, dim3(plan_groups(job)), dim3(PLAN_THREADS), plan_lds, stream, rp.ids, (int)pairs, e_lo, e_n, shared_rows, ws.plan, ws.order,
            rp, m, slot_rows, (int)moe_max_slots(pairs, e_n, shared_rows, slot_rows), ws.plan_wide, 1, 0, job ? *job : QuantJob{});
  return HB_OK;
}

int moe_launch_route_plan(const float* logits, int m, int e, int topk, int32_t* ids, float* weights, int e_lo, int e_n, int shared_rows,
                          const MoeWorkspace& ws, hipStream_t stream, int slot_rows, const QuantJob* job) {
  if (int err = moe_check_route(m, e, topk)) return err;
  RouteParams rp{};
  rp.logits = logits;
  rp.stride = e;
  rp.e = e;
  rp.k = topk;
  rp.per = (e + 63) / 64;
  rp.steps = 1;
  rp.pad_id = e;
  rp.ids = ids;
  rp.weights = weights;
  return launch_route_plan(rp, m, e_lo, e_n, shared_rows, ws, stream, slot_rows, job);
}

int moe_launch_budget_plan(const BudgetRoute& b, int m, int topk, int32_t* ids, float* weights, int e_lo, int e_n, int shared_rows,
                           const MoeWorkspace& ws, void* scratch, hipStream_t stream, int slot_rows) {
  static_assert(BUDGET_THREADS == PLAN_THREADS, "the selection and the plan share a workgroup");
  const int64_t pairs = (int64_t)m * topk;
  const size_t plan_lds = ((size_t)(PLAN_WAVES + 1) * e_n + 3 * (PLAN_WAVES + 1)) * sizeof(int);
  if (plan_lds > 64 * 1024 || e_n > PLAN_THREADS || pairs > 0x3fffffff) return HB_EINVAL;
  if (!b.logits || !scratch) return HB_ENULL;
  if (b.e < BUDGET_CANDIDATES || b.e > BUDGET_THREADS || topk > BUDGET_CANDIDATES || b.keep < 0 || b.keep > BUDGET_CANDIDATES || b.budget < 0 ||
      b.steps <= 0 || m % b.steps || b.per_request < 0 || b.min_cap < 0 || !aligned(b.logits, 2) || !aligned(b.slots, 4) || !aligned(scratch, 4))
    return HB_EINVAL;
  BudgetParams q{};
  q.logits = b.logits;
  q.slots = b.slots;
  q.r = m, q.e = b.e, q.k = topk, q.keep = b.keep, q.budget = b.budget, q.per_request = b.per_request, q.min_cap = b.min_cap, q.steps = b.steps,
  q.repeat = b.repeat;
  q.cands = BUDGET_CANDIDATES;
  q.cand = static_cast<int32_t*>(scratch);
  q.prob = reinterpret_cast<float*>(q.cand + (int64_t)m * BUDGET_CANDIDATES);
  q.share = q.prob;
  q.ids = ids, q.weights = weights;
  const bool small = b.e <= 512;
  if (small) {
    HB_LAUNCH((route_rank_kernel<8>), dim3((unsigned)m), dim3(64), 0, stream, q);
  } else {
    HB_LAUNCH((route_rank_kernel<16>), dim3((unsigned)m), dim3(64), 0, stream, q);
  }
  const int copies_n = small ? BUDGET_WAVES : BUDGET_WAVES / 2;
  const size_t pick_lds = (size_t)copies_n * b.e * sizeof(float);
  const int slot_cap = (int)moe_max_slots(pairs, e_n, shared_rows, slot_rows);
  if (pairs < PLAN_WIDE_PAIRS) {
    const size_t lds = std::max(pick_lds, plan_lds);
    if (small) {
      HB_LAUNCH((moe_budget_plan_kernel<8, true>), dim3(1), dim3(PLAN_THREADS), lds, stream, q, copies_n, e_lo, e_n, shared_rows, ws.plan, ws.order, slot_rows,
                slot_cap);
    } else {
      HB_LAUNCH((moe_budget_plan_kernel<16, true>), dim3(1), dim3(PLAN_THREADS), lds, stream, q, copies_n, e_lo, e_n, shared_rows, ws.plan, ws.order, slot_rows,
                slot_cap);
    }
    return HB_OK;
  }
  if (small) {
    HB_LAUNCH((moe_budget_plan_kernel<8, false>), dim3(1), dim3(PLAN_THREADS), pick_lds, stream, q, copies_n, e_lo, e_n, shared_rows, ws.plan, ws.order,
              slot_rows, slot_cap);
  } else {
    HB_LAUNCH((moe_budget_plan_kernel<16, false>), dim3(1), dim3(PLAN_THREADS), pick_lds, stream, q, copies_n, e_lo, e_n, shared_rows, ws.plan, ws.order,
              slot_rows, slot_cap);
  }
  return moe_launch_plan(ids, pairs, e_lo, e_n, shared_rows, ws, stream, slot_rows, nullptr);
}

int latent_launch_router(const LatentRouter& r, hipStream_t stream) {
  const int n = r.experts + r.latent;
  if (r.m <= 0 || r.m > LATENT_MAX_ROWS || r.hidden <= 0 || r.hidden % 512 || r.latent < 0 || r.steps <= 0) return HB_EINVAL;
  if (int err = moe_check_route(r.m, r.experts, r.topk)) return err;
  RouterGemv g{r.w, r.x, r.fused, r.lat, n, r.hidden, r.m, r.experts};
  HB_LAUNCH(latent_router_kernel, dim3((unsigned)((n + 15) / 16)), dim3(1024), 0, stream, g);
  if (!r.route) return HB_OK;
  RouteParams rp{};
  rp.sigmoid = 1;
  rp.logits = r.fused;
  rp.stride = n;
  rp.bias = r.bias;
  rp.slots = r.slots;
  rp.steps = r.steps;
  rp.repeat = r.pad_id < 0;
  rp.pad_id = r.pad_id;
  rp.e = r.experts;
  rp.k = r.topk;
  rp.per = (r.experts + 63) / 64;
  rp.latent = r.latent;
  rp.ids = r.ids;
  rp.weights = r.weights;
  rp.lat = nullptr;  // the product's epilogue has written them
  if (!r.ws) {  // no plan to fill: the routing alone
    launch_route<true>(rp, r.m, stream);
    return HB_OK;
  }
  return launch_route_plan(rp, r.m, r.e_lo, r.e_n, 0, *r.ws, stream, ROWS_PER_SLOT, nullptr);
}

int latent_launch_out(const uint16_t* fc2, const uint16_t* routed, const uint16_t* shared, uint16_t* out, int m, int hidden, int latent, hipStream_t stream) {
  if (m <= 0 || m > LATENT_MAX_ROWS || hidden <= 0 || latent <= 0 || latent % 32) return HB_EINVAL;
  const int steps = latent / 32;
  int waves = 1;
  while (waves < 16 && (steps % waves || steps / waves > 8)) waves *= 2;
  if (steps % waves || steps / waves > 8) return HB_EINVAL;
  OutGemv g{fc2, routed, shared, out, hidden, latent, m, waves};
  HB_LAUNCH(latent_out_kernel, dim3((unsigned)((hidden + 15) / 16)), dim3((unsigned)std::max(256, 64 * waves)), 0, stream, g);
  return HB_OK;
}

void moe_launch_combine(const CombineParams& c, hipStream_t stream) {
  const dim3 grid((unsigned)c.m, (unsigned)((c.h + COMBINE_SPAN - 1) / COMBINE_SPAN));
  if (c.topk <= 8 || (c.topk > 12 && c.m > 64)) {  // a long call is bound by its traffic: fewer registers, more wavefronts
    HB_LAUNCH(moe_combine_kernel<8>, grid, dim3(256), 0, stream, c);
  } else if (c.topk <= 12) {
    HB_LAUNCH(moe_combine_kernel<12>, grid, dim3(256), 0, stream, c);
  } else {
    HB_LAUNCH(moe_combine_kernel<24>, grid, dim3(256), 0, stream, c);
  }
}

}  // namespace hb

using namespace hb;

extern "C" int hb_moe_combine_pairs(const void* pairs, int pairs_bf16, const int32_t* ids, const float* weights, const void* shared,
                                    const void* x, const float* gate_vec, int e_lo, int e_n, int m, int topk, int h, void* out,
                                    void* stream) {
  if (!pairs || !ids || !weights || !out) return HB_ENULL;
  if (gate_vec && shared && !x) return HB_ENULL;
  if (m <= 0 || topk <= 0 || h <= 0 || h % 2) return HB_EINVAL;
  if (!aligned(pairs, 8) || !aligned(ids, 4) || !aligned(weights, 4) || !aligned(shared, 4) || !aligned(x, 2) || !aligned(gate_vec, 4) || !aligned(out, 4))
    return HB_EINVAL;
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
  moe_launch_combine(c, as_stream(stream));
  return launch_status();
}

// out[r, c] = bf16( bf16(silu(gate)) * up ) of BF16 rows holding `half` gate and `half` up columns: [gate | up]
// (pairs == 0) or alternating blocks of `pairs` gate columns and their `pairs` up columns. The roundings are those of
// the BF16 tensor expression silu(gate) * up (hibana/kernels/ops.py:86-92 of the reference); without CHAIN the FP32
// product is rounded once. Two columns a thread.
template <bool CHAIN>
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const uint16_t* __restrict__ x, int64_t rows, int half, int pairs, uint16_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // column pair i % (half / 2) of row i / (half / 2)
  const int per_row = half >> 1;
  if (i >= rows * per_row) return;
  const int64_t r = i / per_row;
  const int c = 2 * (int)(i - r * per_row);
  const int gate_at = pairs ? (c / pairs) * 2 * pairs + c % pairs : c, up_at = pairs ? gate_at + pairs : half + c;
  const uint16_t* row = x + r * 2 * half;
  const uint32_t g2 = *reinterpret_cast<const uint32_t*>(row + gate_at), u2 = *reinterpret_cast<const uint32_t*>(row + up_at);
  const float g0 = __uint_as_float(g2 << 16), g1 = __uint_as_float(g2 & 0xffff0000u);
  const float u0 = __uint_as_float(u2 << 16), u1 = __uint_as_float(u2 & 0xffff0000u);
  float s0 = g0 / (1.0f + expf(-g0)), s1 = g1 / (1.0f + expf(-g1));
  if (CHAIN) s0 = round_bf16(s0), s1 = round_bf16(s1);
  *reinterpret_cast<uint32_t*>(out + r * half + c) = (uint32_t)f32_to_bf16_bits(s0 * u0) | ((uint32_t)f32_to_bf16_bits(s1 * u1) << 16);
}

static int silu_mul_launch(const void* gate_up, int64_t rows, int half, int pairs, bool chain, void* out, void* stream) {
  if (!gate_up || !out) return HB_ENULL;
  if (rows <= 0 || half <= 0 || half % 2 || pairs < 0 || (pairs && (pairs % 2 || half % pairs))) return HB_EINVAL;
  if (!aligned(gate_up, 4) || !aligned(out, 4)) return HB_EINVAL;
  const int64_t threads = rows * (half / 2);
  const dim3 grid((unsigned)((threads + 255) / 256));
  if (chain) {
    hipLaunchKernelGGL(silu_and_mul_kernel<true>, grid, dim3(256), 0, as_stream(stream), static_cast<const uint16_t*>(gate_up), rows, half, pairs,
                       static_cast<uint16_t*>(out));
  } else {
    hipLaunchKernelGGL(silu_and_mul_kernel<false>, grid, dim3(256), 0, as_stream(stream), static_cast<const uint16_t*>(gate_up), rows, half, pairs,
                       static_cast<uint16_t*>(out));
  }
  return launch_status();
}

extern "C" int hb_silu_and_mul(const void* gate_up, int64_t rows, int half, int pairs, void* out, void* stream) {
  return silu_mul_launch(gate_up, rows, half, pairs, true, out, stream);
}

// bf16(silu(gate) * up) from the FP32 product: one rounding (silu_mul, hibana/kernels/flashnext_fused.py:624-639).
extern "C" int hb_silu_mul(const void* gate_up, int64_t rows, int half, int pairs, void* out, void* stream) {
  return silu_mul_launch(gate_up, rows, half, pairs, false, out, stream);
}

// (q, scales) = the per-(row, 32-group) E4M3 rounding of silu(gate) * up in one launch: BF16 [rows, 2 half] with the
// gate | up columns as in silu_and_mul_kernel -> E4M3 [rows, half], FP32 scales [rows, half / 32]. The product is
// rounded to BF16 as that kernel does it (`torch_chain`: silu to BF16 first, then the BF16 product) or from the FP32
// product with one rounding; the rounding to E4M3 is quant_groups_lane's, value for value (silu_mul_quant_groups,
// hibana/kernels/flashnext_fused.py:814-853 of the reference, with the exact divisions of its torch statement). A lane
// takes eight consecutive output columns, four lanes a group.
__global__ __launch_bounds__(256) void silu_mul_quant_groups_kernel(const uint16_t* __restrict__ x, int64_t rows, int half, int pairs, int torch_chain,
                                                                    uint8_t* __restrict__ q, float* __restrict__ scales) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // eight columns from 8 (i % (half / 8)) of row i / (half / 8)
  const int per_row = half >> 3;
  if (i >= rows * per_row) return;  // whole groups leave together: rows * per_row is a multiple of four
  const int64_t r = i / per_row;
  const int c = 8 * (int)(i - r * per_row);
  const int gate_at = pairs ? (c / pairs) * 2 * pairs + c % pairs : c, up_at = pairs ? gate_at + pairs : half + c;
  const uint16_t* row = x + r * 2 * half;
  const u32x4_t g4 = *reinterpret_cast<const u32x4_t*>(row + gate_at), u4 = *reinterpret_cast<const u32x4_t*>(row + up_at);
  float v[8];
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const float g = __uint_as_float((j & 1) ? g4[j >> 1] & 0xffff0000u : g4[j >> 1] << 16);
    const float u = __uint_as_float((j & 1) ? u4[j >> 1] & 0xffff0000u : u4[j >> 1] << 16);
    const float silu = g / (1.0f + expf(-g));
    v[j] = round_bf16(torch_chain ? round_bf16(silu) * u : silu * u);
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
  *reinterpret_cast<i32x2_t*>(q + r * half + c) = i32x2_t{lo, hi};
  if ((c & 31) == 0) scales[r * (half >> 5) + (c >> 5)] = s;
}

extern "C" int hb_silu_mul_quant_groups(const void* gate_up, int64_t rows, int half, int pairs, int torch_chain, void* q, float* scales, void* stream) {
  if (!gate_up || !q || !scales) return HB_ENULL;
  if (rows <= 0 || half <= 0 || half % 32 || pairs < 0 || (pairs && (pairs % 32 || half % pairs))) return HB_EINVAL;
  if (!aligned(gate_up, 16) || !aligned(q, 8) || !aligned(scales, 4)) return HB_EINVAL;
  const int64_t threads = rows * (half / 8);
  hipLaunchKernelGGL(silu_mul_quant_groups_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, as_stream(stream),
                     static_cast<const uint16_t*>(gate_up), rows, half, pairs, torch_chain, static_cast<uint8_t*>(q), scales);
  return launch_status();
}

// x[r, c] = bf16(relu(x[r, c])^2) in place for BF16 rows `stride` elements apart: the square in FP32, one rounding
// (torch's relu(x) ** 2; relu2_, hibana/model/nemotron/moe.py:316-321 of the reference). Two columns a thread.
__global__ __launch_bounds__(256) void relu2_kernel(uint16_t* __restrict__ x, int64_t rows, int n, int64_t stride) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int per_row = n >> 1;
  if (i >= rows * per_row) return;
  const int64_t r = i / per_row;
  uint32_t* at = reinterpret_cast<uint32_t*>(x + r * stride + 2 * (i - r * per_row));
  const uint32_t two = *at;
  const float a = fmaxf(__uint_as_float(two << 16), 0.f), b = fmaxf(__uint_as_float(two & 0xffff0000u), 0.f);
  *at = (uint32_t)f32_to_bf16_bits(a * a) | ((uint32_t)f32_to_bf16_bits(b * b) << 16);
}

extern "C" int hb_relu2(void* x, int64_t rows, int n, int64_t stride, void* stream) {
  if (!x) return HB_ENULL;
  if (rows <= 0 || n <= 0 || n % 2 || stride < n || stride % 2) return HB_EINVAL;
  if (!aligned(x, 4)) return HB_EINVAL;
  const int64_t threads = rows * (n / 2);
  hipLaunchKernelGGL(relu2_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, as_stream(stream), static_cast<uint16_t*>(x), rows, n, stride);
  return launch_status();
}

extern "C" int hb_route_softmax_topk(const float* logits, int m, int e, int k, const int32_t* slots, int steps, int repeat, int32_t* ids,
                                     float* weights, void* stream) {
  if (!logits || !ids || !weights) return HB_ENULL;
  if (m <= 0 || e <= 0 || k <= 0 || k > e || k > 64 || e > 64 * ROUTE_PER_LANE || steps <= 0) return HB_EINVAL;
  if (!aligned(logits, 4) || !aligned(slots, 4) || !aligned(ids, 4) || !aligned(weights, 4)) return HB_EINVAL;
  RouteParams p{};
  p.logits = logits;
  p.stride = e;
  p.slots = slots;
  p.steps = steps;
  p.repeat = repeat;
  p.e = e;
  p.k = k;
  p.per = (e + 63) / 64;
  p.pad_id = e;
  p.ids = ids;
  p.weights = weights;
  launch_route<false>(p, m, as_stream(stream));
  return launch_status();
}

extern "C" int hb_route_sigmoid_topk(const float* fused, int64_t stride, const float* bias, int m, int e, int k, int latent,
                                     const int32_t* slots, int steps, int repeat, int32_t* ids, float* weights, void* lat, void* stream) {
  if (!fused || !bias || !ids || !weights || (latent > 0 && !lat)) return HB_ENULL;
  if (m <= 0 || e <= 0 || k <= 0 || k > e || k > 64 || e > 64 * ROUTE_PER_LANE || latent < 0 || stride < (int64_t)e + latent || steps <= 0)
    return HB_EINVAL;
  RouteParams p{};
  p.logits = fused;
  p.stride = stride;
  p.bias = bias;
  p.slots = slots;
  p.steps = steps;
  p.repeat = repeat;
  p.e = e;
  p.k = k;
  p.per = (e + 63) / 64;
  p.pad_id = e;
  p.latent = latent;
  p.ids = ids;
  p.weights = weights;
  p.lat = static_cast<uint16_t*>(lat);
  launch_route<true>(p, m, as_stream(stream));
  return launch_status();
}

static std::mutex g_trace_lock;
static int64_t* g_trace = nullptr;
static int64_t g_trace_records = 0;
int64_t* hb::moe_trace_buffer(int64_t* records) {
  std::lock_guard<std::mutex> hold(g_trace_lock);
  *records = g_trace_records;
  return g_trace;
}
#ifndef HB_NO_DEBUG_HOOKS
extern "C" int hb_debug_trace(void* buffer, int64_t records) {
  if (records < 0 || !aligned(buffer, 8)) return HB_EINVAL;
  std::lock_guard<std::mutex> hold(g_trace_lock);
  g_trace = records > 0 ? static_cast<int64_t*>(buffer) : nullptr;
  g_trace_records = g_trace ? records : 0;
  return HB_OK;
}

extern "C" int hb_debug_events(void* const* events, int count) {
  if (count < 0 || (count > 0 && !events)) return HB_EINVAL;
  std::lock_guard<std::mutex> hold(g_events_lock);
  g_events.assign(reinterpret_cast<hipEvent_t const*>(events), reinterpret_cast<hipEvent_t const*>(events) + count);
  g_event_next = 0;
  g_events_armed.store(count > 0, std::memory_order_relaxed);
  return HB_OK;
}
#endif

extern "C" int hb_version(void) { return 1005; }  // minor: the entry points added since 1.0 (the small latent block, hb_nvfp4_gemm_ws, budgeted routing, the layer under a budget, the ring skeleton hook, hb_workspace_reset / hb_workspace_status with the counters in the caller's workspace)

extern "C" const char* hb_error_string(int code) {
  switch (code) {
    case HB_OK: return "ok";
    case HB_EINVAL: return "unsupported shape, alignment or flag";
    case HB_ENULL: return "a required pointer is null";
    case HB_EWORKSPACE: return "workspace too small";
    case HB_ELAUNCH: return "the HIP runtime refused a launch";
    case HB_ESCRATCH: return "the call needs more scratch than the library's static buffer holds";
    default: return "unknown error";
  }
}
