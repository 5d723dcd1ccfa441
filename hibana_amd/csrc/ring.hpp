// The weight ring of the stream kernels.
//
// Weight chunks do not wait in registers. A wavefront owns RING_CHUNKS block-sized slots of LDS and fills them with
// LDS-direct loads (buffer_load ... lds: memory to LDS, no register in between), two chunks ahead of the one it expands;
// when a chunk's turn comes its block is read from the slot into registers and the slot is given to the chunk
// two further on. Only the lanes that asked for a block read it back, so no barrier is involved: a wavefront waits on
// its own vector-memory counter. A chunk in flight costs no registers this way: two of them stand behind the one
// being expanded where register double-buffering affords one, and a wavefront's registers go to one chunk's codes, its
// activations and the accumulators.
//
// The counter is shared by everything a wavefront has asked of memory, in order. A chunk's block is a few LDS-direct
// loads (Ring::LOADS), asked for two chunks ahead, right after the slot it goes to has been read; the chunk's
// activation loads (Acts::LOADS of them) are asked for one chunk later, when their registers are free. The compiler may move those
// among the other requests made between two reads of the ring, but not across a read (the reads are volatile
// statements that clobber memory). So when chunk i is due, everything asked for since the read before stands behind
// its block: the block of chunk i + 1 and one chunk's activation loads at least. Waiting until at most that many
// requests remain outstanding is waiting for chunk i, and hardly longer. The last chunk waits for everything. The
// LDS-direct loads go through a buffer descriptor of the block row (the MUBUF form: around it the compiler keeps exact
// count of its own loads, which it gives up around the FLAT form), and the ring is read with explicit ds_read_b128, so
// the only waits on these transfers are the ones written here.
#pragma once

#include "stream_common.hpp"

namespace hb {

constexpr int RING_CHUNKS = 2;
template <class Ring>
constexpr int ring_bytes() { return RING_CHUNKS * Ring::BLOCK_BYTES; }
typedef __attribute__((address_space(3))) uint8_t* lds_ptr_t;

struct RingSource {
  __amdgpu_buffer_rsrc_t row;  // the block row: chunks x Ring::BLOCK_BYTES
  uint32_t codes, scales;      // the lane's byte offsets in a block for its loads of codes and of scales
};

// A format's Ring gives: Chunk (the registers of a block), BLOCK_BYTES, LOADS (LDS-direct loads a block),
// lanes() (the lane's offsets for asking and for reading back), request() (ask for a chunk's block into a slot) and
// take<BEHIND, SLOT>() (wait until at most BEHIND requests are outstanding, read slot SLOT into the registers, wait for
// the reads). A body's Acts gives: LOADS (activation loads a chunk), start() and step<ODD, MORE2, MORE1>().

// Chunks c0 .. c1 - 1 (at least one) of block row `nb`, through the wavefront's ring, for the slot's rows from row0 (the
// four-row bodies: row0 .. row0 + 3; the sixteen-row body: all, row0 = 0).
// `acts`: the body's state (the caller's object when the body keeps results of its own beside the four accumulators).
template <int EPI, class Acts, class Ring>
__device__ __forceinline__ void stream_block(const StreamParams& p, const Slot& sl, int row0, int nb, int c0, int c1, int lane, uint8_t* ring,
                                             f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3, Acts& acts) {
  constexpr int BEHIND = Ring::LOADS + Acts::LOADS;
  const int r16 = lane & 15, n = c1 - c0;
  RingSource src;
  src.row = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(sl.w + (int64_t)nb * p.chunks * Ring::BLOCK_BYTES), 0,
                                              p.chunks * Ring::BLOCK_BYTES, 0x00020000);
  const lds_ptr_t slot0 = (lds_ptr_t)ring, slot1 = (lds_ptr_t)(ring + Ring::BLOCK_BYTES);
  uint32_t codes, scales;  // LDS byte addresses of what the lane reads back from slot 0; the reads select the slot by their offset
  Ring::lanes(src, lane, r16, (uint32_t)(uintptr_t)slot0, codes, scales);
  typename Ring::Chunk ch;
  Ring::request(src, c0, slot0);
  asm volatile("" ::: "memory");  // whatever else the prologue asks for stands behind the first block
  acts.template start<EPI>(p, sl, row0, c0, n, lane);
  if (n == 1) {
    Ring::template take<0, 0>(ch, codes, scales);
    acts.template step<0, false, false>(ch, 0, acc0, acc1, acc2, acc3, sl);
  } else {
    Ring::request(src, c0 + 1, slot1);
    int i = 0;
    for (; i + 3 < n; i += 2) {  // chunks i and i + 1, asking for the blocks of i + 2 and i + 3
      Ring::template take<BEHIND, 0>(ch, codes, scales);
      Ring::request(src, c0 + i + 2, slot0);
      acts.template step<0, true, true>(ch, i, acc0, acc1, acc2, acc3, sl);
      Ring::template take<BEHIND, 1>(ch, codes, scales);
      Ring::request(src, c0 + i + 3, slot1);
      acts.template step<1, true, true>(ch, i + 1, acc0, acc1, acc2, acc3, sl);
    }
    if (i + 3 == n) {  // three left: the block of i + 2 is still to ask for
      Ring::template take<BEHIND, 0>(ch, codes, scales);
      Ring::request(src, c0 + i + 2, slot0);
      acts.template step<0, true, true>(ch, i, acc0, acc1, acc2, acc3, sl);
      Ring::template take<BEHIND, 1>(ch, codes, scales);
      acts.template step<1, false, true>(ch, i + 1, acc0, acc1, acc2, acc3, sl);
      Ring::template take<0, 0>(ch, codes, scales);
      acts.template step<0, false, false>(ch, i + 2, acc0, acc1, acc2, acc3, sl);
    } else {  // two left, both asked for
      Ring::template take<BEHIND, 0>(ch, codes, scales);
      acts.template step<0, false, true>(ch, i, acc0, acc1, acc2, acc3, sl);
      Ring::template take<0, 1>(ch, codes, scales);
      acts.template step<1, false, false>(ch, i + 1, acc0, acc1, acc2, acc3, sl);
    }
  }
}

template <int EPI, class Acts, class Ring>
__device__ __forceinline__ void stream_block(const StreamParams& p, const Slot& sl, int row0, int nb, int c0, int c1, int lane, uint8_t* ring,
                                             f32x4_t& acc0, f32x4_t& acc1, f32x4_t& acc2, f32x4_t& acc3) {
  Acts acts;
  stream_block<EPI, Acts, Ring>(p, sl, row0, nb, c0, c1, lane, ring, acc0, acc1, acc2, acc3, acts);
}

}  // namespace hb
