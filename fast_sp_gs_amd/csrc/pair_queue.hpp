// Per-wavefront queue of blended (pixel, entry) pairs, in LDS: the bookkeeping the two-pass blend backwards share.
//
// The order-bound pass of a backward kernel walks a tile's list one entry per pass; the pixels that blend the entry
// (a quarter of the 64 on average) each leave one 16-byte item. The items of an entry are padded to whole 16-lane
// rows, so that the order-free pass -- 64 items at a time, every lane one item -- can sum a row's gradient components
// with DPP row shifts alone: a row never mixes entries. The ring holds 128 items in two halves of 64; a pass appends
// at most 64, a full half is drained as soon as there is one, so a drain always starts at a half and the ring never
// holds more than 48 + 64 items. Which entry each of the ring's eight rows holds is kept in a 64-bit scalar, a byte
// per row; everything here is wave-uniform except the item a lane writes or reads.
#pragma once
#include "blend.hpp"

namespace fsgs {

constexpr int kQueueItems = 128;
// item.w: pixel of the quadrant (6 bits) | blends (bit 12) | met by the ray-splat intersection rather than by its
// projected centre (bit 13)
constexpr int kItemHit = 1 << 12, kItemRay = 1 << 13;

struct PairQueue {
  int head = 0, count = 0;        // items [head, head + count) of the ring; multiples of 16, head is 0 or 64
  unsigned long long rows = 0ull;  // entry (staging slot, < 256) of each of the ring's eight rows
};

// Appends the items of entry `j`: lanes with `hit` (the lanes of `pass`) store (a, b, c, own pixel | flags) in lane
// order, the next lanes fill the last row up with neutral items (zeros, no flags, their own pixel: every number a drain
// forms from such an item is finite and multiplies a zero). Returns true when a half is full and must be drained.
__device__ __forceinline__ bool queue_append(float4* __restrict__ ring, PairQueue& q, int j, bool hit,
                                             unsigned long long pass, float a, float b, float c, int flags) {
  const int lane  = __lane_id();
  const int n_hit = (int) __popcll(pass), n_pad = (n_hit + 15) & ~15;
  const int below = (int) __builtin_amdgcn_mbcnt_hi((unsigned) (pass >> 32),
                                                    __builtin_amdgcn_mbcnt_lo((unsigned) pass, 0u));
  const int place = hit ? below : n_hit + (lane - below);
  const int tail  = q.head + q.count;  // first free place of the ring (mod its size), a multiple of 16
  if (place < n_pad)
    ring[(tail + place) & (kQueueItems - 1)] =
        make_float4(hit ? a : 0.0f, hit ? b : 0.0f, hit ? c : 0.0f, __int_as_float(lane | (hit ? flags : 0)));
  for (int r = 0; r < n_pad; r += 16) {
    const int sh = (((tail + r) & (kQueueItems - 1)) >> 4) * 8;
    q.rows = (q.rows & ~(0xffull << sh)) | ((unsigned long long) j << sh);
  }
  q.count += n_pad;
  return q.count >= kWave;
}

// The four rows at the front of the queue: byte r of the result = entry of row r.
__device__ __forceinline__ unsigned queue_front_rows(const PairQueue& q) { return (unsigned) (q.rows >> (q.head >> 1)); }

// After a drain of n_valid items: a full pass leaves the other half of the ring in front; the last, partial pass of a
// batch empties the queue.
__device__ __forceinline__ void queue_pop(PairQueue& q, int n_valid) {
  if (n_valid >= kWave) q.head ^= kWave, q.count -= kWave;
  else q.head = 0, q.count = 0;
}

// Adds the row totals a drain formed (`own`: lane (row, c) holds its row's total of component c) to the accumulator
// rows of the rows' entries. The accumulator belongs to this wavefront alone, so a row adds with a plain read and write,
// provided no two rows of the pass write the same entry: rows 2k and 2k + 1 of one entry are added in registers first
// (one row swap) and row 2k writes for both; a run that continues from row 1 into row 2 makes row 2 wait for a second
// round. Rows past n_valid hold old items and stay silent. `acc`: this lane's component of its row's entry;
// `before`: its value, read when the drain began (the read is then off the critical path); `active`: the lane holds a
// component at all (the same lanes of every row).
__device__ __forceinline__ void queue_accumulate(float* acc, float before, float own, unsigned jrows, int n_valid,
                                                 bool active) {
  const int lane = __lane_id(), row = lane >> 4;
  const int rows_valid = (n_valid + 15) >> 4;
  const int j0 = (int) (jrows & 255u), j1 = rows_valid > 1 ? (int) ((jrows >> 8) & 255u) : -1;
  const int j2 = rows_valid > 2 ? (int) ((jrows >> 16) & 255u) : -2, j3 = rows_valid > 3 ? (int) ((jrows >> 24) & 255u) : -3;
  const bool s01 = j0 == j1, s12 = j1 == j2, s23 = j2 == j3;
  float lo = own, hi = own;  // after the swap: lo = rows (0, 0, 2, 2), hi = rows (1, 1, 3, 3) of `own`
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32_e32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
  const float pair = lo + hi;
  const bool joined = (row == 0 && s01) || (row == 2 && s23);  // this row writes for its odd neighbour too
  const bool silent = (row == 1 && s01) || (row == 3 && s23) || row >= rows_valid || !active;
  const float mine  = joined ? pair : own;
  if (!silent && !(row == 2 && s12)) *acc = before + mine;
  if (s12) {  // wave-uniform; the LDS serves a wavefront's accesses in order, so this read sees row 0 / 1's store
    if (row == 2 && !silent) *acc = *(volatile float*) acc + mine;  // re-read: rows 0 / 1 may just have written it
  }
}

}  // namespace fsgs
