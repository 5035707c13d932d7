// Tile GEMMs whose K range is split over workgroups: which workgroup of a launch computes which (tile, K part), and
// how the K parts of a tile become one result.
#pragma once
#include "vaq_common.h"

namespace vaq {

// The (tile, K part) of a workgroup.  Two launch forms:
//  * every tile in `sk` parts: grid (tiles, sk), the part is blockIdx.y;
//  * only the tiles from `tail_first` on (in the order the workgroups take tiles) in `sk` parts, the ones before it whole:
//    grid (tail_first + (tiles - tail_first) * sk).  For tile counts that end in a partly filled round of workgroups:
//    the whole tiles fill the full rounds, the parts of the others fill the last one.
// Consecutive workgroup ids land on different XCDs (round-robin over 8); each XCD gets one contiguous range of tile
// positions (of the whole tiles and of the split ones separately), so that the tiles resident on an XCD are neighbours
// and share operand rows in its L2.  `pos` is the position in tile order, `unit` = the tile's index among the split
// tiles (scratch and counters are laid out by it).
struct TileSlot {
  int pos, split, nsplit, unit, units;
};

__device__ inline TileSlot tile_slot(int tiles, int sk, int tail_first) {
  TileSlot r;
  int b = blockIdx.x;
  if (tail_first > 0) {
    const int rest = tiles - tail_first;
    if (b < tail_first) {
      if (tail_first % 8 == 0) b = (b & 7) * (tail_first / 8) + (b >> 3);
      r.pos = b;
      r.split = 0;
      r.nsplit = 1;
      r.unit = 0;
    } else {
      int q = b - tail_first;
      r.split = q / rest;
      q -= r.split * rest;
      if (rest % 8 == 0 && tail_first % 8 == 0) q = (q & 7) * (rest / 8) + (q >> 3);
      r.pos = tail_first + q;
      r.nsplit = sk;
      r.unit = q;
    }
    r.units = rest;
    return r;
  }
  if (tiles % 8 == 0) b = (b & 7) * (tiles / 8) + (b >> 3);
  r.pos = b;
  r.split = blockIdx.y;
  r.nsplit = sk;
  r.unit = b;
  r.units = tiles;
  return r;
}

// Hand-over of partial tiles.  Each wavefront owns WMB x WNB accumulator blocks of its workgroup's tile and one arrival
// counter per (split tile, wavefront) in the caller's zeroed `counters`.  Every wavefront stores its partial blocks
// (16-byte buffer stores with the sc1 cache-policy bit: device scope, written through to and read from memory that all
// XCDs share -- each XCD has its own L2), waits for their acknowledgement and adds one to the counter; the one that
// finds nsplit - 1 there is the last and sums all parts in split order, starting from zero (the same additions whoever
// is last, so the result does not depend on the order of arrival), and leaves the counter zero.
// (Measured against it on 4096 x 4096 at M = 1024 / 2048 in 2, 4 and 8 parts: a number drawn at the start of the
// kernel that names the summing wavefront, so that it need not store and the others need not be read twice, with a
// bounded wait for the others -- same time in 2 parts, 16-30 % slower in 4 and 8: the wait and its polling cost more
// than the stores they save.  Without any hand-over the same launches take 68 against 83 us in 2 parts of 128 tiles.)
//
// true: this wavefront holds the tile's full sums in `acc` and runs the epilogue; false: it has handed its part over.
template <int WMB, int WNB, int NW>
__device__ inline bool handover_finish(float* c_tmp, int32_t* counters, v16f (&acc)[WMB][WNB], const TileSlot& sl, int wave,
                                       int lane) {
  constexpr int NV4 = WMB * WNB * 4;                       // 16-byte pieces per lane; one unit = NV4 KiB per wavefront
  constexpr int SC1 = 16;
  const int nsplit = sl.nsplit;
  const uint32_t unit = (uint32_t)((sl.unit * NW + wave) * NV4) * 1024u;          // bytes
  const uint32_t split_stride = (uint32_t)sl.units * (uint32_t)(NW * NV4) * 1024u;
  const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc(c_tmp, 0, (int)(split_stride * (uint32_t)nsplit), 0x00020000);
#pragma unroll
  for (int i = 0; i < WMB; ++i)
#pragma unroll
    for (int j = 0; j < WNB; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v4f v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v), rt, lane * 16,
                                               (int)(sl.split * split_stride + unit + ((i * WNB + j) * 4 + q) * 1024), SC1);
      }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // the part is acknowledged before the counter moves
  int32_t* ctr = counters + (int64_t)sl.unit * NW + wave;
  int old = 0;
  if (lane == 0) old = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  old = __builtin_amdgcn_readfirstlane(old);      // lane 0 holds it; a scalar keeps what depends on it scalar
  if (old != nsplit - 1) return false;
  // CH pieces of two parts in flight at a time (one piece after the other, every load waited for, the last arriver
  // spent NV4 x nsplit memory round trips here); each element is summed in split order, starting from zero.  The last
  // arriver reads its own part back as well: keeping it in registers across this loop instead costs the kernels that
  // run at the register limit more (spills in their main loops) than the reads it saves.
  constexpr int CH = NV4 < 8 ? NV4 : 8;
#pragma unroll
  for (int c0 = 0; c0 < NV4; c0 += CH) {
    v4f sum[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) sum[c] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < nsplit; s0 += 2) {
      const int s1 = s0 + 1 < nsplit ? s0 + 1 : s0;
      v4u r0[CH], r1[CH];
#pragma unroll
      for (int c = 0; c < CH; ++c)
        r0[c] = __builtin_amdgcn_raw_buffer_load_b128(rt, lane * 16, (int)(s0 * split_stride + unit + (c0 + c) * 1024), SC1);
#pragma unroll
      for (int c = 0; c < CH; ++c)
        r1[c] = __builtin_amdgcn_raw_buffer_load_b128(rt, lane * 16, (int)(s1 * split_stride + unit + (c0 + c) * 1024), SC1);
#pragma unroll
      for (int c = 0; c < CH; ++c) sum[c] += __builtin_bit_cast(v4f, r0[c]);
      if (s0 + 1 < nsplit) {
#pragma unroll
        for (int c = 0; c < CH; ++c) sum[c] += __builtin_bit_cast(v4f, r1[c]);
      }
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int pc = c0 + c, ij = pc / 4, q = pc % 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[ij / WNB][ij % WNB][4 * q + e] = sum[c][e];
    }
  }
  if (lane == 0) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return true;
}

}  // namespace vaq
