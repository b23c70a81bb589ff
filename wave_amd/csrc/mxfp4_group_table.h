// M tile table of a grouped GEMM: group e's rows offsets[e] .. offsets[e+1]-1 cut into tiles of bm rows.
// Entry 0 = {number of tiles}; entry 1 + t = {first row, rows, group, band}, in group order.
// band = 16 * (first tile of the tile's band) + (tiles in the band): a group's tiles form bands of at most 8
// (as equal as possible), the unit inside which the GEMM walks column by column, so that the tiles running
// together share one expert's B panels.
// The offsets are clamped, not validated: each group's range is cut to [0, total_rows] with end >= begin, and
// tiles beyond the table's capacity (total_rows / bm + num_groups entries, enough for any non-decreasing offsets)
// are dropped; a band that the capacity cuts is recorded with the height that was written, so every tile the
// walk reaches is an entry of the table and a malformed offsets array cannot make the builder or the GEMM leave
// their buffers.
// Built by one workgroup: by a launch of its own, or by the first workgroup of the launch that re-lays the
// scales out (one launch less in front of the GEMM).
//
// The arithmetic (group_tile_range, group_tile_entry, grouped_tile_of_seq) is plain C++ without any device
// intrinsic, so that a host program can run the builder and the walk over arbitrary offsets
// (tests/host_group_table.cpp does, with WAVE_GROUP_TABLE_HOST defined).
#pragma once
#include <stdint.h>

#ifdef WAVE_GROUP_TABLE_HOST
#define WAVE_HD inline
#else
#include "mxfp4_common.h"
#define WAVE_HD __host__ __device__ inline
#endif

namespace wave_mxfp4 {

WAVE_HD int group_table_capacity(int total_rows, int bm, int num_groups) { return total_rows / bm + num_groups; }

// Rows [lo, hi) of group e and the number of bm-row tiles they make.
WAVE_HD int group_tile_range(const int32_t *offsets, int e, int total_rows, int bm, int &lo, int &hi) {
  const int a = offsets[e], b = offsets[e + 1];
  lo = a < 0 ? 0 : a > total_rows ? total_rows : a;
  hi = b < lo ? lo : b > total_rows ? total_rows : b;
  return hi > lo ? (hi - lo + bm - 1) / bm : 0;
}

// Entry of tile i of a group of `tiles` tiles over rows [lo, hi) whose first tile is table tile `first_tile`;
// only called for first_tile + i < cap.
WAVE_HD void group_tile_entry(int lo, int hi, int bm, int tiles, int first_tile, int i, int e, int cap, int32_t *ent) {
  const int nb = (tiles + 7) >> 3;  // bands of the group: `rem` of height hb + 1, then the rest of height hb
  const int hb = tiles / nb, rem = tiles - hb * nb;
  const int tall = rem * (hb + 1);
  const int start = i < tall ? i / (hb + 1) * (hb + 1) : tall + (i - tall) / hb * hb;
  int height = i < tall ? hb + 1 : hb;
  if (first_tile + start + height > cap) height = cap - (first_tile + start);  // the band the capacity cuts
  ent[0] = lo + i * bm;
  ent[1] = hi - lo - i * bm < bm ? hi - lo - i * bm : bm;
  ent[2] = e;
  ent[3] = 16 * (first_tile + start) + height;
}

// Position `seq` of the tile walk (0 .. tiles * tiles_n - 1) -> (M tile, N tile): the bands one after the other,
// each column by column.  `band` is entry [3] of M tile seq / tiles_n.
WAVE_HD void grouped_tile_of_seq(int band, int seq, int tiles_n, int &tm, int &tn) {
  const int start = band >> 4, height = band & 15;
  const int in_band = seq - start * tiles_n;
  tn = in_band / height;
  tm = start + in_band - tn * height;
}

#ifndef WAVE_GROUP_TABLE_HOST
// Inclusive sum over a workgroup's threads (one value each); wave_sums: one int of LDS per wave.
__device__ __forceinline__ int block_inclusive_scan(int v, int *wave_sums, int lane, int wave) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int o = __shfl_up(v, d, 64);
    if (lane >= d) v += o;
  }
  if (lane == 63) wave_sums[wave] = v;
  __syncthreads();
  int before = 0;
  for (int w = 0; w < wave; ++w) before += wave_sums[w];
  __syncthreads();
  return v + before;
}

// All NT threads of one workgroup call this; wave_sums: NT / 64 ints of LDS, carry: one.
template <int NT>
__device__ __forceinline__ void build_group_tile_table(const GroupTableArgs &g, int *wave_sums, int *carry) {
  const int cap = group_table_capacity(g.total_rows, g.bm, g.num_groups);
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  if (t == 0) *carry = 0;
  __syncthreads();
  for (int e0 = 0; e0 < g.num_groups; e0 += NT) {
    const int e = e0 + t;
    int lo = 0, tiles = 0, hi = 0;
    if (e < g.num_groups) tiles = group_tile_range(g.offsets, e, g.total_rows, g.bm, lo, hi);
    const int base = *carry;  // read before anyone moves it on
    const int end = block_inclusive_scan(tiles, wave_sums, lane, wave);
    const int first_tile = base + end - tiles;
    for (int i = 0; i < tiles && first_tile + i < cap; ++i)
      group_tile_entry(lo, hi, g.bm, tiles, first_tile, i, e, cap, g.table + 4 * (1 + first_tile + i));
    __syncthreads();
    if (t == NT - 1) *carry = base + end;
    __syncthreads();
  }
  if (t == 0) g.table[0] = min(*carry, cap);
}
#endif  // WAVE_GROUP_TABLE_HOST

}  // namespace wave_mxfp4
