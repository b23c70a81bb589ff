// M tile table of a grouped GEMM: group e's rows offsets[e] .. offsets[e+1]-1 cut into tiles of bm rows.
// Entry 0 = {number of tiles T, number of full tiles F}; entry 1 + t = {first row, rows, group, band}.
// With short_rows = 0 every tile is "full": F = T, tiles in group order.  With short_rows > 0 a group's last
// tile of at most short_rows rows is a "short" tile: the full tiles come first (entries 1 .. F, in group order),
// the short ones after them (entries F + 1 .. T), and the GEMM runs the full tiles first and the short ones last,
// with a cheaper loop (a short tile costs about a third of a full one; among the full ones it would take a whole
// turn of its workgroup, and the problem would end as late as if it were full).
// band = 16 * (first tile of the tile's band) + (tiles in the band): a group's full tiles form bands of at most 8
// (as equal as possible), the unit inside which the GEMM walks column by column, so that the tiles running
// together share one expert's B panels; a short tile is a band of its own.
// The offsets are clamped, not validated: each group's range is cut to [0, total_rows] with end >= begin, and
// tiles beyond the table's capacity (total_rows / bm + num_groups entries, enough for any non-decreasing offsets)
// are dropped; a band that the capacity cuts is recorded with the height that was written, so every tile the
// walk reaches is an entry of the table and a malformed offsets array cannot make the builder or the GEMM leave
// their buffers.
// Built by one workgroup: by a launch of its own, or by the first workgroup of the launch that re-lays the
// scales out (one launch less in front of the GEMM).
//
// The arithmetic (group_tile_range, group_tile_entry, grouped_tile_of_id) is plain C++ without any device
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

// Rows [lo, hi) of group e, the number of bm-row tiles they make, and whether the last of them is a short tile.
WAVE_HD int group_tile_range(const int32_t *offsets, int e, int total_rows, int bm, int short_rows, int &lo, int &hi,
                             int &has_short) {
  const int a = offsets[e], b = offsets[e + 1];
  lo = a < 0 ? 0 : a > total_rows ? total_rows : a;
  hi = b < lo ? lo : b > total_rows ? total_rows : b;
  const int tiles = hi > lo ? (hi - lo + bm - 1) / bm : 0;
  has_short = tiles > 0 && hi - lo - (tiles - 1) * bm <= short_rows ? 1 : 0;
  return tiles;
}

// Entry of full tile i of a group with `full` full tiles over rows [lo, hi) whose first full tile is table tile
// `first_tile`; only called for first_tile + i < cap_full (the entries left for full tiles).
WAVE_HD void group_tile_entry(int lo, int hi, int bm, int full, int first_tile, int i, int e, int cap_full, int32_t *ent) {
  const int nb = (full + 7) >> 3;  // bands of the group: `rem` of height hb + 1, then the rest of height hb
  const int hb = full / nb, rem = full - hb * nb;
  const int tall = rem * (hb + 1);
  const int start = i < tall ? i / (hb + 1) * (hb + 1) : tall + (i - tall) / hb * hb;
  int height = i < tall ? hb + 1 : hb;
  if (first_tile + start + height > cap_full) height = cap_full - (first_tile + start);  // the band the capacity cuts
  ent[0] = lo + i * bm;
  ent[1] = hi - lo - i * bm < bm ? hi - lo - i * bm : bm;
  ent[2] = e;
  ent[3] = 16 * (first_tile + start) + height;
}

// Entry of a group's short tile (its last, tile `tiles - 1` of the group), table tile `index`.
WAVE_HD void group_short_entry(int lo, int hi, int bm, int tiles, int index, int e, int32_t *ent) {
  ent[0] = lo + (tiles - 1) * bm;
  ent[1] = hi - lo - (tiles - 1) * bm;
  ent[2] = e;
  ent[3] = 16 * index + 1;
}

// Position `seq` of the walk over the full tiles (0 .. F * tiles_n - 1) -> (M tile, N tile): the bands one after
// the other, each column by column.  `band` is entry [3] of M tile seq / tiles_n.
WAVE_HD void grouped_tile_of_seq(int band, int seq, int tiles_n, int &tm, int &tn) {
  const int start = band >> 4, height = band & 15;
  const int in_band = seq - start * tiles_n;
  tn = in_band / height;
  tm = start + in_band - tn * height;
}

// The walk.  Workgroup ids are dealt round-robin over the 8 XCDs (each with its own L2), so ids are regrouped: an
// XCD owns one contiguous run of the full tiles' sequence (ids 0 .. PF - 1, PF = F * tiles_n rounded up to 8) and
// one of the short tiles' (ids PF .. PF + PS - 1).  Returns the number of ids; an id maps to a tile or (padding of
// either part) to none.
WAVE_HD int grouped_walk_ids(int tiles, int full, int tiles_n) {
  return (full * tiles_n + 7) / 8 * 8 + ((tiles - full) * tiles_n + 7) / 8 * 8;
}
// `band_of(t)` returns entry [3] of table tile t.
template <class BandOf>
WAVE_HD bool grouped_tile_of_id(int tiles, int full, int tiles_n, int id, BandOf band_of, int &tm, int &tn) {
  const int nf = full * tiles_n, per_f = (nf + 7) / 8;
  if (id < per_f * 8) {
    const int seq = (id % 8) * per_f + id / 8;
    if (seq >= nf) return false;
    grouped_tile_of_seq(band_of(seq / tiles_n), seq, tiles_n, tm, tn);
    return true;
  }
  const int ns = (tiles - full) * tiles_n, per_s = (ns + 7) / 8, ids = id - per_f * 8;
  const int seq = (ids % 8) * per_s + ids / 8;
  if (ids >= per_s * 8 || seq >= ns) return false;
  tm = full + seq / tiles_n;
  tn = seq - (seq / tiles_n) * tiles_n;
  return true;
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

// All NT threads of one workgroup call this; wave_sums: NT / 64 ints of LDS, carry: two.
template <int NT>
__device__ __forceinline__ void build_group_tile_table(const GroupTableArgs &g, int *wave_sums, int *carry) {
  const int cap = group_table_capacity(g.total_rows, g.bm, g.num_groups);
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  // first pass: the number of full tiles (the short ones' entries start behind them)
  if (t == 0) carry[0] = carry[1] = 0;
  __syncthreads();
  for (int e0 = 0; e0 < g.num_groups; e0 += NT) {
    const int e = e0 + t;
    int lo, hi, has_short = 0, tiles = 0;
    if (e < g.num_groups) tiles = group_tile_range(g.offsets, e, g.total_rows, g.bm, g.short_rows, lo, hi, has_short);
    const int end = block_inclusive_scan(tiles - has_short, wave_sums, lane, wave);
    if (t == NT - 1) carry[0] += end;
    __syncthreads();
  }
  const int full_all = carry[0], cap_full = min(full_all, cap);
  __syncthreads();
  if (t == 0) carry[0] = 0;
  __syncthreads();
  for (int e0 = 0; e0 < g.num_groups; e0 += NT) {
    const int e = e0 + t;
    int lo = 0, hi = 0, has_short = 0, tiles = 0;
    if (e < g.num_groups) tiles = group_tile_range(g.offsets, e, g.total_rows, g.bm, g.short_rows, lo, hi, has_short);
    const int full = tiles - has_short;
    const int base_f = carry[0], base_s = carry[1];  // read before anyone moves them on
    const int end_f = block_inclusive_scan(full, wave_sums, lane, wave);
    const int end_s = block_inclusive_scan(has_short, wave_sums, lane, wave);
    const int first_tile = base_f + end_f - full;
    for (int i = 0; i < full && first_tile + i < cap_full; ++i)
      group_tile_entry(lo, hi, g.bm, full, first_tile, i, e, cap_full, g.table + 4 * (1 + first_tile + i));
    const int short_index = cap_full + base_s + end_s - has_short;
    if (has_short && short_index < cap) group_short_entry(lo, hi, g.bm, tiles, short_index, e, g.table + 4 * (1 + short_index));
    __syncthreads();
    if (t == NT - 1) carry[0] = base_f + end_f, carry[1] = base_s + end_s;
    __syncthreads();
  }
  if (t == 0) {
    g.table[0] = min(cap_full + carry[1], cap);
    g.table[1] = cap_full;
  }
}
#endif  // WAVE_GROUP_TABLE_HOST

}  // namespace wave_mxfp4
