// M tile table of a grouped GEMM: group e's rows offsets[e] .. offsets[e+1]-1 cut into tiles of bm rows.
// Entry 0 = {number of tiles}; entry 1 + t = {first row, rows, group, band}, in group order.
// band = 16 * (first tile of the tile's band) + (tiles in the band): a group's tiles form bands of at most 8
// (as equal as possible), the unit inside which the GEMM walks column by column, so that the tiles running
// together share one expert's B panels.
// The offsets are clamped, not validated: each group's range is cut to [0, total_rows] with end >= begin, and
// tiles beyond the table's capacity (total_rows / bm + num_groups entries, enough for any non-decreasing offsets)
// are dropped, so a malformed offsets array cannot make the builder or the GEMM leave their buffers.
// Built by one workgroup: by a launch of its own, or by the first workgroup of the launch that re-lays the
// scales out (one launch less in front of the GEMM).
#pragma once
#include "mxfp4_common.h"

namespace wave_mxfp4 {

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
  const int cap = g.total_rows / g.bm + g.num_groups;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  if (t == 0) *carry = 0;
  __syncthreads();
  for (int e0 = 0; e0 < g.num_groups; e0 += NT) {
    const int e = e0 + t;
    int lo = 0, tiles = 0, hi = 0;
    if (e < g.num_groups) {
      lo = min(max(g.offsets[e], 0), g.total_rows), hi = min(max(g.offsets[e + 1], lo), g.total_rows);
      tiles = hi > lo ? (hi - lo + g.bm - 1) / g.bm : 0;
    }
    const int base = *carry;  // read before anyone moves it on
    const int end = block_inclusive_scan(tiles, wave_sums, lane, wave);
    const int nb = (tiles + 7) >> 3;  // bands of the group: `rem` of height hb + 1, then the rest of height hb
    const int hb = nb ? tiles / nb : 0, rem = nb ? tiles - hb * nb : 0;
    const int first_tile = base + end - tiles;
    for (int i = 0; i < tiles && first_tile + i < cap; ++i) {
      int32_t *ent = g.table + 4 * (1 + first_tile + i);
      ent[0] = lo + i * g.bm;
      ent[1] = min(g.bm, hi - lo - i * g.bm);
      ent[2] = e;
      const int tall = rem * (hb + 1);
      const int start = i < tall ? i / (hb + 1) * (hb + 1) : tall + (i - tall) / hb * hb;
      ent[3] = 16 * (first_tile + start) + (i < tall ? hb + 1 : hb);
    }
    __syncthreads();
    if (t == NT - 1) *carry = base + end;
    __syncthreads();
  }
  if (t == 0) g.table[0] = min(*carry, cap);
}

}  // namespace wave_mxfp4
