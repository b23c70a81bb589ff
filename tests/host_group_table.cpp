// Host harness for the M tile table of the grouped GEMM (wave_amd/csrc/mxfp4_group_table.h): runs the builder's
// and the tile walk's own arithmetic on the CPU over offsets arrays read from stdin and checks that every tile
// the walk reaches is an entry the builder wrote, with rows, group and N tile in range.
// Input: lines "total_rows bm tiles_n short_rows num_groups off_0 ... off_G".  Output per line: "ok <tiles> <short
// tiles>" or "BAD <why>".
// Built and driven by tests/test_group_table_host.py (g++, no GPU).
#define WAVE_GROUP_TABLE_HOST
#include "../wave_amd/csrc/mxfp4_group_table.h"

#include <cstdio>
#include <vector>

using namespace wave_mxfp4;

int main() {
  int total_rows, bm, tiles_n, groups, short_rows;
  while (std::scanf("%d %d %d %d %d", &total_rows, &bm, &tiles_n, &short_rows, &groups) == 5) {
    std::vector<int32_t> off(groups + 1);
    for (auto &o : off)
      if (std::scanf("%d", &o) != 1) return 2;
    const int cap = group_table_capacity(total_rows, bm, groups);
    const int32_t unwritten = INT32_MIN;
    std::vector<int32_t> table(4 * (1 + cap), unwritten);
    // what the device builder's two passes and scans hand each group
    int full_all = 0;
    for (int e = 0; e < groups; ++e) {
      int lo, hi, has_short;
      full_all += group_tile_range(off.data(), e, total_rows, bm, short_rows, lo, hi, has_short) - has_short;
    }
    const int cap_full = full_all < cap ? full_all : cap;
    int carry_f = 0, carry_s = 0;
    for (int e = 0; e < groups; ++e) {
      int lo, hi, has_short;
      const int tiles = group_tile_range(off.data(), e, total_rows, bm, short_rows, lo, hi, has_short);
      const int full = tiles - has_short;
      for (int i = 0; i < full && carry_f + i < cap_full; ++i)
        group_tile_entry(lo, hi, bm, full, carry_f, i, e, cap_full, table.data() + 4 * (1 + carry_f + i));
      const int short_index = cap_full + carry_s;
      if (has_short && short_index < cap) group_short_entry(lo, hi, bm, tiles, short_index, e, table.data() + 4 * (1 + short_index));
      carry_f += full;
      carry_s += has_short;
    }
    const int count = cap_full + carry_s < cap ? cap_full + carry_s : cap;
    table[0] = count;
    table[1] = cap_full;
    const char *bad = nullptr;
    std::vector<int> seen((size_t)count * tiles_n, 0);
    const int ids = grouped_walk_ids(count, cap_full, tiles_n);
    int shorts_seen = 0;
    for (int id = 0; id < ids && !bad; ++id) {
      int tm = -1, tn = -1;
      bool unwritten_band = false;
      const bool hit = grouped_tile_of_id(count, cap_full, tiles_n, id, [&](int t) {
        if (t < 0 || t >= count || table[4 * (1 + t) + 3] == unwritten) { unwritten_band = true; return 16 * 0 + 1; }
        return (int)table[4 * (1 + t) + 3];
      }, tm, tn);
      if (unwritten_band) { bad = "band of an unwritten entry"; break; }
      if (!hit) continue;
      if (tm < 0 || tm >= count) { bad = "M tile outside the table"; break; }
      if (tn < 0 || tn >= tiles_n) { bad = "N tile out of range"; break; }
      const int32_t *ent = table.data() + 4 * (1 + tm);
      if (ent[0] == unwritten) { bad = "unwritten entry"; break; }
      if (ent[0] < 0 || ent[1] < 1 || ent[1] > bm || ent[0] + ent[1] > total_rows) { bad = "rows out of range"; break; }
      if (ent[2] < 0 || ent[2] >= groups) { bad = "group out of range"; break; }
      if ((ent[3] & 15) < 1) { bad = "empty band"; break; }
      if (tm >= cap_full) {
        if (ent[1] > short_rows) { bad = "a short tile with too many rows"; break; }
        ++shorts_seen;
      }
      // the full tiles come first: a short tile's id is beyond every full tile's
      if (tm >= cap_full && id < (cap_full * tiles_n + 7) / 8 * 8) { bad = "short tile among the full ones"; break; }
      if (seen[(size_t)tm * tiles_n + tn]++) { bad = "tile visited twice"; break; }
    }
    if (!bad)
      for (int v : seen)
        if (v != 1) { bad = "tile never visited"; break; }
    if (bad) std::printf("BAD %s\n", bad);
    else std::printf("ok %d %d\n", count, count - cap_full);
  }
  return 0;
}
