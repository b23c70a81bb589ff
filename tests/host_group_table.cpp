// Host harness for the M tile table of the grouped GEMM (wave_amd/csrc/mxfp4_group_table.h): runs the builder's
// and the tile walk's own arithmetic on the CPU over offsets arrays read from stdin and checks that every tile
// the walk reaches is an entry the builder wrote, with rows, group and N tile in range.
// Input: lines "total_rows bm tiles_n num_groups off_0 ... off_G".  Output per line: "ok <tiles>" or "BAD <why>".
// Built and driven by tests/test_group_table_host.py (g++, no GPU).
#define WAVE_GROUP_TABLE_HOST
#include "../wave_amd/csrc/mxfp4_group_table.h"

#include <cstdio>
#include <vector>

using namespace wave_mxfp4;

int main() {
  int total_rows, bm, tiles_n, groups;
  while (std::scanf("%d %d %d %d", &total_rows, &bm, &tiles_n, &groups) == 4) {
    std::vector<int32_t> off(groups + 1);
    for (auto &o : off)
      if (std::scanf("%d", &o) != 1) return 2;
    const int cap = group_table_capacity(total_rows, bm, groups);
    const int32_t unwritten = INT32_MIN;
    std::vector<int32_t> table(4 * (1 + cap), unwritten);
    int carry = 0;  // what the device builder's scan hands each group
    for (int e = 0; e < groups; ++e) {
      int lo, hi;
      const int tiles = group_tile_range(off.data(), e, total_rows, bm, lo, hi);
      for (int i = 0; i < tiles && carry + i < cap; ++i)
        group_tile_entry(lo, hi, bm, tiles, carry, i, e, cap, table.data() + 4 * (1 + carry + i));
      carry += tiles;
    }
    const int count = carry < cap ? carry : cap;
    table[0] = count;
    const char *bad = nullptr;
    std::vector<int> seen((size_t)count * tiles_n, 0);
    for (int seq = 0; seq < count * tiles_n && !bad; ++seq) {
      const int32_t band = table[4 * (1 + seq / tiles_n) + 3];
      if (band == unwritten) { bad = "band of an unwritten entry"; break; }
      if ((band & 15) < 1) { bad = "empty band"; break; }
      int tm, tn;
      grouped_tile_of_seq(band, seq, tiles_n, tm, tn);
      if (tm < 0 || tm >= count) { bad = "M tile outside the table"; break; }
      if (tn < 0 || tn >= tiles_n) { bad = "N tile out of range"; break; }
      const int32_t *ent = table.data() + 4 * (1 + tm);
      if (ent[0] == unwritten) { bad = "unwritten entry"; break; }
      if (ent[0] < 0 || ent[1] < 1 || ent[1] > bm || ent[0] + ent[1] > total_rows) { bad = "rows out of range"; break; }
      if (ent[2] < 0 || ent[2] >= groups) { bad = "group out of range"; break; }
      if (seen[(size_t)tm * tiles_n + tn]++) { bad = "tile visited twice"; break; }
    }
    if (!bad)
      for (int v : seen)
        if (v != 1) { bad = "tile never visited"; break; }
    if (bad) std::printf("BAD %s\n", bad);
    else std::printf("ok %d\n", count);
  }
  return 0;
}
