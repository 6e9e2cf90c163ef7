// Host-only check of the attention kernels' workgroup -> (head, q-block) map:
// over a launch of grid_for() ids every (head, q-block) of the range must be
// produced exactly once and nothing else.  Prints one line per case; exit
// status 0 when all hold.  No GPU call is made.
#include <cstdio>
#include <vector>

#include "attn_tiles.h"

int main() {
  const int cases[][4] = {
      // H, Hkv, q-block begin, q-block end
      {32, 8, 0, 1024}, {32, 8, 128, 256}, {28, 4, 0, 512}, {24, 24, 0, 931}, {4, 4, 0, 1},   {7, 1, 0, 19},
      {64, 1, 0, 33},   {71, 1, 0, 40},    {128, 1, 0, 17}, {128, 2, 3, 30},  {130, 1, 0, 9}, {96, 3, 0, 25},
      {1, 1, 0, 300},   {6, 3, 5, 6},      {256, 1, 0, 5},  {40, 8, 0, 77},
  };
  int bad = 0;
  for (const auto& c : cases) {
    const int H = c[0], Hkv = c[1], b = c[2], e = c[3];
    const long grid = (long)xattn::grid_for(H, Hkv, e - b);
    std::vector<int> seen((size_t)H * (e - b), 0);
    long stray = 0;
    for (long id = 0; id < grid; ++id) {
      int head = -1, qb = -1;
      if (!xattn::map_workgroup((int)id, H, Hkv, b, e, &head, &qb)) continue;
      if (head < 0 || head >= H || qb < b || qb >= e) {
        ++stray;
        continue;
      }
      ++seen[(size_t)head * (e - b) + (qb - b)];
    }
    long missing = 0, twice = 0;
    for (int v : seen) {
      missing += v == 0;
      twice += v > 1;
    }
    // the 64 ids that reach one XCD one after the other must share their KV head
    long mixed = 0;
    for (long u = 0; u * 512 < grid; ++u)
      for (int x = 0; x < 8; ++x) {
        int kv = -1;
        for (int w = 0; w < 64; ++w) {
          int head, qb;
          if (!xattn::map_workgroup((int)(u * 512 + w * 8 + x), H, Hkv, b, e, &head, &qb)) continue;
          const int g = head / (H / Hkv);
          if (kv >= 0 && g != kv) ++mixed;
          kv = g;
        }
      }
    std::printf("H=%d Hkv=%d q-blocks [%d,%d): grid %ld missing %ld twice %ld stray %ld mixed-units %ld\n", H, Hkv, b, e,
                grid, missing, twice, stray, mixed);
    bad += (missing || twice || stray || mixed) ? 1 : 0;
  }
  return bad ? 1 : 0;
}
