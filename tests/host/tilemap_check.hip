// Host-side check of the block -> tile maps used by the asynchronous-copy kernels (no GPU needed):
// every tile of every batch entry is visited by exactly one block of the launched grid, the blocks of a
// group share their id mod 8 (the XCD they are dealt to), and the split chooser stays inside its slot budget.
#include <cstdio>
#include <cstdlib>
#include <vector>
#include "../../lact_amd/csrc/gemm_dma.h"

using lact::TileMap;

static int check_map(int gx, int gy, int gz) {
  const TileMap m = lact::make_tile_map(gx, gy, gz);
  std::vector<int> seen((size_t)gx * gy * gz, 0);
  std::vector<int> group_xcd((size_t)m.groups(), -1);
  for (int L = 0; L < m.grid(); ++L) {
    int x = -1, y = -1, z = -1;
    if (!m.locate_host(L, x, y, z)) continue;
    if (x < 0 || x >= gx || y < 0 || y >= gy || z < 0 || z >= gz) { printf("out of range: %d %d %d -> %d %d %d at %d\n", gx, gy, gz, x, y, z, L); return 1; }
    ++seen[((size_t)z * gx + x) * gy + y];
    const int g = m.by_batch ? z : z * gx + x;
    if (group_xcd[g] >= 0 && group_xcd[g] != (L & 7)) { printf("group %d split over XCDs (%d %d %d)\n", g, gx, gy, gz); return 1; }
    group_xcd[g] = L & 7;
  }
  for (size_t i = 0; i < seen.size(); ++i)
    if (seen[i] != 1) { printf("tile %zu visited %d times (%d %d %d)\n", i, seen[i], gx, gy, gz); return 1; }
  return 0;
}

int main() {
  int bad = 0, n = 0;
  for (int gx : {1, 2, 3, 8, 16, 37, 128})
    for (int gy : {1, 2, 3, 4, 9})
      for (int gz : {1, 2, 3, 4, 6, 8, 12, 16, 36, 48, 96}) { bad += check_map(gx, gy, gz); ++n; }
  printf("%d maps checked, %d bad\n", n, bad);
  return bad ? 1 : 0;
}
