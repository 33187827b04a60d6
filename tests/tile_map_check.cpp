// Host-only check of the workgroup -> tile map (verl_amd/csrc/tile_map.hpp), compiled and run by test_abi_on_cpu.py:
// for every tile grid up to 70 x 70 (and a few large ones), both walk orders and every block shape, each tile is decoded
// by exactly one workgroup id, ids beyond the tiles decode to nothing, and the 8 XCDs (id % 8) get equal shares.
#include <stdio.h>

#include <vector>

#include "../verl_amd/csrc/tile_map.hpp"

using lce::TileMap;

static int check(const TileMap& m, int nr, int nc, const char* what) {
  std::vector<int> seen((size_t)nr * nc, 0);
  int count[8] = {0};
  for (int bid = 0; bid < m.total + 16; ++bid) {
    int rt = -1, ct = -1;
    if (!m.decode(bid, rt, ct)) continue;
    if (bid >= m.total || rt < 0 || rt >= nr || ct < 0 || ct >= nc) {
      printf("%s %dx%d: id %d decodes outside the grid (%d, %d)\n", what, nr, nc, bid, rt, ct);
      return 1;
    }
    ++seen[(size_t)rt * nc + ct];
    ++count[bid & 7];
  }
  for (size_t i = 0; i < seen.size(); ++i)
    if (seen[i] != 1) {
      printf("%s %dx%d: tile (%d, %d) decoded %d times\n", what, nr, nc, (int)(i / nc), (int)(i % nc), seen[i]);
      return 1;
    }
  if (m.total % 8 != 0 || m.total < nr * nc || m.total >= nr * nc + 8) {
    printf("%s %dx%d: %d workgroups\n", what, nr, nc, m.total);
    return 1;
  }
  for (int x = 0; x < 8; ++x)
    if (count[x] > m.per || count[x] < m.per - 7) {
      printf("%s %dx%d: XCD %d has %d tiles of %d per XCD\n", what, nr, nc, x, count[x], m.per);
      return 1;
    }
  return 0;
}

int main() {
  long maps = 0;
  for (int nr = 1; nr <= 70; ++nr)
    for (int nc = 1; nc <= 70; ++nc)
      for (int order = 0; order < 2; ++order) {
        for (int br = 1; br <= 8; br <<= 1) {
          if (check(TileMap::make(nr, nc, br, order), nr, nc, "make")) return 1;
          ++maps;
        }
        // the device-side map over fewer rows of a grid that the host sized for nr
        const TileMap host = TileMap::make(nr, nc, TileMap::block_rows(nr), order);
        for (int rows = 1; rows <= nr; rows += (nr > 16 ? 7 : 1)) {
          const TileMap dev = host.with_rows(rows);
          if (dev.total > host.total || check(dev, rows, nc, "with_rows")) return 1;
          ++maps;
        }
      }
  const int big[][2] = {{1024, 19}, {1024, 594}, {64, 594}, {594, 14}, {3, 501}, {4097, 5}};
  for (auto& g : big)
    for (int order = 0; order < 2; ++order) {
      if (check(TileMap::make(g[0], g[1], TileMap::block_rows(g[0]), order), g[0], g[1], "make")) return 1;
      ++maps;
    }
  // the 32 consecutive tiles that an XCD holds at a time stay inside two blocks' rows and columns
  {
    const TileMap m = TileMap::make(12, 20, 8, 1);
    int rmin = 1 << 30, rmax = -1, cmin = 1 << 30, cmax = -1;
    for (int l = 0; l < m.per; ++l) {
      int rt, ct;
      if (!m.decode(l * 8, rt, ct)) continue;
      rmin = rt < rmin ? rt : rmin; rmax = rt > rmax ? rt : rmax;
      cmin = ct < cmin ? ct : cmin; cmax = ct > cmax ? ct : cmax;
    }
    if (m.per != 30 || rmax - rmin >= 8 || cmax - cmin >= 4) {
      printf("12x20: XCD 0 spans rows %d..%d, columns %d..%d\n", rmin, rmax, cmin, cmax);
      return 1;
    }
  }
  printf("ok %ld maps\n", maps);
  return 0;
}
