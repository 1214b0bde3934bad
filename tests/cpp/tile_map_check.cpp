// Host check of the prefill GEMMs' workgroup -> tile map (torchlette_amd/csrc/tile_map.h):
// every tile of a launch is taken by exactly one workgroup id, the host's account of the
// busiest XCD matches what the ids really give, and a launch that fits the chip in one or
// two rounds never crowds an XCD into more.  Prints "ok <cases>" or the first failure.
#include <cstdio>
#include <vector>

#include "tile_map.h"

using namespace tlhip;

int main() {
  long cases = 0;
  const TileCost costs[] = {{256, 64}, {256, 128}, {512, 128}, {512, 256}, {128, 128}};
  for (const TileCost cost : costs)
    for (int tiles_m = 1; tiles_m <= 70; ++tiles_m)
      for (int tiles_n = 1; tiles_n <= 2100; tiles_n += (tiles_n < 70 ? 1 : 97)) {
        int grid = 0;
        const TileMap t = make_tile_map(tiles_m, tiles_n, cost, &grid);
        std::vector<int> seen((size_t)tiles_m * tiles_n, 0);
        long load[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int id = 0; id < grid; ++id) {
          int tm, tn;
          if (!tile_of(t, id, tm, tn)) continue;
          if (tm < 0 || tm >= tiles_m || tn < 0 || tn >= tiles_n) {
            printf("tile out of range: %d x %d, id %d -> (%d, %d)\n", tiles_m, tiles_n, id, tm, tn);
            return 1;
          }
          ++seen[(size_t)tm * tiles_n + tn];
          ++load[id & 7];
        }
        for (size_t i = 0; i < seen.size(); ++i)
          if (seen[i] != 1) {
            printf("%d x %d: tile %zu taken %d times\n", tiles_m, tiles_n, i, seen[i]);
            return 1;
          }
        long busiest = 0;
        for (long l : load) busiest = l > busiest ? l : busiest;
        if (busiest != busiest_xcd_tiles(t)) {
          printf("%d x %d: busiest XCD %ld, the host says %ld\n", tiles_m, tiles_n, busiest, (long)busiest_xcd_tiles(t));
          return 1;
        }
        const long total = (long)tiles_m * tiles_n, chip_rounds = (total + 255) / 256;
        if (chip_rounds <= 2 && (busiest + 31) / 32 > chip_rounds) {
          printf("%d x %d: %ld tiles on one XCD, %ld rounds where the chip needs %ld\n", tiles_m, tiles_n, busiest,
                 (busiest + 31) / 32, chip_rounds);
          return 1;
        }
        if (chip_rounds > 2 && busiest * 8 * 20 > total * 21 && (busiest + 31) / 32 > chip_rounds) {
          printf("%d x %d: busiest XCD holds %ld of %ld tiles\n", tiles_m, tiles_n, busiest, total);
          return 1;
        }
        ++cases;
      }
  // the shape rule: few column tiles -> blocks as wide as the matrix; large problems 4 x 8
  int grid = 0;
  TileMap t = make_tile_map(24, 8, TileCost{512, 128}, &grid);
  if ((1 << t.gn_shift) < 4) {
    printf("24 x 8 tiles: blocks of %d x %d\n", 1 << t.gm_shift, 1 << t.gn_shift);
    return 1;
  }
  t = make_tile_map(16, 48, TileCost{256, 128}, &grid);
  if (t.gm_shift != 2 || t.gn_shift != 3) {
    printf("16 x 48 tiles: blocks of %d x %d\n", 1 << t.gm_shift, 1 << t.gn_shift);
    return 1;
  }
  printf("ok %ld\n", cases);
  return 0;
}
