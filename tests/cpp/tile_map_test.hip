// Host-side check of the workgroup -> output tile map that the tile kernels share (tile_of / tile_grid in
// csrc/ksq_internal.h): for every grid size in a range, the logical ids 0 .. tile_grid - 1 hit every (row block, column
// block) exactly once, the ids past the last tile are refused, and consecutive ids inside a band of eight row blocks
// walk down the band first.  Prints "OK <cases>" or the first failure.  No device is touched.
#include <cstdio>
#include <vector>

#include "ksq_internal.h"

int main() {
  long cases = 0;
  for (int mblocks = 1; mblocks <= 40; ++mblocks) {
    for (int nblocks = 1; nblocks <= 97; nblocks += (nblocks < 20 ? 1 : 7)) {
      const unsigned grid = ksq::tile_grid((size_t)mblocks, (size_t)nblocks);
      if (grid % 8 != 0 || grid < (unsigned)(mblocks * nblocks) || grid >= (unsigned)(mblocks * nblocks) + 8) {
        std::printf("FAIL grid %d x %d -> %u\n", mblocks, nblocks, grid);
        return 1;
      }
      std::vector<int> seen((size_t)mblocks * nblocks, 0);
      int prev_mb = -1, prev_nb = -1;
      for (unsigned lid = 0; lid < grid; ++lid) {
        int mb = -1, nb = -1;
        const bool live = ksq::tile_of((int)lid, mblocks, nblocks, &mb, &nb);
        if (live != (lid < (unsigned)(mblocks * nblocks))) {
          std::printf("FAIL live %d x %d lid %u\n", mblocks, nblocks, lid);
          return 1;
        }
        if (!live) continue;
        if (mb < 0 || mb >= mblocks || nb < 0 || nb >= nblocks || seen[(size_t)mb * nblocks + nb]++) {
          std::printf("FAIL tile %d x %d lid %u -> (%d, %d)\n", mblocks, nblocks, lid, mb, nb);
          return 1;
        }
        // inside a band: the next id is the next row block of the same column block, or the band's first row block of
        // the next column block
        if (prev_mb >= 0 && mb / 8 == prev_mb / 8) {
          const int h = mblocks - 8 * (mb / 8) < 8 ? mblocks - 8 * (mb / 8) : 8;
          const bool down = nb == prev_nb && mb == prev_mb + 1;
          const bool next_col = nb == prev_nb + 1 && mb == 8 * (mb / 8) && prev_mb == 8 * (mb / 8) + h - 1;
          if (!down && !next_col) {
            std::printf("FAIL order %d x %d lid %u\n", mblocks, nblocks, lid);
            return 1;
          }
        }
        prev_mb = mb;
        prev_nb = nb;
      }
      ++cases;
    }
  }
  std::printf("OK %ld\n", cases);
  return 0;
}
