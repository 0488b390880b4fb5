// CPU check of the FIFO consumer's host/device arithmetic (fx_fifo_share.hpp):
// the grid never exceeds what the device holds at once, and for every grid,
// trigger number and tile count the takers are exactly `takers` distinct
// workgroups whose tile lists cover every tile once; workgroup 0 computes only
// when it is alone.
#include <cstdio>
#include <vector>

#include "fx_fifo_share.hpp"

using namespace fx;

int main() {
  long cases = 0;
  // grid clamp
  for (int cus : {1, 8, 256, 304})
    for (int res : {1, 2, 8})
      for (long wanted : {0L, 1L, 2L, 255L, 256L, 257L, 512L, 100000L}) {
        const uint32_t g = fifoGridFor(cus, res, wanted);
        if (g < 1 || (long)g > (long)cus * res) { printf("FAIL grid %u cus %d res %d wanted %ld\n", g, cus, res, wanted); return 1; }
        if (wanted > 0 && wanted <= (long)cus * res && (long)g != wanted) { printf("FAIL grid ignores wanted\n"); return 1; }
        if (wanted == 0 && (long)g != cus) { printf("FAIL default grid\n"); return 1; }
        cases++;
      }
  // shares
  for (uint32_t grid : {1u, 2u, 3u, 64u, 255u, 256u, 257u, 513u})
    for (uint64_t seq : {0ull, 1ull, 2ull, 60ull, 61ull, 255ull, 256ull, 1000003ull, (1ull << 40) + 7})
      for (uint64_t tiles : {0ull, 1ull, 2ull, 7ull, 8ull, 9ull, 63ull, 64ull, 254ull, 255ull, 256ull, 257ull, 1024ull, 100000ull})
        for (bool bulk : {false, true}) {
          std::vector<int> owner;
          uint32_t takers = 0;
          for (uint32_t b = 0; b < grid; b++) {
            const Share s = shareFor(grid, b, seq, tiles, bulk);
            if (b == 0) { takers = s.takers; owner.assign(takers, -1); }
            if (s.takers != takers) { printf("FAIL takers differ between workgroups\n"); return 1; }
            if (s.idx < s.takers) {
              if (b == 0 && grid > 1) { printf("FAIL workgroup 0 takes tiles in a grid of %u\n", grid); return 1; }
              if (owner[s.idx] != -1) { printf("FAIL two workgroups share index %u\n", s.idx); return 1; }
              owner[s.idx] = (int)b;
            }
          }
          const uint64_t eff = bulk ? ((tiles >> kBulkShift) ? (tiles >> kBulkShift) : 1) : (tiles ? tiles : 1);
          const uint64_t pool = grid > 1 ? grid - 1 : 1;
          if (takers != (eff < pool ? eff : pool) || takers == 0) { printf("FAIL takers %u for %llu tiles, grid %u\n", takers, (unsigned long long)tiles, grid); return 1; }
          for (uint32_t i = 0; i < takers; i++)
            if (owner[i] == -1) { printf("FAIL index %u has no workgroup (grid %u seq %llu tiles %llu)\n", i, grid, (unsigned long long)seq, (unsigned long long)tiles); return 1; }
          cases++;
        }
  // the rotation carried from trigger to trigger is the one worked out from the trigger's number
  for (uint32_t pool : {1u, 2u, 3u, 60u, 61u, 62u, 122u, 255u, 256u, 512u})
    for (uint64_t start : {0ull, 5ull, 1000003ull, (1ull << 40) + 7}) {
      uint32_t rot = rotOf(start, pool);
      const uint32_t step = rotStep(pool);
      for (uint64_t seq = start; seq < start + 2000; seq++, rot = nextRot(rot, step, pool)) {
        if (rot != rotOf(seq, pool) || rot >= pool) { printf("FAIL rotation drifts: pool %u seq %llu\n", pool, (unsigned long long)seq); return 1; }
        cases++;
      }
    }
  printf("ok %ld cases\n", cases);
  return 0;
}
