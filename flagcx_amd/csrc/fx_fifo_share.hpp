// Host/device arithmetic of the FIFO consumer that decides how many workgroups
// run and which of them take which tiles of a trigger.  Kept free of HIP types
// so that a plain C++ check can exercise it on the CPU.
#pragma once
#include <stdint.h>

#ifdef __HIPCC__
#define FX_HD __host__ __device__
#else
#define FX_HD
#endif

namespace fx {

// Workgroups of the consumer: `wanted` (0 = the default, one per compute unit;
// 257 and 513 on a 256-unit device measured the same or slower), never more
// than the device holds at the same time -- a trigger completes only when all
// its takers have reported in, so a workgroup that is not resident would hold
// up every trigger it is a taker of.
FX_HD inline uint32_t fifoGridFor(int cus, int residentPerCu, long wanted) {
  if (cus < 1) cus = 1;
  if (residentPerCu < 1) residentPerCu = 1;
  const long most = (long)cus * residentPerCu;
  long g = wanted > 0 ? wanted : (long)cus;
  if (g > most) g = most;
  if (g < 1) g = 1;
  return (uint32_t)g;
}

// Which part of a trigger a workgroup takes: tiles idx, idx + takers, ...;
// idx >= takers means none.
struct Share {
  uint32_t idx, takers;
};

constexpr int kBulkShift = 3;   // a trigger that arrived in bulk is shared out over an eighth of its tiles' worth

// Who works on a trigger that has `tiles` tiles (0 counts as 1: an empty or
// unsupported trigger still needs somebody to complete it).  At most grid - 1
// workgroups: workgroup 0 never computes, so it is always free to talk to the
// host -- unless it is alone.  The workers of a small trigger start at a
// position `rot` that rotates with the trigger's number (rotOf), so consecutive
// small triggers run side by side on different workgroups.  Every workgroup
// computes the same answer from the trigger words alone, so the ones left out
// neither work nor report in.  No division in here or in nextRot: every
// workgroup of the consumer does this once per trigger.
FX_HD inline uint32_t rotOf(uint64_t seq, uint32_t pool) { return pool ? (uint32_t)((seq * 61u) % pool) : 0u; }
FX_HD inline uint32_t rotStep(uint32_t pool) { return pool ? 61u % pool : 0u; }
FX_HD inline uint32_t nextRot(uint32_t rot, uint32_t step, uint32_t pool) {   // rotOf(seq + 1) from rotOf(seq)
  const uint32_t r = rot + step;
  return r >= pool ? r - pool : r;
}

FX_HD inline Share shareForRot(uint32_t grid, uint32_t block, uint32_t rot, uint64_t tiles, bool bulk) {
  Share sh;
  if (tiles == 0) tiles = 1;
  if (grid <= 1) {  // a one-workgroup launch does everything itself
    sh.takers = 1;
    sh.idx = 0;
    return sh;
  }
  const uint32_t pool = grid - 1;
  if (bulk) tiles = (tiles >> kBulkShift) ? (tiles >> kBulkShift) : 1;
  sh.takers = (uint32_t)(tiles < pool ? tiles : pool);
  if (block == 0) {
    sh.idx = sh.takers;
  } else {
    const uint32_t x = block - 1 + pool - rot;   // in [1, 2 * pool)
    sh.idx = x >= pool ? x - pool : x;
  }
  return sh;
}

FX_HD inline Share shareFor(uint32_t grid, uint32_t block, uint64_t seq, uint64_t tiles, bool bulk) {
  return shareForRot(grid, block, grid > 1 ? rotOf(seq, grid - 1) : 0u, tiles, bulk);
}

}  // namespace fx
