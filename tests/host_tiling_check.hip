// Host-side check of the kernels' index arithmetic (no GPU needed): for a grid
// of output addresses, lengths, element sizes, unrolls and alignment classes,
// every 16-byte vector that overlaps the segment must be handled by exactly one
// (tile, lane, u), the fast path must only ever see whole in-segment vectors,
// and nothing outside [0, nv) may be touched.  Uses the very functions the
// kernels call (fx::planTiles, fx::laneOfTile).
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "fx_launch.hpp"

using namespace fx;

// `shift` plays the part of (workgroup number - tile) mod 8 in a launch whose first workgroup is not tile 0.
static long checkOne(uint64_t outAddr, uint64_t count, int es, int U, HandOut how, uint32_t shift = 0) {
  const TilePlan tp = planTiles(outAddr, count, es, U, how);
  if (tp.grouped != (how == kGrouped)) return 9;
  if (how == kContiguous && tp.zoneTiles) return 3;          // no striped tiles when asked for none
  const uint64_t ve = 16u / (uint32_t)es, lead = (outAddr & 15u) / (uint32_t)es, end = lead + count;
  if (count == 0) return 0;  // empty segments never reach a kernel (the launchers return first)
  std::vector<unsigned char> seen(tp.nv, 0);
  const uint64_t tiles = tp.tiles();
  for (uint64_t tile = 0; tile < tiles; tile++) {
    bool fast0 = false;
    for (uint32_t tid = 0; tid < (uint32_t)kBlock; tid++) {
      const TileLane tl = laneOfTile(tp, (uint32_t)tile, tid, U, shift);
      if (tid == 0) fast0 = tl.fast;
      if (tl.fast != fast0) return 2;                       // the path must be uniform in a workgroup
      for (int u = 0; u < U; u++) {
        const uint64_t j = tl.j + (uint64_t)u * tl.stride;
        if (tl.fast) {
          if (j < tp.firstFull || j >= tp.endFull) return 4;  // whole vectors inside the segment only
          if (seen[j]++) return 5;
        } else {
          if (j >= tl.limit) continue;                        // the checked path's own guard
          if (j >= tp.nv) return 6;
          const uint64_t e0 = j * ve;
          if (e0 >= end || e0 + ve <= lead) continue;         // reduceVectorChecked returns at once
          if (seen[j]++) return 7;
        }
      }
    }
  }
  for (uint64_t j = 0; j < tp.nv; j++) {
    const uint64_t e0 = j * ve;
    const bool overlaps = !(e0 >= end || e0 + ve <= lead);
    if (overlaps != (seen[j] == 1)) return 8;
  }
  // Grouped flavour: within a region, the workgroups whose number is the same modulo 8 (one die) own eight
  // neighbouring columns; plain flavour: tile i owns column i.
  for (uint64_t tile = 0; tile < tp.zoneTiles; tile++) {
    const uint64_t col = ((laneOfTile(tp, (uint32_t)tile, 0, U, shift).j - tp.zs) % kRowVecs) / kPieceVecs;
    const uint64_t t = tile % kStripeTiles;
    if (tp.grouped ? (col / (kStripeTiles / 8) != (t + shift) % 8) : (col != t)) return 10;
  }
  return 0;
}

int main() {
  long cases = 0;
  const uint64_t MiB = 1ull << 20;
  const uint64_t bases[] = {0x7f0000000000ull, 0x7f0000000000ull + 512, 0x7f0000000000ull + 96 * 1024 + 16,
                            0x7f0000000000ull + MiB - 16, 0x7f0000000000ull + 3 * MiB + 4096};
  for (int es : {1, 2, 4, 8})
    for (int U : {1, 2, 4, 8})
      for (HandOut co : {kStriped, kGrouped, kContiguous})
        for (uint64_t base : bases)
          for (uint64_t mis = 0; mis < 16; mis += (uint64_t)es * (es == 1 ? 5 : 1)) {
            const uint64_t V = (uint64_t)U * kBlock * 16 / es;   // elements per tile
            const uint64_t small[] = {0, 1, 2, 16 / (uint64_t)es - 1, 16 / (uint64_t)es, 16 / (uint64_t)es + 1, V - 1, V,
                                      V + 1, 3 * V + 7};
            const uint64_t zone = kStripeMinBytes / es;   // lengths around the striping threshold, and well above it
            const uint64_t big[] = {zone - 1, zone, zone + 1, zone + V * 64 - 3, 2 * zone + 12345, 4 * MiB / es + 1, 9 * MiB / es + 1};
            for (uint64_t c : small) {
              long rc = checkOne(base + mis, c, es, U, co);
              cases++;
              if (rc) { printf("FAIL rc=%ld es=%d U=%d co=%d addr=%llx count=%llu\n", rc, es, U, (int)co, (unsigned long long)(base + mis), (unsigned long long)c); return 1; }
            }
            if (mis == 0 || mis == 8 || (es == 2 && mis == 2))
              for (uint64_t c : big) {
                long rc = checkOne(base + mis, c, es, U, co, (uint32_t)((c + mis + (uint64_t)U) % 8));
                cases++;
                if (rc) { printf("FAIL rc=%ld es=%d U=%d co=%d addr=%llx count=%llu\n", rc, es, U, (int)co, (unsigned long long)(base + mis), (unsigned long long)c); return 1; }
              }
          }
  // The striping criterion: every stream at the output's offset within a 128-byte line.  16 bytes apart is
  // not enough (a 512-byte piece of such an input would cut five lines instead of covering four).
  {
    char *o = (char *)0x7f0000001000ull;
    const void *same[3] = {o + 128, o + (1 << 20), o - 4096};
    const void *off16[3] = {o + 128, o + 16, o};
    const void *off4[2] = {o + 4, o};
    void *outs[2] = {o + 256, o + 64};
    if (!coAlignedHost(o, same, 3) || coAlignedHost(o, off16, 3) || coAlignedHost(o, off4, 2) ||
        !coAlignedHost(o, same, 3, outs, 1) || coAlignedHost(o, same, 3, outs, 2)) {
      printf("FAIL striping criterion\n");
      return 1;
    }
    const uint64_t count = (16ull << 20) / 4;
    const void *in1[1] = {o + 16};
    const TilePlan off = planTiles((uint64_t)(uintptr_t)o, count, 4, 4, handOutFor(coAlignedHost(o, in1, 1), 1));
    const TilePlan on = planTiles((uint64_t)(uintptr_t)o, count, 4, 4, handOutFor(coAlignedHost(o, same, 3), 3));
    const TilePlan red = planTiles((uint64_t)(uintptr_t)o, count, 4, 4, handOutFor(coAlignedHost(o, off16, 3), 3));
    if (tilesFor(o, in1, 1, count, 4, 4) != off.tiles() || off.zoneTiles == 0 || !off.grouped ||    // copy: striped, grouped columns
        on.zoneTiles != off.zoneTiles || on.grouped ||                                             // same phase: striped, column i
        red.zoneTiles != 0 || tilesFor(o, off16, 3, count, 4, 4) != (count * 4 + 16383) / 16384) { // reduction off phase: contiguous
      printf("FAIL striping decision\n");
      return 1;
    }
    cases += 8;
  }
  // Which batches of one-input slices read with ordinary loads: those that read at least half of their bytes twice.
  {
    char *src = (char *)0x7f0000100000ull, *dst = (char *)0x7f4000000000ull;
    const uint64_t chunk = 1 << 20;
    std::vector<fxSliceDesc> ag;                 // the all-gather copy phase of 8 ranks: chunk r to the 7 other ranks
    for (int r = 0; r < 8; r++)
      for (int q = 0; q < 8; q++)
        if (q != r) ag.push_back(fxSliceDesc{{src + r * chunk}, dst + (q * 8 + r) * chunk, chunk});
    std::vector<fxSliceDesc> pack;               // a pack: every slice another source
    for (int i = 0; i < 64; i++) pack.push_back(fxSliceDesc{{src + i * chunk}, dst + i * chunk, chunk});
    std::vector<fxSliceDesc> half = pack, less = pack, lens = pack, many;
    for (int i = 0; i < 32; i++) half[2 * i + 1].in[0] = half[2 * i].in[0];      // 32 of 64 slices read again: exactly half
    for (int i = 0; i < 31; i++) less[2 * i + 1].in[0] = less[2 * i].in[0];      // 31 of 64
    for (int i = 0; i < 64; i++) lens[i].in[0] = src, lens[i].count = chunk - i; // one address, 64 different lengths
    for (int i = 0; i < (int)kRereadMaxSlices + 1; i++) many.push_back(fxSliceDesc{{src}, dst + i * chunk, chunk});
    std::vector<fxSliceDesc> shuffled = ag;      // the order of the slices does not matter
    for (size_t i = 0; i < shuffled.size(); i++) std::swap(shuffled[i], shuffled[(i * 37 + 11) % shuffled.size()]);
    if (rereadHint(ag.data(), ag.size(), 1, 1) != kKeepAllLoads || rereadHint(shuffled.data(), shuffled.size(), 1, 2) != kKeepAllLoads ||
        rereadHint(pack.data(), pack.size(), 1, 1) != 0 || rereadHint(half.data(), half.size(), 1, 4) != kKeepAllLoads ||
        rereadHint(less.data(), less.size(), 1, 4) != 0 || rereadHint(lens.data(), lens.size(), 1, 1) != 0 ||
        rereadHint(ag.data(), 1, 1, 1) != 0 || rereadHint(ag.data(), ag.size(), 2, 1) != 0 ||
        rereadHint(many.data(), many.size(), 1, 1) != 0 || rereadHint(many.data(), kRereadMaxSlices, 1, 1) != kKeepAllLoads ||
        touchedBytes(1000, 2, 8, 1) != 18000 || touchedBytes(3ull << 30, 8, 8, 8) != (3ull << 37) ||
        // store-heavy launches whose results fit the memory-side cache leave them there; reductions into one output
        // and larger results stream (no forced policy in this process)
        (getenv("FX_CACHE_POLICY") == nullptr && getenv("FX_TEMPORAL_MAX_BYTES") == nullptr &&
         (cachePolicyFor(256ull << 20, 256ull << 20) != kKeepStores || cachePolicyFor(256ull << 20, (256ull << 20) + 1) != 0 ||
          cachePolicyFor((256ull << 20) + 1, 256ull << 20) != 0 || cachePolicyFor(8ull << 20, 1ull << 20) != 0 ||
          cachePolicyFor(1ull << 20, 8ull << 20) != kKeepStores ||
          cachePolicyFor(1, 1, kKeepAllLoads) != (kKeepAllLoads | kKeepStores)))) {
      printf("FAIL re-read detection\n");
      return 1;
    }
    cases += 12;
  }
  printf("ok %ld cases\n", cases);
  return 0;
}
