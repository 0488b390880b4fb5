// Host-side launch tables for the reduce / copy kernel family.  One
// translation unit per element type instantiates a KernelSet per reduction
// op; the C-ABI layer picks the entry for (dtype, op, k) at run time.
#pragma once
#include "flagcx_amd/fx_kernels.h"
#include "fx_reduce_body.hpp"

namespace fx {

// Vectors per lane per input, measured on MI355X.
//  * One, for three inputs and more, while a launch writes less than 32 MiB (4 MiB per output buffer for the
//    multi-output kernels; the run-time-k kernels likewise).  With four, such a launch has few workgroups per compute
//    unit and every lane waits for 32 loads before its first store: an eight-input bf16 reduction of 4 MiB per input
//    takes 6.9 us against 4.8 us (12.1 against 10.2 from cold), 16 MiB 25.2 against 23.8 (29.4 against 28.0), a
//    four-input fp32 one of 4 MiB 4.4 against 3.9; the eight-rank all-reduce of 64 KiB per rank 6.2 against 4.3 us,
//    but at 8 MiB per rank 20.0 us with four against 22.7 with one, hence its lower limit.
//  * Above that: four (two for one and two inputs).  From 32 MiB of output up the difference between one and four
//    is within 1 % either way (eight inputs of 512 MiB: 747 us with four, 751 with one).
// LEAN kernel sets (the types only the host path of the reference carries, and
// the element-type fold) have one variant per input count: no separate
// small-launch kernels and one table size.
constexpr int unrollFor(int K) { return K <= 2 ? 2 : 4; }
constexpr int smallUnrollFor(int K, bool lean) {
  return (!lean && (K >= 3 || K == 0)) ? 1 : unrollFor(K);   // K = 0: run-time k, nine inputs and more
}
constexpr uint64_t kSmallLaunchVecs = 2048 * 1024;      // single-output kernels: fewer 16-byte vectors of output than this (32 MiB) -> one vector per lane
constexpr uint64_t kSmallBcastVecs = 256 * 1024;        // multi-output and many-rank kernels: 4 MiB per output buffer
constexpr int kBcastUnroll = 4;
constexpr int smallBcastUnroll(bool lean) { return lean ? kBcastUnroll : 1; }   // the multi-output kernels, any number of inputs
constexpr int kOrderedUnroll = 2;   // the tree / keep-local kernels: one variant for every size

inline uint64_t vectorsOf(uint64_t count, int es) { return (count * (uint64_t)es + 15) / 16; }

// ---- cache policy of a launch ----
//
// Loads.  Every byte of a reduction is used once, so loads are nontemporal:
// they stream past the 4 MiB L2 of each die and the 256 MiB memory-side cache
// behind them.  Measured on MI355X with every launch preceded by a 1 GiB fill
// (nothing of the operands cached), ordinary loads are 40-70 % SLOWER than
// nontemporal ones from 4 MiB to 256 MiB per input (two fp32 inputs of 64 MiB:
// 57 against 34 us; eight bf16 inputs of 16 MiB: 51 against 30 us), and with the
// operands cached they are within +-10 % of them, better at some sizes and worse
// at others.  (The fill leaves the caches full of dirty lines, and a load that
// allocates a line evicts one: a write to memory per line read.  Behind caches
// full of clean lines the two kinds of load take the same time, and inputs that
// were written just before the launch and fit the memory-side cache are read
// 8-10 % faster with ordinary loads.)  The loss is several times the gain, and
// a launch cannot know what the caches hold, so the operands' size alone does
// not choose ordinary loads.  What does:
//  * a launch that reads the same bytes more than once -- the all-gather copy
//    phase hands one source chunk to every other rank, seven copies of it --
//    reads with ordinary loads, so that the later readers find the chunk in a
//    cache (56 copies of 8 MiB: 75 against 118 us, and 97 against 126 us from
//    cold); the batch entry points detect that (rereadHint);
//  * FX_TEMPORAL_MAX_BYTES (environment, read once; default 0 = never) makes
//    every launch that touches no more than that many bytes use ordinary loads,
//    for a caller who knows that its operands are cache-resident.
// Stores.  A launch in which stores are at least half of the traffic (copies,
// pack / unpack, the one-read-n-stores collectives) and which writes no more
// than the memory-side cache holds (kCachedStoreMaxBytes) leaves its results
// there -- write-back stores at agent scope, stg_keep -- for whoever reads them
// next; everything else streams its results (nontemporal stores).  Measured
// against nontemporal stores, same box, alternating: alltoallv pack of 19.6 MB
// 6.2 against 7.4 us and unpack 6.2 against 7.6 (behind a 1 GiB fill 15.5
// against 15.0 and 14.9 against 15.1), seven copies of 8 MiB 16.8 against
// 18.7 us, an eight-rank all-reduce of 16 MiB per rank 46.1 against 50.1 us and
// all-gather 26.4 against 27.7 (behind a fill both within 0.5 %).  Reductions
// into one output gain 1-10 % by them when the same buffers are used over and
// over -- the output is then never written to memory at all, which a benchmark
// loop rewards and an application does not -- and lose 1-6 % behind a fill, so
// they stream.  Above the limit cached stores lose 0.3-2.4 % (eight inputs of
// 512 MiB: 741 against 736 us).  Plain stores without a scope (what a C++
// assignment compiles to) are slower than either everywhere.
// FX_CACHE_POLICY = stream | keep | keep-loads | keep-stores forces one policy
// for every launch (measurements).
struct CachePolicyConfig {
  uint64_t maxBytes;
  int forced;        // -1: by the rules above; otherwise the policy bits for every launch
};
inline CachePolicyConfig readCachePolicyConfig() {
  CachePolicyConfig c = {0, -1};
  if (const char *e = getenv("FX_TEMPORAL_MAX_BYTES")) {
    char *end = nullptr;
    const unsigned long long v = strtoull(e, &end, 0);
    if (end != e) c.maxBytes = v;
  }
  if (const char *e = getenv("FX_CACHE_POLICY")) {
    if (!strcmp(e, "stream")) c.forced = 0;
    else if (!strcmp(e, "keep")) c.forced = (int)(kKeepAllLoads | kKeepStores);
    else if (!strcmp(e, "keep-loads")) c.forced = (int)kKeepAllLoads;
    else if (!strcmp(e, "keep-stores")) c.forced = (int)kKeepStores;
  }
  return c;
}
constexpr uint64_t kCachedStoreMaxBytes = 256ull << 20;   // the memory-side cache
// `hint`: policy bits the caller has a reason for (rereadHint).
inline uint32_t cachePolicyFor(uint64_t bytesRead, uint64_t bytesWritten, uint32_t hint = 0) {
  static const CachePolicyConfig cfg = readCachePolicyConfig();
  if (cfg.forced >= 0) return (uint32_t)cfg.forced;
  return hint | (bytesRead + bytesWritten <= cfg.maxBytes ? kKeepAllLoads : 0u) |
         (bytesWritten >= bytesRead && bytesWritten <= kCachedStoreMaxBytes ? kKeepStores : 0u);
}
// Bytes a reduction of `count` elements of `es` bytes touches: k inputs, nout outputs.
inline uint64_t touchedBytes(uint64_t count, int es, int k, int nout) {
  return count * (uint64_t)es * (uint64_t)(k + nout);
}

// kKeepAllLoads when at least half of the input bytes of a batch of one-input
// slices are read by more than one slice (same address and length), else 0.
// Batches of 2..kRereadMaxSlices slices are looked at; the cost is a sort of
// that many pointers.
constexpr size_t kRereadMaxSlices = 128;
inline uint32_t rereadHint(const fxSliceDesc *slices, size_t n, int k, size_t es) {
  if (k != 1 || n < 2 || n > kRereadMaxSlices) return 0;
  struct Src {
    uintptr_t p;
    uint64_t bytes;
  };
  Src src[kRereadMaxSlices];
  uint64_t total = 0;
  for (size_t i = 0; i < n; i++) {
    src[i].p = (uintptr_t)slices[i].in[0];
    src[i].bytes = slices[i].count * (uint64_t)es;
    total += src[i].bytes;
  }
  for (size_t i = 1; i < n; i++) {   // insertion sort: the lists are short and mostly grouped already
    const Src v = src[i];
    size_t j = i;
    for (; j > 0 && (src[j - 1].p > v.p || (src[j - 1].p == v.p && src[j - 1].bytes > v.bytes)); j--) src[j] = src[j - 1];
    src[j] = v;
  }
  uint64_t again = 0;
  for (size_t i = 1; i < n; i++)
    if (src[i].p == src[i - 1].p && src[i].bytes == src[i - 1].bytes) again += src[i].bytes;
  return again * 2 >= total ? kKeepAllLoads : 0u;
}

struct KernelSet {
  // index = compile-time input count, 0 = runtime-k kernel
  flagcxResult_t (*direct[kMaxFixedK + 1])(void *out, const void *const *in, int k, uint64_t count, hipStream_t s);
  // n validated, non-empty slices; as many launches as their kernel-argument tables need
  flagcxResult_t (*slicesInline[kMaxFixedK + 1])(const fxSliceDesc *slices, size_t n, uint32_t hint, hipStream_t s);
  // device-resident tables, tile counts made with unrollFor(k)
  flagcxResult_t (*slicesTable[kMaxFixedK + 1])(const SliceDescDev *d, const uint32_t *tileStart, uint32_t n,
                                                uint32_t grid, uint32_t keep, hipStream_t s);
  // n validated, non-empty multi-output slices
  flagcxResult_t (*bcastInline[kMaxFixedK + 1])(const BcastDescDev *d, size_t n, hipStream_t s);
  // the same with the inputs combined in the tree ([0]) or keep-local ([1]) association; nullptr where the
  // association cannot differ from the input-order fold (integers) or is not defined (avg)
  flagcxResult_t (*ordered[2][kMaxFixedK + 1])(const BcastDescDev *d, size_t n, hipStream_t s);
  // one segment, up to kMaxK inputs and kMaxK outputs (outputs aligned alike within 16 bytes)
  flagcxResult_t (*bcastRuntime)(void *const *out, int nout, const void *const *in, int k, uint64_t count,
                                 hipStream_t s);
  // chunks of a collective over up to kMaxK ranks; tileStart is filled here
  flagcxResult_t (*chunksRuntime)(ChunkedArgs *a, hipStream_t s);
  // copy sets only: all-to-all of n * n equal blocks in one launch
  flagcxResult_t (*allToAll)(void *const *recv, const void *const *send, int n, uint64_t blockElems, hipStream_t s);
  int elemSize;
};

// Tiles (workgroups) a segment of `count` elements needs with unroll U.
inline uint64_t tilesFor(const void *out, const void *const *in, int k, uint64_t count, int es, int U,
                         void *const *more = nullptr, int nmore = 0) {
  if (count == 0) return 0;
  return planTiles((uint64_t)(uintptr_t)out, count, es, U, handOutFor(coAlignedHost(out, in, k, more, nmore), k)).tiles();
}

template <class R, int K, int U>
flagcxResult_t launchDirectU(void *out, const void *const *in, int k, uint64_t count, hipStream_t s) {
  DirectArgs<K> a;
  const int kk = (K > 0) ? K : k;
  for (int p = 0; p < kk; p++) a.in[p] = in[p];
  a.out = out;
  a.count = count;
  a.k = kk;
  a.keep = cachePolicyFor(touchedBytes(count, R::ES, kk, 0), touchedBytes(count, R::ES, 0, 1));
  uint64_t ntiles = tilesFor(out, in, kk, count, R::ES, U);
  if (ntiles == 0) return flagcxSuccess;
  if (ntiles > 0x7ffffff0ull) return flagcxInvalidArgument;
  return launchKernel(reduceCopyDirect<R, K, U>, (uint32_t)ntiles, s, a);
}

template <class R, int K, bool LEAN>
flagcxResult_t launchDirect(void *out, const void *const *in, int k, uint64_t count, hipStream_t s) {
  constexpr int US = smallUnrollFor(K, LEAN), UD = unrollFor(K);
  if constexpr (US != UD)
    if (vectorsOf(count, R::ES) < kSmallLaunchVecs) return launchDirectU<R, K, US>(out, in, k, count, s);
  return launchDirectU<R, K, UD>(out, in, k, count, s);
}

template <class R, int K, int U, int NS>
flagcxResult_t launchSlicesInlineSized(const fxSliceDesc *slices, size_t n, uint32_t keep, hipStream_t s) {
  InlineSliceTable<K, NS> t;
  t.n = 0;
  t.keep = keep;
  t.tileStart[0] = 0;
  for (size_t i = 0; i <= n; i++) {
    uint64_t tiles = 0;
    if (i < n) {
      tiles = tilesFor(slices[i].out, slices[i].in, K, slices[i].count, R::ES, U);
      if (tiles > 0x7ffffff0ull) return flagcxInvalidArgument;
    }
    const bool full = t.n == (uint32_t)InlineSliceTable<K, NS>::kSlots ||
                      (i < n && (uint64_t)t.tileStart[t.n] + tiles > 0x7ffffff0ull);
    if ((i == n || full) && t.n > 0) {
      const flagcxResult_t rc = launchKernel(reduceSlicesInline<R, K, U, NS>, t.tileStart[t.n], s, t);
      if (rc != flagcxSuccess) return rc;
      t.n = 0;
    }
    if (i == n) break;
    SliceDescK<K> &d = t.d[t.n];
    for (int p = 0; p < K; p++) d.in[p] = slices[i].in[p];
    d.out = slices[i].out;
    d.count = slices[i].count;
    t.tileStart[t.n + 1] = t.tileStart[t.n] + (uint32_t)tiles;
    t.n++;
  }
  return flagcxSuccess;
}

// The policy follows what the whole call touches (a batch that spreads over
// several launches still shares the caches).
template <class R, int K, bool LEAN>
flagcxResult_t launchSlicesInline(const fxSliceDesc *slices, size_t n, uint32_t hint, hipStream_t s) {
  constexpr int US = smallUnrollFor(K, LEAN), UD = unrollFor(K);
  uint64_t vecs = 0, elems = 0;
  for (size_t i = 0; i < n; i++) {
    vecs += vectorsOf(slices[i].count, R::ES);
    elems += slices[i].count;
  }
  const uint32_t keep = cachePolicyFor(touchedBytes(elems, R::ES, K, 0), touchedBytes(elems, R::ES, 0, 1), hint);
  if constexpr (LEAN) return launchSlicesInlineSized<R, K, UD, kSmallSliceTable>(slices, n, keep, s);
  if (n > (size_t)kSmallSliceTable) return launchSlicesInlineSized<R, K, UD, 0>(slices, n, keep, s);
  if constexpr (US != UD)
    if (vecs < kSmallLaunchVecs) return launchSlicesInlineSized<R, K, US, kSmallSliceTable>(slices, n, keep, s);
  return launchSlicesInlineSized<R, K, UD, kSmallSliceTable>(slices, n, keep, s);
}

template <class R, int K>
flagcxResult_t launchSlicesTable(const SliceDescDev *d, const uint32_t *tileStart, uint32_t n, uint32_t grid,
                                 uint32_t keep, hipStream_t s) {
  constexpr int U = unrollFor(K);
  if (grid == 0) return flagcxSuccess;
  return launchKernel(reduceSlicesTable<R, K, U>, grid, s, d, tileStart, n, keep);
}

inline uint64_t bcastTiles(const BcastDescDev &d, int k, int es, int U) {
  return tilesFor(d.out[0], d.in, k, d.count, es, U, d.out + 1, (int)d.nout - 1);
}

template <class R, int K, int U>
flagcxResult_t launchBcastOne(const BcastDescDev &d, uint32_t keep, hipStream_t s) {  // the one-slot table
  const uint64_t tiles = bcastTiles(d, K, R::ES, U);
  if (tiles > 0x7ffffff0ull) return flagcxInvalidArgument;
  InlineBcastTable<1> t;
  t.d[0] = d;
  t.tileStart[0] = 0;
  t.tileStart[1] = (uint32_t)tiles;
  t.n = 1;
  t.keep = keep;
  return launchKernel(reduceBcastInline<R, K, U, 1, kChain>, (uint32_t)tiles, s, t);
}

template <class R, int K, int U, int SCHED>
flagcxResult_t launchBcastMany(const BcastDescDev *d, size_t n, uint32_t keep, hipStream_t s) {  // the eight-slot table
  InlineBcastTable<kInlineBcast> t;
  t.n = 0;
  t.keep = keep;
  t.tileStart[0] = 0;
  for (size_t i = 0; i <= n; i++) {
    uint64_t tiles = 0;
    if (i < n) {
      tiles = bcastTiles(d[i], K, R::ES, U);
      if (tiles > 0x7ffffff0ull) return flagcxInvalidArgument;
    }
    const bool full = t.n == (uint32_t)kInlineBcast || (i < n && (uint64_t)t.tileStart[t.n] + tiles > 0x7ffffff0ull);
    if ((i == n || full) && t.n > 0) {
      const flagcxResult_t rc = launchKernel(reduceBcastInline<R, K, U, kInlineBcast, SCHED>, t.tileStart[t.n], s, t);
      if (rc != flagcxSuccess) return rc;
      t.n = 0;
    }
    if (i == n) break;
    t.d[t.n] = d[i];
    t.tileStart[t.n + 1] = t.tileStart[t.n] + (uint32_t)tiles;
    t.n++;
  }
  return flagcxSuccess;
}

inline uint32_t bcastPolicy(const BcastDescDev *d, size_t n, int es, int k, uint64_t *vecsPerOutput) {
  uint64_t vecs = 0, read = 0, written = 0;
  for (size_t i = 0; i < n; i++) {
    vecs += vectorsOf(d[i].count, es);
    read += touchedBytes(d[i].count, es, k, 0);
    written += touchedBytes(d[i].count, es, 0, (int)d[i].nout);
  }
  *vecsPerOutput = vecs;
  return cachePolicyFor(read, written);
}

template <class R, int K, bool LEAN>
flagcxResult_t launchBcastInline(const BcastDescDev *d, size_t n, hipStream_t s) {
  constexpr int US = smallBcastUnroll(LEAN), UD = kBcastUnroll;
  uint64_t vecs = 0;   // per output buffer, all descriptors together
  const uint32_t keep = bcastPolicy(d, n, R::ES, K, &vecs);
  if constexpr (LEAN) return launchBcastMany<R, K, UD, kChain>(d, n, keep, s);
  const bool small = vecs < kSmallBcastVecs;
  if (n == 1) return small ? launchBcastOne<R, K, US>(d[0], keep, s) : launchBcastOne<R, K, UD>(d[0], keep, s);
  return small ? launchBcastMany<R, K, US, kChain>(d, n, keep, s) : launchBcastMany<R, K, UD, kChain>(d, n, keep, s);
}

template <class R, int K, int SCHED>
flagcxResult_t launchOrdered(const BcastDescDev *d, size_t n, hipStream_t s) {
  uint64_t vecs = 0;
  const uint32_t keep = bcastPolicy(d, n, R::ES, K, &vecs);
  return launchBcastMany<R, K, kOrderedUnroll, SCHED>(d, n, keep, s);
}

template <class R, int U>
flagcxResult_t launchBcastRuntimeU(void *const *out, int nout, const void *const *in, int k, uint64_t count,
                                   hipStream_t s) {
  ManyArgs a = {};
  for (int p = 0; p < k; p++) a.in[p] = in[p];
  for (int o = 0; o < nout; o++) a.out[o] = out[o];
  a.count = count;
  a.k = k;
  a.nout = nout;
  a.keep = cachePolicyFor(touchedBytes(count, R::ES, k, 0), touchedBytes(count, R::ES, 0, nout));
  if (count == 0) return flagcxSuccess;
  a.co = coAlignedHost(out[0], in, k, out + 1, nout - 1) ? 1 : 0;
  const uint64_t ntiles = planTiles((uint64_t)(uintptr_t)out[0], count, R::ES, U, handOutFor(a.co != 0, k)).tiles();
  if (ntiles == 0) return flagcxSuccess;
  if (ntiles > 0x7ffffff0ull) return flagcxInvalidArgument;
  return launchKernel(reduceBcastRuntime<R, U>, (uint32_t)ntiles, s, a);
}

// One vector per lane while a launch writes less than 4 MiB per buffer, as for the fixed-k kernels.
template <class R, bool LEAN>
flagcxResult_t launchBcastRuntime(void *const *out, int nout, const void *const *in, int k, uint64_t count,
                                  hipStream_t s) {
  if constexpr (!LEAN)
    if (vectorsOf(count, R::ES) < kSmallBcastVecs) return launchBcastRuntimeU<R, 1>(out, nout, in, k, count, s);
  return launchBcastRuntimeU<R, unrollFor(0)>(out, nout, in, k, count, s);
}

template <class R, int U>
flagcxResult_t launchChunksRuntimeU(ChunkedArgs *a, hipStream_t s) {
  uint64_t total = 0, read = 0, written = 0;
  a->tileStart[0] = 0;
  for (int c = 0; c < a->nchunks; c++) {
    a->co[c] = chunkCoAligned(*a, c) ? 1 : 0;
    total += a->cnt[c] ? chunkPlan<R::ES, U>(*a, c).tiles() : 0;
    if (total > 0x7ffffff0ull) return flagcxInvalidArgument;
    a->tileStart[c + 1] = (uint32_t)total;
    read += touchedBytes(a->cnt[c], R::ES, a->only[c] >= 0 ? 1 : a->k, 0);
    written += touchedBytes(a->cnt[c], R::ES, 0, a->outSel[c] >= 0 ? 1 : a->nout);
  }
  if (total == 0) return flagcxSuccess;
  a->keep = cachePolicyFor(read, written);
  return launchKernel(reduceChunksRuntime<R, U>, (uint32_t)total, s, *a);
}

template <class R, bool LEAN>
flagcxResult_t launchChunksRuntime(ChunkedArgs *a, hipStream_t s) {
  if constexpr (!LEAN) {
    uint64_t vecs = 0;
    for (int c = 0; c < a->nchunks; c++) vecs += vectorsOf(a->cnt[c], R::ES);
    if (vecs < kSmallBcastVecs) return launchChunksRuntimeU<R, 1>(a, s);
  }
  return launchChunksRuntimeU<R, unrollFor(0)>(a, s);
}

// The workgroups a block of the all-to-all can need at most: its tiles, plus one for a head before the first
// region boundary and one for a tail after the last (where the block lies in memory decides, block by block).
template <class R, int U>
flagcxResult_t launchAllToAllU(void *const *recv, const void *const *send, int n, uint64_t blockElems, hipStream_t s) {
  AllToAllArgs a = {};
  for (int r = 0; r < n; r++) {
    a.send[r] = send[r];
    a.recv[r] = recv[r];
  }
  a.blockElems = blockElems;
  a.n = n;
  const uint64_t moved = touchedBytes(blockElems * (uint64_t)n * (uint64_t)n, R::ES, 1, 0);
  a.keep = cachePolicyFor(moved, moved);
  const uint64_t V = (uint64_t)U * kBlock, nv = vectorsOf(blockElems, R::ES) + 1;   // + 1: a block off 16-byte alignment spans one vector more
  const uint64_t striped = blockElems * (uint64_t)R::ES >= kStripeMinBytes ? 2 : 0;   // shorter blocks have no regions
  const uint64_t per = (nv + V - 1) / V + striped, total = per * (uint64_t)n * (uint64_t)n;
  if (total > 0x7ffffff0ull) return flagcxInvalidArgument;
  a.tilesPerBlock = (uint32_t)per;
  return launchKernel(allToAllBlocks<R, U>, (uint32_t)total, s, a);
}

template <class R>
flagcxResult_t launchAllToAll(void *const *recv, const void *const *send, int n, uint64_t blockElems, hipStream_t s) {
  if (blockElems == 0) return flagcxSuccess;
  return launchAllToAllU<R, unrollFor(1)>(recv, send, n, blockElems, s);
}

// Which associations other than the input-order fold a reducer is built for:
// the tree for every floating type and sum / prod / max / min (integers give the
// same bits in any association; a mean is not a tree of two-input means), the
// keep-local chain for floating max / min (sums and products commute bit for
// bit in each step, so the input-order fold over suitably ordered inputs
// already is that chain).
template <class R>
struct OrderedFolds {
  static constexpr bool tree = false, keepLocal = false;
};
template <int DT, int OP>
struct OrderedFolds<Red<DT, OP>> {
  static constexpr bool floating = DT == flagcxFloat16 || DT == flagcxBfloat16 || DT == flagcxFloat32 || DT == flagcxFloat64;
  static constexpr bool tree = floating && OP != flagcxAvg;
  static constexpr bool keepLocal = floating && (OP == flagcxMax || OP == flagcxMin);
};

template <class R, int K, bool LEAN>
void fillSet(KernelSet &ks) {
  ks.direct[K] = &launchDirect<R, K, LEAN>;
  ks.ordered[0][K] = ks.ordered[1][K] = nullptr;
  if constexpr (K > 0) {
    ks.slicesInline[K] = &launchSlicesInline<R, K, LEAN>;
    ks.slicesTable[K] = &launchSlicesTable<R, K>;
    ks.bcastInline[K] = &launchBcastInline<R, K, LEAN>;
    if constexpr (K >= 3) {   // one and two inputs: every association is the input-order fold of suitably ordered inputs
      if constexpr (OrderedFolds<R>::tree) ks.ordered[0][K] = &launchOrdered<R, K, kTree>;
      if constexpr (OrderedFolds<R>::keepLocal) ks.ordered[1][K] = &launchOrdered<R, K, kKeepLocal>;
    }
  } else {
    ks.slicesInline[0] = nullptr;
    ks.slicesTable[0] = nullptr;
    ks.bcastInline[0] = nullptr;
  }
}

template <class R, bool LEAN>
KernelSet makeSet() {
  KernelSet ks = {};
  fillSet<R, 0, LEAN>(ks);
  fillSet<R, 1, LEAN>(ks);
  fillSet<R, 2, LEAN>(ks);
  fillSet<R, 3, LEAN>(ks);
  fillSet<R, 4, LEAN>(ks);
  fillSet<R, 5, LEAN>(ks);
  fillSet<R, 6, LEAN>(ks);
  fillSet<R, 7, LEAN>(ks);
  fillSet<R, 8, LEAN>(ks);
  ks.bcastRuntime = &launchBcastRuntime<R, LEAN>;
  ks.chunksRuntime = &launchChunksRuntime<R, LEAN>;
  ks.elemSize = R::ES;
  return ks;
}

// Only k = 1 is meaningful for the byte mover.
template <int ES>
KernelSet makeCopySet() {
  KernelSet ks = {};
  fillSet<CopyRed<ES>, 1, false>(ks);
  ks.bcastRuntime = &launchBcastRuntime<CopyRed<ES>, false>;
  ks.chunksRuntime = &launchChunksRuntime<CopyRed<ES>, false>;
  ks.allToAll = &launchAllToAll<CopyRed<ES>>;
  ks.elemSize = ES;
  return ks;
}

// The four types of the device path (fp32, fp16, bf16, int32) get the full set
// of variants; the types only the reference's host loops carry get the lean one.
template <int DT, bool LEAN>
const KernelSet *makeSets() {
  static const KernelSet sets[5] = {makeSet<Red<DT, flagcxSum>, LEAN>(), makeSet<Red<DT, flagcxProd>, LEAN>(),
                                    makeSet<Red<DT, flagcxMax>, LEAN>(), makeSet<Red<DT, flagcxMin>, LEAN>(),
                                    makeSet<Red<DT, flagcxAvg>, LEAN>()};  // indexed by flagcxRedOp_t
  return sets;
}

// Defined one per translation unit (fx_reduce_<type>.hip, fx_copy.hip).
const KernelSet *kernelSetsF32();
const KernelSet *kernelSetsI32();
const KernelSet *kernelSetsBF16();
const KernelSet *kernelSetsF16();
const KernelSet *kernelSetsU32();
const KernelSet *kernelSetsI8();
const KernelSet *kernelSetsU8();
const KernelSet *kernelSetsI64();
const KernelSet *kernelSetsU64();
const KernelSet *kernelSetsF64();
const KernelSet *kernelSetsCopy();  // index log2(ES): 0 -> 1 byte, 1 -> 2, 2 -> 4
const KernelSet *kernelSetsElem();  // RedElem: index 3 * (dtype == bf16) + (sum 0, max 1, min 2)

}  // namespace fx
