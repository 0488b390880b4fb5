// Host-side launch tables for the reduce / copy kernel family.  One
// translation unit per element type instantiates a KernelSet per reduction
// op; the C-ABI layer picks the entry for (dtype, op, k) at run time.
#pragma once
#include "flagcx_amd/fx_kernels.h"
#include "fx_reduce_body.hpp"

namespace fx {

// Vectors per lane per input, measured on MI355X.
//  * Launches that write less than 4 MiB (per output buffer): 1 for three inputs
//    and more, and for the multi-output kernels.  With 4, such a launch has fewer
//    workgroups than the device has compute units and each lane waits for 32
//    loads: an eight-input reduction of 1 MiB per input takes 4.8 us against
//    2.9 us, the eight-rank all-reduce of 64 KiB per rank 6.2 against 4.3 us.
//    The run-time-k kernels (nine inputs and more, 2 otherwise) likewise: the
//    all-reduce of 16 KiB per rank over 12 / 16 / 32 ranks 5.0 / 5.8 / 10.4
//    against 4.0 / 4.5 / 8.2 us.
//  * Larger launches: 4 (2 for one and two inputs); 8 for 8 inputs once the
//    launch is large enough not to miss the extra workgroups and every input is
//    aligned like the output (256 VGPRs; unaligned: 4 is 7-10 % faster).  Between
//    1, 2 and 4 the difference at these sizes is within 1 % and changes sign with
//    where the buffers sit: builds that differ only in this number, run
//    alternately on one box, gave the same figures for two-input sums, copies,
//    pack / unpack and four-input sums from 8 MiB to 1 GiB, and 0.5-1 % in favour
//    of 4 over 1 for the eight-rank all-reduce from 64 MiB per rank.
constexpr int unrollFor(int K) { return K <= 2 ? 2 : 4; }
constexpr int smallUnrollFor(int K) { return (K >= 3 || K == 0) ? 1 : unrollFor(K); }   // K = 0: run-time k, nine inputs and more
constexpr int bigUnrollFor(int K) { return K == 8 ? 8 : unrollFor(K); }
constexpr uint64_t kBigLaunchTiles = 1024;  // use bigUnrollFor only above this many of its tiles (32 MiB per input)
constexpr uint64_t kSmallLaunchVecs = 256 * 1024;  // fewer 16-byte vectors of output than this: one vector per lane
constexpr int kBcastUnroll = 4, kSmallBcastUnroll = 1;   // the multi-output kernels, any number of inputs

inline uint64_t vectorsOf(uint64_t count, int es) { return (count * (uint64_t)es + 15) / 16; }

struct KernelSet {
  // index = compile-time input count, 0 = runtime-k kernel
  flagcxResult_t (*direct[kMaxFixedK + 1])(void *out, const void *const *in, int k, uint64_t count, hipStream_t s);
  // n validated, non-empty slices; as many launches as their kernel-argument tables need
  flagcxResult_t (*slicesInline[kMaxFixedK + 1])(const fxSliceDesc *slices, size_t n, hipStream_t s);
  // device-resident tables, tile counts made with unrollFor(k)
  flagcxResult_t (*slicesTable[kMaxFixedK + 1])(const SliceDescDev *d, const uint32_t *tileStart, uint32_t n,
                                                uint32_t grid, hipStream_t s);
  // n validated, non-empty multi-output slices
  flagcxResult_t (*bcastInline[kMaxFixedK + 1])(const BcastDescDev *d, size_t n, hipStream_t s);
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
  uint64_t ntiles = tilesFor(out, in, kk, count, R::ES, U);
  if (ntiles == 0) return flagcxSuccess;
  if (ntiles > 0x7ffffff0ull) return flagcxInvalidArgument;
  return launchKernel(reduceCopyDirect<R, K, U>, (uint32_t)ntiles, s, a);
}

template <class R, int K>
flagcxResult_t launchDirect(void *out, const void *const *in, int k, uint64_t count, hipStream_t s) {
  constexpr int US = smallUnrollFor(K), UD = unrollFor(K), UB = bigUnrollFor(K);
  if constexpr (US != UD)
    if (vectorsOf(count, R::ES) < kSmallLaunchVecs) return launchDirectU<R, K, US>(out, in, k, count, s);
  if constexpr (UB != UD)
    if (coAlignedHost(out, in, (K > 0) ? K : k) && tilesFor(out, in, (K > 0) ? K : k, count, R::ES, UB) >= kBigLaunchTiles)
      return launchDirectU<R, K, UB>(out, in, k, count, s);
  return launchDirectU<R, K, UD>(out, in, k, count, s);
}

template <class R, int K, int U, int NS>
flagcxResult_t launchSlicesInlineSized(const fxSliceDesc *slices, size_t n, hipStream_t s) {
  InlineSliceTable<K, NS> t;
  t.n = 0;
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

template <class R, int K>
flagcxResult_t launchSlicesInline(const fxSliceDesc *slices, size_t n, hipStream_t s) {
  constexpr int US = smallUnrollFor(K), UD = unrollFor(K);
  if (n > (size_t)kSmallSliceTable) return launchSlicesInlineSized<R, K, UD, 0>(slices, n, s);
  if constexpr (US != UD) {
    uint64_t vecs = 0;
    for (size_t i = 0; i < n; i++) vecs += vectorsOf(slices[i].count, R::ES);
    if (vecs < kSmallLaunchVecs) return launchSlicesInlineSized<R, K, US, kSmallSliceTable>(slices, n, s);
  }
  return launchSlicesInlineSized<R, K, UD, kSmallSliceTable>(slices, n, s);
}

template <class R, int K>
flagcxResult_t launchSlicesTable(const SliceDescDev *d, const uint32_t *tileStart, uint32_t n, uint32_t grid,
                                 hipStream_t s) {
  constexpr int U = unrollFor(K);
  if (grid == 0) return flagcxSuccess;
  return launchKernel(reduceSlicesTable<R, K, U>, grid, s, d, tileStart, n);
}

inline uint64_t bcastTiles(const BcastDescDev &d, int k, int es, int U) {
  return tilesFor(d.out[0], d.in, k, d.count, es, U, d.out + 1, (int)d.nout - 1);
}

template <class R, int K, int U>
flagcxResult_t launchBcastOne(const BcastDescDev &d, hipStream_t s) {  // the one-slot table
  const uint64_t tiles = bcastTiles(d, K, R::ES, U);
  if (tiles > 0x7ffffff0ull) return flagcxInvalidArgument;
  InlineBcastTable<1> t;
  t.d[0] = d;
  t.tileStart[0] = 0;
  t.tileStart[1] = (uint32_t)tiles;
  t.n = 1;
  return launchKernel(reduceBcastInline<R, K, U, 1>, (uint32_t)tiles, s, t);
}

template <class R, int K, int U>
flagcxResult_t launchBcastMany(const BcastDescDev *d, size_t n, hipStream_t s) {  // the sixteen-slot table
  InlineBcastTable<kInlineBcast> t;
  t.n = 0;
  t.tileStart[0] = 0;
  for (size_t i = 0; i <= n; i++) {
    uint64_t tiles = 0;
    if (i < n) {
      tiles = bcastTiles(d[i], K, R::ES, U);
      if (tiles > 0x7ffffff0ull) return flagcxInvalidArgument;
    }
    const bool full = t.n == (uint32_t)kInlineBcast || (i < n && (uint64_t)t.tileStart[t.n] + tiles > 0x7ffffff0ull);
    if ((i == n || full) && t.n > 0) {
      const flagcxResult_t rc = launchKernel(reduceBcastInline<R, K, U, kInlineBcast>, t.tileStart[t.n], s, t);
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

template <class R, int K>
flagcxResult_t launchBcastInline(const BcastDescDev *d, size_t n, hipStream_t s) {
  uint64_t vecs = 0;   // per output buffer, all descriptors together
  for (size_t i = 0; i < n; i++) vecs += vectorsOf(d[i].count, R::ES);
  const bool small = vecs < kSmallLaunchVecs;
  if (n == 1) return small ? launchBcastOne<R, K, kSmallBcastUnroll>(d[0], s) : launchBcastOne<R, K, kBcastUnroll>(d[0], s);
  return small ? launchBcastMany<R, K, kSmallBcastUnroll>(d, n, s) : launchBcastMany<R, K, kBcastUnroll>(d, n, s);
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
  if (count == 0) return flagcxSuccess;
  a.co = coAlignedHost(out[0], in, k, out + 1, nout - 1) ? 1 : 0;
  const uint64_t ntiles = planTiles((uint64_t)(uintptr_t)out[0], count, R::ES, U, handOutFor(a.co != 0, k)).tiles();
  if (ntiles == 0) return flagcxSuccess;
  if (ntiles > 0x7ffffff0ull) return flagcxInvalidArgument;
  return launchKernel(reduceBcastRuntime<R, U>, (uint32_t)ntiles, s, a);
}

// One vector per lane while a launch writes less than 4 MiB per buffer, as for the fixed-k kernels.
template <class R>
flagcxResult_t launchBcastRuntime(void *const *out, int nout, const void *const *in, int k, uint64_t count,
                                  hipStream_t s) {
  if (vectorsOf(count, R::ES) < kSmallLaunchVecs) return launchBcastRuntimeU<R, 1>(out, nout, in, k, count, s);
  return launchBcastRuntimeU<R, unrollFor(0)>(out, nout, in, k, count, s);
}

template <class R, int U>
flagcxResult_t launchChunksRuntimeU(ChunkedArgs *a, hipStream_t s) {
  uint64_t total = 0;
  a->tileStart[0] = 0;
  for (int c = 0; c < a->nchunks; c++) {
    a->co[c] = chunkCoAligned(*a, c) ? 1 : 0;
    total += a->cnt[c] ? chunkPlan<R::ES, U>(*a, c).tiles() : 0;
    if (total > 0x7ffffff0ull) return flagcxInvalidArgument;
    a->tileStart[c + 1] = (uint32_t)total;
  }
  if (total == 0) return flagcxSuccess;
  return launchKernel(reduceChunksRuntime<R, U>, (uint32_t)total, s, *a);
}

template <class R>
flagcxResult_t launchChunksRuntime(ChunkedArgs *a, hipStream_t s) {
  uint64_t vecs = 0;
  for (int c = 0; c < a->nchunks; c++) vecs += vectorsOf(a->cnt[c], R::ES);
  if (vecs < kSmallLaunchVecs) return launchChunksRuntimeU<R, 1>(a, s);
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

template <class R, int K, bool BCAST = true>
void fillSet(KernelSet &ks) {
  ks.direct[K] = &launchDirect<R, K>;
  if (K > 0) {
    ks.slicesInline[K] = &launchSlicesInline<R, (K > 0 ? K : 1)>;
    ks.slicesTable[K] = &launchSlicesTable<R, (K > 0 ? K : 1)>;
    if constexpr (BCAST) ks.bcastInline[K] = &launchBcastInline<R, (K > 0 ? K : 1)>;
    else ks.bcastInline[K] = nullptr;
  } else {
    ks.slicesInline[0] = nullptr;
    ks.slicesTable[0] = nullptr;
    ks.bcastInline[0] = nullptr;
  }
}

template <class R>
KernelSet makeSet() {
  KernelSet ks;
  fillSet<R, 0>(ks);
  fillSet<R, 1>(ks);
  fillSet<R, 2>(ks);
  fillSet<R, 3>(ks);
  fillSet<R, 4>(ks);
  fillSet<R, 5>(ks);
  fillSet<R, 6>(ks);
  fillSet<R, 7>(ks);
  fillSet<R, 8>(ks);
  ks.bcastRuntime = &launchBcastRuntime<R>;
  ks.chunksRuntime = &launchChunksRuntime<R>;
  ks.elemSize = R::ES;
  return ks;
}

// Only k = 1 is meaningful for the byte mover.
template <int ES>
KernelSet makeCopySet() {
  KernelSet ks = {};
  fillSet<CopyRed<ES>, 1, true>(ks);
  ks.bcastRuntime = &launchBcastRuntime<CopyRed<ES>>;
  ks.chunksRuntime = &launchChunksRuntime<CopyRed<ES>>;
  ks.allToAll = &launchAllToAll<CopyRed<ES>>;
  ks.elemSize = ES;
  return ks;
}

template <int DT>
const KernelSet *makeSets() {
  static const KernelSet sets[5] = {makeSet<Red<DT, flagcxSum>>(), makeSet<Red<DT, flagcxProd>>(),
                                    makeSet<Red<DT, flagcxMax>>(), makeSet<Red<DT, flagcxMin>>(),
                                    makeSet<Red<DT, flagcxAvg>>()};  // indexed by flagcxRedOp_t
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
