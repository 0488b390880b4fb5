// Device code of the k-way element-wise reduce-copy for gfx950 (wave64).
//
// Arithmetic contract (order follows FlagCX's peer loop,
// flagcx/adaptor/kernel/nvidia/custom_allreduce.cu:345-359):
//   acc = in[0]; acc = acc (op) in[p] for p = 1..k-1, left to right.
//   fp32 / fp64: plain IEEE arithmetic.  Integers of every width: sum/prod
//   wrap modulo 2^width (the host loops of flagcx/service/include/utils.h:664-725
//   on the types FlagCX dispatches there: char = signed 8-bit on x86-64,
//   unsigned char, int32_t, uint32_t, int64_t, uint64_t, float, double).
//   bf16/fp16 sum and prod: every input widened to fp32, accumulated in fp32,
//   rounded to nearest even once.  max = (acc < x) ? x : acc and
//   min = (x < acc) ? x : acc (the std::max / std::min of
//   flagcx/service/include/utils.h:707-725: ties and NaN keep the earlier
//   operand); for 16-bit types the chosen input's own bits are returned.
//   avg = the sum above divided once by the number of inputs before the final
//   rounding: IEEE division for the floating types (16-bit: in fp32), C division
//   (truncating toward zero, on the wrapped sum) for signed integers, unsigned
//   division for unsigned ones.  FlagCX itself only forwards avg to vendor
//   libraries, so this definition is this path's own.
//   Two further associations of the same k inputs (enum Sched) exist for the
//   callers that must reproduce a multi-step schedule of the reference's in one
//   launch: its binomial tree and its host ring's "local operand first" chain.
//   They round to the element type after every step, as those schedules do.
//
// Data movement: one 16-byte vector per lane per input, U vectors per lane in
// flight per input, all K*U loads issued before the first use.  Loads and
// stores bypass the caches (nontemporal) unless the launch's policy word
// (`keep` in every argument block) asks for ordinary accesses: one bit per
// input plus one for the stores, uniform over the launch.  The index
// space is anchored at the output pointer rounded down to 16 bytes, so stores
// are always whole aligned vectors except in the first and last vector of a
// segment, which fall back to element accesses.  An input need not share the
// output's misalignment: its vectors are fetched with 128-bit loads that start
// wherever the matching elements start (see ldg_stream).  Large
// segments are handed to workgroups as 512-byte pieces 32 KiB apart (see
// TilePlan) instead of contiguous 16 KiB runs.
#pragma once
#include "fx_common.hpp"

namespace fx {

// ------------------------------------------------------------------ reducers

// avg accumulates like sum and divides in finish().
constexpr bool isAdd(int op) { return op == flagcxSum || op == flagcxAvg; }

template <int OP>
__device__ __forceinline__ float opF32(float a, float b) {
  if (isAdd(OP)) return a + b;
  if (OP == flagcxProd) return a * b;
  if (OP == flagcxMax) return (a < b) ? b : a;
  return (b < a) ? b : a;
}

template <int OP>
__device__ __forceinline__ uint32_t opI32(uint32_t a, uint32_t b) {
  if (isAdd(OP)) return a + b;
  if (OP == flagcxProd) return a * b;
  if (OP == flagcxMax) return ((int32_t)a < (int32_t)b) ? b : a;
  return ((int32_t)b < (int32_t)a) ? b : a;
}

// fp32 -> bf16 bits in the TOP half of the result (low half is garbage):
// round to nearest even; NaN keeps its sign/payload with the quiet bit forced.
__device__ __forceinline__ uint32_t roundBf16Top(float f) {
  uint32_t u = __float_as_uint(f);
  uint32_t r = u + 0x7fffu + ((u >> 16) & 1u);
  return ((u & 0x7fffffffu) > 0x7f800000u) ? (u | 0x00400000u) : r;
}

__device__ __forceinline__ float halfToF32(uint32_t bits16) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
}
// fp32 -> fp16, round to nearest even, as a step of its own: the empty asm hides
// where f came from.  Without it the compiler fuses a multiplication that feeds
// the conversion into one mixed-precision instruction that rounds the exact
// product to 16 bits once, and a product whose fp32 rounding lands on a tie
// between two fp16 values then comes out one ulp off the accumulate-in-fp32,
// round-once definition (7 of 131,072 four-input products of N(0,1) values).
__device__ __forceinline__ uint32_t f32ToHalf(float f) {
  asm("" : "+v"(f));
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}

template <int DT, int OP>
struct Red;

template <int OP>
struct Red<flagcxFloat32, OP> {
  static constexpr int ES = 4;  // element bytes
  struct Acc {
    float a[4];
  };
  static __device__ __forceinline__ void init(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) c.a[i] = __uint_as_float(v[i]);
  }
  static __device__ __forceinline__ void fold(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) c.a[i] = opF32<OP>(c.a[i], __uint_as_float(v[i]));
  }
  static __device__ __forceinline__ u32x4 finish(const Acc &c, uint32_t k) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = __float_as_uint(OP == flagcxAvg ? c.a[i] / (float)k : c.a[i]);
    return r;
  }
};

template <int OP>
struct Red<flagcxInt32, OP> {
  static constexpr int ES = 4;
  struct Acc {
    uint32_t a[4];
  };
  static __device__ __forceinline__ void init(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) c.a[i] = v[i];
  }
  static __device__ __forceinline__ void fold(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) c.a[i] = opI32<OP>(c.a[i], v[i]);
  }
  static __device__ __forceinline__ u32x4 finish(const Acc &c, uint32_t k) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = (OP == flagcxAvg) ? (uint32_t)((int32_t)c.a[i] / (int32_t)k) : c.a[i];
    return r;
  }
};

// uint32: as int32 with unsigned comparisons.
template <int OP>
struct Red<flagcxUint32, OP> {
  static constexpr int ES = 4;
  struct Acc {
    uint32_t a[4];
  };
  static __device__ __forceinline__ uint32_t op(uint32_t a, uint32_t b) {
    if (isAdd(OP)) return a + b;
    if (OP == flagcxProd) return a * b;
    if (OP == flagcxMax) return (a < b) ? b : a;
    return (b < a) ? b : a;
  }
  static __device__ __forceinline__ void init(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) c.a[i] = v[i];
  }
  static __device__ __forceinline__ void fold(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) c.a[i] = op(c.a[i], v[i]);
  }
  static __device__ __forceinline__ u32x4 finish(const Acc &c, uint32_t k) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = (OP == flagcxAvg) ? c.a[i] / k : c.a[i];
    return r;
  }
};

// 8-bit integers: sixteen per vector, each kept in a 32-bit accumulator
// (sign- or zero-extended).  The low byte of a 32-bit sum or product is the
// 8-bit result modulo 256; max/min compare the extended values.
template <bool SIGNED, int OP>
struct Red8 {
  static constexpr int ES = 1;
  struct Acc {
    int32_t a[16];
  };
  static __device__ __forceinline__ int32_t lane(uint32_t w, int b) {
    return SIGNED ? ((int32_t)(w << (24 - 8 * b)) >> 24) : (int32_t)((w >> (8 * b)) & 0xffu);
  }
  static __device__ __forceinline__ int32_t op(int32_t a, int32_t b) {
    if (isAdd(OP)) return (int32_t)((uint32_t)a + (uint32_t)b);
    if (OP == flagcxProd) return (int32_t)((uint32_t)a * (uint32_t)b);
    if (OP == flagcxMax) return (a < b) ? b : a;
    return (b < a) ? b : a;
  }
  static __device__ __forceinline__ void init(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 16; i++) c.a[i] = lane(v[i / 4], i & 3);
  }
  static __device__ __forceinline__ void fold(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 16; i++) c.a[i] = op(c.a[i], lane(v[i / 4], i & 3));
  }
  // avg divides the sum as it would read in 8 bits (wrapped), not the wide accumulator
  static __device__ __forceinline__ uint32_t byteOf(int32_t a, uint32_t k) {
    if (OP != flagcxAvg) return (uint32_t)a & 0xffu;
    if (SIGNED) return (uint32_t)(((int32_t)(a << 24) >> 24) / (int32_t)k) & 0xffu;
    return ((uint32_t)a & 0xffu) / k;
  }
  static __device__ __forceinline__ u32x4 finish(const Acc &c, uint32_t k) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++)
      r[i] = byteOf(c.a[4 * i], k) | (byteOf(c.a[4 * i + 1], k) << 8) | (byteOf(c.a[4 * i + 2], k) << 16) |
             (byteOf(c.a[4 * i + 3], k) << 24);
    return r;
  }
};
template <int OP>
struct Red<flagcxInt8, OP> : Red8<true, OP> {};
template <int OP>
struct Red<flagcxUint8, OP> : Red8<false, OP> {};

// 64-bit integers and doubles: two per vector.
template <bool SIGNED, int OP>
struct RedI64 {
  static constexpr int ES = 8;
  struct Acc {
    uint64_t a[2];
  };
  static __device__ __forceinline__ uint64_t op(uint64_t a, uint64_t b) {
    if (isAdd(OP)) return a + b;
    if (OP == flagcxProd) return a * b;
    const bool lt = SIGNED ? ((int64_t)a < (int64_t)b) : (a < b);
    const bool gt = SIGNED ? ((int64_t)b < (int64_t)a) : (b < a);
    if (OP == flagcxMax) return lt ? b : a;
    return gt ? b : a;
  }
  static __device__ __forceinline__ uint64_t word(u32x4 v, int i) {
    return (uint64_t)v[2 * i] | ((uint64_t)v[2 * i + 1] << 32);
  }
  static __device__ __forceinline__ void init(Acc &c, u32x4 v) {
    c.a[0] = word(v, 0);
    c.a[1] = word(v, 1);
  }
  static __device__ __forceinline__ void fold(Acc &c, u32x4 v) {
    c.a[0] = op(c.a[0], word(v, 0));
    c.a[1] = op(c.a[1], word(v, 1));
  }
  static __device__ __forceinline__ uint64_t mean(uint64_t a, uint32_t k) {
    if (OP != flagcxAvg) return a;
    return SIGNED ? (uint64_t)((int64_t)a / (int64_t)k) : a / (uint64_t)k;
  }
  static __device__ __forceinline__ u32x4 finish(const Acc &c, uint32_t k) {
    const uint64_t x = mean(c.a[0], k), y = mean(c.a[1], k);
    u32x4 r = {(uint32_t)x, (uint32_t)(x >> 32), (uint32_t)y, (uint32_t)(y >> 32)};
    return r;
  }
};
template <int OP>
struct Red<flagcxInt64, OP> : RedI64<true, OP> {};
template <int OP>
struct Red<flagcxUint64, OP> : RedI64<false, OP> {};

template <int OP>
struct Red<flagcxFloat64, OP> {
  static constexpr int ES = 8;
  struct Acc {
    double a[2];
  };
  static __device__ __forceinline__ double op(double a, double b) {
    if (isAdd(OP)) return a + b;
    if (OP == flagcxProd) return a * b;
    if (OP == flagcxMax) return (a < b) ? b : a;
    return (b < a) ? b : a;
  }
  static __device__ __forceinline__ double word(u32x4 v, int i) {
    return __longlong_as_double((long long)((uint64_t)v[2 * i] | ((uint64_t)v[2 * i + 1] << 32)));
  }
  static __device__ __forceinline__ void init(Acc &c, u32x4 v) {
    c.a[0] = word(v, 0);
    c.a[1] = word(v, 1);
  }
  static __device__ __forceinline__ void fold(Acc &c, u32x4 v) {
    c.a[0] = op(c.a[0], word(v, 0));
    c.a[1] = op(c.a[1], word(v, 1));
  }
  static __device__ __forceinline__ u32x4 finish(const Acc &c, uint32_t k) {
    const double d0 = (OP == flagcxAvg) ? c.a[0] / (double)k : c.a[0], d1 = (OP == flagcxAvg) ? c.a[1] / (double)k : c.a[1];
    const uint64_t x = (uint64_t)__double_as_longlong(d0), y = (uint64_t)__double_as_longlong(d1);
    u32x4 r = {(uint32_t)x, (uint32_t)(x >> 32), (uint32_t)y, (uint32_t)(y >> 32)};
    return r;
  }
};

// bf16: widening is a shift, so for max/min the accumulator's top half IS the
// selected input's bit pattern and no rounding is needed.
template <int OP>
struct Red<flagcxBfloat16, OP> {
  static constexpr int ES = 2;
  struct Acc {
    float a[8];
  };
  static __device__ __forceinline__ void init(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      c.a[2 * i] = __uint_as_float(v[i] << 16);
      c.a[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void fold(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      c.a[2 * i] = opF32<OP>(c.a[2 * i], __uint_as_float(v[i] << 16));
      c.a[2 * i + 1] = opF32<OP>(c.a[2 * i + 1], __uint_as_float(v[i] & 0xffff0000u));
    }
  }
  static __device__ __forceinline__ u32x4 finish(const Acc &c, uint32_t k) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t lo, hi;
      if (OP == flagcxAvg) {
        lo = roundBf16Top(c.a[2 * i] / (float)k);
        hi = roundBf16Top(c.a[2 * i + 1] / (float)k);
      } else if (OP == flagcxSum || OP == flagcxProd) {
        lo = roundBf16Top(c.a[2 * i]);
        hi = roundBf16Top(c.a[2 * i + 1]);
      } else {
        lo = __float_as_uint(c.a[2 * i]);
        hi = __float_as_uint(c.a[2 * i + 1]);
      }
      r[i] = (hi & 0xffff0000u) | (lo >> 16);
    }
    return r;
  }
};

// fp16: widened with the hardware converter (exact); max/min also carry the
// raw 16-bit pattern of the current winner so the output is bit-preserving.
template <int OP>
struct Red<flagcxFloat16, OP> {
  static constexpr int ES = 2;
  static constexpr bool kSelect = (OP == flagcxMax || OP == flagcxMin);
  struct Acc {
    float a[8];
    uint32_t b[kSelect ? 8 : 1];
  };
  static __device__ __forceinline__ void init(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t lo = v[i] & 0xffffu, hi = v[i] >> 16;
      c.a[2 * i] = halfToF32(lo);
      c.a[2 * i + 1] = halfToF32(hi);
      if (kSelect) {
        c.b[2 * i] = lo;
        c.b[2 * i + 1] = hi;
      }
    }
  }
  static __device__ __forceinline__ void fold1(Acc &c, int i, uint32_t bits) {
    float x = halfToF32(bits);
    if (kSelect) {
      bool take = (OP == flagcxMax) ? (c.a[i] < x) : (x < c.a[i]);
      c.a[i] = take ? x : c.a[i];
      c.b[i] = take ? bits : c.b[i];
    } else {
      c.a[i] = opF32<OP>(c.a[i], x);
    }
  }
  static __device__ __forceinline__ void fold(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      fold1(c, 2 * i, v[i] & 0xffffu);
      fold1(c, 2 * i + 1, v[i] >> 16);
    }
  }
  static __device__ __forceinline__ u32x4 finish(const Acc &c, uint32_t k) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t lo, hi;
      if (kSelect) {
        lo = c.b[2 * i];
        hi = c.b[2 * i + 1];
      } else if (OP == flagcxAvg) {
        lo = f32ToHalf(c.a[2 * i] / (float)k);
        hi = f32ToHalf(c.a[2 * i + 1] / (float)k);
      } else {
        lo = f32ToHalf(c.a[2 * i]);
        hi = f32ToHalf(c.a[2 * i + 1]);
      }
      r[i] = (hi << 16) | lo;
    }
    return r;
  }
};

// The 16-bit types folded in the element type itself, as the reference's device
// kernel does (custom_allreduce.cu:326-361: acc = reduceOp(acc, x) on half /
// nv_bfloat16 values): a sum is rounded to 16 bits after every addition, and
// max / min hand on the LATER operand unless the earlier one compares greater /
// smaller (a > b ? a : b), so a NaN or a zero of the other sign replaces the
// accumulator where the host rule keeps it.  Sum, max and min only, the ops
// that kernel accepts.  The accumulator is the eight raw 16-bit patterns.
template <int DT, int OP>
struct RedElem {
  static_assert(DT == flagcxFloat16 || DT == flagcxBfloat16, "16-bit element types only");
  static_assert(OP == flagcxSum || OP == flagcxMax || OP == flagcxMin, "sum, max, min only");
  static constexpr int ES = 2;
  struct Acc {
    uint32_t h[8];
  };
  static __device__ __forceinline__ float widen(uint32_t bits16) {
    return DT == flagcxBfloat16 ? __uint_as_float(bits16 << 16) : halfToF32(bits16);
  }
  // One rounding per step: the hardware converters (round to nearest even; gfx950 has one for bf16 too), where
  // the default reducer's single bf16 rounding is integer arithmetic.
  static __device__ __forceinline__ uint32_t narrow(float f) {
    return DT == flagcxBfloat16 ? (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f) : f32ToHalf(f);
  }
  static __device__ __forceinline__ uint32_t step(uint32_t a, uint32_t b) {
    const float x = widen(a), y = widen(b);
    if (OP == flagcxSum) return narrow(x + y);   // the exact sum of two 16-bit values, rounded once: what a native add gives
    if (OP == flagcxMax) return (x > y) ? a : b;
    return (x < y) ? a : b;
  }
  static __device__ __forceinline__ void init(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      c.h[2 * i] = v[i] & 0xffffu;
      c.h[2 * i + 1] = v[i] >> 16;
    }
  }
  static __device__ __forceinline__ void fold(Acc &c, u32x4 v) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      c.h[2 * i] = step(c.h[2 * i], v[i] & 0xffffu);
      c.h[2 * i + 1] = step(c.h[2 * i + 1], v[i] >> 16);
    }
  }
  static __device__ __forceinline__ u32x4 finish(const Acc &c, uint32_t) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = (c.h[2 * i + 1] << 16) | (c.h[2 * i] & 0xffffu);
    return r;
  }
};

// Plain byte mover with ES-byte granularity (ES = 1, 2 or 4), used with k = 1
// for the all-gather copy phase and the alltoallv pack / unpack.
template <int ESZ>
struct CopyRed {
  static constexpr int ES = ESZ;
  struct Acc {
    u32x4 v;
  };
  static __device__ __forceinline__ void init(Acc &c, u32x4 v) { c.v = v; }
  static __device__ __forceinline__ void fold(Acc &, u32x4) {}
  static __device__ __forceinline__ u32x4 finish(const Acc &c, uint32_t) { return c.v; }
};

// ------------------------------------------------------------- one segment

// Tiling of a segment.  The index space is anchored at the output pointer
// rounded down to 16 bytes: vector j covers bytes [16j, 16j+16) from there and
// the valid elements are [lead, end).  A tile is V = U*kBlock vectors.
//
// Striped zone.  On MI355X a workgroup that touches one contiguous 16 KiB per
// stream spreads its few stores thinly over many DRAM channels, and a sparse
// write stream mixed into reads is expensive (measured: 5.9 TB/s for 8 inputs).
// The same bytes moved as 512-byte pieces 32 KiB apart reach 6.4-6.5 TB/s.  So
// the part of a segment that consists of whole regions of kStripeTiles tiles,
// aligned in ABSOLUTE address of the output, is handed out striped: tile i of a
// region owns one 512-byte column of every 32 KiB row of that region.  The rest
// (head before the first region boundary, tail after the last) is handed out
// contiguously.
//
// Two flavours.  When every stream sits at the output's offset within a
// 128-byte cache line, a piece is four whole lines in every stream: tile i
// takes column i and all loads are nontemporal.  When some stream does not, its
// piece cuts five lines and the fifth is the first line of the next column's
// piece: then tile i takes column 8 * (i % 8) + i / 8 -- workgroups are dealt
// round-robin to the eight dies, so eight neighbouring columns land on one die
// and share its L2 -- and the loads are ordinary (temporal) ones, so that the
// shared line is still in that L2 when the neighbour asks for it.  Measured on
// copies of 1-2 GiB whose source is 4-132 bytes off: contiguous tiles 5.6-5.9
// TB/s; striped by column i with nontemporal loads 5.8 (1.25 x the bytes
// fetched); grouped columns and temporal loads 6.3-6.4 (1.11 x).  Aligned
// streams keep column i and nontemporal loads (grouped columns cost 1-2 % for
// 8 inputs of 512 MiB, temporal loads 4 % for large aligned streams).
constexpr uint32_t kPieceVecs = 32;                         // 512 bytes (a divisor of the workgroup size)
constexpr uint32_t kStripeTiles = 64;                       // tiles per region (a multiple of 8)
constexpr uint32_t kRowVecs = kPieceVecs * kStripeTiles;    // 32 KiB
// Segments shorter than this (output bytes) stay contiguous: the smallest region
// (two vectors per lane) is 512 KiB.
constexpr uint64_t kStripeMinBytes = 1ull << 19;

// Streams a and b sit at the same offset within a cache line.
constexpr uint64_t kLineBytes = 128;
__host__ __device__ inline bool sameLinePhase(uint64_t a, uint64_t b) { return ((a ^ b) & (kLineBytes - 1)) == 0; }

struct TilePlan {
  uint64_t nv;                 // vectors spanned by the segment
  uint64_t firstFull, endFull; // vectors [firstFull, endFull) lie wholly inside the segment
  uint64_t zs, ze;             // striped zone [zs, ze) in vectors; empty when zs == ze
  uint32_t zoneTiles, headTiles, tailTiles;
  bool grouped;                // striped zone of a segment with a stream off the output's line phase (see above)
  __host__ __device__ uint64_t tiles() const { return (uint64_t)zoneTiles + headTiles + tailTiles; }
};

// Same function on host (grid size, tile prefix tables) and device (mapping).
// How the whole regions of a segment are handed out.
enum HandOut {
  kContiguous = 0,  // not striped at all
  kStriped = 1,     // tile i owns column i, nontemporal loads: every stream at the output's line phase
  kGrouped = 2      // eight neighbouring columns per die, temporal loads: a copy whose source is off that phase
};

// Reductions of several inputs with one off the line phase stay contiguous:
// measured with every other input off by one element, the grouped flavour
// (temporal loads for the aligned inputs too) read 6.0-6.2 TB/s for 2 inputs and
// 6.0 for 4 where contiguous tiles read 6.45-6.58 and 6.37; for 8 inputs the two
// were equal (6.0).
__host__ __device__ inline HandOut handOutFor(bool samePhase, int k) {
  return samePhase ? kStriped : (k == 1 ? kGrouped : kContiguous);
}

// Element sizes, vectors per tile and tiles per region are powers of two, so
// the plan is shifts and masks only: a persistent kernel works it out once per
// trigger in every workgroup, with an element size it only knows at run time,
// and a 64-bit division there is a hundred instructions.
__host__ __device__ constexpr uint32_t log2Of(uint32_t x) {   // x a power of two
  uint32_t l = 0;
  while ((1u << l) < x) l++;
  return l;
}
__host__ __device__ inline TilePlan planTiles(uint64_t outAddr, uint64_t count, int es, int U, HandOut how) {
  TilePlan tp;
  const uint32_t esShift = (es == 1) ? 0u : (es == 2) ? 1u : (es == 4) ? 2u : 3u;
  const uint32_t veShift = 4u - esShift;                                     // elements per vector
  const uint32_t vShift = log2Of(kBlock) + ((U == 1) ? 0u : (U == 2) ? 1u : (U == 4) ? 2u : 3u);   // vectors per tile
  const uint32_t rvShift = vShift + log2Of(kStripeTiles);                    // vectors per region
  const uint64_t V = 1ull << vShift, RV = 1ull << rvShift, ve = 1ull << veShift;
  const uint64_t mis = outAddr & 15u, lead = mis >> esShift, end = lead + count;
  tp.nv = (end + ve - 1) >> veShift;
  tp.firstFull = (lead + ve - 1) >> veShift;
  tp.endFull = end >> veShift;
  const uint64_t a0 = (outAddr - mis) >> 4;  // absolute vector number of vector 0
  const uint64_t zs = ((a0 + tp.firstFull + RV - 1) >> rvShift) << rvShift, ze = ((a0 + tp.endFull) >> rvShift) << rvShift;
  tp.grouped = (how == kGrouped);
  if (how == kContiguous || ze <= zs || (count << esShift) < kStripeMinBytes) {
    tp.zs = tp.ze = 0;
  } else {
    tp.zs = zs - a0;
    tp.ze = ze - a0;
  }
  tp.zoneTiles = (uint32_t)((tp.ze - tp.zs) >> vShift);
  tp.headTiles = (uint32_t)((tp.zs + V - 1) >> vShift);
  tp.tailTiles = (uint32_t)((tp.nv - tp.ze + V - 1) >> vShift);
  return tp;
}

// Every buffer these kernels touch is device-visible global memory.  Pointers
// that reach a kernel through a table in memory or through LDS carry no address
// space, and the compiler would then use flat instructions for them; passing
// them through the global address space once lets it pick global ones.
typedef __attribute__((address_space(1))) char GlobalByte;
__device__ __forceinline__ const char *asGlobal(const void *p) {
  return (const char *)(const GlobalByte *)(uintptr_t)p;
}
__device__ __forceinline__ char *asGlobal(void *p) { return (char *)(GlobalByte *)(uintptr_t)p; }

template <int K>
struct Seg {
  const char *in[K];
  char *out;
  uint64_t lead, end;
  uint32_t keep;   // cache policy of the launch (kKeepAllLoads / kKeepStores bits), wave-uniform
  __device__ __forceinline__ const char *inp(int p) const { return in[p]; }
  __device__ __forceinline__ int inputs() const { return K; }
};

// Runtime-k variant: the pointer table stays where it is (kernel argument
// block) and is read through scalar loads instead of being copied.
template <>
struct Seg<0> {
  const void *const *raw;
  uint64_t mis;
  char *out;
  uint64_t lead, end;
  uint32_t keep;
  int k;
  __device__ __forceinline__ const char *inp(int p) const { return asGlobal(raw[p]) - mis; }
  __device__ __forceinline__ int inputs() const { return k; }
};

template <int ES>
__device__ __forceinline__ u32x4 gatherElems(const char *base, uint64_t e0, int lo, int hi) {
  constexpr int VE = 16 / ES;
  u32x4 r = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int s = 0; s < VE; s++) {
    if (s >= lo && s < hi) {
      if constexpr (ES == 8) {
        const uint64_t w = *reinterpret_cast<const uint64_t *>(base + (e0 + s) * 8);
        r[2 * s] = (uint32_t)w;
        r[2 * s + 1] = (uint32_t)(w >> 32);
      } else if constexpr (ES == 4) {
        r[s] = *reinterpret_cast<const uint32_t *>(base + (e0 + s) * 4);
      } else if constexpr (ES == 2) {
        uint32_t h = *reinterpret_cast<const uint16_t *>(base + (e0 + s) * 2);
        r[s / 2] |= h << (16 * (s & 1));
      } else {
        uint32_t h = *reinterpret_cast<const uint8_t *>(base + e0 + s);
        r[s / 4] |= h << (8 * (s & 3));
      }
    }
  }
  return r;
}

template <int ES>
__device__ __forceinline__ void scatterElems(char *base, uint64_t e0, int lo, int hi, u32x4 v) {
  constexpr int VE = 16 / ES;
#pragma unroll
  for (int s = 0; s < VE; s++) {
    if (s >= lo && s < hi) {
      if constexpr (ES == 8)
        *reinterpret_cast<uint64_t *>(base + (e0 + s) * 8) = (uint64_t)v[2 * s] | ((uint64_t)v[2 * s + 1] << 32);
      else if constexpr (ES == 4)
        *reinterpret_cast<uint32_t *>(base + (e0 + s) * 4) = v[s];
      else if constexpr (ES == 2)
        *reinterpret_cast<uint16_t *>(base + (e0 + s) * 2) = (uint16_t)(v[s / 2] >> (16 * (s & 1)));
      else
        *reinterpret_cast<uint8_t *>(base + e0 + s) = (uint8_t)(v[s / 4] >> (8 * (s & 3)));
    }
  }
}

// Segment with several outputs: the result of every vector is stored to out
// and to each of more[0..nmore-1] (the software form of a multicast store: one
// read of the k inputs serves every rank's receive buffer).  All outputs share
// out's misalignment within 16 bytes; the host checks that.
template <int K>
struct SegB : Seg<K> {
  char *more[kMaxFixedK - 1];
  int nmore;
};

// One result vector to memory, streaming or ordinary as the launch's policy says
// (the choice is the same for every lane of the launch).
__device__ __forceinline__ void stg_as(uint32_t keep, void *p, u32x4 v) {
  if (keep & kKeepStores) stg_keep(p, v);
  else stg_stream(p, v);
}
template <int K>
__device__ __forceinline__ void storeVector(const Seg<K> &sg, uint64_t byteOff, u32x4 v) {
  stg_as(sg.keep, sg.out + byteOff, v);
}
template <int K>
__device__ __forceinline__ void storeVector(const SegB<K> &sg, uint64_t byteOff, u32x4 v) {
  stg_as(sg.keep, sg.out + byteOff, v);
#pragma unroll
  for (int o = 0; o < kMaxFixedK - 1; o++)   // constant indices keep the pointers in scalar registers
    if (o < sg.nmore) stg_as(sg.keep, sg.more[o] + byteOff, v);
}
template <int ES, int K>
__device__ __forceinline__ void storeElems(const Seg<K> &sg, uint64_t e0, int lo, int hi, u32x4 v) {
  scatterElems<ES>(sg.out, e0, lo, hi, v);
}

// Segment whose results are written THROUGH the caches (system-scope stores):
// nothing of it stays dirty in a die's L2, so a kernel that must publish its
// results to other agents while it keeps running (the FIFO consumer) needs no
// cache write-back afterwards, only to wait for its stores.
template <int K>
struct SegWT : Seg<K> {};

template <class T>
__device__ __forceinline__ void storeThrough(void *p, T v) {
  __hip_atomic_store(reinterpret_cast<T *>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
// A whole vector: one 128-bit buffer store carrying the system-scope and
// streaming cache-policy bits (two 64-bit atomic stores reach only 3.7 TB/s on
// a large segment).  The buffer descriptor is based at the first active lane's
// address; lane addresses only grow with the lane number in every tiling used
// here, so the 32-bit offsets are small and non-negative.
typedef int i32x4 __attribute__((ext_vector_type(4)));
template <int K>
__device__ __forceinline__ void storeVector(const SegWT<K> &sg, uint64_t byteOff, u32x4 v) {
  const uint64_t a = (uint64_t)(uintptr_t)(sg.out + byteOff);
  const uint64_t base = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a) |
                        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32)) << 32);
  __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(uintptr_t)base, 0, 0x7fffffff, 0x00020000);
  constexpr int kSc0 = 1, kNt = 2, kSc1 = 16;
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, v), rsrc, (int)(uint32_t)(a - base), 0,
                                         kSc0 | kSc1 | kNt);
}
template <int ES, int K>
__device__ __forceinline__ void storeElems(const SegWT<K> &sg, uint64_t e0, int lo, int hi, u32x4 v) {
  constexpr int VE = 16 / ES;
#pragma unroll
  for (int s = 0; s < VE; s++) {
    if (s >= lo && s < hi) {
      if constexpr (ES == 8)
        storeThrough<uint64_t>(sg.out + (e0 + s) * 8, (uint64_t)v[2 * s] | ((uint64_t)v[2 * s + 1] << 32));
      else if constexpr (ES == 4)
        storeThrough<uint32_t>(sg.out + (e0 + s) * 4, v[s]);
      else if constexpr (ES == 2)
        storeThrough<uint16_t>(sg.out + (e0 + s) * 2, (uint16_t)(v[s / 2] >> (16 * (s & 1))));
      else
        storeThrough<uint8_t>(sg.out + e0 + s, (uint8_t)(v[s / 4] >> (8 * (s & 3))));
    }
  }
}
template <int ES, int K>
__device__ __forceinline__ void storeElems(const SegB<K> &sg, uint64_t e0, int lo, int hi, u32x4 v) {
  scatterElems<ES>(sg.out, e0, lo, hi, v);
#pragma unroll
  for (int o = 0; o < kMaxFixedK - 1; o++)
    if (o < sg.nmore) scatterElems<ES>(sg.more[o], e0, lo, hi, v);
}

// Runtime number of inputs AND of outputs (more ranks than a descriptor has
// slots): both pointer tables stay in the kernel argument block and are read
// through scalar loads.  All outputs share out's misalignment within 16 bytes.
struct SegMany : Seg<0> {
  void *const *rawOut;   // the outputs after the first
  int nmore;
  __device__ __forceinline__ char *outp(int o) const { return asGlobal(rawOut[o]) - mis; }
};
// The extra outputs four at a time: their pointers come through scalar loads,
// and four independent ones are fetched together where a loop of single ones
// would wait for each in turn.
template <class SG>
__device__ __forceinline__ void storeToMore(const SG &sg, uint64_t byteOff, u32x4 v) {
  for (int o = 0; o < sg.nmore; o += 4) {
    char *q[4];
#pragma unroll
    for (int i = 0; i < 4; i++) q[i] = sg.outp(o + i < sg.nmore ? o + i : o);
#pragma unroll
    for (int i = 0; i < 4; i++)
      if (o + i < sg.nmore) stg_as(sg.keep, q[i] + byteOff, v);
  }
}
__device__ __forceinline__ void storeVector(const SegMany &sg, uint64_t byteOff, u32x4 v) {
  stg_as(sg.keep, sg.out + byteOff, v);
  storeToMore(sg, byteOff, v);
}
template <int ES>
__device__ __forceinline__ void storeElems(const SegMany &sg, uint64_t e0, int lo, int hi, u32x4 v) {
  scatterElems<ES>(sg.out, e0, lo, hi, v);
  for (int o = 0; o < sg.nmore; o++) scatterElems<ES>(sg.outp(o), e0, lo, hi, v);
}

// One chunk of a chunked collective over many ranks: the fold starts at input
// `first` and wraps, or reads the single input `only`; the result goes to one
// output or to all of them.  Pointer tables stay in the kernel argument block.
struct SegChunk {
  const void *const *rawIn;
  void *const *rawOut;   // outputs after the primary one (nmore of them)
  uint64_t inAdj;        // byte offset of the chunk in every input, minus the output's misalignment
  uint64_t outAdj;       // the same for the extra outputs
  char *out;
  uint64_t lead, end;
  uint32_t keep;
  int k, first, only, nmore;
  __device__ __forceinline__ int inputs() const { return only >= 0 ? 1 : k; }
  __device__ __forceinline__ const char *inp(int p) const {
    int idx = only;
    if (idx < 0) {
      idx = first + p;
      if (idx >= k) idx -= k;
    }
    return asGlobal(rawIn[idx]) + inAdj;
  }
  __device__ __forceinline__ char *outp(int o) const { return asGlobal(rawOut[o]) + outAdj; }
};
__device__ __forceinline__ void storeVector(const SegChunk &sg, uint64_t byteOff, u32x4 v) {
  stg_as(sg.keep, sg.out + byteOff, v);
  storeToMore(sg, byteOff, v);
}
template <int ES>
__device__ __forceinline__ void storeElems(const SegChunk &sg, uint64_t e0, int lo, int hi, u32x4 v) {
  scatterElems<ES>(sg.out, e0, lo, hi, v);
  for (int o = 0; o < sg.nmore; o++) scatterElems<ES>(sg.outp(o), e0, lo, hi, v);
}

// ------------------------------------------------------- fold associations
//
// How the K input vectors of one output vector are combined.
//   kChain      acc = in[0]; acc = acc (op) in[p], p = 1..K-1: the peer loop of
//               flagcx/adaptor/kernel/nvidia/custom_allreduce.cu:345-359.
//   kTree       the binomial tree of the reference's flagcxReduce
//               (flagcx/runner/uni_runner_impl.cc:1314-1326,1372-1477), in[a] being
//               tree rank a (rank (a + root) % n): in round i every tree rank a with
//               more than i receive steps computes
//               partial(a) = partial(a + 2^i) (op) partial(a), the received operand
//               first; the result is partial(0).
//   kKeepLocal  the host ring's chain (flagcx/service/bootstrap.cc:853-871 with the
//               std::max / std::min of flagcx/service/include/utils.h:707-725):
//               res = in[0]; res = in[j] (op) res, j = 1..K-1 -- the operand that is
//               local to the rank of that step comes FIRST, so it is the one kept
//               when the comparison is false (a NaN on either side), and a NaN met
//               on the way hides what was folded before it exactly as on the ring.
// In the tree and in the keep-local chain every step is a complete two-input
// reduction in the element type (16-bit sums and products are rounded after
// every step), as when each step is a launch of its own writing a buffer.
enum Sched { kChain = 0, kTree = 1, kKeepLocal = 2 };

// Receive steps of tree rank a among n (uni_runner_impl.cc:1314-1326): the root
// takes ceil(log2 n); others the number of trailing zero bits of a, clipped so
// that a + 2^i stays below n.
__host__ __device__ constexpr int treeStepsOf(int a, int n) {
  int total = 0;
  while ((1 << total) < n) total++;
  if (a == 0) return total;
  int st = 0;
  while (((a >> st) & 1) == 0) st++;
  if (st && n - a <= (1 << (st - 1))) {
    int rest = n - a - 1;
    for (st = 0; rest; rest >>= 1) st++;
  }
  return st;
}

template <class R>
__device__ __forceinline__ u32x4 combineTwo(u32x4 x, u32x4 y) {
  typename R::Acc acc;
  R::init(acc, x);
  R::fold(acc, y);
  return R::finish(acc, 2u);
}

template <class R, int K, int SCHED>
__device__ __forceinline__ u32x4 foldVectors(u32x4 (&v)[K]) {
  if constexpr (SCHED == kChain) {
    typename R::Acc acc;
    R::init(acc, v[0]);
#pragma unroll
    for (int p = 1; p < K; p++) R::fold(acc, v[p]);
    return R::finish(acc, (uint32_t)K);
  } else if constexpr (SCHED == kTree) {
    constexpr int total = treeStepsOf(0, K);
#pragma unroll
    for (int i = 0; i < total; i++) {
#pragma unroll
      for (int a = 0; a < K; a++)   // a + 2^i takes no step in round i, so the order of a within a round is free
        if (treeStepsOf(a, K) > i) v[a] = combineTwo<R>(v[a + (1 << i)], v[a]);
    }
    return v[0];
  } else {
    u32x4 r = v[0];
#pragma unroll
    for (int j = 1; j < K; j++) r = combineTwo<R>(v[j], r);
    return r;
  }
}

// Reduce vector j of the segment with full bounds / alignment handling.
template <class R, int K, int SCHED, class SG>
__device__ __forceinline__ void reduceVectorChecked(const SG &sg, uint64_t j) {
  constexpr int VE = 16 / R::ES;
  const uint64_t e0 = j * VE;
  if (e0 >= sg.end || e0 + VE <= sg.lead) return;
  const int lo = (sg.lead > e0) ? (int)(sg.lead - e0) : 0;
  const int hi = (sg.end - e0 < (uint64_t)VE) ? (int)(sg.end - e0) : VE;
  const bool full = (lo == 0 && hi == VE);
  auto fetch = [&](int p) -> u32x4 {
    if (!full) return gatherElems<R::ES>(sg.inp(p), e0, lo, hi);
    return ldg_stream(sg.inp(p) + j * 16);
  };
  u32x4 r;
  if constexpr (SCHED != kChain) {
    static_assert(K > 0, "the tree and keep-local associations need a compile-time input count");
    u32x4 v[K > 0 ? K : 1];
#pragma unroll
    for (int p = 0; p < K; p++) v[p] = fetch(p);
    r = foldVectors<R, (K > 0 ? K : 1), SCHED>(v);
  } else {
    typename R::Acc acc;
    const int k = sg.inputs();
    R::init(acc, fetch(0));
    // Sixteen inputs in flight at a time, folded in their order: a launch smaller than one full tile comes through
    // here, and with a run-time k nothing else overlaps the loads -- one after the other they cost 0.3 us per input.
    constexpr int kGroup = 16;
    int p = 1;
    for (; p + kGroup <= k; p += kGroup) {
      u32x4 v[kGroup];
#pragma unroll
      for (int q = 0; q < kGroup; q++) v[q] = fetch(p + q);
#pragma unroll
      for (int q = 0; q < kGroup; q++) R::fold(acc, v[q]);
    }
    for (; p < k; p++) R::fold(acc, fetch(p));
    r = R::finish(acc, (uint32_t)k);
  }
  if (full)
    storeVector(sg, j * 16, r);
  else
    storeElems<R::ES>(sg, e0, lo, hi, r);
}

// Branch-free body: lane handles U whole vectors at byte offsets off + u*ustride
// of every stream, all K*U loads in flight before the first use.  `keep` is the
// launch's cache policy: input p is read with ordinary loads when bit p is set,
// with nontemporal ones otherwise (the same for every lane, so the choice is a
// scalar branch around the U loads of that input).
template <class R, int K, int U, int SCHED, class SG>
__device__ __forceinline__ void reduceVectorsFixed(const SG &sg, uint64_t off, uint64_t ustride, uint32_t keep) {
  u32x4 v[U][K];
#pragma unroll
  for (int p = 0; p < K; p++) {
    const char *ip = sg.inp(p) + off;
    if ((keep >> p) & 1u) {
#pragma unroll
      for (int u = 0; u < U; u++) v[u][p] = ldg_keep(ip + u * ustride);
    } else {
#pragma unroll
      for (int u = 0; u < U; u++) v[u][p] = ldg_stream(ip + u * ustride);
    }
  }
#pragma unroll
  for (int u = 0; u < U; u++) storeVector(sg, off + u * ustride, foldVectors<R, K, SCHED>(v[u]));
}

constexpr int kRuntimeGroup = 4;   // inputs a lane of a run-time-k kernel keeps in flight

template <bool KEEP>
__device__ __forceinline__ u32x4 ldg_as(const void *p) {
  return KEEP ? ldg_keep(p) : ldg_stream(p);
}

// The same for a run-time number of inputs, folded in their order.  The load
// flavour is a template parameter here and the caller branches once.
template <class R, int U, bool KEEP, class SG>
__device__ __forceinline__ void reduceVectorsRuntime(const SG &sg, uint64_t off, uint64_t ustride) {
  typename R::Acc acc[U];
#pragma unroll
  for (int u = 0; u < U; u++) R::init(acc[u], ldg_as<KEEP>(sg.inp(0) + off + u * ustride));
  // kRuntimeGroup inputs in flight at a time (folded in their order): a lane that waits for
  // every input in turn is what a small launch of many inputs spends its time on
  const int k = sg.inputs();
  int p = 1;
  for (; p + kRuntimeGroup <= k; p += kRuntimeGroup) {
    u32x4 v[kRuntimeGroup][U];
#pragma unroll
    for (int q = 0; q < kRuntimeGroup; q++) {
      const char *ip = sg.inp(p + q);
#pragma unroll
      for (int u = 0; u < U; u++) v[q][u] = ldg_as<KEEP>(ip + off + u * ustride);
    }
#pragma unroll
    for (int q = 0; q < kRuntimeGroup; q++)
#pragma unroll
      for (int u = 0; u < U; u++) R::fold(acc[u], v[q][u]);
  }
  for (; p < k; p++) {
    const char *ip = sg.inp(p);
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = ldg_as<KEEP>(ip + off + u * ustride);
#pragma unroll
    for (int u = 0; u < U; u++) R::fold(acc[u], v[u]);
  }
#pragma unroll
  for (int u = 0; u < U; u++) storeVector(sg, off + u * ustride, R::finish(acc[u], (uint32_t)sg.inputs()));
}

template <class R, int K, int U, int SCHED, class SG>
__device__ __forceinline__ void reduceVectorsFast(const SG &sg, uint64_t off, uint64_t ustride, uint32_t keep) {
  if constexpr (K > 0) {
    reduceVectorsFixed<R, K, U, SCHED>(sg, off, ustride, keep);
  } else {
    static_assert(SCHED == kChain, "run-time input counts fold in input order only");
    if (keep & kKeepAllLoads) reduceVectorsRuntime<R, U, true>(sg, off, ustride);
    else reduceVectorsRuntime<R, U, false>(sg, off, ustride);
  }
}

// Which vectors lane `tid` of the workgroup that owns tile `tile` handles:
// j, j + stride, .., U of them.  `fast` (the same for the whole workgroup) says
// that all U * kBlock vectors of the tile are whole and inside the segment;
// otherwise every vector below `limit` goes through the checked path.  Shared by the kernels and by the host-side check of
// this index arithmetic.
struct TileLane {
  uint64_t j, stride, limit;
  bool fast;
};

// xcdShift = (number of the workgroup that executes the tile - tile) mod 8:
// workgroups are dealt to the eight dies round-robin by their number, and the
// grouped flavour wants eight neighbouring columns on one die.
__host__ __device__ inline TileLane laneOfTile(const TilePlan &tp, uint32_t tile, uint32_t tid, int U,
                                               uint32_t xcdShift = 0) {
  const uint64_t V = (uint64_t)U * kBlock;
  TileLane tl;
  if (tile < tp.zoneTiles) {
    // tile i of region r owns vectors zs + r*RV + row*kRowVecs + i*kPieceVecs + [0, kPieceVecs)
    // for row = 0 .. V/kPieceVecs-1; lane (u, tid) takes row u*(kBlock/kPieceVecs) + tid/kPieceVecs.
    const uint32_t r = tile / kStripeTiles, t = tile % kStripeTiles;
    const uint32_t i = tp.grouped ? ((t + xcdShift) % 8) * (kStripeTiles / 8) + t / 8 : t;   // which column this tile owns
    tl.j = tp.zs + (uint64_t)r * (V * kStripeTiles) + (uint64_t)(tid / kPieceVecs) * kRowVecs + i * kPieceVecs +
           (tid % kPieceVecs);
    tl.stride = (uint64_t)(kBlock / kPieceVecs) * kRowVecs;
    tl.limit = tp.ze;
    tl.fast = true;
    return tl;
  }
  const uint32_t t = tile - tp.zoneTiles;
  uint64_t j0;
  if (t < tp.headTiles) {
    j0 = (uint64_t)t * V;
    tl.limit = (tp.ze > tp.zs) ? tp.zs : tp.nv;   // the head stops where the zone begins
  } else {
    j0 = tp.ze + (uint64_t)(t - tp.headTiles) * V;
    tl.limit = tp.nv;
  }
  const uint64_t fastEnd = (tl.limit < tp.endFull) ? tl.limit : tp.endFull;
  tl.j = j0 + tid;
  tl.stride = kBlock;
  tl.fast = j0 >= tp.firstFull && j0 + V <= fastEnd;
  return tl;
}

// Tile `tile` of the segment: striped zone first, then head, then tail.
// xcdShift must be the same for every tile of the segment (it decides which
// column a tile owns in the grouped flavour): a launch whose workgroup b runs
// tile b - first passes (b - tile) mod 8 = first mod 8, so that the grouping
// follows the dies; a kernel that hands tiles out differently passes 0.
template <class R, int K, int U, class SG, int SCHED = kChain>
__device__ __forceinline__ void reduceTile(const SG &sg, const TilePlan &tp, uint32_t tile, uint32_t xcdShift) {
  const TileLane tl = laneOfTile(tp, tile, threadIdx.x, U, xcdShift);
  if (tl.fast) {
    // The grouped flavour only occurs for one-input segments (handOutFor): its
    // loads are ordinary ones whatever the launch's policy says.
    const uint32_t keep = sg.keep | ((K == 1 && tp.grouped && tile < tp.zoneTiles) ? 1u : 0u);
    reduceVectorsFast<R, K, U, SCHED>(sg, tl.j * 16, tl.stride * 16, keep);
  } else {
#pragma unroll 1
    for (int u = 0; u < U; u++) {
      const uint64_t j = tl.j + (uint64_t)u * tl.stride;
      if (j < tl.limit) reduceVectorChecked<R, K, SCHED>(sg, j);
    }
  }
}

// Build the output-anchored segment from raw element pointers.
// `co` carries what the caller already knows about further streams (the extra
// outputs of a multi-output segment).
template <int ES, int U, int K>
__device__ __forceinline__ TilePlan makeSeg(Seg<K> &sg, const void *const *in, void *out, uint64_t count, int,
                                            bool co = true) {
  const uint64_t mis = (uint64_t)(uintptr_t)out & 15u;
  sg.out = asGlobal(out) - mis;
  sg.lead = mis / ES;
  sg.end = sg.lead + count;
#pragma unroll
  for (int p = 0; p < K; p++) {
    co = co && sameLinePhase((uint64_t)(uintptr_t)in[p], (uint64_t)(uintptr_t)out);
    sg.in[p] = asGlobal(in[p]) - mis;
  }
  return planTiles((uint64_t)(uintptr_t)out, count, ES, U, handOutFor(co, K));
}

template <int ES, int U>
__device__ __forceinline__ TilePlan makeSeg(Seg<0> &sg, const void *const *in, void *out, uint64_t count, int k) {
  const uint64_t mis = (uint64_t)(uintptr_t)out & 15u;
  sg.raw = in;
  sg.mis = mis;
  sg.out = asGlobal(out) - mis;
  sg.lead = mis / ES;
  sg.end = sg.lead + count;
  sg.k = k;
  bool co = true;
  for (int p = 0; p < k; p++) co = co && sameLinePhase((uint64_t)(uintptr_t)in[p], (uint64_t)(uintptr_t)out);
  return planTiles((uint64_t)(uintptr_t)out, count, ES, U, handOutFor(co, k));
}

// Host twin of the co-alignment test above; `more` are further outputs.
inline bool coAlignedHost(const void *out, const void *const *in, int k, void *const *more = nullptr, int nmore = 0) {
  for (int p = 0; p < k; p++)
    if (!sameLinePhase((uint64_t)(uintptr_t)in[p], (uint64_t)(uintptr_t)out)) return false;
  for (int o = 0; o < nmore; o++)
    if (!sameLinePhase((uint64_t)(uintptr_t)more[o], (uint64_t)(uintptr_t)out)) return false;
  return true;
}

// --------------------------------------------------------- kernel arguments

template <int K>
struct DirectArgs {
  const void *in[K > 0 ? K : kMaxK];
  void *out;
  uint64_t count;
  int k;
  uint32_t keep;   // cache policy, see kKeepAllLoads
};

struct ManyArgs {
  const void *in[kMaxK];
  void *out[kMaxK];
  uint64_t count;
  int k, nout;
  uint32_t keep;
  int co;   // every stream sits at out[0]'s offset within a cache line (the host has looked at all k + nout pointers)
};

// k inputs (rotated by the host) folded once and stored to nout buffers.
template <class R, int U>
__global__ void __launch_bounds__(kBlock) reduceBcastRuntime(ManyArgs a) {
  SegMany sg;
  const uint64_t mis = (uint64_t)(uintptr_t)a.out[0] & 15u;
  sg.raw = a.in;
  sg.mis = mis;
  sg.out = asGlobal(a.out[0]) - mis;
  sg.lead = mis / R::ES;
  sg.end = sg.lead + a.count;
  sg.k = a.k;
  sg.keep = a.keep;
  sg.rawOut = a.out + 1;
  sg.nmore = a.nout - 1;
  const TilePlan tp = planTiles((uint64_t)(uintptr_t)a.out[0], a.count, R::ES, U, handOutFor(a.co != 0, a.k));
  reduceTile<R, 0, U>(sg, tp, blockIdx.x, 0u);
}

__device__ __forceinline__ uint32_t findSlice(const uint32_t *tileStart, uint32_t n, uint32_t b);

// Up to kMaxK chunks over up to kMaxK inputs and outputs in one launch.
struct ChunkedArgs {
  const void *in[kMaxK];
  void *out[kMaxK];
  uint64_t inOff[kMaxK], outOff[kMaxK];   // bytes
  uint64_t cnt[kMaxK];                    // elements
  uint32_t tileStart[kMaxK + 1];
  int8_t first[kMaxK];                    // fold order starts at this input
  int8_t only[kMaxK];                     // >= 0: this input alone
  int8_t outSel[kMaxK];                   // >= 0: this output alone; -1: all nout
  int8_t co[kMaxK];                       // chunkCoAligned of the chunk, worked out once on the host
  int k, nout, nchunks;
  uint32_t keep;
};

// Whether every stream of a chunk sits at the primary output's offset within a
// cache line.  The host works it out (it reads up to k + nout pointers) and
// leaves it in co[c] for the kernel.
__host__ __device__ inline bool chunkCoAligned(const ChunkedArgs &a, int c) {
  const int primary = a.outSel[c] >= 0 ? a.outSel[c] : 0;
  const uint64_t o = (uint64_t)(uintptr_t)a.out[primary] + a.outOff[c];
  bool co = true;
  if (a.only[c] >= 0) {
    co = sameLinePhase((uint64_t)(uintptr_t)a.in[a.only[c]] + a.inOff[c], o);
  } else {
    for (int p = 0; p < a.k; p++) co = co && sameLinePhase((uint64_t)(uintptr_t)a.in[p] + a.inOff[c], o);
  }
  if (a.outSel[c] < 0)
    for (int r = 1; r < a.nout; r++) co = co && sameLinePhase((uint64_t)(uintptr_t)a.out[r] + a.outOff[c], o);
  return co;
}
template <int ES, int U>
__host__ __device__ inline TilePlan chunkPlan(const ChunkedArgs &a, int c) {
  const int primary = a.outSel[c] >= 0 ? a.outSel[c] : 0;
  return planTiles((uint64_t)(uintptr_t)a.out[primary] + a.outOff[c], a.cnt[c], ES, U,
                   handOutFor(a.co[c] != 0, a.only[c] >= 0 ? 1 : a.k));
}

template <class R, int U>
__global__ void __launch_bounds__(kBlock) reduceChunksRuntime(ChunkedArgs a) {
  const uint32_t b = blockIdx.x;
  const uint32_t c = findSlice(a.tileStart, (uint32_t)a.nchunks, b);
  const int primary = a.outSel[c] >= 0 ? a.outSel[c] : 0;
  const uint64_t o = (uint64_t)(uintptr_t)a.out[primary] + a.outOff[c];
  const uint64_t mis = o & 15u;
  SegChunk sg;
  sg.rawIn = a.in;
  sg.rawOut = a.out + 1;
  sg.inAdj = a.inOff[c] - mis;
  sg.outAdj = a.outOff[c] - mis;
  sg.out = asGlobal((void *)(uintptr_t)o) - mis;
  sg.lead = mis / R::ES;
  sg.end = sg.lead + a.cnt[c];
  sg.k = a.k;
  sg.keep = a.keep;
  sg.first = a.first[c];
  sg.only = a.only[c];
  sg.nmore = a.outSel[c] >= 0 ? 0 : a.nout - 1;
  const TilePlan tp = chunkPlan<R::ES, U>(a, (int)c);
  reduceTile<R, 0, U>(sg, tp, b - a.tileStart[c], a.tileStart[c] & 7u);
}

template <class R, int K, int U>
__global__ void __launch_bounds__(kBlock) reduceCopyDirect(DirectArgs<K> a) {
  Seg<K> sg;
  sg.keep = a.keep;
  const TilePlan tp = makeSeg<R::ES, U>(sg, a.in, a.out, a.count, a.k);
  reduceTile<R, K, U>(sg, tp, blockIdx.x, 0u);
}

// Batched slices: a table of independent segments sharing dtype, op and k.
// tileStart[i] is the first workgroup of slice i, tileStart[n] the grid size.
struct SliceDescDev {
  const void *in[kMaxFixedK];
  void *out;
  uint64_t count;
};

// Slices carried in the kernel argument block itself (no device table to fill
// first).  The block is kept under 4 KiB, so a table for K inputs holds as many
// descriptors of K+2 words as fit: 142 for copies (K = 1), 110 for two-input
// reduces, 47 for K = 8.
template <int K>
struct SliceDescK {
  const void *in[K];
  void *out;
  uint64_t count;
};

template <int K>
constexpr int inlineSlicesFor() {
  return (4000 - 12) / (int)(sizeof(SliceDescK<K>) + sizeof(uint32_t));
}

// NS = 0 means as many slots as fit under 4 KiB.  A second, small size exists
// because the argument block is copied at every launch (about 0.3 us per KiB)
// and most batches -- one descriptor per rank or per peer -- have eight
// entries or fewer.
constexpr int kSmallSliceTable = 8;

template <int K, int NS = 0>
struct InlineSliceTable {
  static constexpr int kSlots = NS > 0 ? NS : inlineSlicesFor<K>();
  SliceDescK<K> d[kSlots];
  uint32_t tileStart[kSlots + 1];
  uint32_t n;
  uint32_t keep;
};

__device__ __forceinline__ uint32_t findSlice(const uint32_t *tileStart, uint32_t n, uint32_t b) {
  uint32_t lo = 0, hi = n;  // invariant: tileStart[lo] <= b < tileStart[hi]
  while (hi - lo > 1) {
    uint32_t mid = (lo + hi) >> 1;
    if (tileStart[mid] <= b) lo = mid; else hi = mid;
  }
  return lo;
}

template <class R, int K, int U, class D>
__device__ __forceinline__ void reduceSlicesBody(const D *d, const uint32_t *tileStart, uint32_t n, uint32_t keep) {
  const uint32_t b = blockIdx.x;
  const uint32_t i = findSlice(tileStart, n, b);
  Seg<K> sg;
  sg.keep = keep;
  const TilePlan tp = makeSeg<R::ES, U>(sg, d[i].in, d[i].out, d[i].count, K);
  reduceTile<R, K, U>(sg, tp, b - tileStart[i], tileStart[i] & 7u);
}

template <class R, int K, int U, int NS>
__global__ void __launch_bounds__(kBlock) reduceSlicesInline(InlineSliceTable<K, NS> t) {
  reduceSlicesBody<R, K, U>(t.d, t.tileStart, t.n, t.keep);
}

template <class R, int K, int U>
__global__ void __launch_bounds__(kBlock)
reduceSlicesTable(const SliceDescDev *d, const uint32_t *tileStart, uint32_t n, uint32_t keep) {
  reduceSlicesBody<R, K, U>(d, tileStart, n, keep);
}

// All-to-all of equal blocks over up to kMaxK ranks in one launch: block (r, i)
// -- block i of rank r's send buffer, which becomes block r of rank i's receive
// buffer -- is a copy segment whose two addresses follow from the 2 n base
// pointers, so no table of n * n descriptors has to travel (4,096 of them for
// 64 ranks, 29 argument blocks).  Every block gets the same number of
// workgroups, the most any of them can need; those a block has no tile for
// leave at once.
struct AllToAllArgs {
  const void *send[kMaxK];
  void *recv[kMaxK];
  uint64_t blockElems;      // elements of the kernel's copy type per block
  uint32_t tilesPerBlock;
  int n;
  uint32_t keep;
};

template <class R, int U>
__global__ void __launch_bounds__(kBlock) allToAllBlocks(AllToAllArgs a) {
  const uint32_t blk = blockIdx.x / a.tilesPerBlock, tile = blockIdx.x % a.tilesPerBlock;
  const uint32_t r = blk / (uint32_t)a.n, i = blk % (uint32_t)a.n;
  const uint64_t bytes = a.blockElems * R::ES;
  const void *in = (const char *)a.send[r] + (uint64_t)i * bytes;
  void *out = (char *)a.recv[i] + (uint64_t)r * bytes;
  Seg<1> sg;
  sg.keep = a.keep;
  const TilePlan tp = makeSeg<R::ES, U>(sg, &in, out, a.blockElems, 1);
  if (tile >= tp.tiles()) return;
  reduceTile<R, 1, U>(sg, tp, tile, (blockIdx.x - tile) & 7u);
}

// One read of the inputs, several outputs: slices whose result goes to up to
// kMaxFixedK buffers at once.
struct BcastDescDev {
  const void *in[kMaxFixedK];
  void *out[kMaxFixedK];
  uint64_t count;
  uint32_t nout;
};

// Two table sizes: the kernel-argument block is copied at every launch (about
// 0.3 us per KiB), and the common case -- a whole all-reduce merged into one
// descriptor -- should not carry seven empty slots.  Eight slots hold one
// descriptor per chunk of a collective over eight ranks.
constexpr int kInlineBcast = 8;

template <int NS>
struct InlineBcastTable {
  BcastDescDev d[NS];
  uint32_t tileStart[NS + 1];
  uint32_t n;
  uint32_t keep;
};

// SCHED other than kChain: the same launch with the inputs combined in the
// reference's tree or host-ring association (see Sched).
template <class R, int K, int U, int NS, int SCHED = kChain>
__global__ void __launch_bounds__(kBlock) reduceBcastInline(InlineBcastTable<NS> t) {
  const uint32_t b = blockIdx.x;
  const uint32_t i = findSlice(t.tileStart, t.n, b);
  const BcastDescDev &d = t.d[i];
  SegB<K> sg;
  sg.keep = t.keep;
  const uint64_t mis = (uint64_t)(uintptr_t)d.out[0] & 15u;
  sg.nmore = (int)d.nout - 1;
  bool co = true;   // every output at the same place in its cache line, or the striped pieces would split lines
#pragma unroll
  for (int o = 0; o < kMaxFixedK - 1; o++) {
    sg.more[o] = (o < sg.nmore) ? asGlobal(d.out[o + 1]) - mis : nullptr;
    if (o < sg.nmore) co = co && sameLinePhase((uint64_t)(uintptr_t)d.out[o + 1], (uint64_t)(uintptr_t)d.out[0]);
  }
  const TilePlan tp = makeSeg<R::ES, U>(static_cast<Seg<K> &>(sg), d.in, d.out[0], d.count, K, co);
  reduceTile<R, K, U, SegB<K>, SCHED>(sg, tp, b - t.tileStart[i], t.tileStart[i] & 7u);
}

}  // namespace fx
