// Shared host/device definitions for the gfx950 reduce / copy / pack kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>
#include <new>
#include <tuple>
#include <utility>

#include "flagcx_amd/fx_types.h"

namespace fx {

constexpr int kBlock = 256;     // 4 wavefronts of 64 lanes per workgroup
constexpr int kMaxFixedK = 8;   // inputs unrolled at compile time
constexpr int kMaxK = 64;       // inputs accepted by the runtime-k kernel

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__host__ __device__ inline size_t dtypeSize(int dt) {
  switch (dt) {
    case flagcxInt8:
    case flagcxUint8: return 1;
    case flagcxFloat16:
    case flagcxBfloat16: return 2;
    case flagcxInt32:
    case flagcxUint32:
    case flagcxFloat32: return 4;
    case flagcxInt64:
    case flagcxUint64:
    case flagcxFloat64: return 8;
    default: return 0;
  }
}

inline bool opSupported(int op) { return op >= flagcxSum && op <= flagcxAvg; }

// Launch `kernel` on a grid of `grid` workgroups of kBlock threads and report
// THIS launch's own status: the return value of hipLaunchKernel, not the
// thread's last-error slot, which an unrelated earlier call (say an allocation
// the caller saw fail and handled) may still occupy.
template <class Tuple, size_t... I>
inline void argPointers(Tuple &vals, void **argv, std::index_sequence<I...>) {
  ((argv[I] = static_cast<void *>(&std::get<I>(vals))), ...);
}
template <class... P, class... A>
inline flagcxResult_t launchKernel(void (*kernel)(P...), uint32_t grid, hipStream_t s, const A &...args) {
  static_assert(sizeof...(P) == sizeof...(A), "one argument per kernel parameter");
  std::tuple<P...> vals{static_cast<P>(args)...};  // each argument in the kernel's own parameter type
  void *argv[sizeof...(P)];
  argPointers(vals, argv, std::index_sequence_for<P...>{});
  return hipLaunchKernel(reinterpret_cast<const void *>(kernel), dim3(grid), dim3(kBlock), argv, 0, s) == hipSuccess
             ? flagcxSuccess
             : flagcxUnhandledDeviceError;
}

// No C++ exception may cross the C ABI: host entry points that allocate run
// their body through this.
template <class F>
inline int guarded(F body) noexcept {
  try {
    return body();
  } catch (const std::bad_alloc &) {
    return flagcxSystemError;
  } catch (...) {
    return flagcxInternalError;
  }
}

// Array of trivially copyable T that lives on the stack up to N elements and
// moves to the heap beyond: the descriptor lists of a call are almost always a
// handful (one per rank or per peer), and a heap allocation per call is a
// measurable part of a 3 us launch.
template <class T, size_t N>
class SmallVec {
 public:
  SmallVec() : p_(inl_), n_(0), cap_(N) {}
  ~SmallVec() {
    if (p_ != inl_) free(p_);
  }
  SmallVec(const SmallVec &) = delete;
  SmallVec &operator=(const SmallVec &) = delete;
  void push_back(const T &v) {
    if (n_ == cap_) reserve(cap_ * 2);
    p_[n_++] = v;
  }
  void reserve(size_t want) {
    if (want <= cap_) return;
    T *q = static_cast<T *>(malloc(want * sizeof(T)));
    if (!q) throw std::bad_alloc();
    memcpy(static_cast<void *>(q), static_cast<const void *>(p_), n_ * sizeof(T));
    if (p_ != inl_) free(p_);
    p_ = q;
    cap_ = want;
  }
  void resize(size_t n) {   // new elements are left uninitialised
    reserve(n);
    n_ = n;
  }
  void clear() { n_ = 0; }
  bool empty() const { return n_ == 0; }
  size_t size() const { return n_; }
  T *data() { return p_; }
  const T *data() const { return p_; }
  T &operator[](size_t i) { return p_[i]; }
  const T &operator[](size_t i) const { return p_[i]; }
  T &back() { return p_[n_ - 1]; }
  T *begin() { return p_; }
  T *end() { return p_ + n_; }
  const T *begin() const { return p_; }
  const T *end() const { return p_ + n_; }

 private:
  T inl_[N];
  T *p_;
  size_t n_, cap_;
};

// 128-bit streaming accesses: every byte is touched once, so keep it out of
// the caches' way (nontemporal).  Loads may start at any byte: gfx950 under HSA
// serves global loads of every width at unaligned addresses (the compiler itself
// emits one 128-bit load for an under-aligned pointer), so an input that is only
// element-aligned relative to the output's 16-byte grid costs no extra
// instructions.  Stores are always whole aligned vectors.
typedef u32x4 u32x4_anywhere __attribute__((aligned(1)));
__device__ __forceinline__ u32x4 ldg_stream(const void *p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4_anywhere *>(p));
}
// A load without the streaming hint: the line stays in the die's L2 for a
// neighbouring workgroup that needs its other half.  Issued as a buffer load
// (descriptor based at the first active lane's address; lane addresses only
// grow with the lane number in every tiling used here, so the 32-bit offsets
// are small and non-negative) rather than as a plain global load: two code
// paths that differ only in the hint of otherwise identical loads get merged by
// the optimiser, which drops the hint from both.
typedef int i32x4_raw __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x4 ldg_keep(const void *p) {
  const uint64_t a = (uint64_t)(uintptr_t)p;
  const uint64_t base = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a) |
                        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32)) << 32);
  __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(uintptr_t)base, 0, 0x7fffffff, 0x00020000);
  return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(uint32_t)(a - base), 0, 0));
}
__device__ __forceinline__ void stg_stream(void *p, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
}
// A write-back store at agent scope (sc1, no streaming hint): the line stays in
// the caches for whoever reads the result next.  For launches whose results fit
// the memory-side cache these are faster than the streaming ones (and than
// stores without a scope, which a plain assignment would give).  A buffer store:
// the instruction carries the scope bit.
__device__ __forceinline__ void stg_keep(void *p, u32x4 v) {
  const uint64_t a = (uint64_t)(uintptr_t)p;
  const uint64_t base = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a) |
                        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32)) << 32);
  __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(uintptr_t)base, 0, 0x7fffffff, 0x00020000);
  constexpr int kSc1 = 16;   // agent scope
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4_raw, v), rsrc, (int)(uint32_t)(a - base), 0, kSc1);
}

// Cache policy of one launch, decided on the host from the bytes the launch
// reads and writes (see cachePolicyFor in fx_launch.hpp) and carried in the
// kernel arguments: bit p (p < 8) = input p is read with ordinary loads,
// kKeepStores = results are written with stg_keep.  Zero = everything streams.
constexpr uint32_t kKeepAllLoads = 0xffu;
constexpr uint32_t kKeepStores = 0x100u;

}  // namespace fx
