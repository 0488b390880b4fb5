// Shared host/device definitions for the gfx950 reduce / copy / pack kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <new>

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

#define FX_HIP(call)                                                           \
  do {                                                                         \
    hipError_t e_ = (call);                                                    \
    if (e_ != hipSuccess) return flagcxUnhandledDeviceError;                   \
  } while (0)

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
__device__ __forceinline__ void stg_stream(void *p, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
}

}  // namespace fx
