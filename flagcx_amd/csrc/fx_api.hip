// C ABI over the gfx950 kernels: argument checking, batching of slice
// descriptors into launches, and device-resident plans.
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

#include "flagcx_amd/fx_kernels.h"
#include "fx_launch.hpp"

using namespace fx;

namespace {

// dtype / op screening.  Types FlagCX knows but this path does not carry
// return flagcxNotSupported so a caller can fall through to another path;
// values outside the enums are invalid arguments.
flagcxResult_t screen(int dtype, int op) {
  if (dtype < 0 || dtype >= flagcxNumTypes) return flagcxInvalidArgument;
  if (op >= 0 && (op & FX_OP_ELEMENT_FOLD)) {   // the reference device kernel's own arithmetic, where it differs from the default
    const int base = op & ~FX_OP_ELEMENT_FOLD;
    if (base >= flagcxNumRedOps) return flagcxInvalidArgument;
    const bool sixteen = dtype == flagcxFloat16 || dtype == flagcxBfloat16;
    return (sixteen && (base == flagcxSum || base == flagcxMax || base == flagcxMin)) ? flagcxSuccess : flagcxNotSupported;
  }
  if (op < 0 || op >= flagcxNumRedOps) return flagcxInvalidArgument;
  if (dtypeSize(dtype) == 0) return flagcxNotSupported;
  if (!opSupported(op)) return flagcxNotSupported;
  return flagcxSuccess;
}

const KernelSet *setFor(int dtype, int op) {
  if (op & FX_OP_ELEMENT_FOLD) {
    const int base = op & ~FX_OP_ELEMENT_FOLD;
    return &kernelSetsElem()[3 * (dtype == flagcxBfloat16) + (base == flagcxSum ? 0 : base == flagcxMax ? 1 : 2)];
  }
  switch (dtype) {
    case flagcxFloat32: return &kernelSetsF32()[op];
    case flagcxInt32: return &kernelSetsI32()[op];
    case flagcxBfloat16: return &kernelSetsBF16()[op];
    case flagcxFloat16: return &kernelSetsF16()[op];
    case flagcxUint32: return &kernelSetsU32()[op];
    case flagcxInt8: return &kernelSetsI8()[op];
    case flagcxUint8: return &kernelSetsU8()[op];
    case flagcxInt64: return &kernelSetsI64()[op];
    case flagcxUint64: return &kernelSetsU64()[op];
    case flagcxFloat64: return &kernelSetsF64()[op];
    default: return nullptr;
  }
}

const KernelSet *copySetFor(int es) { return &kernelSetsCopy()[es == 4 ? 2 : (es == 2 ? 1 : 0)]; }

bool aligned(const void *p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

// Validate one slice: pointers present and aligned to the element size.
flagcxResult_t sliceOk(const fxSliceDesc &s, int k, int es) {
  if (s.count == 0) return flagcxSuccess;
  if (!s.out || !aligned(s.out, es)) return flagcxInvalidArgument;
  for (int p = 0; p < k; p++)
    if (!s.in[p] || !aligned(s.in[p], es)) return flagcxInvalidArgument;
  return flagcxSuccess;
}

// Validate one slice and return the number of workgroups it needs with U vectors per lane.
flagcxResult_t sliceTiles(const fxSliceDesc &s, int k, int es, int U, uint64_t *tiles) {
  *tiles = 0;
  const flagcxResult_t rc = sliceOk(s, k, es);
  if (rc != flagcxSuccess || s.count == 0) return rc;
  *tiles = tilesFor(s.out, s.in, k, s.count, es, U);
  return flagcxSuccess;
}

// Slices that continue each other in every input and in the output are one
// longer slice (the operation is element-wise).  Partitions such as the
// reference's slice / red-slice split produce long runs of them, and a long
// segment gets the striped hand-out where 512 KiB pieces would not.
constexpr size_t kFewSlices = 16;   // descriptor lists up to this length stay on the stack
typedef SmallVec<fxSliceDesc, kFewSlices> SliceList;

void mergeAdjacent(SliceList &out, const fxSliceDesc *slices, size_t n, int k, size_t es, uint64_t div = 1) {
  out.reserve(n);
  for (size_t i = 0; i < n; i++) {
    fxSliceDesc d = slices[i];
    d.count /= div;          // copies are given in bytes and moved in units of `div` bytes
    if (d.count == 0) continue;
    if (!out.empty()) {
      fxSliceDesc &l = out.back();
      const size_t bytes = l.count * es;
      bool cont = (const char *)d.out == (const char *)l.out + bytes;
      for (int p = 0; p < k && cont; p++) cont = (const char *)d.in[p] == (const char *)l.in[p] + bytes;
      if (cont) {
        l.count += d.count;
        continue;
      }
    }
    out.push_back(d);
  }
}

// Launch n slices through kernel-argument tables (as many launches as the tables need).
flagcxResult_t launchSliceBatches(const KernelSet *ks, const fxSliceDesc *slicesIn, size_t nIn, int k, hipStream_t s,
                                  uint64_t div = 1) {
  for (size_t i = 0; i < nIn; i++)   // validate before merging so a bad slice is still reported
    if (slicesIn[i].count) {
      if (!slicesIn[i].out) return flagcxInvalidArgument;
      for (int p = 0; p < k; p++)
        if (!slicesIn[i].in[p]) return flagcxInvalidArgument;
    }
  SliceList merged;
  mergeAdjacent(merged, slicesIn, nIn, k, (size_t)ks->elemSize, div);   // drops empty slices
  for (size_t i = 0; i < merged.size(); i++) {
    const flagcxResult_t rc = sliceOk(merged[i], k, ks->elemSize);
    if (rc != flagcxSuccess) return rc;
  }
  if (merged.empty()) return flagcxSuccess;
  // A single segment needs no table: the direct kernel's argument block is 100
  // bytes instead of the eight-slot table's 700.
  if (merged.size() == 1) return ks->direct[k](merged[0].out, merged[0].in, k, merged[0].count, s);
  return ks->slicesInline[k](merged.data(), merged.size(), rereadHint(merged.data(), merged.size(), k, (size_t)ks->elemSize), s);
}

// Largest power-of-two granularity (4, 2 or 1 bytes) shared by all copy slices.
int copyGranularity(const fxSliceDesc *slices, size_t n) {
  uintptr_t bits = 0;
  for (size_t i = 0; i < n; i++) {
    if (slices[i].count == 0) continue;
    bits |= (uintptr_t)slices[i].in[0] | (uintptr_t)slices[i].out | (uintptr_t)slices[i].count;
  }
  return (bits & 1) ? 1 : ((bits & 2) ? 2 : 4);
}


// ---------------------------------------------- table in static device memory

// Descriptor table and tile-prefix table of fx_reduce_slices_static: the same
// two arrays a plan keeps in allocated device memory, here in a file-scope
// array so that the call path allocates nothing.  Every GPU holds its own copy
// of the array, at its own address, until the process ends.
constexpr size_t kStaticSlices = FX_STATIC_MAX_SLICES;
constexpr size_t kStaticDescBytes = kStaticSlices * sizeof(SliceDescDev);
constexpr size_t kStaticBytes = kStaticDescBytes + (kStaticSlices + 1) * sizeof(uint32_t);
static __device__ __align__(256) unsigned char scratch[(kStaticBytes + 255) / 256 * 256];

// Descriptors travel to the table in the argument block of a small kernel
// (an upload from pageable host memory would stage through the runtime's own
// buffers and could not be captured).
constexpr int kWriterSlots = 32;
struct TableChunk {
  SliceDescDev d[kWriterSlots];
  uint32_t tileStart[kWriterSlots];  // first workgroup of descriptor base + i
  uint32_t base, n, gridEnd;         // gridEnd = tileStart of the entry after this chunk
};

__global__ void __launch_bounds__(kBlock) writeSliceTable(TableChunk c, SliceDescDev *d, uint32_t *tileStart) {
  constexpr uint32_t kWords = sizeof(SliceDescDev) / sizeof(uint64_t);
  const uint64_t *src = reinterpret_cast<const uint64_t *>(c.d);
  uint64_t *dst = reinterpret_cast<uint64_t *>(d + c.base);
  for (uint32_t w = threadIdx.x; w < c.n * kWords; w += kBlock) dst[w] = src[w];
  for (uint32_t i = threadIdx.x; i < c.n; i += kBlock) tileStart[c.base + i] = c.tileStart[i];
  if (threadIdx.x == 0) tileStart[c.base + c.n] = c.gridEnd;   // the next chunk overwrites it with the same value
}

constexpr int kMaxDevices = 64;
unsigned char *g_scratchOf[kMaxDevices];  // device address of `scratch` per GPU, filled on first use

// Address of this GPU's copy of `scratch`.  In host code the array's name is
// only a handle for the runtime; the address kernels and copies need comes from
// hipGetSymbolAddress, asked once per device with that device current.
flagcxResult_t staticTable(unsigned char **ptr) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return flagcxUnhandledDeviceError;
  unsigned char *p = __atomic_load_n(&g_scratchOf[dev], __ATOMIC_ACQUIRE);
  if (!p) {
    if (hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return flagcxUnhandledDeviceError;
    __atomic_store_n(&g_scratchOf[dev], p, __ATOMIC_RELEASE);   // racing first calls store the same value
  }
  *ptr = p;
  return flagcxSuccess;
}

// Walk the descriptors the way launchSliceBatches / fx_plan_create see them:
// empty ones dropped, counts divided by `div` (copies count bytes), runs that
// continue each other in every stream merged.  emit(desc) is called once per
// merged descriptor; a non-zero return stops the walk and is handed back.
template <class F>
int forEachMerged(const fxSliceDesc *slices, size_t n, int k, size_t es, uint64_t div, F emit) {
  fxSliceDesc cur;
  bool have = false;
  for (size_t i = 0; i < n; i++) {
    fxSliceDesc d = slices[i];
    d.count /= div;
    if (d.count == 0) continue;
    if (have) {
      const size_t bytes = cur.count * es;
      bool cont = (const char *)d.out == (const char *)cur.out + bytes;
      for (int p = 0; p < k && cont; p++) cont = (const char *)d.in[p] == (const char *)cur.in[p] + bytes;
      if (cont) {
        cur.count += d.count;
        continue;
      }
      const int rc = emit(cur);
      if (rc) return rc;
    }
    cur = d;
    have = true;
  }
  return have ? emit(cur) : 0;
}

}  // namespace

struct fxPlan {
  const KernelSet *ks;
  SliceDescDev *dDesc;
  uint32_t *dTileStart;
  uint32_t n, grid;
  uint32_t keep;   // cache policy for what the whole plan touches
  int k;
};

extern "C" {
#pragma GCC visibility push(default)

const char *fx_version(void) { return "flagcx_amd 0.1 (gfx950)"; }

size_t fx_dtype_size(int dtype) {
  switch (dtype) {
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

int fx_reduce_copy(void *out, const void *const *in, int k, size_t count, int dtype, int op, int first,
                   void *stream) {
  flagcxResult_t rc = screen(dtype, op);
  if (rc != flagcxSuccess) return rc;
  if (!in || k < 1 || k > FX_MAX_INPUTS || first < 0 || first >= k) return flagcxInvalidArgument;
  if (count == 0) return flagcxSuccess;
  const size_t es = dtypeSize(dtype);
  if (!out || !aligned(out, es)) return flagcxInvalidArgument;
  const void *rot[FX_MAX_INPUTS];
  for (int j = 0; j < k; j++) {
    const void *p = in[(first + j) % k];
    if (!p || !aligned(p, es)) return flagcxInvalidArgument;
    rot[j] = p;
  }
  const KernelSet *ks = setFor(dtype, op);
  return ks->direct[k <= kMaxFixedK ? k : 0](out, rot, k, count, (hipStream_t)stream);
}

int fx_reduce2(void *out, const void *in1, const void *in2, size_t count, int dtype, int op, void *stream) {
  const void *in[2] = {in1, in2};
  return fx_reduce_copy(out, in, 2, count, dtype, op, 0, stream);
}

void fx_trigger_set(fxReduceTrigger *t, uint64_t in1, uint64_t in2, uint64_t out, size_t count, size_t nthreads,
                    int dtype, int op, int state) {
  t->value[0] = in1;
  t->value[1] = in2;
  t->value[2] = out;
  t->value[3] = ((uint64_t)count & 0xffffffffull) | (((uint64_t)nthreads & 0xffffull) << 32) |
                (((uint64_t)dtype & 0xfull) << 48) | (((uint64_t)op & 0xfull) << 52) |
                (((uint64_t)state & 0x3ull) << 56);
}

void fx_trigger_get(const fxReduceTrigger *t, uint64_t *in1, uint64_t *in2, uint64_t *out, uint64_t *count,
                    uint64_t *nthreads, int *dtype, int *op, int *state) {
  const uint64_t w = t->value[3];
  if (in1) *in1 = t->value[0];
  if (in2) *in2 = t->value[1];
  if (out) *out = t->value[2];
  if (count) *count = w & 0xffffffffull;
  if (nthreads) *nthreads = (w >> 32) & 0xffffull;
  if (dtype) *dtype = (int)((w >> 48) & 0xfull);
  if (op) *op = (int)((w >> 52) & 0xfull);
  if (state) *state = (int)((w >> 56) & 0x3ull);
}

int fx_reduce_slices(const fxSliceDesc *slices, size_t n, int k, int dtype, int op, void *stream) {
  flagcxResult_t rc = screen(dtype, op);
  if (rc != flagcxSuccess) return rc;
  if (k < 1 || k > FX_MAX_SLICE_INPUTS) return flagcxInvalidArgument;
  if (n == 0) return flagcxSuccess;
  if (!slices) return flagcxInvalidArgument;
  return guarded([&] { return (int)launchSliceBatches(setFor(dtype, op), slices, n, k, (hipStream_t)stream); });
}

int fx_reduce_triggers(const fxReduceTrigger *triggers, size_t n, void *stream) {
  if (n == 0) return flagcxSuccess;
  if (!triggers) return flagcxInvalidArgument;
  return guarded([&]() -> int {
    SliceList run;
    size_t i = 0;
    while (i < n) {
      int dtype, op;
      fx_trigger_get(&triggers[i], nullptr, nullptr, nullptr, nullptr, nullptr, &dtype, &op, nullptr);
      run.clear();
      size_t j = i;
      for (; j < n; j++) {
        uint64_t a, b, o, c;
        int dt, rop;
        fx_trigger_get(&triggers[j], &a, &b, &o, &c, nullptr, &dt, &rop, nullptr);
        if (dt != dtype || rop != op) break;
        fxSliceDesc d;
        memset(&d, 0, sizeof(d));
        d.in[0] = (const void *)(uintptr_t)a;
        d.in[1] = (const void *)(uintptr_t)b;
        d.out = (void *)(uintptr_t)o;
        d.count = c;
        run.push_back(d);
      }
      int rc = fx_reduce_slices(run.data(), run.size(), 2, dtype, op, stream);
      if (rc != flagcxSuccess) return rc;
      i = j;
    }
    return flagcxSuccess;
  });
}

int fx_copy_slices(const fxSliceDesc *slices, size_t n, void *stream) {
  if (n == 0) return flagcxSuccess;
  if (!slices) return flagcxInvalidArgument;
  for (size_t i = 0; i < n; i++)
    if (slices[i].count && (!slices[i].in[0] || !slices[i].out)) return flagcxInvalidArgument;
  return guarded([&]() -> int {
    const int es = copyGranularity(slices, n);
    return launchSliceBatches(copySetFor(es), slices, n, 1, (hipStream_t)stream, (uint64_t)es);
  });
}

int fx_reduce_bcast_slices(const fxBcastDesc *slices, size_t n, int k, int nout, int dtype, int op, void *stream) {
  const bool copy = (op == -1);
  if (copy) {
    k = 1;
  } else {
    flagcxResult_t rc = screen(dtype, op);
    if (rc != flagcxSuccess) return rc;
  }
  if (k < 1 || k > FX_MAX_SLICE_INPUTS || nout < 1 || nout > FX_MAX_SLICE_INPUTS) return flagcxInvalidArgument;
  if (n == 0) return flagcxSuccess;
  if (!slices) return flagcxInvalidArgument;
  return guarded([&]() -> int {
    hipStream_t s = (hipStream_t)stream;
    // element size: the dtype's, or for copies the widest unit every pointer and count allows
    uintptr_t bits = 0;
    for (size_t i = 0; i < n; i++) {
      if (slices[i].count == 0) continue;
      for (int p = 0; p < k; p++) {
        if (!slices[i].in[p]) return flagcxInvalidArgument;
        bits |= (uintptr_t)slices[i].in[p];
      }
      for (int o = 0; o < nout; o++) {
        if (!slices[i].out[o]) return flagcxInvalidArgument;
        bits |= (uintptr_t)slices[i].out[o];
      }
      if (copy) bits |= (uintptr_t)slices[i].count;
    }
    const int es = copy ? ((bits & 1) ? 1 : ((bits & 2) ? 2 : 4)) : (int)dtypeSize(dtype);
    if (!copy && (bits & (uintptr_t)(es - 1))) return flagcxInvalidArgument;
    const KernelSet *ks = copy ? copySetFor(es) : setFor(dtype, op);
    // merge slices that continue each other in every stream
    SmallVec<fxBcastDesc, kFewSlices> merged;
    merged.reserve(n);
    for (size_t i = 0; i < n; i++) {
      fxBcastDesc d = slices[i];
      if (d.count == 0) continue;
      if (copy) d.count /= (uint64_t)es;
      if (!merged.empty()) {
        fxBcastDesc &l = merged.back();
        const size_t bytes = l.count * (size_t)es;
        bool cont = true;
        for (int p = 0; p < k && cont; p++) cont = (const char *)d.in[p] == (const char *)l.in[p] + bytes;
        for (int o = 0; o < nout && cont; o++) cont = (const char *)d.out[o] == (const char *)l.out[o] + bytes;
        if (cont) {
          l.count += d.count;
          continue;
        }
      }
      merged.push_back(d);
    }
    SliceList plainReduce, plainCopy;  // slices whose outputs are not co-aligned
    SmallVec<BcastDescDev, kFewSlices> dev;
    for (const fxBcastDesc &d : merged) {
      bool same = true;
      for (int o = 1; o < nout; o++) same = same && (((uintptr_t)d.out[o] & 15u) == ((uintptr_t)d.out[0] & 15u));
      if (!same) {
        fxSliceDesc r;
        memset(&r, 0, sizeof(r));
        for (int p = 0; p < k; p++) r.in[p] = d.in[p];
        r.out = d.out[0];
        r.count = d.count;
        plainReduce.push_back(r);
        for (int o = 1; o < nout; o++) {
          fxSliceDesc c;
          memset(&c, 0, sizeof(c));
          c.in[0] = d.out[0];
          c.out = d.out[o];
          c.count = d.count * (uint64_t)es;
          plainCopy.push_back(c);
        }
        continue;
      }
      BcastDescDev dd;
      for (int p = 0; p < kMaxFixedK; p++) dd.in[p] = (p < k) ? d.in[p] : nullptr;
      for (int o = 0; o < kMaxFixedK; o++) dd.out[o] = (o < nout) ? d.out[o] : nullptr;
      dd.count = d.count;
      dd.nout = (uint32_t)nout;
      dev.push_back(dd);
    }
    flagcxResult_t rc = dev.empty() ? flagcxSuccess : ks->bcastInline[k](dev.data(), dev.size(), s);
    if (rc != flagcxSuccess) return rc;
    if (!plainReduce.empty()) {
      rc = launchSliceBatches(ks, plainReduce.data(), plainReduce.size(), k, s);
      if (rc != flagcxSuccess) return rc;
      return fx_copy_slices(plainCopy.data(), plainCopy.size(), stream);
    }
    return flagcxSuccess;
  });
}

int fx_reduce_ordered(const fxBcastDesc *slices, size_t n, int k, int nout, int dtype, int op, int order, void *stream) {
  flagcxResult_t rc = screen(dtype, op);
  if (rc != flagcxSuccess) return rc;
  if (order != FX_FOLD_CHAIN && order != FX_FOLD_TREE && order != FX_FOLD_KEEP_LOCAL) return flagcxInvalidArgument;
  if (k < 1 || k > FX_MAX_SLICE_INPUTS || nout < 1 || nout > FX_MAX_SLICE_INPUTS) return flagcxInvalidArgument;
  if ((op & FX_OP_ELEMENT_FOLD) || (op == flagcxAvg && order != FX_FOLD_CHAIN)) return flagcxNotSupported;
  if (n == 0) return flagcxSuccess;
  if (!slices) return flagcxInvalidArgument;
  const KernelSet *ks = setFor(dtype, op);
  const bool select = (op == flagcxMax || op == flagcxMin);
  const bool floating = dtype == flagcxFloat16 || dtype == flagcxBfloat16 || dtype == flagcxFloat32 || dtype == flagcxFloat64;
  // Which association has a kernel of its own.  Everything else is the
  // input-order fold of the inputs in a suitable order:
  //  * integers give the same bits in every association and operand order
  //    (sum / prod wrap, max / min pick one of two equal patterns on a tie);
  //  * two inputs: tree and keep-local are both in[1] (op) in[0];
  //  * keep-local sums and products: the two operands of a step commute bit for
  //    bit, so res = in[j] (op) res is res = res (op) in[j].
  const bool reversePair = (k == 2 && order != FX_FOLD_CHAIN);
  int kernel = -1;   // index into KernelSet::ordered, -1 = the input-order fold
  if (floating && k >= 3) {
    if (order == FX_FOLD_TREE) kernel = 0;
    else if (order == FX_FOLD_KEEP_LOCAL && select) kernel = 1;
  }
  // 16-bit sums and products in the keep-local chain would round after every
  // step; the host ring does not carry those types (utils.h:690-694), so there is
  // no kernel for them.
  const bool sixteen = dtype == flagcxFloat16 || dtype == flagcxBfloat16;
  if (sixteen && !select && order == FX_FOLD_KEEP_LOCAL && k >= 3) return flagcxNotSupported;
  if (kernel < 0 && !reversePair) return fx_reduce_bcast_slices(slices, n, k, nout, dtype, op, stream);
  return guarded([&]() -> int {
    const int es = (int)dtypeSize(dtype);
    SmallVec<fxBcastDesc, kFewSlices> swapped;
    SmallVec<BcastDescDev, kFewSlices> dev;
    for (size_t i = 0; i < n; i++) {
      fxBcastDesc d = slices[i];
      if (d.count == 0) continue;
      uintptr_t bits = 0;
      for (int p = 0; p < k; p++) {
        if (!d.in[p]) return flagcxInvalidArgument;
        bits |= (uintptr_t)d.in[p];
      }
      for (int o = 0; o < nout; o++) {
        if (!d.out[o]) return flagcxInvalidArgument;
        bits |= (uintptr_t)d.out[o];
      }
      if (bits & (uintptr_t)(es - 1)) return flagcxInvalidArgument;
      if (reversePair) {
        const void *t = d.in[0];
        d.in[0] = d.in[1];
        d.in[1] = t;
        swapped.push_back(d);
        continue;
      }
      for (int o = 1; o < nout; o++)   // the one-read-n-stores kernels share byte offsets between the outputs
        if ((((uintptr_t)d.out[o] ^ (uintptr_t)d.out[0]) & 15u) != 0) return flagcxInvalidArgument;
      // descriptors that continue each other in every stream are one longer descriptor
      if (!dev.empty()) {
        BcastDescDev &l = dev.back();
        const size_t bytes = l.count * (size_t)es;
        bool cont = true;
        for (int p = 0; p < k && cont; p++) cont = (const char *)d.in[p] == (const char *)l.in[p] + bytes;
        for (int o = 0; o < nout && cont; o++) cont = (const char *)d.out[o] == (const char *)l.out[o] + bytes;
        if (cont) {
          l.count += d.count;
          continue;
        }
      }
      BcastDescDev dd;
      for (int p = 0; p < kMaxFixedK; p++) dd.in[p] = (p < k) ? d.in[p] : nullptr;
      for (int o = 0; o < kMaxFixedK; o++) dd.out[o] = (o < nout) ? d.out[o] : nullptr;
      dd.count = d.count;
      dd.nout = (uint32_t)nout;
      dev.push_back(dd);
    }
    if (reversePair) return fx_reduce_bcast_slices(swapped.data(), swapped.size(), k, nout, dtype, op, stream);
    if (dev.empty()) return flagcxSuccess;
    return ks->ordered[kernel][k](dev.data(), dev.size(), (hipStream_t)stream);
  });
}

int fx_reduce_bcast(void *const *outs, int nout, const void *const *ins, int k, size_t count, int dtype, int op,
                    int first, void *stream) {
  const bool copy = (op == -1);
  if (copy) {
    if (k != 1) return flagcxInvalidArgument;
  } else {
    flagcxResult_t rc = screen(dtype, op);
    if (rc != flagcxSuccess) return rc;
  }
  if (!outs || !ins || k < 1 || k > FX_MAX_INPUTS || nout < 1 || nout > FX_MAX_INPUTS || first < 0 || first >= k)
    return flagcxInvalidArgument;
  if (count == 0) return flagcxSuccess;
  return guarded([&]() -> int {
    hipStream_t s = (hipStream_t)stream;
    uintptr_t bits = copy ? (uintptr_t)count : 0;
    const void *rot[FX_MAX_INPUTS];
    for (int j = 0; j < k; j++) {
      rot[j] = ins[(first + j) % k];
      if (!rot[j]) return flagcxInvalidArgument;
      bits |= (uintptr_t)rot[j];
    }
    bool alike = true;
    for (int o = 0; o < nout; o++) {
      if (!outs[o]) return flagcxInvalidArgument;
      bits |= (uintptr_t)outs[o];
      alike = alike && (((uintptr_t)outs[o] & 15u) == ((uintptr_t)outs[0] & 15u));
    }
    const int es = copy ? ((bits & 1) ? 1 : ((bits & 2) ? 2 : 4)) : (int)dtypeSize(dtype);
    if (!copy && (bits & (uintptr_t)(es - 1))) return flagcxInvalidArgument;
    const KernelSet *ks = copy ? copySetFor(es) : setFor(dtype, op);
    const uint64_t n = copy ? (uint64_t)count / (uint64_t)es : (uint64_t)count;
    if (alike) return ks->bcastRuntime(outs, nout, rot, k, n, s);
    // outputs at different offsets within 16 bytes: one reduce, then copies of its result
    flagcxResult_t rc = ks->direct[k <= kMaxFixedK ? k : 0](outs[0], rot, k, n, s);
    if (rc != flagcxSuccess) return rc;
    SliceList copies;
    for (int o = 1; o < nout; o++) {
      fxSliceDesc c;
      memset(&c, 0, sizeof(c));
      c.in[0] = outs[0];
      c.out = outs[o];
      c.count = n * (uint64_t)es;
      copies.push_back(c);
    }
    return copies.empty() ? flagcxSuccess : fx_copy_slices(copies.data(), copies.size(), stream);
  });
}

int fx_reduce_chunks(void *const *outs, int nout, const void *const *ins, int k, const fxChunk *chunks, int nchunks,
                     int dtype, int op, void *stream) {
  const bool copy = (op == -1);
  if (!copy) {
    flagcxResult_t rc = screen(dtype, op);
    if (rc != flagcxSuccess) return rc;
  }
  if (!outs || !ins || k < 1 || k > FX_MAX_INPUTS || nout < 1 || nout > FX_MAX_INPUTS || nchunks < 0) return flagcxInvalidArgument;
  if (nchunks == 0) return flagcxSuccess;
  if (!chunks) return flagcxInvalidArgument;
  return guarded([&]() -> int {
    uintptr_t bits = 0;
    for (int j = 0; j < k; j++) {
      if (!ins[j]) return flagcxInvalidArgument;
      bits |= (uintptr_t)ins[j];
    }
    for (int o = 0; o < nout; o++) {
      if (!outs[o]) return flagcxInvalidArgument;
      bits |= (uintptr_t)outs[o];
    }
    for (int c = 0; c < nchunks; c++) {
      const fxChunk &ch = chunks[c];
      if (ch.in_sel >= k || ch.out_sel >= nout || (ch.in_sel < 0 && (ch.first < 0 || ch.first >= k))) return flagcxInvalidArgument;
      if (copy && ch.in_sel < 0) return flagcxInvalidArgument;
      if (copy) bits |= (uintptr_t)ch.in_off | (uintptr_t)ch.out_off | (uintptr_t)ch.count;
      if (ch.out_sel < 0 && ch.count)   // the outputs of one chunk share their byte offset, so their bases must agree within 16
        for (int o = 1; o < nout; o++)
          if ((((uintptr_t)outs[o] ^ (uintptr_t)outs[0]) & 15u) != 0) return flagcxInvalidArgument;
    }
    const int es = copy ? ((bits & 1) ? 1 : ((bits & 2) ? 2 : 4)) : (int)dtypeSize(dtype);
    if (!copy && (bits & (uintptr_t)(es - 1))) return flagcxInvalidArgument;
    const KernelSet *ks = copy ? copySetFor(es) : setFor(dtype, op);
    const uint64_t scale = copy ? 1 : (uint64_t)es;        // offsets to bytes
    const uint64_t unit = copy ? (uint64_t)es : 1;         // counts to elements of the kernel's type
    for (int base = 0; base < nchunks; base += kMaxK) {
      ChunkedArgs a;
      memset(&a, 0, sizeof(a));
      for (int j = 0; j < k; j++) a.in[j] = ins[j];
      for (int o = 0; o < nout; o++) a.out[o] = outs[o];
      a.k = k;
      a.nout = nout;
      a.nchunks = (nchunks - base < kMaxK) ? nchunks - base : kMaxK;
      for (int c = 0; c < a.nchunks; c++) {
        const fxChunk &ch = chunks[base + c];
        a.inOff[c] = ch.in_off * scale;
        a.outOff[c] = ch.out_off * scale;
        a.cnt[c] = ch.count / unit;
        a.first[c] = (int8_t)(ch.in_sel < 0 ? ch.first : 0);
        a.only[c] = (int8_t)(ch.in_sel < 0 ? -1 : ch.in_sel);
        a.outSel[c] = (int8_t)(ch.out_sel < 0 ? -1 : ch.out_sel);
      }
      const flagcxResult_t rc = ks->chunksRuntime(&a, (hipStream_t)stream);
      if (rc != flagcxSuccess) return rc;
    }
    return flagcxSuccess;
  });
}

int fx_alltoall(void *const *recv, const void *const *send, int n, size_t block_bytes, void *stream) {
  if (!recv || !send || n < 1 || n > FX_MAX_INPUTS) return flagcxInvalidArgument;
  if (block_bytes == 0) return flagcxSuccess;
  return guarded([&]() -> int {
    uintptr_t bits = (uintptr_t)block_bytes;
    for (int r = 0; r < n; r++) {
      if (!recv[r] || !send[r]) return flagcxInvalidArgument;
      bits |= (uintptr_t)recv[r] | (uintptr_t)send[r];
    }
    const int es = (bits & 1) ? 1 : ((bits & 2) ? 2 : 4);   // the widest unit every address and the block size allow
    return copySetFor(es)->allToAll(recv, send, n, (uint64_t)block_bytes / (uint64_t)es, (hipStream_t)stream);
  });
}

int fx_plan_create(fxPlan_t *plan, const fxSliceDesc *slices, size_t n, int k, int dtype, int op) {
  if (!plan) return flagcxInvalidArgument;
  *plan = nullptr;
  if (n && !slices) return flagcxInvalidArgument;
  if (n > 0x7fffffffull) return flagcxInvalidArgument;
  return guarded([&]() -> int {
    const KernelSet *ks;
    uint64_t div = 1;
    if (op == -1) {
      k = 1;
      for (size_t i = 0; i < n; i++)
        if (slices[i].count && (!slices[i].in[0] || !slices[i].out)) return flagcxInvalidArgument;
      int es = copyGranularity(slices, n);
      ks = copySetFor(es);
      div = (uint64_t)es;
    } else {
      flagcxResult_t rc = screen(dtype, op);
      if (rc != flagcxSuccess) return rc;
      if (k < 1 || k > FX_MAX_SLICE_INPUTS) return flagcxInvalidArgument;
      ks = setFor(dtype, op);
    }
    const int U = unrollFor(k);
    std::vector<SliceDescDev> desc;
    std::vector<uint32_t> start(1, 0u);
    uint64_t elems = 0;
    std::vector<fxSliceDesc> scaled(slices, slices + n);
    for (auto &d : scaled) {
      if (d.count && !d.out) return flagcxInvalidArgument;
      for (int p = 0; p < k; p++)
        if (d.count && !d.in[p]) return flagcxInvalidArgument;
      d.count /= div;
    }
    SliceList merged;
    mergeAdjacent(merged, scaled.data(), scaled.size(), k, (size_t)ks->elemSize);
    for (size_t i = 0; i < merged.size(); i++) {
      fxSliceDesc s = merged[i];
      uint64_t tiles;
      flagcxResult_t rc = sliceTiles(s, k, ks->elemSize, U, &tiles);
      if (rc != flagcxSuccess) return rc;
      if (tiles == 0) continue;
      if ((uint64_t)start.back() + tiles > 0x7ffffff0ull) return flagcxInvalidArgument;
      SliceDescDev d;
      for (int p = 0; p < kMaxFixedK; p++) d.in[p] = (p < k) ? s.in[p] : nullptr;
      d.out = s.out;
      d.count = s.count;
      elems += s.count;
      desc.push_back(d);
      start.push_back(start.back() + (uint32_t)tiles);
    }
    fxPlan *pl = new (std::nothrow) fxPlan();
    if (!pl) return flagcxSystemError;
    pl->ks = ks;
    pl->k = k;
    pl->n = (uint32_t)desc.size();
    pl->grid = start.back();
    pl->keep = cachePolicyFor(touchedBytes(elems, ks->elemSize, k, 0), touchedBytes(elems, ks->elemSize, 0, 1),
                              rereadHint(merged.data(), merged.size(), k, (size_t)ks->elemSize));
    pl->dDesc = nullptr;
    pl->dTileStart = nullptr;
    if (pl->n) {
      if (hipMalloc((void **)&pl->dDesc, desc.size() * sizeof(SliceDescDev)) != hipSuccess ||
          hipMalloc((void **)&pl->dTileStart, start.size() * sizeof(uint32_t)) != hipSuccess ||
          hipMemcpy(pl->dDesc, desc.data(), desc.size() * sizeof(SliceDescDev), hipMemcpyHostToDevice) != hipSuccess ||
          hipMemcpy(pl->dTileStart, start.data(), start.size() * sizeof(uint32_t), hipMemcpyHostToDevice) !=
              hipSuccess) {
        fx_plan_destroy(pl);
        return flagcxUnhandledDeviceError;
      }
    }
    *plan = pl;
    return flagcxSuccess;
  });
}

int fx_plan_launch(fxPlan_t plan, void *stream) {
  if (!plan) return flagcxInvalidArgument;
  if (plan->n == 0) return flagcxSuccess;
  return plan->ks->slicesTable[plan->k](plan->dDesc, plan->dTileStart, plan->n, plan->grid, plan->keep,
                                        (hipStream_t)stream);
}

int fx_plan_destroy(fxPlan_t plan) {
  if (!plan) return flagcxSuccess;
  if (plan->dDesc) (void)hipFree(plan->dDesc);
  if (plan->dTileStart) (void)hipFree(plan->dTileStart);
  delete plan;
  return flagcxSuccess;
}

int fx_reduce_slices_static(const fxSliceDesc *slices, size_t n, int k, int dtype, int op, void *stream) {
  const KernelSet *ks;
  uint64_t div = 1;
  if (n && !slices) return flagcxInvalidArgument;
  if (op == -1) {
    k = 1;
    for (size_t i = 0; i < n; i++)
      if (slices[i].count && (!slices[i].in[0] || !slices[i].out)) return flagcxInvalidArgument;
    const int es = copyGranularity(slices, n);
    ks = copySetFor(es);
    div = (uint64_t)es;
  } else {
    flagcxResult_t rc = screen(dtype, op);
    if (rc != flagcxSuccess) return rc;
    if (k < 1 || k > FX_MAX_SLICE_INPUTS) return flagcxInvalidArgument;
    ks = setFor(dtype, op);
  }
  if (n == 0) return flagcxSuccess;
  for (size_t i = 0; i < n; i++)
    if (slices[i].count) {
      if (!slices[i].out) return flagcxInvalidArgument;
      for (int p = 0; p < k; p++)
        if (!slices[i].in[p]) return flagcxInvalidArgument;
    }
  const int U = unrollFor(k);
  const size_t es = (size_t)ks->elemSize;
  // first walk: validate everything and size the table, so that an error leaves nothing enqueued
  size_t entries = 0;
  uint64_t grid = 0, elems = 0;
  int rc = forEachMerged(slices, n, k, es, div, [&](const fxSliceDesc &d) -> int {
    uint64_t t = 0;
    const flagcxResult_t r = sliceTiles(d, k, (int)es, U, &t);
    if (r != flagcxSuccess) return r;
    if (t == 0) return 0;
    entries++;
    grid += t;
    elems += d.count;
    return (grid > 0x7ffffff0ull) ? (int)flagcxInvalidArgument : 0;
  });
  if (rc) return rc;
  if (entries == 0) return flagcxSuccess;
  if (entries > kStaticSlices) return flagcxInvalidArgument;   // more descriptors than the static table holds
  unsigned char *base = nullptr;
  flagcxResult_t st = staticTable(&base);
  if (st != flagcxSuccess) return st;
  SliceDescDev *dDesc = reinterpret_cast<SliceDescDev *>(base);
  uint32_t *dTileStart = reinterpret_cast<uint32_t *>(base + kStaticDescBytes);
  hipStream_t s = (hipStream_t)stream;
  // second walk: fill the table chunk by chunk on the caller's stream
  TableChunk c;
  c.base = 0;
  c.n = 0;
  uint32_t next = 0;   // tileStart of the descriptor being added
  auto flush = [&]() -> int {
    if (c.n == 0) return 0;
    c.gridEnd = next;
    const flagcxResult_t r = launchKernel(writeSliceTable, 1, s, c, dDesc, dTileStart);
    c.base += c.n;
    c.n = 0;
    return r;
  };
  rc = forEachMerged(slices, n, k, es, div, [&](const fxSliceDesc &d) -> int {
    uint64_t t = 0;
    (void)sliceTiles(d, k, (int)es, U, &t);
    if (t == 0) return 0;
    SliceDescDev &o = c.d[c.n];
    for (int p = 0; p < kMaxFixedK; p++) o.in[p] = (p < k) ? d.in[p] : nullptr;
    o.out = d.out;
    o.count = d.count;
    c.tileStart[c.n] = next;
    next += (uint32_t)t;
    c.n++;
    return (c.n == (uint32_t)kWriterSlots) ? flush() : 0;
  });
  if (rc) return rc;
  rc = flush();
  if (rc) return rc;
  const uint32_t keep = cachePolicyFor(touchedBytes(elems, (int)es, k, 0), touchedBytes(elems, (int)es, 0, 1));
  return ks->slicesTable[k](dDesc, dTileStart, (uint32_t)entries, next, keep, s);
}

static int packOrUnpack(bool pack, void *a, const void *b, const size_t *counts, const size_t *displs, int npeers,
                        int dtype, void *stream) {
  if (npeers < 0) return flagcxInvalidArgument;
  const size_t es = fx_dtype_size(dtype);
  if (es == 0) return flagcxInvalidArgument;
  if (npeers == 0) return flagcxSuccess;
  if (!counts || !displs) return flagcxInvalidArgument;
  return guarded([&]() -> int {
    SliceList sl;
    size_t slot = 0;
    for (int i = 0; i < npeers; i++) {
      if (counts[i]) {
        if (!a || !b) return flagcxInvalidArgument;
        fxSliceDesc d;
        memset(&d, 0, sizeof(d));
        if (pack) {  // a = packed, b = sendbuff
          d.in[0] = (const char *)b + displs[i] * es;
          d.out = (char *)a + slot * es;
        } else {     // a = recvbuff, b = packed
          d.in[0] = (const char *)b + slot * es;
          d.out = (char *)a + displs[i] * es;
        }
        d.count = counts[i] * es;
        sl.push_back(d);
      }
      slot += counts[i];
    }
    return fx_copy_slices(sl.data(), sl.size(), stream);
  });
}

int fx_pack(void *packed, const void *sendbuff, const size_t *sendcounts, const size_t *sdispls, int npeers,
            int dtype, void *stream) {
  return packOrUnpack(true, packed, sendbuff, sendcounts, sdispls, npeers, dtype, stream);
}

int fx_unpack(void *recvbuff, const void *packed, const size_t *recvcounts, const size_t *rdispls, int npeers,
              int dtype, void *stream) {
  return packOrUnpack(false, recvbuff, packed, recvcounts, rdispls, npeers, dtype, stream);
}

void fx_split(size_t total, size_t parts, size_t idx, size_t *cnt, size_t *off) {
  if (parts == 0) {
    if (cnt) *cnt = 0;
    if (off) *off = 0;
    return;
  }
  const size_t base = total / parts, rem = total % parts;
  if (cnt) *cnt = base + (idx < rem ? 1 : 0);
  if (off) *off = idx * base + (idx < rem ? idx : rem);
}

size_t fx_nredslices(size_t count, int nranks, size_t nslices, size_t nredslices, size_t redslicesize) {
  if (nredslices != 0) return nredslices;
  if (count == 0 || redslicesize == 0 || nranks < 1 || nslices == 0) return 1;
  float v = (float)count / nranks / nslices / redslicesize;
  size_t r = (size_t)ceilf(v);
  return r ? r : 1;
}

#pragma GCC visibility pop
}  // extern "C"
