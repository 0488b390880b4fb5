// A stand-in for FlagCX's uniRunner (flagcx/runner/uni_runner_impl.cc) that drives
// this build's reduce kernels the way the unmodified scheduler does: it declares
// flagcxLaunchCollectiveKernel exactly as flagcx/include/flagcx_kernel_internal.h:56
// does and takes NOTHING else from the kernel library -- the host side of the
// trigger ring below is this program's own, as libflagcx.so's is its own
// (flagcx/core/flagcx_reduce_kernel_host.cc).  Device memory, streams and the
// pinned ring come through the device-adaptor plugin, as in the reference
// (initUniRunner, uni_runner_impl.cc:1795-1840).
//
//   unirunner_client <plugin.so> <in.bin> <out.bin> <nslices> <nredslices>
//
// in.bin:  uint64 nranks, uint64 count, then nranks * count floats (rank-major send buffers).
// out.bin: nranks * count floats (every rank's receive buffer), written after each of
//          two all-reduces in a row (the second in place on the first's result is NOT
//          done: both start from the same inputs; the file holds the second's output).
//
// One process plays all ranks: the P2P steps of the ring are device-to-device
// copies, the Red nodes are triggers in the ring, one ring and one consumer
// launch per collective (runUniRunner, uni_runner_impl.cc:1864-1901).
#include <dlfcn.h>
#include <sched.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "flagcx_amd/fx_device_adaptor.h"

// flagcx/include/flagcx_kernel_internal.h:56, verbatim
void flagcxLaunchCollectiveKernel(void *fifoBuffer, size_t nthreads, size_t nblocks, flagcxStream_t stream);

namespace {

// ---- the ring, host side (layout: flagcx/include/flagcx_kernel_core.h:53-67,146-162) ----
enum { kIdxCapacity = 0, kIdxConsumed = 1, kIdxProduced = 2, kIdxTerminate = 3, kIdxData = 4 };
enum { kAvailable = 0, kEnqueued = 1, kInprogress = 2, kComplete = 3 };
constexpr uint64_t kCapacity = 128;   // FLAGCX_FIFO_CAPACITY

struct Trigger {
  uint64_t value[4];
};

uint64_t pollState(Trigger *t) { return (__atomic_load_n(&t->value[3], __ATOMIC_ACQUIRE) >> 56) & 0x3; }

void setState(Trigger *t, uint64_t state) {
  uint64_t v = __atomic_load_n(&t->value[3], __ATOMIC_ACQUIRE);
  v = (v & ~(0x3ull << 56)) | ((state & 0x3) << 56);
  __atomic_store_n(&t->value[3], v, __ATOMIC_RELEASE);
}

// enqueue() of flagcx_reduce_kernel_host.cc:46-80: -1 when the ring is full or the slot is not collected yet
int enqueue(uint64_t *ring, uint64_t in1, uint64_t in2, uint64_t out, uint64_t count, uint64_t nthreads, int dtype, int op) {
  const int capacity = (int)ring[kIdxCapacity];
  const int distance = (int)(ring[kIdxProduced] - __atomic_load_n(&ring[kIdxConsumed], __ATOMIC_ACQUIRE));
  if (distance >= capacity) {
    sched_yield();
    return -1;
  }
  const int idx = (int)(ring[kIdxProduced] % (uint64_t)capacity);
  Trigger *t = reinterpret_cast<Trigger *>(ring + kIdxData) + idx;
  if (pollState(t) != kAvailable) {
    sched_yield();
    return -1;
  }
  uint64_t tmp[4] = {in1, in2, out,
                     (count & 0xffffffffull) | ((nthreads & 0xffffull) << 32) | (((uint64_t)dtype & 0xf) << 48) |
                         (((uint64_t)op & 0xf) << 52) | ((uint64_t)kEnqueued << 56)};
  memcpy(t->value, tmp, sizeof(tmp));
  __atomic_fetch_add(&ring[kIdxProduced], 1ul, __ATOMIC_RELEASE);
  return idx;
}

// ---- the partition (uni_runner_impl.cc:100-131,433-457,854-866) ----
void split(size_t total, size_t parts, size_t idx, size_t *cnt, size_t *off) {
  const size_t base = total / parts, rem = total % parts;
  *cnt = base + (idx < rem ? 1 : 0);
  *off = idx * base + (idx < rem ? idx : rem);
}
int mod(int a, int n) { return ((a % n) + n) % n; }

#define CHECK(call)                                                              \
  do {                                                                           \
    const flagcxResult_t rc_ = (call);                                           \
    if (rc_ != flagcxSuccess) {                                                  \
      fprintf(stderr, "%s:%d %s -> %d\n", __FILE__, __LINE__, #call, (int)rc_); \
      return 3;                                                                  \
    }                                                                            \
  } while (0)

struct Red {
  uint64_t in1, in2, out, count;
};

// Whatever way a collective is left, its consumer is told to end and waited for.
struct ConsumerGuard {
  flagcxDeviceAdaptor_v1 *dev;
  uint64_t *ring;
  flagcxStream_t stream;
  ~ConsumerGuard() {
    __atomic_store_n(ring + kIdxTerminate, 1, __ATOMIC_RELEASE);
    dev->streamSynchronize(stream);
  }
};

// Enqueue every node of `nodes` as slots free up, collect each when it is Complete
// (processReadyQueue + processInflightQueue, uni_runner_impl.cc:1701-1794).
int runNodes(uint64_t *ring, const std::vector<Red> &nodes) {
  std::vector<int> slot(nodes.size(), -1);
  size_t issued = 0, collected = 0;
  uint64_t idle = 0;
  while (collected < nodes.size()) {
    bool progress = false;
    if (issued < nodes.size()) {
      const Red &r = nodes[issued];
      const int idx = enqueue(ring, r.in1, r.in2, r.out, r.count, 32, flagcxFloat32, flagcxSum);
      if (idx >= 0) {
        slot[issued++] = idx;
        progress = true;
      }
    }
    while (collected < issued) {
      Trigger *t = reinterpret_cast<Trigger *>(ring + kIdxData) + slot[collected];
      if (pollState(t) != kComplete) break;
      setState(t, kAvailable);
      collected++;
      progress = true;
    }
    idle = progress ? 0 : idle + 1;
    if (idle > 200000000ull) {
      fprintf(stderr, "no trigger completed for a long time: is the consumer running?\n");
      return 4;
    }
  }
  return 0;
}

}  // namespace

int main(int argc, char **argv) {
  if (argc != 6) {
    fprintf(stderr, "usage: %s plugin.so in.bin out.bin nslices nredslices\n", argv[0]);
    return 2;
  }
  void *h = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  if (!h) {
    fprintf(stderr, "dlopen: %s\n", dlerror());
    return 2;
  }
  auto *dev = static_cast<flagcxDeviceAdaptor_v1 *>(dlsym(h, FX_DEVICE_ADAPTOR_SYMBOL));
  if (!dev) return 2;
  FILE *f = fopen(argv[2], "rb");
  uint64_t hdr[2];
  if (!f || fread(hdr, sizeof(hdr), 1, f) != 1) return 2;
  const int n = (int)hdr[0];
  const size_t count = (size_t)hdr[1], S = (size_t)atol(argv[4]), R = (size_t)atol(argv[5]);
  std::vector<float> host((size_t)n * count);
  if (fread(host.data(), sizeof(float), host.size(), f) != host.size()) return 2;
  fclose(f);

  CHECK(dev->setDevice(0));
  flagcxStream_t redStream, cpyStream;
  CHECK(dev->streamCreate(&redStream));
  CHECK(dev->streamCreate(&cpyStream));
  std::vector<char *> send(n), recv(n);
  for (int r = 0; r < n; r++) {
    CHECK(dev->deviceMalloc((void **)&send[r], count * 4, flagcxMemDevice, NULL));
    CHECK(dev->deviceMalloc((void **)&recv[r], count * 4, flagcxMemDevice, NULL));
    CHECK(dev->deviceMemcpy(send[r], host.data() + (size_t)r * count, count * 4, flagcxMemcpyHostToDevice, NULL, NULL));
  }
  auto copy = [&](void *dst, void *src, size_t bytes) {
    return bytes ? dev->deviceMemcpy(dst, src, bytes, flagcxMemcpyDeviceToDevice, cpyStream, NULL) : flagcxSuccess;
  };

  for (int round = 0; round < 2; round++) {
    for (int r = 0; r < n; r++) CHECK(dev->deviceMemset(recv[r], 0xff, count * 4, flagcxMemDevice, NULL));
    // flagcxRedFifoInit (flagcx_reduce_kernel_host.cc:82-98): a fresh pinned ring per collective
    uint64_t *ring = nullptr;
    CHECK(dev->deviceMalloc((void **)&ring, (kIdxData + 4 * kCapacity) * sizeof(uint64_t), flagcxMemHost, NULL));
    ring[kIdxCapacity] = kCapacity;
    ring[kIdxConsumed] = ring[kIdxProduced] = ring[kIdxTerminate] = 0;
    memset(ring + kIdxData, 0, kCapacity * sizeof(Trigger));
    __sync_synchronize();
    void *ringDev = nullptr;
    CHECK(dev->hostGetDevicePointer(&ringDev, ring));

    flagcxLaunchCollectiveKernel(ringDev, 32, 1, redStream);   // uniRunnerNThreads / NBlocks defaults
    {
    ConsumerGuard guard{dev, ring, redStream};

    // reduce-scatter: step i, rank r receives chunk (r-i-1)%n from rank r-1 and adds its own data
    std::vector<Red> nodes;
    for (int i = 0; i < n - 1; i++) {
      for (int r = 0; r < n; r++) {
        const int prev = mod(r - 1, n), rx = mod(r - i - 1, n);
        size_t ccnt, coff;
        split(count, n, rx, &ccnt, &coff);
        CHECK(copy(recv[r] + coff * 4, (i == 0 ? send[prev] : recv[prev]) + coff * 4, ccnt * 4));
      }
      CHECK(dev->streamSynchronize(cpyStream));
      nodes.clear();
      for (int r = 0; r < n; r++) {
        const int rx = mod(r - i - 1, n);
        size_t ccnt, coff;
        split(count, n, rx, &ccnt, &coff);
        for (size_t s = 0; s < S; s++) {
          size_t scnt, soff;
          split(ccnt, S, s, &scnt, &soff);
          for (size_t q = 0; q < R; q++) {
            size_t rcnt, roff;
            split(scnt, R, q, &rcnt, &roff);
            if (rcnt == 0) continue;
            const size_t off = (coff + soff + roff) * 4;
            nodes.push_back(Red{(uint64_t)(uintptr_t)(recv[r] + off), (uint64_t)(uintptr_t)(send[r] + off),
                                (uint64_t)(uintptr_t)(recv[r] + off), rcnt});
          }
        }
      }
      const int rc = runNodes(ring, nodes);
      if (rc) return rc;
    }
    // all-gather: step i, rank r receives chunk (r-i)%n from rank r-1
    for (int i = 0; i < n - 1; i++) {
      for (int r = 0; r < n; r++) {
        const int prev = mod(r - 1, n), rx = mod(r - i, n);
        size_t ccnt, coff;
        split(count, n, rx, &ccnt, &coff);
        CHECK(copy(recv[r] + coff * 4, recv[prev] + coff * 4, ccnt * 4));
      }
      CHECK(dev->streamSynchronize(cpyStream));
    }
    __atomic_store_n(ring + kIdxTerminate, 1, __ATOMIC_RELEASE);
    CHECK(dev->streamSynchronize(redStream));
    CHECK(dev->streamSynchronize(cpyStream));
    }
    CHECK(dev->deviceFree(ring, flagcxMemHost, NULL));   // flagcxRedFifoDestroy
  }

  for (int r = 0; r < n; r++)
    CHECK(dev->deviceMemcpy(host.data() + (size_t)r * count, recv[r], count * 4, flagcxMemcpyDeviceToHost, NULL, NULL));
  f = fopen(argv[3], "wb");
  if (!f || fwrite(host.data(), sizeof(float), host.size(), f) != host.size()) return 2;
  fclose(f);
  for (int r = 0; r < n; r++) {
    CHECK(dev->deviceFree(send[r], flagcxMemDevice, NULL));
    CHECK(dev->deviceFree(recv[r], flagcxMemDevice, NULL));
  }
  CHECK(dev->streamDestroy(redStream));
  CHECK(dev->streamDestroy(cpyStream));
  printf("unirunner_client ok: %d ranks x %zu floats, %zu slices x %zu red-slices, 2 collectives\n", n, count, S, R);
  return 0;
}
