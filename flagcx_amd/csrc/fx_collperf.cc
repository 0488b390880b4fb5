// fx_collperf: the host-API performance tests of FlagCX as one native program
// over simulated ranks on one GPU.
//
//   fx_collperf <allreduce|reduce|reducescatter|allgather|broadcast|gather|
//                scatter|alltoall|alltoallv|sendrecv> [options]
//
// Options, defaults, the meaning of a "size" per collective and the result
// line are the reference's (test/tools.cc:123-250: -b 1M -e 1G -f 2 -w 5 -n 20
// -r root -o op -d datatype; test/perf_common.cc:183-240: "Comm size: ..
// Elapsed time: .. Algo bandwidth: .. Bus bandwidth: .."; the bus factors of
// test/perf/host_api/test_*.cpp), so a sweep made with those programs and a
// sweep made here can be laid side by side.  Added here: -N ranks (default 8),
// -A direct|ring, -O rank|ring|host, -a default|element, -c 1 to check every rank's result after the
// timed loop (long results by sample), and a second figure per line: the bytes the GPU's memory moved
// for one collective, divided by the time between two device events around
// the timed calls.
//
// One host thread posts rank after rank on one stream, as a test program with
// one process per rank would, minus the processes; with -T 1 every rank has a
// host thread and a stream of its own and a call blocks until all ranks have
// made it (FX_SYNC_RENDEZVOUS), which is how separate processes behave.  Host code only: buffers,
// streams and events come through flagcxDeviceHandleInit's table, as in the
// reference's tests (test/perf_common.cc:27-60).
#include <getopt.h>
#include <unistd.h>

#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <string>
#include <thread>
#include <vector>

#include "flagcx_amd/fx_handle.h"
#include "flagcx_amd/fx_sim.h"

namespace {

flagcxDeviceHandle_t dev = nullptr;   // flagcxDeviceHandleInit: the device operations an application may call

[[noreturn]] void die(const char *what, int rc) {
  fprintf(stderr, "fx_collperf: %s failed: %s (%d)\n", what, flagcxGetErrorString((flagcxResult_t)rc), rc);
  exit(1);
}
#define OK(call)                              \
  do {                                        \
    const int rc_ = (int)(call);              \
    if (rc_ != flagcxSuccess) die(#call, rc_); \
  } while (0)

struct TypeInfo {
  const char *name;
  flagcxDataType_t code;
  size_t size;
};
const TypeInfo kTypes[] = {{"int8", flagcxInt8, 1},      {"uint8", flagcxUint8, 1},   {"int32", flagcxInt32, 4},
                           {"uint32", flagcxUint32, 4},  {"int64", flagcxInt64, 8},   {"uint64", flagcxUint64, 8},
                           {"half", flagcxFloat16, 2},   {"float", flagcxFloat32, 4}, {"double", flagcxFloat64, 8},
                           {"bfloat16", flagcxBfloat16, 2}};
const char *kOps[] = {"sum", "prod", "max", "min", "avg"};

double parseSize(const char *s) {
  char *end = nullptr;
  const double v = strtod(s, &end);
  if (end == s || v < 0) return -1;
  switch (*end) {
    case 'G': case 'g': return v * 1024 * 1024 * 1024;
    case 'M': case 'm': return v * 1024 * 1024;
    case 'K': case 'k': return v * 1024;
    case 0: return v;
    default: return -1;
  }
}

// Small whole numbers: exact in every datatype, and their sums over 64 ranks in
// every 4- and 8-byte one.
double valueAt(size_t i, int rank) { return (double)(i % 10) + rank; }

void encode(void *dst, size_t i, double v, flagcxDataType_t t) {
  switch (t) {
    case flagcxInt8: ((int8_t *)dst)[i] = (int8_t)v; break;
    case flagcxUint8: ((uint8_t *)dst)[i] = (uint8_t)v; break;
    case flagcxInt32: ((int32_t *)dst)[i] = (int32_t)v; break;
    case flagcxUint32: ((uint32_t *)dst)[i] = (uint32_t)v; break;
    case flagcxInt64: ((int64_t *)dst)[i] = (int64_t)v; break;
    case flagcxUint64: ((uint64_t *)dst)[i] = (uint64_t)v; break;
    case flagcxFloat32: ((float *)dst)[i] = (float)v; break;
    case flagcxFloat64: ((double *)dst)[i] = v; break;
    case flagcxBfloat16: {   // v < 256 and whole: the top 16 bits of the float are exact
      const float f = (float)v;
      uint32_t w;
      memcpy(&w, &f, 4);
      ((uint16_t *)dst)[i] = (uint16_t)(w >> 16);
      break;
    }
    case flagcxFloat16: {    // whole numbers below 2048: sign 0, exponent and 10 mantissa bits by hand
      const unsigned u = (unsigned)v;
      uint16_t h = 0;
      if (u) {
        int e = 31 - __builtin_clz(u);
        h = (uint16_t)(((e + 15) << 10) | (((u << (10 - e)) & 0x3ff)));
      }
      ((uint16_t *)dst)[i] = h;
      break;
    }
    default: break;
  }
}

double decode(const void *src, size_t i, flagcxDataType_t t) {
  switch (t) {
    case flagcxInt32: return ((const int32_t *)src)[i];
    case flagcxUint32: return ((const uint32_t *)src)[i];
    case flagcxInt64: return (double)((const int64_t *)src)[i];
    case flagcxUint64: return (double)((const uint64_t *)src)[i];
    case flagcxFloat32: return ((const float *)src)[i];
    case flagcxFloat64: return ((const double *)src)[i];
    default: return NAN;
  }
}

enum Coll { kAllReduce, kReduce, kReduceScatter, kAllGather, kBroadcast, kGather, kScatter, kAlltoAll, kAlltoAllv, kSendRecv, kUnknown };
const char *kCollNames[] = {"allreduce", "reduce", "reducescatter", "allgather", "broadcast", "gather", "scatter", "alltoall",
                            "alltoallv", "sendrecv"};

struct Options {
  std::string coll;
  Coll kind = kUnknown;
  size_t minBytes = 1ull << 20, maxBytes = 1ull << 30;
  int factor = 2, warmup = 5, iters = 20, root = 0, nranks = 8, check = 0;
  int type = 7 /* float */, op = 0;
  int algo = -1, order = -1;
  int arith = -1;    // -a element: fp16 / bf16 folded in the element type, as the reference's device kernel does
  int threads = 0;   // -T 1: one host thread and one stream per rank, calls that block until every rank has posted
};

void usage(const char *argv0) {
  printf("Usage: %s <allreduce|reduce|reducescatter|allgather|broadcast|gather|scatter|alltoall|alltoallv|sendrecv>\n\t"
         "[-b <minbytes K/M/G>] [-e <maxbytes K/M/G>] [-f <stepfactor>] [-w <warmupiters>] [-n <iters>]\n\t"
         "[-r <root>] [-o <sum|prod|max|min|avg>] [-d <int8|uint8|int32|uint32|int64|uint64|half|float|double|bfloat16>]\n\t"
         "[-N <simulated ranks, 1..64>] [-A <direct|ring>] [-O <rank|ring|host>] [-c <check 0/1>]\n\t"
         "[-T <0: one thread posts every rank on one stream | 1: a thread and a stream per rank>]\n\t"
         "[-a <default|element: how fp16 / bf16 are folded>]\n",
         argv0);
}

Options parse(int argc, char **argv) {
  Options o;
  if (argc < 2 || argv[1][0] == '-') {
    usage(argv[0]);
    exit(argc < 2 ? 1 : 0);
  }
  o.coll = argv[1];
  for (int i = 0; i < (int)kUnknown; i++)
    if (o.coll == kCollNames[i]) o.kind = (Coll)i;
  if (o.kind == kUnknown) {
    fprintf(stderr, "fx_collperf: unknown collective '%s'\n", o.coll.c_str());
    usage(argv[0]);
    exit(1);
  }
  static option longOpts[] = {{"minbytes", required_argument, 0, 'b'}, {"maxbytes", required_argument, 0, 'e'},
                              {"stepfactor", required_argument, 0, 'f'}, {"warmup_iters", required_argument, 0, 'w'},
                              {"iters", required_argument, 0, 'n'}, {"root", required_argument, 0, 'r'},
                              {"op", required_argument, 0, 'o'}, {"datatype", required_argument, 0, 'd'},
                              {"nranks", required_argument, 0, 'N'}, {"algo", required_argument, 0, 'A'},
                              {"order", required_argument, 0, 'O'}, {"check", required_argument, 0, 'c'},
                              {"threads", required_argument, 0, 'T'}, {"arith", required_argument, 0, 'a'},
                              {"help", no_argument, 0, 'h'}, {}};
  optind = 2;
  for (int c; (c = getopt_long(argc, argv, "b:e:f:w:n:r:o:d:N:A:O:c:T:a:h", longOpts, nullptr)) != -1;) {
    const std::string a = optarg ? optarg : "";
    bool bad = false;
    switch (c) {
      case 'b': { const double v = parseSize(optarg); bad = v < 1; o.minBytes = (size_t)v; break; }
      case 'e': { const double v = parseSize(optarg); bad = v < 1; o.maxBytes = (size_t)v; break; }
      case 'f': o.factor = atoi(optarg); bad = o.factor <= 1; break;
      case 'w': o.warmup = atoi(optarg); bad = o.warmup < 0; break;
      case 'n': o.iters = atoi(optarg); bad = o.iters < 1; break;
      case 'r': o.root = atoi(optarg); break;
      case 'N': o.nranks = atoi(optarg); bad = o.nranks < 1 || o.nranks > 64; break;
      case 'c': o.check = atoi(optarg); break;
      case 'a': o.arith = a == "default" ? FX_ARITH_DEFAULT : a == "element" ? FX_ARITH_ELEMENT : -1; bad = o.arith < 0; break;
      case 'T': o.threads = atoi(optarg); bad = o.threads != 0 && o.threads != 1; break;
      case 'o':
        bad = true;
        for (int i = 0; i < 5; i++)
          if (a == kOps[i]) o.op = i, bad = false;
        break;
      case 'd':
        bad = true;
        for (int i = 0; i < 10; i++)
          if (a == kTypes[i].name) o.type = i, bad = false;
        break;
      case 'A': o.algo = a == "direct" ? FX_ALGO_DIRECT : a == "ring" ? FX_ALGO_RING : -1; bad = o.algo < 0; break;
      case 'O':
        o.order = a == "rank" ? FX_ORDER_RANK : a == "ring" ? FX_ORDER_RING : a == "host" ? FX_ORDER_HOST : -1;
        bad = o.order < 0;
        break;
      case 'h': usage(argv[0]); exit(0);
      default: bad = true;
    }
    if (bad) {
      fprintf(stderr, "fx_collperf: bad value for -%c\n", c);
      usage(argv[0]);
      exit(1);
    }
  }
  if (o.root < 0 || o.root >= o.nranks) {
    fprintf(stderr, "fx_collperf: root %d is not a rank of %d\n", o.root, o.nranks);
    exit(1);
  }
  return o;
}

// What one collective is, for this tool: how big each rank's buffers are for a
// "size", how a rank posts it, the bus factor, the bytes the GPU's memory moves
// and what a rank must hold afterwards.
struct Shape {
  size_t sendElems, recvElems;   // per rank, for `count` elements of "size"
  double busFactor;
  double hbmBytes;               // read + written by the whole collective
};

struct Run {
  Options o;
  TypeInfo t;
  int n;
  std::vector<flagcxComm_t> comms;
  std::vector<void *> send, recv;
  flagcxStream_t stream = nullptr;         // rank 0's, and everybody's without -T 1
  std::vector<flagcxStream_t> streams;     // one per rank (all the same without -T 1)
  std::vector<size_t> sc, sd, rc, rd;   // alltoallv, one row of n per rank

  Shape shape(size_t count) const {
    const double N = n, sz = (double)count * t.size, part = (double)(count / n) * t.size;
    switch (o.kind) {
      case kAllReduce: return {count, count, 2 * (N - 1) / N, 2 * N * sz};
      case kReduce: return {count, count, 1, (N + 1) * sz};
      case kReduceScatter: return {count, count / n, (N - 1) / N, (N * N + N) * part};
      case kAllGather: return {count / n, count, (N - 1) / N, (N + N * N) * part};
      case kBroadcast: return {count, count, 1, (1 + N) * sz};
      case kGather: return {count / n, count, (N - 1) / N, 2 * N * part};
      case kScatter: return {count, count / n, (N - 1) / N, 2 * N * part};
      case kAlltoAll: return {count, count, (N - 1) / N, 2 * N * N * part};
      case kAlltoAllv: {   // slots of two blocks for every rank of one's own parity (see layoutV)
        double moved = 0;
        for (size_t v : sc) moved += (double)v * t.size;
        return {count + 2 * (count / n), count + 2 * (count / n), (N - 1) / N, 2 * moved};
      }
      default: return {count, count, 1, 2 * N * sz};   // sendrecv
    }
  }

  int post(int r, size_t count) {
    const flagcxRedOp_t op = (flagcxRedOp_t)o.op;
    switch (o.kind) {
      case kAllReduce: return flagcxAllReduce(send[r], recv[r], count, t.code, op, comms[r], streams[r]);
      case kReduce: return flagcxReduce(send[r], recv[r], count, t.code, op, o.root, comms[r], streams[r]);
      case kReduceScatter: return flagcxReduceScatter(send[r], recv[r], count / n, t.code, op, comms[r], streams[r]);
      case kAllGather: return flagcxAllGather(send[r], recv[r], count / n, t.code, comms[r], streams[r]);
      case kBroadcast: return flagcxBroadcast(send[r], recv[r], count, t.code, o.root, comms[r], streams[r]);
      case kGather: return flagcxGather(send[r], recv[r], count / n, t.code, o.root, comms[r], streams[r]);
      case kScatter: return flagcxScatter(send[r], recv[r], count / n, t.code, o.root, comms[r], streams[r]);
      case kAlltoAll: return flagcxAlltoAll(send[r], recv[r], count / n, t.code, comms[r], streams[r]);
      case kAlltoAllv:
        return flagcxAlltoAllv(send[r], &sc[(size_t)r * n], &sd[(size_t)r * n], recv[r], &rc[(size_t)r * n], &rd[(size_t)r * n],
                               t.code, comms[r], streams[r]);
      default: return flagcxInvalidArgument;
    }
  }

  // every rank sends to the next and receives from the previous, inside one bracket per rank
  void sendrecvOnce(size_t count) {
    for (int r = 0; r < n; r++) {
      OK(flagcxGroupStart(comms[r]));
      OK(flagcxSend(send[r], count, t.code, (r + 1) % n, comms[r], stream));
      OK(flagcxRecv(recv[r], count, t.code, (r + n - 1) % n, comms[r], stream));
    }
    for (int r = 0; r < n; r++) OK(flagcxGroupEnd(comms[r]));
  }

  void once(size_t count) {
    if (o.kind == kSendRecv) return sendrecvOnce(count);
    for (int r = 0; r < n; r++) {
      const int rc_ = post(r, count);
      if (rc_ != flagcxSuccess) die(o.coll.c_str(), rc_);
    }
  }

  // -T 1: every rank's thread makes `times` calls of its own; a call returns when all ranks have made theirs
  void threaded(size_t count, int times) {
    std::vector<std::thread> ts;
    for (int r = 0; r < n; r++)
      ts.emplace_back([this, r, count, times] {
        for (int i = 0; i < times; i++) {
          if (o.kind == kSendRecv) {
            OK(flagcxGroupStart(comms[r]));
            OK(flagcxSend(send[r], count, t.code, (r + 1) % n, comms[r], streams[r]));
            OK(flagcxRecv(recv[r], count, t.code, (r + n - 1) % n, comms[r], streams[r]));
            OK(flagcxGroupEnd(comms[r]));
          } else {
            const int rc_ = post(r, count);
            if (rc_ != flagcxSuccess) die(o.coll.c_str(), rc_);
          }
        }
      });
    for (auto &th : ts) th.join();
  }

  void repeat(size_t count, int times) {
    if (o.threads) return threaded(count, times);
    for (int i = 0; i < times; i++) once(count);
  }

  void syncAll() {
    for (int r = 0; r < (o.threads ? n : 1); r++) OK(dev->streamSynchronize(streams[r]));
  }

  // alltoallv with the ragged pattern of the reference's test (test_alltoallv.cpp:10-52): a rank
  // exchanges two blocks of count / n elements with every other rank of its own parity and nothing
  // with the rest; the slots sit back to back in peer order, the rank's own slot left empty.
  void layoutV(size_t count) {
    const size_t two = 2 * (count / n);
    sc.assign((size_t)n * n, 0);
    sd = rc = rd = sc;
    for (int r = 0; r < n; r++) {
      size_t at = 0;
      for (int j = 0; j < n; j++) {
        const size_t k = (size_t)r * n + j;
        sd[k] = rd[k] = at;
        if ((j & 1) != (r & 1)) continue;
        sc[k] = rc[k] = (j == r) ? 0 : two;
        at += two;
      }
    }
  }

  double expected(int r, size_t i, size_t count, bool *defined) const {
    const size_t part = count / n;
    const Coll c = o.kind;
    *defined = true;
    // the n parts of count / n elements may not fill the whole size
    if ((c == kAllGather || c == kGather || c == kAlltoAll) && (part == 0 || i >= part * (size_t)n)) return (*defined = false, 0.0);
    auto fold = [&](size_t at) {
      double acc = valueAt(at, 0);
      for (int q = 1; q < n; q++) {
        const double v = valueAt(at, q);
        acc = o.op == flagcxSum ? acc + v : o.op == flagcxMax ? std::max(acc, v) : std::min(acc, v);
      }
      return acc;
    };
    switch (c) {
      case kAllReduce: return fold(i);
      case kReduce: return r == o.root ? fold(i) : (*defined = false, 0.0);
      case kReduceScatter: return fold((size_t)r * part + i);
      case kAllGather: return valueAt(i % part, (int)(i / part));
      case kBroadcast: return valueAt(i, o.root);
      case kGather: return r == o.root ? valueAt(i % part, (int)(i / part)) : (*defined = false, 0.0);
      case kScatter: return valueAt((size_t)r * part + i, o.root);
      case kAlltoAll: return valueAt((size_t)r * part + i % part, (int)(i / part));
      case kAlltoAllv: {   // slot q of rank r holds what the q-th rank of r's parity sent from its slot for r
        const size_t two = 2 * part;
        const int from = two ? (r & 1) + 2 * (int)(i / two) : n;
        if (from >= n || from == r) return (*defined = false, 0.0);
        return valueAt(sd[(size_t)from * n + r] + i % two, from);
      }
      case kSendRecv: return valueAt(i, (r + n - 1) % n);
      default: return (*defined = false, 0.0);
    }
  }
};

bool reduces(Coll c) { return c == kAllReduce || c == kReduce || c == kReduceScatter; }

double seconds() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

}  // namespace

int main(int argc, char **argv) {
  Run run;
  run.o = parse(argc, argv);
  run.t = kTypes[run.o.type];
  run.n = run.o.nranks;
  const int n = run.n;
  OK(flagcxDeviceHandleInit(&dev));
  OK(dev->setDevice(0));
  run.comms.resize(n);
  OK(fxSimCommInitAll(run.comms.data(), n));
  if (run.o.algo >= 0) OK(fxSimCommConfig(run.comms[0], FX_SIM_ALGO, run.o.algo));
  if (run.o.order >= 0) OK(fxSimCommConfig(run.comms[0], FX_SIM_ORDER, run.o.order));
  if (run.o.arith >= 0) OK(fxSimCommConfig(run.comms[0], FX_SIM_ARITH, run.o.arith));
  OK(dev->streamCreate(&run.stream));
  run.streams.assign(n, run.stream);
  if (run.o.threads) {
    OK(fxSimCommConfig(run.comms[0], FX_SIM_SYNC, FX_SYNC_RENDEZVOUS));
    for (int r = 1; r < n; r++) OK(dev->streamCreate(&run.streams[r]));
  }
  flagcxEvent_t t0, t1;
  OK(dev->eventCreate(&t0, flagcxEventDefault));
  OK(dev->eventCreate(&t1, flagcxEventDefault));

  const size_t maxCount = run.o.maxBytes / run.t.size;
  if (run.o.kind == kAlltoAllv) run.layoutV(maxCount);
  const Shape big = run.shape(maxCount);
  run.send.resize(n);
  run.recv.resize(n);
  for (int r = 0; r < n; r++) {
    OK(dev->deviceMalloc(&run.send[r], std::max<size_t>(big.sendElems, 1) * run.t.size, flagcxMemDevice, nullptr));
    OK(dev->deviceMalloc(&run.recv[r], std::max<size_t>(big.recvElems, 1) * run.t.size, flagcxMemDevice, nullptr));
  }
  std::vector<char> host(std::max<size_t>(std::max(big.sendElems, big.recvElems), 1) * run.t.size);

  const bool exactType = run.t.size >= 4;
  const bool checkable = run.o.check && (!reduces(run.o.kind) || (exactType && run.o.op != flagcxProd && run.o.op != flagcxAvg));
  char vendor[128] = "";
  OK(dev->getVendor(vendor));
  printf("# %s over %d simulated ranks on one GPU; buffers, stream and events through the device handle (%s); %s\n",
         run.o.coll.c_str(), n, vendor,
         run.o.threads ? "a host thread and a stream per rank, calls block until every rank has posted"
                       : "one host thread posts rank after rank on one stream");
  printf("#\n# datatype: %s, op: %s\n#\n", run.t.name, kOps[run.o.op]);
  if (run.o.check && !checkable)
    printf("# no check for this datatype / op: the pattern's sums are exact only in 4- and 8-byte types\n");

  int failures = 0;
  for (size_t size = run.o.minBytes; size <= run.o.maxBytes; size *= (size_t)run.o.factor) {
    const size_t count = size / run.t.size;
    if (run.o.kind == kAlltoAllv) run.layoutV(count);
    const Shape sh = run.shape(count);
    for (int r = 0; r < n; r++) {
      for (size_t i = 0; i < sh.sendElems; i++) encode(host.data(), i, valueAt(i, r), run.t.code);
      if (sh.sendElems)
        OK(dev->deviceMemcpy(run.send[r], host.data(), sh.sendElems * run.t.size, flagcxMemcpyHostToDevice, nullptr));
      if (sh.recvElems) OK(dev->deviceMemset(run.recv[r], 0xff, sh.recvElems * run.t.size, flagcxMemDevice, nullptr));
    }
    OK(dev->deviceSynchronize());
    run.repeat(count, run.o.warmup);
    run.syncAll();

    OK(dev->eventRecord(t0, run.stream));
    const double w0 = seconds();
    run.repeat(count, run.o.iters);
    OK(dev->eventRecord(t1, run.stream));
    run.syncAll();
    const double elapsed = (seconds() - w0) / run.o.iters;
    float ms = 0;
    OK(dev->eventElapsedTime(&ms, t0, t1));
    const double onDevice = (double)ms * 1e-3 / run.o.iters;

    const double algBw = (double)size / 1.0e9 / elapsed;
    printf("Comm size: %zu bytes; Elapsed time: %lf sec; Algo bandwidth: %lf GB/s; Bus bandwidth: %lf GB/s", size, elapsed,
           algBw, algBw * sh.busFactor);
    printf("; on the device: %.2f us, %.1f GB/s of memory traffic\n", onDevice * 1e6, sh.hbmBytes / 1.0e9 / onDevice);

    if (checkable) {
      for (int r = 0; r < n && failures < 10; r++) {
        if (!sh.recvElems) continue;
        OK(dev->deviceMemcpy(host.data(), run.recv[r], sh.recvElems * run.t.size, flagcxMemcpyDeviceToHost, nullptr));
        std::vector<char> want(run.t.size);
        // every element up to 4 Mi of them; of longer results the first and last 64 Ki and every 4099th between
        const size_t edge = 65536, all = sh.recvElems <= (4u << 20) ? sh.recvElems : 0;
        for (size_t i = 0; i < sh.recvElems; i += (all || i < edge || i + edge >= sh.recvElems) ? 1 : std::min<size_t>(4099, sh.recvElems - edge - i)) {
          bool defined;
          const double v = run.expected(r, i, count, &defined);
          if (!defined) continue;
          bool same;
          if (exactType) {
            same = decode(host.data(), i, run.t.code) == v;
          } else {   // data movement of a narrow type: compare the bytes
            encode(want.data(), 0, v, run.t.code);
            same = memcmp(want.data(), host.data() + i * run.t.size, run.t.size) == 0;
          }
          if (!same) {
            printf("# MISMATCH size %zu rank %d element %zu: expected %g\n", size, r, i, v);
            failures++;
            break;
          }
        }
      }
    }
    fflush(stdout);
  }
  if (run.o.check && checkable) printf("# check: %s\n", failures ? "FAILED" : "every rank's result as expected");

  for (int r = 0; r < n; r++) {
    OK(dev->deviceFree(run.send[r], flagcxMemDevice, nullptr));
    OK(dev->deviceFree(run.recv[r], flagcxMemDevice, nullptr));
  }
  OK(dev->eventDestroy(t0));
  OK(dev->eventDestroy(t1));
  for (int r = 1; r < n && run.o.threads; r++) OK(dev->streamDestroy(run.streams[r]));
  OK(dev->streamDestroy(run.stream));
  OK(fxSimCommDestroyAll(run.comms.data(), n));
  OK(flagcxDeviceHandleFree(dev));
  return failures ? 2 : 0;
}
