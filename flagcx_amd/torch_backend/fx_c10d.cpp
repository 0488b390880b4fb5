// torch.distributed backend "flagcx" over the FlagCX-named C entry points of
// libflagcx_amd.so: the counterpart of the reference's torch plugin
// (plugin/torch/flagcx/src/backend_flagcx.cpp), which drives flagcxAllReduce &
// co. from c10d.  Collectives are enqueued on the caller's current HIP stream,
// so a Work is complete in stream order as soon as the call returns; wait()
// only has to order another stream after it.
//
// Ranks are the simulated ranks of one process on one GPU: every rank's backend
// object joins the same in-process group through the unique id rank 0 leaves in
// the store, and a collective is launched by the last rank that posts it.  A
// rank's results are therefore defined once every rank has posted; wait() on a
// Work is meant to be called then (with one rank, at once).  Copies that a
// call owes its caller behind the collective (out of a staging tensor into a
// list of output tensors) are enqueued, on the rank's own stream, by whichever
// call finds the collective launched -- normally the last rank's.
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include <torch/csrc/distributed/c10d/Backend.hpp>
#include <torch/csrc/distributed/c10d/Store.hpp>
#include <torch/csrc/distributed/c10d/Types.hpp>
#include <torch/csrc/distributed/c10d/Work.hpp>
#include <torch/extension.h>

#include <algorithm>
#include <cstring>
#include <functional>
#include <map>
#include <mutex>
#include <numeric>
#include <string>
#include <vector>

#include "flagcx_amd/fx_device_adaptor.h"
#include "flagcx_amd/fx_sim.h"

namespace {

using c10d::OpType;
using c10d::Work;
using Tensors = std::vector<at::Tensor>;

void ok(flagcxResult_t rc, const char *what) {
  TORCH_CHECK(rc == flagcxSuccess, what, " failed: ", flagcxGetErrorString(rc), " (flagcxResult_t ", (int)rc, ")");
}

// The device adaptor that owns the flagcxStream_t handle type lives in the
// plugin library beside this module's kernel library.
const flagcxDeviceAdaptor_v1 *deviceAdaptor() {
  static const flagcxDeviceAdaptor_v1 *table = [] {
    Dl_info me;
    TORCH_CHECK(dladdr((const void *)&flagcxAllReduce, &me) && me.dli_fname, "cannot locate libflagcx_amd.so");
    std::string dir(me.dli_fname);
    dir.erase(dir.find_last_of('/') + 1);
    const std::string path = dir + "libflagcx-device-mi355x.so";
    void *h = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
    TORCH_CHECK(h, "cannot load ", path, ": ", dlerror());
    void *sym = dlsym(h, FX_DEVICE_ADAPTOR_SYMBOL);
    TORCH_CHECK(sym, path, " does not export ", FX_DEVICE_ADAPTOR_SYMBOL);
    return (const flagcxDeviceAdaptor_v1 *)sym;
  }();
  return table;
}

// flagcxStream_t around the caller's current stream for the duration of one call.
class BorrowedStream {
 public:
  explicit BorrowedStream(hipStream_t raw) { ok(deviceAdaptor()->streamCopy(&h_, (void *)raw), "streamCopy"); }
  ~BorrowedStream() { (void)deviceAdaptor()->streamFree(h_); }
  BorrowedStream(const BorrowedStream &) = delete;
  BorrowedStream &operator=(const BorrowedStream &) = delete;
  flagcxStream_t get() const { return h_; }

 private:
  flagcxStream_t h_ = nullptr;
};

// dtype and op tables: the reference's (backend_flagcx.cpp:21-84).  Bool and
// the 8-bit floats travel as uint8; a sum over bools is an "or", sent as max.
flagcxDataType_t dtypeOf(const at::Tensor &t) {
  switch (t.scalar_type()) {
    case at::kChar: return flagcxInt8;
    case at::kByte:
    case at::kBool:
    case at::kFloat8_e5m2:
    case at::kFloat8_e4m3fn: return flagcxUint8;
    case at::kInt: return flagcxInt32;
    case at::kLong: return flagcxInt64;
    case at::kHalf: return flagcxFloat16;
    case at::kBFloat16: return flagcxBfloat16;
    case at::kFloat: return flagcxFloat32;
    case at::kDouble: return flagcxFloat64;
    default: C10_THROW_ERROR(TypeError, c10::str("tensor type ", t.scalar_type(), " has no FlagCX datatype"));
  }
}

flagcxRedOp_t opOf(const c10d::ReduceOp &op, const at::Tensor &t) {
  const bool boolean = t.scalar_type() == at::kBool;
  const bool raw8 = t.scalar_type() == at::kFloat8_e5m2 || t.scalar_type() == at::kFloat8_e4m3fn;
  if (raw8) C10_THROW_ERROR(TypeError, "8-bit floats can be moved but not reduced");
  switch (op) {
    case c10d::ReduceOp::SUM: return boolean ? flagcxMax : flagcxSum;
    case c10d::ReduceOp::PRODUCT: return flagcxProd;
    case c10d::ReduceOp::MIN: return flagcxMin;
    case c10d::ReduceOp::MAX: return flagcxMax;
    case c10d::ReduceOp::AVG:
      if (boolean) C10_THROW_ERROR(TypeError, "ReduceOp.AVG has no meaning for boolean tensors");
      return flagcxAvg;
    default: C10_THROW_ERROR(ValueError, "this ReduceOp has no FlagCX reduction (sum, product, min, max, avg do)");
  }
}

void checkOne(const Tensors &v, const char *what) {
  TORCH_CHECK(v.size() == 1, what, " takes exactly one tensor per rank, got ", v.size());
}

void checkDense(const at::Tensor &t, const char *what) {
  TORCH_CHECK(t.is_cuda(), what, ": tensor must live on the GPU");
  // the call goes to the current device's current stream
  TORCH_CHECK(t.get_device() == c10::hip::current_device(), what, ": tensor is on GPU ", t.get_device(),
              " but the current device is ", (int)c10::hip::current_device());
  TORCH_CHECK(t.is_contiguous(), what, ": tensor must be contiguous");
  TORCH_CHECK(!t.is_sparse(), what, ": sparse tensors are not supported");
}

class FxWork : public Work {
 public:
  FxWork(int rank, OpType op, hipStream_t stream, Tensors outputs)
      : Work(rank, op), stream_(stream), outputs_(std::move(outputs)) {
    std::vector<c10::Device> devices;
    for (const auto &t : outputs_)
      if (std::find(devices.begin(), devices.end(), t.device()) == devices.end()) devices.push_back(t.device());
    future_ = c10::make_intrusive<c10::ivalue::Future>(c10::ListType::create(c10::TensorType::get()), devices);
    future_->markCompleted(c10::IValue(outputs_));
  }
  ~FxWork() override {
    if (event_) (void)hipEventDestroy(event_);
  }
  bool isCompleted() override {
    mark();
    return hipEventQuery(event_) == hipSuccess;
  }
  bool isSuccess() const override { return true; }
  // Orders the caller's current stream after the collective; never blocks the host.
  bool wait(std::chrono::milliseconds /*timeout*/ = kNoTimeout) override {
    const hipStream_t cur = c10::hip::getCurrentHIPStream().stream();
    if (cur != stream_) {
      mark();
      TORCH_CHECK(hipStreamWaitEvent(cur, event_, 0) == hipSuccess, "hipStreamWaitEvent failed");
    }
    return true;
  }
  void synchronize() override { (void)wait(); }
  Tensors result() override { return outputs_; }
  c10::intrusive_ptr<c10::ivalue::Future> getFuture() override { return future_; }

 private:
  // An event on the collective's stream, recorded when first asked for: with
  // simulated ranks the launch may come from a later rank's call, which also
  // makes this rank's stream wait for it, so "now" covers it once every rank
  // has posted.
  void mark() {
    if (!event_) TORCH_CHECK(hipEventCreateWithFlags(&event_, hipEventDisableTiming) == hipSuccess, "hipEventCreate failed");
    TORCH_CHECK(hipEventRecord(event_, stream_) == hipSuccess, "hipEventRecord failed");
  }
  hipStream_t stream_;
  hipEvent_t event_ = nullptr;
  Tensors outputs_;
  c10::intrusive_ptr<c10::ivalue::Future> future_;
};

// Copies owed behind collectives that have not been launched yet, per group of
// simulated ranks (the key is the group's unique id).
struct Owed {
  uint64_t joined;                 // the group's launch count when the collective was posted
  c10::hip::HIPStream stream;      // the posting rank's stream
  std::function<void()> finish;
};
std::mutex owedMu;
std::map<std::string, std::vector<Owed>> owed;

// Enqueue every owed copy of `group` whose collective has been launched, each on its own rank's stream.
void payOwed(const std::string &group, uint64_t launched) {
  std::vector<Owed> due;
  {
    std::lock_guard<std::mutex> lock(owedMu);
    auto &v = owed[group];
    for (size_t i = 0; i < v.size();) {
      if (v[i].joined < launched) {
        due.push_back(std::move(v[i]));
        v.erase(v.begin() + (long)i);
      } else {
        i++;
      }
    }
  }
  const c10::hip::HIPStream before = c10::hip::getCurrentHIPStream();
  try {
    for (auto &o : due) {
      c10::hip::setCurrentHIPStream(o.stream);
      o.finish();
    }
  } catch (...) {
    c10::hip::setCurrentHIPStream(before);
    throw;
  }
  c10::hip::setCurrentHIPStream(before);
}

class FxBackend : public c10d::Backend {
 public:
  FxBackend(const c10::intrusive_ptr<c10d::Store> &store, int rank, int size) : Backend(rank, size) {
    TORCH_CHECK(size >= 1 && rank >= 0 && rank < size, "bad rank ", rank, " of ", size);
    // rank 0 makes the id; the others read it from the store (blocking until it is there).  The key names the
    // group: a store may be shared by several groups one after the other (simulated ranks over one HashStore
    // without torch's per-group prefix), and the id of an earlier group must not be found by a later one's ranks.
    // Every rank counts the groups it has joined through this store; ranks join their groups in the same order,
    // so the count is the same number for all ranks of one group.
    const int64_t generation = store->add("flagcx_amd/groups_joined/" + std::to_string(rank), 1);
    const std::string key = "flagcx_amd/unique_id/" + std::to_string(generation);
    flagcxUniqueId id;
    if (rank == 0) {
      ok(flagcxGetUniqueId(&id), "flagcxGetUniqueId");
      store->set(key, std::vector<uint8_t>(id.internal, id.internal + sizeof(id.internal)));
    } else {
      store->wait({key});
      const std::vector<uint8_t> bytes = store->get(key);
      TORCH_CHECK(bytes.size() == sizeof(id.internal), "unique id in the store has ", bytes.size(), " bytes");
      std::memcpy(id.internal, bytes.data(), sizeof(id.internal));
    }
    ok(flagcxCommInitRank(&comm_, size, &id, rank), "flagcxCommInitRank");
    group_.assign(id.internal, id.internal + sizeof(id.internal));
  }
  ~FxBackend() override {
    if (comm_) (void)flagcxCommDestroy(comm_);
    if (getRank() == 0) {
      std::lock_guard<std::mutex> lock(owedMu);
      owed.erase(group_);
    }
  }

  const std::string getBackendName() const override { return "flagcx"; }

  // A coalescing bracket is the library's group bracket (the reference's backend does the same,
  // backend_flagcx.cpp:525-537): sends and recvs that meet inside it leave as one copy launch when it closes.
  // What torch.distributed.batch_isend_irecv uses.
  bool supportsCoalescing() const override { return true; }
  void startCoalescing() override { ok(flagcxGroupStart(comm_), "flagcxGroupStart"); }
  c10::intrusive_ptr<Work> endCoalescing() override {
    ok(flagcxGroupEnd(comm_), "flagcxGroupEnd");
    return c10::make_intrusive<FxWork>(getRank(), OpType::COALESCED, c10::hip::getCurrentHIPStream().stream(), Tensors{});
  }

  c10::intrusive_ptr<Work> allreduce(Tensors &tensors, const c10d::AllreduceOptions &opts) override {
    checkOne(tensors, "allreduce");
    at::Tensor &t = tensors[0];
    checkDense(t, "allreduce");
    return run(OpType::ALLREDUCE, {t}, [&](flagcxStream_t s) {
      return flagcxAllReduce(t.data_ptr(), t.data_ptr(), (size_t)t.numel(), dtypeOf(t), opOf(opts.reduceOp, t), comm_, s);
    });
  }

  // One collective over the tensors laid end to end: with simulated ranks a
  // rank may not post a second collective before the others have posted the first.
  c10::intrusive_ptr<Work> allreduce_coalesced(Tensors &tensors, const c10d::AllreduceCoalescedOptions &opts) override {
    if (tensors.size() == 1) {
      c10d::AllreduceOptions one;
      one.reduceOp = opts.reduceOp;
      return allreduce(tensors, one);
    }
    TORCH_CHECK(!tensors.empty(), "allreduce_coalesced: no tensors");
    std::vector<size_t> displs, counts;
    at::Tensor flat = flatten(tensors, "allreduce_coalesced", displs, counts);
    return run(OpType::ALLREDUCE_COALESCED, tensors, [&](flagcxStream_t s) {
      return flagcxAllReduce(flat.data_ptr(), flat.data_ptr(), (size_t)flat.numel(), dtypeOf(flat), opOf(opts.reduceOp, flat), comm_, s);
    }, unpacker(flat, tensors, displs, counts), {flat});
  }

  c10::intrusive_ptr<Work> broadcast(Tensors &tensors, const c10d::BroadcastOptions &opts) override {
    checkOne(tensors, "broadcast");
    at::Tensor &t = tensors[0];
    checkDense(t, "broadcast");
    const int root = (int)opts.rootRank;
    return run(OpType::BROADCAST, {t}, [&](flagcxStream_t s) {
      return flagcxBroadcast(t.data_ptr(), t.data_ptr(), (size_t)t.numel(), dtypeOf(t), root, comm_, s);
    });
  }

  c10::intrusive_ptr<Work> reduce(Tensors &tensors, const c10d::ReduceOptions &opts) override {
    checkOne(tensors, "reduce");
    at::Tensor &t = tensors[0];
    checkDense(t, "reduce");
    const int root = (int)opts.rootRank;
    return run(OpType::REDUCE, {t}, [&](flagcxStream_t s) {
      return flagcxReduce(t.data_ptr(), t.data_ptr(), (size_t)t.numel(), dtypeOf(t), opOf(opts.reduceOp, t), root, comm_, s);
    });
  }

  c10::intrusive_ptr<Work> _allgather_base(at::Tensor &out, at::Tensor &in, const c10d::AllgatherOptions &) override {
    checkDense(out, "allgather_into_tensor");
    checkDense(in, "allgather_into_tensor");
    TORCH_CHECK(out.scalar_type() == in.scalar_type(), "allgather_into_tensor: input and output types differ");
    TORCH_CHECK(out.numel() == in.numel() * getSize(), "allgather_into_tensor: output must hold world_size inputs");
    return run(OpType::_ALLGATHER_BASE, {out}, [&](flagcxStream_t s) {
      return flagcxAllGather(in.data_ptr(), out.data_ptr(), (size_t)in.numel(), dtypeOf(in), comm_, s);
    }, nullptr, {in});
  }

  c10::intrusive_ptr<Work> allgather(std::vector<Tensors> &outs, Tensors &ins, const c10d::AllgatherOptions &opts) override {
    checkOne(ins, "allgather");
    TORCH_CHECK(outs.size() == 1 && (int)outs[0].size() == getSize(), "allgather: one output list of world_size tensors");
    at::Tensor &in = ins[0];
    checkDense(in, "allgather");
    for (auto &o : outs[0])
      TORCH_CHECK(o.numel() == in.numel() && o.scalar_type() == in.scalar_type(), "allgather: outputs must match the input");
    at::Tensor flat = at::empty({(int64_t)getSize() * in.numel()}, in.options());
    std::vector<size_t> displs(getSize()), counts(getSize(), (size_t)in.numel());
    for (int r = 0; r < getSize(); r++) displs[r] = (size_t)r * (size_t)in.numel();
    return run(OpType::ALLGATHER, outs[0], [&](flagcxStream_t s) {
      return flagcxAllGather(in.data_ptr(), flat.data_ptr(), (size_t)in.numel(), dtypeOf(in), comm_, s);
    }, unpacker(flat, outs[0], displs, counts), {flat});
  }

  // Every rank's inputs end to end, gathered once; output i is then rank 0's
  // input i, rank 1's input i, ... copied out of the gathered rows.
  c10::intrusive_ptr<Work> allgather_into_tensor_coalesced(Tensors &outs, Tensors &ins, const c10d::AllgatherOptions &opts) override {
    TORCH_CHECK(outs.size() == ins.size() && !ins.empty(), "allgather_into_tensor_coalesced: as many outputs as inputs, at least one");
    if (ins.size() == 1) return _allgather_base(outs[0], ins[0], opts);
    const int n = getSize();
    for (size_t i = 0; i < ins.size(); i++) {
      checkDense(outs[i], "allgather_into_tensor_coalesced");
      TORCH_CHECK(outs[i].scalar_type() == ins[i].scalar_type() && outs[i].numel() == ins[i].numel() * n,
                  "allgather_into_tensor_coalesced: output ", i, " must hold world_size inputs of the same type");
    }
    std::vector<size_t> displs, counts;
    at::Tensor flat = flatten(ins, "allgather_into_tensor_coalesced", displs, counts);
    const int64_t total = flat.numel();
    at::Tensor all = at::empty({(int64_t)n * total}, flat.options());
    Tensors outsCopy = outs;
    auto finish = [all, outsCopy, displs, counts, n, total]() mutable {
      const at::Tensor rows = all.view({n, total});
      for (size_t i = 0; i < outsCopy.size(); i++)
        if (counts[i])
          outsCopy[i].view({n, (int64_t)counts[i]}).copy_(rows.narrow(1, (int64_t)displs[i], (int64_t)counts[i]), true);
    };
    return run(OpType::COALESCED, outs, [&](flagcxStream_t s) {
      return flagcxAllGather(flat.data_ptr(), all.data_ptr(), (size_t)total, dtypeOf(flat), comm_, s);
    }, std::move(finish), {flat, all});
  }

  c10::intrusive_ptr<Work> _reduce_scatter_base(at::Tensor &out, at::Tensor &in, const c10d::ReduceScatterOptions &opts) override {
    checkDense(out, "reduce_scatter_tensor");
    checkDense(in, "reduce_scatter_tensor");
    TORCH_CHECK(out.scalar_type() == in.scalar_type(), "reduce_scatter_tensor: input and output types differ");
    TORCH_CHECK(in.numel() == out.numel() * getSize(), "reduce_scatter_tensor: input must hold world_size outputs");
    return run(OpType::_REDUCE_SCATTER_BASE, {out}, [&](flagcxStream_t s) {
      return flagcxReduceScatter(in.data_ptr(), out.data_ptr(), (size_t)out.numel(), dtypeOf(in), opOf(opts.reduceOp, in), comm_, s);
    }, nullptr, {in});
  }

  c10::intrusive_ptr<Work> reduce_scatter(Tensors &outs, std::vector<Tensors> &ins, const c10d::ReduceScatterOptions &opts) override {
    checkOne(outs, "reduce_scatter");
    TORCH_CHECK(ins.size() == 1 && (int)ins[0].size() == getSize(), "reduce_scatter: one input list of world_size tensors");
    for (auto &t : ins[0])
      TORCH_CHECK(t.numel() == outs[0].numel() && t.scalar_type() == outs[0].scalar_type(), "reduce_scatter: inputs must match the output");
    Tensors flatParts;
    for (auto &t : ins[0]) flatParts.push_back(t.reshape({-1}));
    at::Tensor flat = at::cat(flatParts);
    return run(OpType::REDUCE_SCATTER, outs, [&](flagcxStream_t s) {
      return flagcxReduceScatter(flat.data_ptr(), outs[0].data_ptr(), (size_t)outs[0].numel(), dtypeOf(flat),
                                 opOf(opts.reduceOp, flat), comm_, s);
    }, nullptr, {flat});
  }

  // Row r of the staged input holds part r of every input end to end, so that one
  // reduce-scatter leaves this rank's part of every output in one row.
  c10::intrusive_ptr<Work> reduce_scatter_tensor_coalesced(Tensors &outs, Tensors &ins, const c10d::ReduceScatterOptions &opts) override {
    TORCH_CHECK(outs.size() == ins.size() && !ins.empty(), "reduce_scatter_tensor_coalesced: as many outputs as inputs, at least one");
    if (ins.size() == 1) return _reduce_scatter_base(outs[0], ins[0], opts);
    const int n = getSize();
    Tensors rows;
    std::vector<size_t> displs, counts;
    size_t total = 0;
    for (size_t i = 0; i < ins.size(); i++) {
      checkDense(ins[i], "reduce_scatter_tensor_coalesced");
      checkDense(outs[i], "reduce_scatter_tensor_coalesced");
      TORCH_CHECK(ins[i].scalar_type() == ins[0].scalar_type() && outs[i].scalar_type() == ins[0].scalar_type(),
                  "reduce_scatter_tensor_coalesced: one element type throughout");
      TORCH_CHECK(ins[i].numel() == outs[i].numel() * n, "reduce_scatter_tensor_coalesced: input ", i, " must hold world_size outputs");
      rows.push_back(ins[i].view({n, outs[i].numel()}));
      displs.push_back(total);
      counts.push_back((size_t)outs[i].numel());
      total += (size_t)outs[i].numel();
    }
    at::Tensor staged = at::cat(rows, 1).contiguous();
    at::Tensor mine = at::empty({(int64_t)total}, staged.options());
    return run(OpType::COALESCED, outs, [&](flagcxStream_t s) {
      return flagcxReduceScatter(staged.data_ptr(), mine.data_ptr(), total, dtypeOf(staged), opOf(opts.reduceOp, staged), comm_, s);
    }, unpacker(mine, outs, displs, counts), {staged, mine});
  }

  c10::intrusive_ptr<Work> alltoall_base(at::Tensor &out, at::Tensor &in, std::vector<int64_t> &outSplit,
                                         std::vector<int64_t> &inSplit, const c10d::AllToAllOptions &) override {
    checkDense(out, "all_to_all_single");
    checkDense(in, "all_to_all_single");
    TORCH_CHECK(out.scalar_type() == in.scalar_type(), "all_to_all_single: input and output types differ");
    const int n = getSize();
    if (outSplit.empty() && inSplit.empty()) {
      TORCH_CHECK(in.numel() == out.numel() && in.numel() % n == 0, "all_to_all_single: sizes must be equal and divide by world_size");
      return run(OpType::ALLTOALL_BASE, {out}, [&](flagcxStream_t s) {
        return flagcxAlltoAll(in.data_ptr(), out.data_ptr(), (size_t)(in.numel() / n), dtypeOf(in), comm_, s);
      }, nullptr, {in});
    }
    // splits count rows of dimension 0; everything below it is one row
    auto layout = [n](const at::Tensor &t, const std::vector<int64_t> &split, std::vector<size_t> &counts, std::vector<size_t> &displs) {
      const int64_t row = t.dim() > 0 && t.size(0) > 0 ? t.numel() / t.size(0) : 0;
      counts.assign(n, 0);
      displs.assign(n, 0);
      if (split.empty()) {
        TORCH_CHECK(t.dim() > 0 && t.size(0) % n == 0, "all_to_all_single: dimension 0 must divide by world_size");
        for (int r = 0; r < n; r++) counts[r] = (size_t)(t.size(0) / n * row);
      } else {
        TORCH_CHECK((int)split.size() == n, "all_to_all_single: one split size per rank");
        TORCH_CHECK(std::accumulate(split.begin(), split.end(), (int64_t)0) == (t.dim() > 0 ? t.size(0) : 0),
                    "all_to_all_single: split sizes must add up to dimension 0");
        for (int r = 0; r < n; r++) counts[r] = (size_t)(split[r] * row);
      }
      for (int r = 1; r < n; r++) displs[r] = displs[r - 1] + counts[r - 1];
    };
    std::vector<size_t> sc, sd, rc, rd;
    layout(in, inSplit, sc, sd);
    layout(out, outSplit, rc, rd);
    return run(OpType::ALLTOALL_BASE, {out}, [&](flagcxStream_t s) {
      return flagcxAlltoAllv(in.data_ptr(), sc.data(), sd.data(), out.data_ptr(), rc.data(), rd.data(), dtypeOf(in), comm_, s);
    }, nullptr, {in});
  }

  c10::intrusive_ptr<Work> alltoall(Tensors &outs, Tensors &ins, const c10d::AllToAllOptions &) override {
    const int n = getSize();
    TORCH_CHECK((int)outs.size() == n && (int)ins.size() == n, "all_to_all: world_size tensors each way");
    std::vector<size_t> sc(n), sd(n, 0), rc(n), rd(n, 0);
    Tensors flatIn;
    for (int r = 0; r < n; r++) {
      TORCH_CHECK(ins[r].scalar_type() == ins[0].scalar_type() && outs[r].scalar_type() == ins[0].scalar_type(),
                  "all_to_all: one element type throughout");
      sc[r] = (size_t)ins[r].numel();
      rc[r] = (size_t)outs[r].numel();
      flatIn.push_back(ins[r].reshape({-1}));
    }
    for (int r = 1; r < n; r++) {
      sd[r] = sd[r - 1] + sc[r - 1];
      rd[r] = rd[r - 1] + rc[r - 1];
    }
    at::Tensor in = at::cat(flatIn);
    at::Tensor out = at::empty({(int64_t)(rd[n - 1] + rc[n - 1])}, ins[0].options());
    checkDense(in, "all_to_all");
    return run(OpType::ALLTOALL, outs, [&](flagcxStream_t s) {
      return flagcxAlltoAllv(in.data_ptr(), sc.data(), sd.data(), out.data_ptr(), rc.data(), rd.data(), dtypeOf(in), comm_, s);
    }, unpacker(out, outs, rd, rc), {in, out});
  }

  c10::intrusive_ptr<Work> gather(std::vector<Tensors> &outs, Tensors &ins, const c10d::GatherOptions &opts) override {
    checkOne(ins, "gather");
    at::Tensor &in = ins[0];
    checkDense(in, "gather");
    const int root = (int)opts.rootRank, n = getSize();
    at::Tensor flat;
    if (getRank() == root) {
      TORCH_CHECK(outs.size() == 1 && (int)outs[0].size() == n, "gather: the root passes one list of world_size tensors");
      flat = at::empty({(int64_t)n * in.numel()}, in.options());
    } else {
      TORCH_CHECK(outs.empty() || outs[0].empty(), "gather: only the root passes outputs");
    }
    std::function<void()> finish;
    if (getRank() == root) {
      std::vector<size_t> rd(n), rc(n, (size_t)in.numel());
      for (int r = 0; r < n; r++) rd[r] = (size_t)r * (size_t)in.numel();
      finish = unpacker(flat, outs[0], rd, rc);
    }
    return run(OpType::GATHER, getRank() == root ? outs[0] : Tensors{}, [&](flagcxStream_t s) {
      return flagcxGather(in.data_ptr(), flat.defined() ? flat.data_ptr() : nullptr, (size_t)in.numel(), dtypeOf(in), root, comm_, s);
    }, std::move(finish), flat.defined() ? Tensors{in, flat} : Tensors{in});
  }

  c10::intrusive_ptr<Work> scatter(Tensors &outs, std::vector<Tensors> &ins, const c10d::ScatterOptions &opts) override {
    checkOne(outs, "scatter");
    at::Tensor &out = outs[0];
    checkDense(out, "scatter");
    const int root = (int)opts.rootRank, n = getSize();
    at::Tensor flat;
    if (getRank() == root) {
      TORCH_CHECK(ins.size() == 1 && (int)ins[0].size() == n, "scatter: the root passes one list of world_size tensors");
      Tensors parts;
      for (auto &t : ins[0]) {
        TORCH_CHECK(t.numel() == out.numel() && t.scalar_type() == out.scalar_type(), "scatter: inputs must match the output");
        parts.push_back(t.reshape({-1}));
      }
      flat = at::cat(parts);
    }
    return run(OpType::SCATTER, outs, [&](flagcxStream_t s) {
      return flagcxScatter(flat.defined() ? flat.data_ptr() : nullptr, out.data_ptr(), (size_t)out.numel(), dtypeOf(out), root, comm_, s);
    }, nullptr, {flat});
  }

  c10::intrusive_ptr<Work> send(Tensors &tensors, int dst, int /*tag*/) override {
    checkOne(tensors, "send");
    at::Tensor &t = tensors[0];
    checkDense(t, "send");
    return run(OpType::SEND, {}, [&](flagcxStream_t s) {
      return flagcxSend(t.data_ptr(), (size_t)t.numel(), dtypeOf(t), dst, comm_, s);
    }, nullptr, {t});
  }

  c10::intrusive_ptr<Work> recv(Tensors &tensors, int src, int /*tag*/) override {
    checkOne(tensors, "recv");
    at::Tensor &t = tensors[0];
    checkDense(t, "recv");
    return run(OpType::RECV, {t}, [&](flagcxStream_t s) {
      return flagcxRecv(t.data_ptr(), (size_t)t.numel(), dtypeOf(t), src, comm_, s);
    });
  }

  c10::intrusive_ptr<Work> barrier(const c10d::BarrierOptions &) override {
    return run(OpType::BARRIER, {}, [&](flagcxStream_t s) { return flagcxBarrier(comm_, s); });
  }

 private:
  // The tensors' elements end to end in a new tensor; where each one starts and how long it is.
  static at::Tensor flatten(const Tensors &v, const char *what, std::vector<size_t> &displs, std::vector<size_t> &counts) {
    Tensors parts;
    size_t total = 0;
    for (const auto &t : v) {
      checkDense(t, what);
      TORCH_CHECK(t.scalar_type() == v[0].scalar_type(), what, ": one element type throughout");
      parts.push_back(t.reshape({-1}));
      displs.push_back(total);
      counts.push_back((size_t)t.numel());
      total += (size_t)t.numel();
    }
    return at::cat(parts);
  }

  // Copy pieces of a staging tensor into a list of output tensors, on the
  // collective's stream, after the launch.
  static std::function<void()> unpacker(at::Tensor flat, Tensors outs, std::vector<size_t> displs, std::vector<size_t> counts) {
    return [flat, outs, displs, counts]() mutable {
      for (size_t r = 0; r < outs.size(); r++)
        if (counts[r]) outs[r].copy_(flat.narrow(0, (int64_t)displs[r], (int64_t)counts[r]).view_as(outs[r]), true);
    };
  }

  // `staging`: tensors of this call that the kernels read or write and that
  // nothing else keeps alive: staging the caller never sees, and inputs the
  // caller may drop as soon as the call returns.  With simulated ranks the
  // launch may come from a later rank's call, so they are held here, not by the
  // Work the caller may drop, until this rank's next collective has been
  // accepted -- which the rank layer only does once the previous one has been
  // launched.
  template <class F>
  c10::intrusive_ptr<Work> run(OpType op, Tensors outputs, F call, std::function<void()> finish = nullptr,
                               Tensors staging = {}) {
    const c10::hip::HIPStream cur = c10::hip::getCurrentHIPStream();
    const hipStream_t raw = cur.stream();
    BorrowedStream s(raw);
    ok(call(s.get()), c10d::opTypeToString(op).c_str());
    if (op == OpType::SEND) {
      // The matching recv may come after this rank's next collective has been
      // accepted, but not after the one that follows: that one is only accepted
      // once the next has been launched, for which the receiver has posted it,
      // and its recv before it.
      for (auto &t : staging) sent_[0].push_back(std::move(t));
    } else if (op != OpType::RECV) {
      sent_[1] = std::move(sent_[0]);
      sent_[0].clear();
      held_ = std::move(staging);
      uint64_t joined = 0, launched = 0;
      ok(fxSimCommProgress(comm_, &joined, &launched), "fxSimCommProgress");
      if (finish) {
        std::lock_guard<std::mutex> lock(owedMu);
        owed[group_].push_back(Owed{joined, cur, std::move(finish)});
      }
      if (launched > joined) payOwed(group_, launched);
    }
    return c10::make_intrusive<FxWork>(getRank(), op, raw, std::move(outputs));
  }

  flagcxComm_t comm_ = nullptr;
  std::string group_;   // the unique id's bytes: what the ranks of one group share
  Tensors held_;
  Tensors sent_[2];   // send buffers of the calls since the last collective, and of those before it
};

c10::intrusive_ptr<c10d::Backend> createBackend(const c10::intrusive_ptr<c10d::Store> &store, int rank, int size) {
  return c10::make_intrusive<FxBackend>(store, rank, size);
}

}  // namespace

PYBIND11_MODULE(fx_c10d, m) {
  m.doc() = "torch.distributed backend over libflagcx_amd.so";
  // without the interpreter lock: a rank other than 0 waits in here for rank 0's id, and rank 0 may be
  // another thread of this process
  m.def("create_backend", &createBackend, py::arg("store"), py::arg("rank"), py::arg("size"),
        py::call_guard<py::gil_scoped_release>());
  // torch binds these two on ProcessGroup only; a backend object on its own reaches them here
  m.def("allgather_into_tensor_coalesced", [](const c10::intrusive_ptr<c10d::Backend> &b, Tensors outs, Tensors ins) {
    return b->allgather_into_tensor_coalesced(outs, ins);
  }, py::arg("backend"), py::arg("outputs"), py::arg("inputs"));
  m.def("reduce_scatter_tensor_coalesced", [](const c10::intrusive_ptr<c10d::Backend> &b, Tensors outs, Tensors ins, const c10d::ReduceOp &op) {
    c10d::ReduceScatterOptions o;
    o.reduceOp = op;
    return b->reduce_scatter_tensor_coalesced(outs, ins, o);
  }, py::arg("backend"), py::arg("outputs"), py::arg("inputs"), py::arg("op") = c10d::ReduceOp(c10d::ReduceOp::SUM));
}
