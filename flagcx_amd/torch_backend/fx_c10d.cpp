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
// Work is meant to be called then (with one rank, at once).
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
  // `finish`: what is left to do on the stream once the collective has been
  // launched (copies out of a staging tensor into a list of output tensors);
  // it runs at the first wait.
  FxWork(int rank, OpType op, hipStream_t stream, Tensors outputs, std::function<void()> finish = nullptr)
      : Work(rank, op), stream_(stream), outputs_(std::move(outputs)), finish_(std::move(finish)) {
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
    finishOnce();
    mark();
    return hipEventQuery(event_) == hipSuccess;
  }
  bool isSuccess() const override { return true; }
  // Orders the caller's current stream after the collective; never blocks the host.
  bool wait(std::chrono::milliseconds /*timeout*/ = kNoTimeout) override {
    finishOnce();
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
  void finishOnce() {
    if (!finish_) return;
    std::function<void()> f;
    f.swap(finish_);
    // the copies go where the collective went, whatever stream is current now
    const c10::hip::HIPStream before = c10::hip::getCurrentHIPStream();
    if (before.stream() == stream_) {
      f();
      return;
    }
    c10::hip::setCurrentHIPStream(c10::hip::getStreamFromExternal(stream_, before.device_index()));
    try {
      f();
    } catch (...) {
      c10::hip::setCurrentHIPStream(before);
      throw;
    }
    c10::hip::setCurrentHIPStream(before);
  }
  hipStream_t stream_;
  hipEvent_t event_ = nullptr;
  Tensors outputs_;
  std::function<void()> finish_;
  c10::intrusive_ptr<c10::ivalue::Future> future_;
};

class FxBackend : public c10d::Backend {
 public:
  FxBackend(const c10::intrusive_ptr<c10d::Store> &store, int rank, int size) : Backend(rank, size) {
    TORCH_CHECK(size >= 1 && rank >= 0 && rank < size, "bad rank ", rank, " of ", size);
    // rank 0 makes the id; the others read it from the store (blocking until it is there)
    const std::string key = "flagcx_amd/unique_id";
    flagcxUniqueId id;
    if (rank == 0) {
      ok(flagcxGetUniqueId(&id), "flagcxGetUniqueId");
      store->set(key, std::vector<uint8_t>(id.internal, id.internal + sizeof(id.internal)));
    } else {
      const std::vector<uint8_t> bytes = store->get(key);
      TORCH_CHECK(bytes.size() == sizeof(id.internal), "unique id in the store has ", bytes.size(), " bytes");
      std::memcpy(id.internal, bytes.data(), sizeof(id.internal));
    }
    ok(flagcxCommInitRank(&comm_, size, &id, rank), "flagcxCommInitRank");
  }
  ~FxBackend() override {
    if (comm_) (void)flagcxCommDestroy(comm_);
  }

  const std::string getBackendName() const override { return "flagcx"; }

  c10::intrusive_ptr<Work> allreduce(Tensors &tensors, const c10d::AllreduceOptions &opts) override {
    checkOne(tensors, "allreduce");
    at::Tensor &t = tensors[0];
    checkDense(t, "allreduce");
    return run(OpType::ALLREDUCE, {t}, [&](flagcxStream_t s) {
      return flagcxAllReduce(t.data_ptr(), t.data_ptr(), (size_t)t.numel(), dtypeOf(t), opOf(opts.reduceOp, t), comm_, s);
    });
  }

  c10::intrusive_ptr<Work> allreduce_coalesced(Tensors &tensors, const c10d::AllreduceCoalescedOptions &opts) override {
    for (auto &t : tensors) checkDense(t, "allreduce_coalesced");
    return run(OpType::ALLREDUCE_COALESCED, tensors, [&](flagcxStream_t s) {
      for (auto &t : tensors) {
        const flagcxResult_t rc = flagcxAllReduce(t.data_ptr(), t.data_ptr(), (size_t)t.numel(), dtypeOf(t),
                                                  opOf(opts.reduceOp, t), comm_, s);
        if (rc != flagcxSuccess) return rc;
      }
      return flagcxSuccess;
    });
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
    });
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

  c10::intrusive_ptr<Work> allgather_into_tensor_coalesced(Tensors &outs, Tensors &ins, const c10d::AllgatherOptions &opts) override {
    TORCH_CHECK(outs.size() == ins.size(), "allgather_into_tensor_coalesced: as many outputs as inputs");
    for (size_t i = 0; i < ins.size(); i++) (void)_allgather_base(outs[i], ins[i], opts);
    return c10::make_intrusive<FxWork>(getRank(), OpType::COALESCED, c10::hip::getCurrentHIPStream().stream(), outs);
  }

  c10::intrusive_ptr<Work> _reduce_scatter_base(at::Tensor &out, at::Tensor &in, const c10d::ReduceScatterOptions &opts) override {
    checkDense(out, "reduce_scatter_tensor");
    checkDense(in, "reduce_scatter_tensor");
    TORCH_CHECK(out.scalar_type() == in.scalar_type(), "reduce_scatter_tensor: input and output types differ");
    TORCH_CHECK(in.numel() == out.numel() * getSize(), "reduce_scatter_tensor: input must hold world_size outputs");
    return run(OpType::_REDUCE_SCATTER_BASE, {out}, [&](flagcxStream_t s) {
      return flagcxReduceScatter(in.data_ptr(), out.data_ptr(), (size_t)out.numel(), dtypeOf(in), opOf(opts.reduceOp, in), comm_, s);
    });
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

  c10::intrusive_ptr<Work> reduce_scatter_tensor_coalesced(Tensors &outs, Tensors &ins, const c10d::ReduceScatterOptions &opts) override {
    TORCH_CHECK(outs.size() == ins.size(), "reduce_scatter_tensor_coalesced: as many outputs as inputs");
    for (size_t i = 0; i < ins.size(); i++) (void)_reduce_scatter_base(outs[i], ins[i], opts);
    return c10::make_intrusive<FxWork>(getRank(), OpType::COALESCED, c10::hip::getCurrentHIPStream().stream(), outs);
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
      });
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
    });
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
    }, std::move(finish), flat.defined() ? Tensors{flat} : Tensors{});
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
    });
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
  // Copy pieces of a staging tensor into a list of output tensors, on the
  // collective's stream, after the launch.
  static std::function<void()> unpacker(at::Tensor flat, Tensors outs, std::vector<size_t> displs, std::vector<size_t> counts) {
    return [flat, outs, displs, counts]() mutable {
      for (size_t r = 0; r < outs.size(); r++)
        if (counts[r]) outs[r].copy_(flat.narrow(0, (int64_t)displs[r], (int64_t)counts[r]).view_as(outs[r]), true);
    };
  }

  // `staging`: tensors of this call that the kernels read or write and the
  // caller never sees.  With simulated ranks the launch may come from a later
  // rank's call, so they are held here, not by the Work the caller may drop,
  // until this rank's next collective has been accepted -- which the rank layer
  // only does once the previous one has been launched.
  template <class F>
  c10::intrusive_ptr<Work> run(OpType op, Tensors outputs, F call, std::function<void()> finish = nullptr,
                               Tensors staging = {}) {
    const hipStream_t raw = c10::hip::getCurrentHIPStream().stream();
    BorrowedStream s(raw);
    ok(call(s.get()), c10d::opTypeToString(op).c_str());
    held_ = std::move(staging);
    auto work = c10::make_intrusive<FxWork>(getRank(), op, raw, std::move(outputs), std::move(finish));
    if (getSize() == 1) (void)work->wait();   // one rank: the launch has happened, finish now
    return work;
  }

  flagcxComm_t comm_ = nullptr;
  Tensors held_;
};

c10::intrusive_ptr<c10d::Backend> createBackend(const c10::intrusive_ptr<c10d::Store> &store, int rank, int size) {
  return c10::make_intrusive<FxBackend>(store, rank, size);
}

}  // namespace

PYBIND11_MODULE(fx_c10d, m) {
  m.doc() = "torch.distributed backend over libflagcx_amd.so";
  m.def("create_backend", &createBackend, py::arg("store"), py::arg("rank"), py::arg("size"));
}
