// Python module on PyTorch-ROCm: a c10d::ProcessGroup whose collectives run
// the hot path of the host core (libmoodist.so) on the caller's current HIP
// stream.
//
// Mirrors the reference's wrapper: the c10d virtuals _allgather_base,
// _reduce_scatter_base, allreduce and the coalesced variants
// (wrapper/processgroup_wrapper.cc:131-190), compile_op_full -> CustomOp ->
// Future (wrapper/processgroup_wrapper.cc:349-444; wrapper/module.cc:689-804,
// :1240-1305), option access (wrapper/module.cc:836-848), the unsupported
// point-to-point calls (wrapper/processgroup_wrapper.h:168-185) and the
// dlopen + version handshake with the core (wrapper/moodist_loader.cc:363-386).
// Tensors cross into the core as plain descriptors; the core never sees torch.
#include <dlfcn.h>

#include <c10/hip/HIPStream.h>
#include <torch/csrc/distributed/c10d/ProcessGroup.hpp>
#include <torch/csrc/distributed/c10d/Work.hpp>
#include <torch/extension.h>

#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "moodist_core.h"

namespace py = pybind11;

namespace {

// ---- the core, loaded at import (wrapper/moodist_loader.cc:363-386) ----

struct CoreApi {
#define MOODIST_CORE_FN(name) decltype(&::name) name = nullptr;
  MOODIST_CORE_FN(moodist_core_check_version)
  MOODIST_CORE_FN(moodist_last_error)
  MOODIST_CORE_FN(moodist_world_create)
  MOODIST_CORE_FN(moodist_world_destroy)
  MOODIST_CORE_FN(moodist_world_group)
  MOODIST_CORE_FN(moodist_pg_rank)
  MOODIST_CORE_FN(moodist_pg_size)
  MOODIST_CORE_FN(moodist_pg_get_option)
  MOODIST_CORE_FN(moodist_pg_set_option)
  MOODIST_CORE_FN(moodist_pg_all_gather)
  MOODIST_CORE_FN(moodist_pg_all_gather_list)
  MOODIST_CORE_FN(moodist_pg_reduce_scatter)
  MOODIST_CORE_FN(moodist_pg_allreduce)
  MOODIST_CORE_FN(moodist_pg_stage_input)
  MOODIST_CORE_FN(moodist_work_is_completed)
  MOODIST_CORE_FN(moodist_work_wait)
  MOODIST_CORE_FN(moodist_work_destroy)
  MOODIST_CORE_FN(moodist_compile_op_full)
  MOODIST_CORE_FN(moodist_op_destroy)
  MOODIST_CORE_FN(moodist_op_call)
  MOODIST_CORE_FN(moodist_future_wait)
  MOODIST_CORE_FN(moodist_future_destroy)
  MOODIST_CORE_FN(moodist_op_plan_count)
  MOODIST_CORE_FN(moodist_op_plan_read)
  MOODIST_CORE_FN(moodist_op_plan_copy)
  MOODIST_CORE_FN(moodist_op_plan_size)
  MOODIST_CORE_FN(moodist_op_plan_message)
#undef MOODIST_CORE_FN
};

CoreApi core;

void load_core() {
  Dl_info info;
  std::string path = "libmoodist.so";
  if (dladdr(reinterpret_cast<void*>(&load_core), &info) && info.dli_fname) {
    std::string self = info.dli_fname;
    size_t slash = self.rfind('/');
    if (slash != std::string::npos) {
      path = self.substr(0, slash + 1) + "libmoodist.so";
    }
  }
  void* lib = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (!lib) {
    throw std::runtime_error("moodist: cannot load " + path + ": " + dlerror());
  }
#define MOODIST_CORE_FN(name)                                                  \
  core.name = reinterpret_cast<decltype(core.name)>(dlsym(lib, #name));        \
  if (!core.name) {                                                            \
    throw std::runtime_error("moodist: libmoodist.so has no symbol " #name); \
  }
  MOODIST_CORE_FN(moodist_core_check_version)
  MOODIST_CORE_FN(moodist_last_error)
  MOODIST_CORE_FN(moodist_world_create)
  MOODIST_CORE_FN(moodist_world_destroy)
  MOODIST_CORE_FN(moodist_world_group)
  MOODIST_CORE_FN(moodist_pg_rank)
  MOODIST_CORE_FN(moodist_pg_size)
  MOODIST_CORE_FN(moodist_pg_get_option)
  MOODIST_CORE_FN(moodist_pg_set_option)
  MOODIST_CORE_FN(moodist_pg_all_gather)
  MOODIST_CORE_FN(moodist_pg_all_gather_list)
  MOODIST_CORE_FN(moodist_pg_reduce_scatter)
  MOODIST_CORE_FN(moodist_pg_allreduce)
  MOODIST_CORE_FN(moodist_pg_stage_input)
  MOODIST_CORE_FN(moodist_work_is_completed)
  MOODIST_CORE_FN(moodist_work_wait)
  MOODIST_CORE_FN(moodist_work_destroy)
  MOODIST_CORE_FN(moodist_compile_op_full)
  MOODIST_CORE_FN(moodist_op_destroy)
  MOODIST_CORE_FN(moodist_op_call)
  MOODIST_CORE_FN(moodist_future_wait)
  MOODIST_CORE_FN(moodist_future_destroy)
  MOODIST_CORE_FN(moodist_op_plan_count)
  MOODIST_CORE_FN(moodist_op_plan_read)
  MOODIST_CORE_FN(moodist_op_plan_copy)
  MOODIST_CORE_FN(moodist_op_plan_size)
  MOODIST_CORE_FN(moodist_op_plan_message)
#undef MOODIST_CORE_FN
  if (!core.moodist_core_check_version(MOODIST_CORE_API_VERSION)) {
    throw std::runtime_error("moodist: libmoodist.so speaks a different API version than this module");
  }
}

void check(int rc) {
  if (rc != 0) {
    throw std::runtime_error(core.moodist_last_error());
  }
}

moodist_tensor describe(const at::Tensor& t) {
  moodist_tensor d{};
  d.data = t.data_ptr();
  d.numel = t.numel();
  d.itemsize = (int32_t)t.element_size();
  d.dtype = (int32_t)t.scalar_type();
  d.device = t.is_cuda() ? (int32_t)t.device().index() : -1;
  d.contiguous = t.is_contiguous() ? 1 : 0;
  d.ndim = (int32_t)std::min<int64_t>(t.dim(), 10);
  for (int i = 0; i < d.ndim; ++i) {
    d.shape[i] = t.size(i);
  }
  return d;
}

// the caller's current stream on the tensor's device (wrapper/processgroup_wrapper.cc:55-57)
void* stream_of(const at::Tensor& t) {
  return t.is_cuda() ? (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream() : nullptr;
}

int reduce_op_code(const c10d::ReduceOp& op) {
  switch (static_cast<int>(op.op_)) {
  case c10d::ReduceOp::SUM:
  case c10d::ReduceOp::AVG:
  case c10d::ReduceOp::PRODUCT:
  case c10d::ReduceOp::MIN:
  case c10d::ReduceOp::MAX:
  case c10d::ReduceOp::PREMUL_SUM:
    return static_cast<int>(op.op_); // the core refuses PRODUCT, as the reference's core does
  default:
    throw std::runtime_error("Unsupported reduce op");
  }
}

// wrapper/processgroup_wrapper.cc:41-53
float premul_value(const c10d::ReduceOp& op, at::ScalarType dtype) {
  if (op.op_ != c10d::ReduceOp::PREMUL_SUM) {
    return 0.0f;
  }
  if (dtype != at::ScalarType::Float) {
    throw std::runtime_error("PREMUL_SUM only supported for float32");
  }
  auto* supplement = reinterpret_cast<c10d::NCCLPreMulSumSupplement*>(op.supplement_.get());
  if (supplement->tensor_factor.defined()) {
    return supplement->tensor_factor.item<float>();
  }
  return static_cast<float>(supplement->double_factor);
}

// ---- Work: complete once every local rank has posted and the launch is enqueued ----

struct WorkImpl : c10d::Work {
  std::vector<moodist_work*> parts;
  std::vector<at::Tensor> tensors;

  ~WorkImpl() override {
    for (moodist_work* w : parts) {
      core.moodist_work_destroy(w);
    }
  }
  void synchronize() override {}
  bool wait(std::chrono::milliseconds = std::chrono::milliseconds(0)) override {
    for (moodist_work* w : parts) {
      check(core.moodist_work_wait(w));
    }
    return true;
  }
  bool isCompleted() override {
    for (moodist_work* w : parts) {
      if (!core.moodist_work_is_completed(w)) {
        return false;
      }
    }
    return true;
  }
  bool isSuccess() const override {
    return true;
  }
  std::vector<at::Tensor> result() override {
    return tensors;
  }
};

struct WorldHolder {
  moodist_world* world = nullptr;
  int size = 0;
  int device = 0;
  ~WorldHolder() {
    if (world) {
      core.moodist_world_destroy(world);
    }
  }
};

// ---- the process group ----

class ProcessGroup : public c10d::ProcessGroup {
public:
  ProcessGroup(std::shared_ptr<WorldHolder> world, int rank)
      : c10d::ProcessGroup(rank, world->size), world_(std::move(world)),
        pg_(core.moodist_world_group(world_->world, rank)) {
    if (!pg_) {
      throw std::runtime_error(core.moodist_last_error());
    }
  }

  const std::string getBackendName() const override {
    return "moodist";
  }

  c10::intrusive_ptr<c10d::Work> _allgather_base(at::Tensor& output, at::Tensor& input,
      const c10d::AllgatherOptions& = c10d::AllgatherOptions()) override {
    auto work = c10::make_intrusive<WorkImpl>();
    moodist_tensor o = describe(output), i = describe(input);
    moodist_work* w = nullptr;
    check(core.moodist_pg_all_gather(pg_, &o, &i, stream_of(input), &w));
    work->parts.push_back(w);
    work->tensors = {output};
    keep(input);
    return work;
  }

  // wrapper/processgroup_wrapper.cc:112-129
  c10::intrusive_ptr<c10d::Work> allgather(std::vector<std::vector<at::Tensor>>& outputLists,
      std::vector<at::Tensor>& inputs, const c10d::AllgatherOptions& = c10d::AllgatherOptions()) override {
    TORCH_CHECK(outputLists.size() == 1 && inputs.size() == 1);
    auto work = c10::make_intrusive<WorkImpl>();
    std::vector<moodist_tensor> outs;
    for (at::Tensor& t : outputLists[0]) {
      outs.push_back(describe(t));
    }
    moodist_tensor i = describe(inputs[0]);
    moodist_work* w = nullptr;
    check(core.moodist_pg_all_gather_list(pg_, outs.data(), outs.size(), &i, stream_of(inputs[0]), &w));
    work->parts.push_back(w);
    work->tensors = outputLists[0];
    keep(inputs[0]);
    return work;
  }

  c10::intrusive_ptr<c10d::Work> _reduce_scatter_base(at::Tensor& output, at::Tensor& input,
      const c10d::ReduceScatterOptions& opts = c10d::ReduceScatterOptions()) override {
    auto work = c10::make_intrusive<WorkImpl>();
    moodist_tensor o = describe(output), i = describe(input);
    moodist_work* w = nullptr;
    check(core.moodist_pg_reduce_scatter(pg_, &o, &i, reduce_op_code(opts.reduceOp), stream_of(input),
        premul_value(opts.reduceOp, input.scalar_type()), &w));
    work->parts.push_back(w);
    work->tensors = {output};
    keep(input);
    return work;
  }

  // wrapper/processgroup_wrapper.cc:139-148
  c10::intrusive_ptr<c10d::Work> allgather_into_tensor_coalesced(std::vector<at::Tensor>& outputs,
      std::vector<at::Tensor>& inputs, const c10d::AllgatherOptions& = c10d::AllgatherOptions()) override {
    TORCH_CHECK(outputs.size() == inputs.size());
    auto work = c10::make_intrusive<WorkImpl>();
    for (size_t k = 0; k < inputs.size(); ++k) {
      moodist_tensor o = describe(outputs[k]), i = describe(inputs[k]);
      moodist_work* w = nullptr;
      check(core.moodist_pg_all_gather(pg_, &o, &i, stream_of(inputs[k]), &w));
      work->parts.push_back(w);
      keep(inputs[k]);
    }
    work->tensors = outputs;
    return work;
  }

  // wrapper/processgroup_wrapper.cc:159-170
  c10::intrusive_ptr<c10d::Work> reduce_scatter_tensor_coalesced(std::vector<at::Tensor>& outputs,
      std::vector<at::Tensor>& inputs, const c10d::ReduceScatterOptions& opts = c10d::ReduceScatterOptions()) override {
    TORCH_CHECK(outputs.size() == inputs.size());
    auto work = c10::make_intrusive<WorkImpl>();
    for (size_t k = 0; k < inputs.size(); ++k) {
      moodist_tensor o = describe(outputs[k]), i = describe(inputs[k]);
      moodist_work* w = nullptr;
      check(core.moodist_pg_reduce_scatter(pg_, &o, &i, reduce_op_code(opts.reduceOp), stream_of(inputs[k]),
          premul_value(opts.reduceOp, inputs[k].scalar_type()), &w));
      work->parts.push_back(w);
      keep(inputs[k]);
    }
    work->tensors = outputs;
    return work;
  }

  // wrapper/processgroup_wrapper.cc:172-190
  c10::intrusive_ptr<c10d::Work> allreduce(std::vector<at::Tensor>& tensors,
      const c10d::AllreduceOptions& opts = c10d::AllreduceOptions()) override {
    TORCH_CHECK(tensors.size() == 1);
    at::Tensor& t = tensors[0];
    auto work = c10::make_intrusive<WorkImpl>();
    moodist_tensor d = describe(t), s{};
    const int64_t n = t.numel(), size = getSize();
    at::Tensor scratch;
    if (n % size != 0) {
      // the padded temporary the reference allocates through torch (core/processgroup.cc:1694-1697)
      scratch = at::empty({(n + size - 1) / size * size}, t.options());
      s = describe(scratch);
      keep(scratch); // allocated, used and later reused on this same stream, so stream order protects it
    }
    moodist_work* w = nullptr;
    check(core.moodist_pg_allreduce(pg_, &d, scratch.defined() ? &s : nullptr, reduce_op_code(opts.reduceOp),
        stream_of(t), premul_value(opts.reduceOp, t.scalar_type()), &w));
    work->parts.push_back(w);
    work->tensors = tensors;
    keep(t);
    return work;
  }

  // wrapper/processgroup_wrapper.cc:182-191
  c10::intrusive_ptr<c10d::Work> allreduce_coalesced(std::vector<at::Tensor>& tensors,
      const c10d::AllreduceCoalescedOptions& opts = c10d::AllreduceCoalescedOptions()) override {
    auto work = c10::make_intrusive<WorkImpl>();
    c10d::AllreduceOptions one;
    one.reduceOp = opts.reduceOp;
    for (at::Tensor& t : tensors) {
      std::vector<at::Tensor> single{t};
      auto part = allreduce(single, one);
      auto* impl = static_cast<WorkImpl*>(part.get());
      work->parts.insert(work->parts.end(), impl->parts.begin(), impl->parts.end());
      impl->parts.clear();
    }
    work->tensors = tensors;
    return work;
  }

  c10::intrusive_ptr<c10d::Work> barrier(const c10d::BarrierOptions& = c10d::BarrierOptions()) override {
    // every local rank lives in this process and on this thread: nothing to wait for
    return c10::make_intrusive<WorkImpl>();
  }

#define MOODIST_UNSUPPORTED(what) throw std::runtime_error("moodist: " what " is not supported")
  c10::intrusive_ptr<c10d::Work> send(std::vector<at::Tensor>&, int, int) override {
    MOODIST_UNSUPPORTED("send");
  }
  c10::intrusive_ptr<c10d::Work> recv(std::vector<at::Tensor>&, int, int) override {
    MOODIST_UNSUPPORTED("recv");
  }
  c10::intrusive_ptr<c10d::Work> recvAnysource(std::vector<at::Tensor>&, int) override {
    MOODIST_UNSUPPORTED("recvAnysource");
  }
  c10::intrusive_ptr<c10d::Work> scatter(std::vector<at::Tensor>&, std::vector<std::vector<at::Tensor>>&,
      const c10d::ScatterOptions& = c10d::ScatterOptions()) override {
    MOODIST_UNSUPPORTED("scatter");
  }
  c10::intrusive_ptr<c10d::Work> broadcast(std::vector<at::Tensor>&,
      const c10d::BroadcastOptions& = c10d::BroadcastOptions()) override {
    MOODIST_UNSUPPORTED("broadcast (outside the single-GPU hot path)");
  }
  c10::intrusive_ptr<c10d::Work> reduce(std::vector<at::Tensor>&,
      const c10d::ReduceOptions& = c10d::ReduceOptions()) override {
    MOODIST_UNSUPPORTED("reduce (outside the single-GPU hot path)");
  }
  c10::intrusive_ptr<c10d::Work> gather(std::vector<std::vector<at::Tensor>>&, std::vector<at::Tensor>&,
      const c10d::GatherOptions& = c10d::GatherOptions()) override {
    MOODIST_UNSUPPORTED("gather (outside the single-GPU hot path)");
  }
  c10::intrusive_ptr<c10d::Work> alltoall(std::vector<at::Tensor>&, std::vector<at::Tensor>&,
      const c10d::AllToAllOptions& = c10d::AllToAllOptions()) override {
    MOODIST_UNSUPPORTED("alltoall (outside the single-GPU hot path)");
  }
#undef MOODIST_UNSUPPORTED

  moodist_pg* handle() const {
    return pg_;
  }

  // A peer that only contributes: its buffer is the staged contribution of that rank.
  c10::intrusive_ptr<c10d::Work> stage_input(const std::string& kind, at::Tensor& input, int reduce_op, float premul) {
    auto work = c10::make_intrusive<WorkImpl>();
    moodist_tensor i = describe(input);
    moodist_work* w = nullptr;
    int k;
    if (kind == "all_gather") {
      k = 0;
    } else if (kind == "reduce_scatter") {
      k = 1;
    } else {
      throw std::runtime_error("moodist: stage_input kind must be 'all_gather' or 'reduce_scatter'");
    }
    check(core.moodist_pg_stage_input(pg_, k, &i, reduce_op, stream_of(input), premul, &w));
    work->parts.push_back(w);
    keep(input);
    return work;
  }

private:
  // Inputs must outlive launches that happen when a later rank posts; the core holds raw
  // pointers, so the last few tensors are kept alive here (the reference keeps peers' memory
  // mapped through its IPC cache instead, core/ipc_mapper.h:30-40).
  void keep(const at::Tensor& t) {
    alive_[next_alive_++ % alive_.size()] = t;
  }
  std::shared_ptr<WorldHolder> world_;
  moodist_pg* pg_;
  std::array<at::Tensor, 64> alive_;
  size_t next_alive_ = 0;
};

ProcessGroup* downcast(const c10::intrusive_ptr<c10d::ProcessGroup>& pg) {
  auto* p = dynamic_cast<ProcessGroup*>(pg.get());
  if (!p) {
    throw std::runtime_error("moodist: not a moodist process group");
  }
  return p;
}

// ---- compile_op_full -> CustomOp -> Future ----

struct FutureObj {
  moodist_future* f = nullptr;
  std::vector<at::Tensor> hold; // inputs and outputs stay alive until the future dies (core/processgroup.cc:3239-3245)
  std::vector<at::Tensor> outputs;
  void* stream = nullptr;
  ~FutureObj() {
    if (f) {
      core.moodist_future_destroy(f);
    }
  }
  void wait() {
    py::gil_scoped_release nogil; // wrapper/module.cc:1211-1214
    check(core.moodist_future_wait(f, stream));
  }
  std::vector<at::Tensor> result() {
    wait();
    return outputs;
  }
};

struct CustomOpObj {
  moodist_op* op = nullptr;
  size_t ndim = 0;
  c10::intrusive_ptr<c10d::ProcessGroup> pg; // keeps the group (and its world) alive
  ~CustomOpObj() {
    if (op) {
      core.moodist_op_destroy(op);
    }
  }

  std::shared_ptr<FutureObj> call(std::vector<at::Tensor> inputs, std::vector<at::Tensor> outputs) {
    std::vector<moodist_tensor> in, out;
    void* stream = nullptr;
    for (const at::Tensor& t : inputs) {
      in.push_back(describe(t));
      if (t.is_cuda()) {
        stream = stream_of(t);
      }
    }
    for (const at::Tensor& t : outputs) {
      out.push_back(describe(t));
      if (t.is_cuda()) {
        stream = stream_of(t);
      }
    }
    // a rank that passes no device tensor (a bystander) launches nothing, so it needs no stream
    auto fut = std::make_shared<FutureObj>();
    fut->stream = stream;
    {
      py::gil_scoped_release nogil; // wrapper/module.cc:1286-1290
      check(core.moodist_op_call(op, in.data(), in.size(), out.data(), out.size(), stream, &fut->f));
    }
    fut->outputs = outputs;
    fut->hold = std::move(inputs);
    fut->hold.insert(fut->hold.end(), outputs.begin(), outputs.end());
    return fut;
  }

  py::dict plan() const {
    py::dict d;
    py::list reads, sizes_in, sizes_out;
    for (int64_t i = 0, n = core.moodist_op_plan_count(op, 0); i < n; ++i) {
      int64_t r[6];
      check(core.moodist_op_plan_read(op, (size_t)i, r));
      reads.append(py::make_tuple(r[0], r[1], r[2], r[3], r[4], r[5]));
    }
    auto copies = [&](int which) {
      py::list l;
      for (int64_t i = 0, n = core.moodist_op_plan_count(op, which); i < n; ++i) {
        int64_t buf[1 + 2 * 10];
        check(core.moodist_op_plan_copy(op, which, (size_t)i, buf, 21));
        l.append(py::make_tuple(buf[0], std::vector<int64_t>(buf + 1, buf + 1 + ndim),
            std::vector<int64_t>(buf + 1 + ndim, buf + 1 + 2 * ndim)));
      }
      return l;
    };
    for (int64_t i = 0, n = core.moodist_op_plan_count(op, 3); i < n; ++i) {
      sizes_in.append(core.moodist_op_plan_size(op, 3, (size_t)i));
    }
    for (int64_t i = 0, n = core.moodist_op_plan_count(op, 4); i < n; ++i) {
      sizes_out.append(core.moodist_op_plan_size(op, 4, (size_t)i));
    }
    d["reads"] = reads;
    d["inputCopies"] = copies(1);
    d["outputCopies"] = copies(2);
    d["inputs"] = sizes_in;
    d["outputs"] = sizes_out;
    // what this rank sends each receiver during compile, in the reference's byte format
    py::list messages;
    for (int receiver = 0;; ++receiver) {
      const int64_t n = core.moodist_op_plan_message(op, receiver, nullptr, 0);
      if (n < 0) {
        break;
      }
      std::string bytes((size_t)n, '\0');
      core.moodist_op_plan_message(op, receiver, bytes.data(), bytes.size());
      messages.append(py::bytes(bytes));
    }
    d["messages"] = messages;
    return d;
  }
};

using Spec = std::tuple<int, std::vector<int>, std::vector<int>>;

// wrapper/processgroup_wrapper.cc:349-383: flatten to int arrays for the core
std::shared_ptr<CustomOpObj> compile_op_full(const c10::intrusive_ptr<c10d::ProcessGroup>& pg, std::vector<int> shape,
    at::ScalarType dtype, const std::vector<Spec>& inputs, const std::vector<Spec>& outputs) {
  const size_t ndim = shape.size();
  auto flatten = [&](const std::vector<Spec>& specs, std::vector<int>& ranks, std::vector<int>& offs,
                     std::vector<int>& shapes) {
    for (const Spec& s : specs) {
      if (std::get<1>(s).size() != ndim || std::get<2>(s).size() != ndim) {
        throw std::runtime_error("moodist.compile_op_full: offset/shape dimension mismatch");
      }
      ranks.push_back(std::get<0>(s));
      offs.insert(offs.end(), std::get<1>(s).begin(), std::get<1>(s).end());
      shapes.insert(shapes.end(), std::get<2>(s).begin(), std::get<2>(s).end());
    }
  };
  std::vector<int> ir, io, is, orr, oo, os;
  flatten(inputs, ir, io, is);
  flatten(outputs, orr, oo, os);
  auto obj = std::make_shared<CustomOpObj>();
  obj->pg = pg;
  obj->ndim = ndim;
  {
    py::gil_scoped_release nogil; // wrapper/module.cc:793-796
    check(core.moodist_compile_op_full(downcast(pg)->handle(), shape.data(), ndim, (int)dtype, ir.data(), io.data(),
        is.data(), ir.size(), orr.data(), oo.data(), os.data(), orr.size(), &obj->op));
  }
  return obj;
}

} // namespace

PYBIND11_MODULE(_C, m) {
  load_core();

  py::class_<WorldHolder, std::shared_ptr<WorldHolder>>(m, "World")
      .def(py::init([](int size, int device) {
        auto w = std::make_shared<WorldHolder>();
        w->size = size;
        w->device = device;
        check(core.moodist_world_create(size, device, &w->world));
        return w;
      }),
          py::arg("size"), py::arg("device") = 0)
      .def_readonly("size", &WorldHolder::size)
      .def_readonly("device", &WorldHolder::device);

  // Returned as the torch.distributed.ProcessGroup it derives from, so that c10d's own Python
  // bindings (rank, size, _allgather_base, _reduce_scatter_base, allreduce, ...) reach the
  // overrides above through the virtual table.
  m.def("create_process_group", [](std::shared_ptr<WorldHolder> world, int rank) {
    return c10::intrusive_ptr<c10d::ProcessGroup>(c10::make_intrusive<ProcessGroup>(std::move(world), rank));
  });
  m.def("moodist_name", [](const c10::intrusive_ptr<c10d::ProcessGroup>& pg) {
    return "moodist-local-" + std::to_string(downcast(pg)->getRank()) + "-of-" + std::to_string(pg->getSize());
  });
  m.def("get_option", [](const c10::intrusive_ptr<c10d::ProcessGroup>& pg, const std::string& name) {
    int64_t v = 0;
    check(core.moodist_pg_get_option(downcast(pg)->handle(), name.c_str(), &v));
    return v;
  });
  m.def("set_option", [](const c10::intrusive_ptr<c10d::ProcessGroup>& pg, const std::string& name, int64_t value) {
    check(core.moodist_pg_set_option(downcast(pg)->handle(), name.c_str(), value));
  });
  m.def("stage_input",
      [](const c10::intrusive_ptr<c10d::ProcessGroup>& pg, const std::string& kind, at::Tensor input, int reduce_op,
          float premul) { return downcast(pg)->stage_input(kind, input, reduce_op, premul); },
      py::arg("pg"), py::arg("kind"), py::arg("input"), py::arg("reduce_op") = 0, py::arg("premul") = 0.0f);
  m.def("compile_op_full", &compile_op_full);

  py::class_<CustomOpObj, std::shared_ptr<CustomOpObj>>(m, "CustomOp")
      .def("__call__", &CustomOpObj::call, py::arg("inputs"), py::arg("outputs"))
      .def("plan", &CustomOpObj::plan);
  py::class_<FutureObj, std::shared_ptr<FutureObj>>(m, "Future")
      .def("wait", &FutureObj::wait)
      .def("result", &FutureObj::result);
}
