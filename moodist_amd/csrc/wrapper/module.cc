// Python module on PyTorch-ROCm: MoodistProcessGroup, a torch.distributed.ProcessGroup whose
// collectives run the hot path of the host core (libmoodist.so) on the caller's current HIP
// stream.
//
// The core is loaded the way the reference's wrapper loads it (wrapper/moodist_loader.cc:363-386):
// dlopen, ONE symbol -- moodistGetApi -- called with this module's API version and a table of
// torch-backed callbacks, a NULL answer or a wrong build magic refused.  Everything the
// reference's table has is called through the table; the few things it has no slot for (a
// peer that only contributes, the list form of all_gather, plan inspection, launch status)
// use the core's plain C functions.
//
// Mirrors the reference's wrapper otherwise: the c10d virtuals _allgather_base,
// _reduce_scatter_base, allreduce and the coalesced variants
// (wrapper/processgroup_wrapper.cc:131-190), compile_op_full -> CustomOp -> Future
// (wrapper/processgroup_wrapper.cc:349-444; wrapper/module.cc:689-804, :1240-1305), option
// access (wrapper/module.cc:836-848), the unsupported point-to-point calls
// (wrapper/processgroup_wrapper.h:168-185), and the Python type itself: a subclass of
// torch.distributed.ProcessGroup built from (store, rank, size) (wrapper/module.cc:547-566,
// :851-865).
#include <dlfcn.h>

#include <c10/hip/HIPCachingAllocator.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/csrc/distributed/c10d/ProcessGroup.hpp>
#include <torch/csrc/distributed/c10d/Store.hpp>
#include <torch/csrc/distributed/c10d/Work.hpp>
#include <torch/extension.h>

#include <memory>
#include <mutex>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

#include "moodist_core.h"
#include "moodist_plugin.h"

namespace py = pybind11;

namespace moodist {

// The tensor the core sees: opaque there, a torch tensor plus its count here
// (wrapper/moodist_loader.cc:27-35).
struct Tensor : ApiRefCounted {
  at::Tensor tensor;
  explicit Tensor(at::Tensor t) : tensor(std::move(t)) {
    refcount.store(1, std::memory_order_relaxed);
  }
};

namespace {

CoreApi* core = nullptr;

// the core's plain C functions used beside the table
struct CoreExtras {
#define MOODIST_EXTRA(name) decltype(&::name) name = nullptr;
  MOODIST_EXTRA(moodistGroupCHandle)
  MOODIST_EXTRA(moodistOpCHandle)
  MOODIST_EXTRA(moodist_last_error)
  MOODIST_EXTRA(moodist_pg_all_gather_list)
  MOODIST_EXTRA(moodist_pg_all_gather_many)
  MOODIST_EXTRA(moodist_pg_allreduce_many)
  MOODIST_EXTRA(moodist_pg_reduce_scatter_many)
  MOODIST_EXTRA(moodist_pg_stage_input)
  MOODIST_EXTRA(moodist_pg_last_work)
  MOODIST_EXTRA(moodist_pg_keep_alive)
  MOODIST_EXTRA(moodist_work_is_completed)
  MOODIST_EXTRA(moodist_work_wait)
  MOODIST_EXTRA(moodist_work_destroy)
  MOODIST_EXTRA(moodist_op_plan_count)
  MOODIST_EXTRA(moodist_op_plan_read)
  MOODIST_EXTRA(moodist_op_plan_copy)
  MOODIST_EXTRA(moodist_op_plan_size)
  MOODIST_EXTRA(moodist_op_plan_message)
#undef MOODIST_EXTRA
} extra;

void check(int rc) {
  if (rc != 0) {
    throw std::runtime_error(extra.moodist_last_error());
  }
}

// ---- WrapperApi: what the core may ask of torch (api/moodist_api.h:61-128) ----

at::TensorOptions options_for(DType dtype, int device) {
  auto o = at::TensorOptions().dtype(static_cast<at::ScalarType>(static_cast<int>(dtype)));
  return device < 0 ? o.device(at::kCPU) : o.device(at::kCUDA, (c10::DeviceIndex)device);
}

std::mutex stores_mutex;
std::set<void*> real_stores; // store arguments that are c10d::Store objects

c10d::Store* as_store(void* store) {
  std::lock_guard<std::mutex> l(stores_mutex);
  if (!real_stores.count(store)) {
    throw std::runtime_error("moodist: this group was not built on a torch.distributed.Store");
  }
  return static_cast<c10d::Store*>(store);
}

WrapperApi make_wrapper_api() {
  WrapperApi w{};
  w.cudaCurrentDevice = []() -> int { return c10::hip::device_count() > 0 ? (int)c10::hip::current_device() : 0; };
  w.cudaGetCurrentStream = []() -> Stream { return c10::hip::getCurrentHIPStream().stream(); };
  w.cudaStreamGuardEnter = [](Stream stream, int device) -> void* {
    return new c10::hip::HIPStreamGuard(c10::hip::getStreamFromExternal(stream, (c10::DeviceIndex)device));
  };
  w.cudaStreamGuardExit = [](void* guard) { delete static_cast<c10::hip::HIPStreamGuard*>(guard); };
  w.cudaCachingAllocatorAlloc = [](size_t bytes, void** cleanup) -> void* {
    auto* held = new c10::DataPtr(c10::hip::HIPCachingAllocator::get()->allocate(bytes));
    *cleanup = held;
    return held->get();
  };
  w.cudaCachingAllocatorFree = [](void* cleanup) { delete static_cast<c10::DataPtr*>(cleanup); };

  w.tensorFromBlob = [](void* data, const int64_t* sizes, int ndim, DType dtype, int device) {
    return new Tensor(at::from_blob(data, at::IntArrayRef(sizes, (size_t)ndim), options_for(dtype, device)));
  };
  w.tensorEmpty = [](const int64_t* sizes, int ndim, DType dtype, int device) {
    return new Tensor(at::empty(at::IntArrayRef(sizes, (size_t)ndim), options_for(dtype, device)));
  };
  w.tensorFromBlobWithDeleter = [](void* data, const int64_t* sizes, int ndim, DType dtype, int device,
                                    void (*deleter)(void*), void* ctx) {
    return new Tensor(at::from_blob(
        data, at::IntArrayRef(sizes, (size_t)ndim), [deleter, ctx](void*) { deleter(ctx); }, options_for(dtype, device)));
  };
  w.tensorAddRef = [](Tensor* t) { t->refcount.fetch_add(1, std::memory_order_relaxed); };
  w.tensorDecRef = [](Tensor* t) {
    if (t->refcount.fetch_sub(1, std::memory_order_acq_rel) == 1) {
      delete t;
    }
  };

  w.tensorDataPtr = [](Tensor* t) -> void* { return t->tensor.data_ptr(); };
  w.tensorNumel = [](Tensor* t) -> int64_t { return t->tensor.numel(); };
  w.tensorNdim = [](Tensor* t) -> int64_t { return t->tensor.dim(); };
  w.tensorSize = [](Tensor* t, int64_t d) -> int64_t { return t->tensor.size(d); };
  w.tensorStride = [](Tensor* t, int64_t d) -> int64_t { return t->tensor.stride(d); };
  w.tensorDtype = [](Tensor* t) -> DType { return static_cast<DType>(static_cast<int>(t->tensor.scalar_type())); };
  w.tensorDevice = [](Tensor* t) -> int { return t->tensor.is_cuda() ? (int)t->tensor.device().index() : -1; };
  w.tensorIsContiguous = [](Tensor* t) -> bool { return t->tensor.is_contiguous(); };
  w.tensorIsCuda = [](Tensor* t) -> bool { return t->tensor.is_cuda(); };
  w.tensorIsCpu = [](Tensor* t) -> bool { return t->tensor.is_cpu(); };
  w.tensorItemsize = [](Tensor* t) -> int64_t { return (int64_t)t->tensor.element_size(); };

  w.tensorView = [](Tensor* t, const int64_t* sizes, int ndim) {
    return new Tensor(t->tensor.view(at::IntArrayRef(sizes, (size_t)ndim)));
  };
  w.tensorNarrow = [](Tensor* t, int dim, int64_t start, int64_t length) {
    return new Tensor(t->tensor.narrow(dim, start, length));
  };
  w.tensorContiguous = [](Tensor* t) { return new Tensor(t->tensor.contiguous()); };
  w.tensorMulScalar = [](Tensor* t, double s) { return new Tensor(t->tensor * s); };
  w.tensorMulScalar_ = [](Tensor* t, double s) { t->tensor.mul_(s); };
  w.tensorRecordStream = [](Tensor* t, Stream stream) {
    if (t->tensor.is_cuda()) {
      c10::hip::HIPCachingAllocator::recordStream(t->tensor.storage().data_ptr(),
          c10::hip::getStreamFromExternal(stream, t->tensor.device().index()));
    }
  };
  w.tensorCopy_ = [](Tensor* dst, Tensor* src) { dst->tensor.copy_(src->tensor); };
  w.tensorSumOut = [](Tensor* dst, Tensor* src, int dim) { at::sum_out(dst->tensor, src->tensor, {dim}); };
  w.tensorAmaxOut = [](Tensor* dst, Tensor* src, int dim) { at::amax_out(dst->tensor, src->tensor, {dim}); };
  w.tensorAminOut = [](Tensor* dst, Tensor* src, int dim) { at::amin_out(dst->tensor, src->tensor, {dim}); };

  w.dtypeSize = [](DType dtype) -> size_t { return c10::elementSize(static_cast<at::ScalarType>(static_cast<int>(dtype))); };
  w.registerFreeMemoryCallback = []() {};

  w.c10dStoreSet = [](void* store, std::string_view key, const std::vector<uint8_t>& value) {
    as_store(store)->set(std::string(key), value);
  };
  w.c10dStoreGet = [](void* store, std::string_view key) { return as_store(store)->get(std::string(key)); };
  w.c10dStoreWait = [](void* store, std::span<const std::string> keys) {
    as_store(store)->wait(std::vector<std::string>(keys.begin(), keys.end()));
  };
  w.checkSignals = []() {
    py::gil_scoped_acquire gil;
    if (PyErr_CheckSignals() != 0) {
      throw py::error_already_set();
    }
  };
  return w;
}

WrapperApi wrapper_api = make_wrapper_api();

// ---- loading the core (wrapper/moodist_loader.cc:363-386) ----

struct CoreInfo {
  std::string path;
  uint32_t version = 0;
  uint64_t magic = 0;
} core_info;

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
  auto get_api = reinterpret_cast<decltype(&::moodistGetApi)>(dlsym(lib, "moodistGetApi"));
  if (!get_api) {
    throw std::runtime_error("moodist: " + path + " has no symbol moodistGetApi");
  }
  core = get_api(kMoodistApiVersion, &wrapper_api);
  if (!core) {
    throw std::runtime_error("moodist: API version mismatch - libmoodist.so does not speak version " +
                             std::to_string(kMoodistApiVersion) + " of the core API");
  }
  if (core->magic != kMoodistBuildMagic) {
    throw std::runtime_error("moodist: build magic mismatch - libmoodist.so and _C are from different builds");
  }
  core_info.path = path;
  core_info.version = kMoodistApiVersion;
  core_info.magic = core->magic;
#define MOODIST_EXTRA(name)                                                    \
  extra.name = reinterpret_cast<decltype(extra.name)>(dlsym(lib, #name));      \
  if (!extra.name) {                                                           \
    throw std::runtime_error("moodist: libmoodist.so has no symbol " #name); \
  }
  MOODIST_EXTRA(moodistGroupCHandle)
  MOODIST_EXTRA(moodistOpCHandle)
  MOODIST_EXTRA(moodist_last_error)
  MOODIST_EXTRA(moodist_pg_all_gather_list)
  MOODIST_EXTRA(moodist_pg_all_gather_many)
  MOODIST_EXTRA(moodist_pg_allreduce_many)
  MOODIST_EXTRA(moodist_pg_reduce_scatter_many)
  MOODIST_EXTRA(moodist_pg_stage_input)
  MOODIST_EXTRA(moodist_pg_last_work)
  MOODIST_EXTRA(moodist_pg_keep_alive)
  MOODIST_EXTRA(moodist_work_is_completed)
  MOODIST_EXTRA(moodist_work_wait)
  MOODIST_EXTRA(moodist_work_destroy)
  MOODIST_EXTRA(moodist_op_plan_count)
  MOODIST_EXTRA(moodist_op_plan_read)
  MOODIST_EXTRA(moodist_op_plan_copy)
  MOODIST_EXTRA(moodist_op_plan_size)
  MOODIST_EXTRA(moodist_op_plan_message)
#undef MOODIST_EXTRA
}

// A torch tensor wrapped for one call into the core; the core takes its own references on
// what it keeps (tensorAddRef), so the wrapper can go when the call returns.
struct Wrapped {
  TensorPtr ptr;
  explicit Wrapped(const at::Tensor& t) : ptr(new Tensor(t)) {}
  Wrapped(const Wrapped&) = delete;
  Wrapped& operator=(const Wrapped&) = delete;
  ~Wrapped() {
    if (Tensor* p = ptr.release()) {
      wrapper_api.tensorDecRef(p);
    }
  }
};

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
Stream stream_of(const at::Tensor& t) {
  return t.is_cuda() ? c10::hip::getCurrentHIPStream(t.device().index()).stream() : nullptr;
}

ReduceOp reduce_op_code(const c10d::ReduceOp& op) {
  switch (static_cast<int>(op.op_)) {
  case c10d::ReduceOp::SUM:
  case c10d::ReduceOp::AVG:
  case c10d::ReduceOp::PRODUCT:
  case c10d::ReduceOp::MIN:
  case c10d::ReduceOp::MAX:
  case c10d::ReduceOp::PREMUL_SUM:
    return static_cast<ReduceOp>(static_cast<int>(op.op_)); // the core refuses PRODUCT, as the reference's does
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
      extra.moodist_work_destroy(w);
    }
  }
  void synchronize() override {}
  bool wait(std::chrono::milliseconds = std::chrono::milliseconds(0)) override {
    for (moodist_work* w : parts) {
      check(extra.moodist_work_wait(w));
    }
    return true;
  }
  bool isCompleted() override {
    for (moodist_work* w : parts) {
      if (!extra.moodist_work_is_completed(w)) {
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

void release_tensors(void* ctx) {
  delete static_cast<std::vector<at::Tensor>*>(ctx);
}

// ---- the process group ----

class ProcessGroup : public c10d::ProcessGroup {
public:
  // `store_key` identifies the group's world: ranks created with the same key are peers.
  ProcessGroup(void* store_key, py::object store_ref, int rank, int size)
      : c10d::ProcessGroup(rank, size), store_ref_(std::move(store_ref)),
        handle_(core->createProcessGroup(store_key, rank, size)), c_(extra.moodistGroupCHandle(handle_.get())) {}

  ~ProcessGroup() override {
    handle_.drop();
    // the store object outlives the group: its address is the world's key
    py::gil_scoped_acquire gil;
    store_ref_ = py::object();
  }

  const std::string getBackendName() const override {
    return "moodist";
  }

  c10::intrusive_ptr<c10d::Work> _allgather_base(at::Tensor& output, at::Tensor& input,
      const c10d::AllgatherOptions& = c10d::AllgatherOptions()) override {
    Wrapped o(output), i(input);
    core->processGroupAllGather(handle_.get(), o.ptr, i.ptr, stream_of(input));
    return work({output});
  }

  // wrapper/processgroup_wrapper.cc:112-129; here every source goes straight into its output
  // tensor (moodist_pg_all_gather_list), so no flat temporary exists
  c10::intrusive_ptr<c10d::Work> allgather(std::vector<std::vector<at::Tensor>>& outputLists,
      std::vector<at::Tensor>& inputs, const c10d::AllgatherOptions& = c10d::AllgatherOptions()) override {
    TORCH_CHECK(outputLists.size() == 1 && inputs.size() == 1);
    std::vector<moodist_tensor> outs;
    for (at::Tensor& t : outputLists[0]) {
      outs.push_back(describe(t));
    }
    moodist_tensor i = describe(inputs[0]);
    auto result = c10::make_intrusive<WorkImpl>();
    moodist_work* w = nullptr;
    check(extra.moodist_pg_all_gather_list(c_, outs.data(), outs.size(), &i, stream_of(inputs[0]), &w));
    result->parts.push_back(w);
    auto held = new std::vector<at::Tensor>(outputLists[0]);
    held->push_back(inputs[0]);
    // the core owns `held` from the call on and releases it exactly once, also when it fails
    check(extra.moodist_pg_keep_alive(c_, held, release_tensors));
    result->tensors = outputLists[0];
    return result;
  }

  c10::intrusive_ptr<c10d::Work> _reduce_scatter_base(at::Tensor& output, at::Tensor& input,
      const c10d::ReduceScatterOptions& opts = c10d::ReduceScatterOptions()) override {
    Wrapped o(output), i(input);
    core->processGroupReduceScatter(handle_.get(), o.ptr, i.ptr, reduce_op_code(opts.reduceOp), stream_of(input),
        premul_value(opts.reduceOp, input.scalar_type()));
    return work({output});
  }

  // wrapper/processgroup_wrapper.cc:139-148 loops over the tensors; here a list of two or more
  // is one collective whose copies share launches (moodist_pg_all_gather_many)
  c10::intrusive_ptr<c10d::Work> allgather_into_tensor_coalesced(std::vector<at::Tensor>& outputs,
      std::vector<at::Tensor>& inputs, const c10d::AllgatherOptions& = c10d::AllgatherOptions()) override {
    TORCH_CHECK(outputs.size() == inputs.size());
    auto result = c10::make_intrusive<WorkImpl>();
    if (inputs.size() < 2) {
      for (size_t k = 0; k < inputs.size(); ++k) {
        Wrapped o(outputs[k]), i(inputs[k]);
        core->processGroupAllGather(handle_.get(), o.ptr, i.ptr, stream_of(inputs[k]));
        add_last(*result);
      }
      result->tensors = outputs;
      return result;
    }
    std::vector<moodist_tensor> outs, ins;
    for (size_t k = 0; k < inputs.size(); ++k) {
      outs.push_back(describe(outputs[k]));
      ins.push_back(describe(inputs[k]));
    }
    moodist_work* w = nullptr;
    check(extra.moodist_pg_all_gather_many(c_, outs.data(), ins.data(), ins.size(), stream_of(inputs[0]), &w));
    result->parts.push_back(w);
    auto held = new std::vector<at::Tensor>(outputs);
    held->insert(held->end(), inputs.begin(), inputs.end());
    // the core owns `held` from the call on and releases it exactly once, also when it fails
    check(extra.moodist_pg_keep_alive(c_, held, release_tensors));
    result->tensors = outputs;
    return result;
  }

  // wrapper/processgroup_wrapper.cc:159-170 loops over the tensors; here a list of two or more of
  // one element type is one collective whose reductions share launches
  // (moodist_pg_reduce_scatter_many)
  c10::intrusive_ptr<c10d::Work> reduce_scatter_tensor_coalesced(std::vector<at::Tensor>& outputs,
      std::vector<at::Tensor>& inputs, const c10d::ReduceScatterOptions& opts = c10d::ReduceScatterOptions()) override {
    TORCH_CHECK(outputs.size() == inputs.size());
    auto result = c10::make_intrusive<WorkImpl>();
    bool one_type = inputs.size() >= 2;
    for (size_t k = 1; k < inputs.size(); ++k) {
      one_type = one_type && inputs[k].scalar_type() == inputs[0].scalar_type();
    }
    if (!one_type) {
      for (size_t k = 0; k < inputs.size(); ++k) {
        Wrapped o(outputs[k]), i(inputs[k]);
        core->processGroupReduceScatter(handle_.get(), o.ptr, i.ptr, reduce_op_code(opts.reduceOp),
            stream_of(inputs[k]), premul_value(opts.reduceOp, inputs[k].scalar_type()));
        add_last(*result);
      }
      result->tensors = outputs;
      return result;
    }
    std::vector<moodist_tensor> outs, ins;
    for (size_t k = 0; k < inputs.size(); ++k) {
      outs.push_back(describe(outputs[k]));
      ins.push_back(describe(inputs[k]));
    }
    moodist_work* w = nullptr;
    check(extra.moodist_pg_reduce_scatter_many(c_, outs.data(), ins.data(), ins.size(),
        static_cast<int>(reduce_op_code(opts.reduceOp)), stream_of(inputs[0]),
        premul_value(opts.reduceOp, inputs[0].scalar_type()), &w));
    result->parts.push_back(w);
    auto held = new std::vector<at::Tensor>(outputs);
    held->insert(held->end(), inputs.begin(), inputs.end());
    // the core owns `held` from the call on and releases it exactly once, also when it fails
    check(extra.moodist_pg_keep_alive(c_, held, release_tensors));
    result->tensors = outputs;
    return result;
  }

  // wrapper/processgroup_wrapper.cc:172-190; the padded temporary of a size that does not
  // divide by the group size is the core's business (core/processgroup.cc:1694-1697)
  c10::intrusive_ptr<c10d::Work> allreduce(std::vector<at::Tensor>& tensors,
      const c10d::AllreduceOptions& opts = c10d::AllreduceOptions()) override {
    TORCH_CHECK(tensors.size() == 1);
    auto result = c10::make_intrusive<WorkImpl>();
    allreduce_one(tensors[0], opts.reduceOp, *result);
    result->tensors = tensors;
    return result;
  }

  // wrapper/processgroup_wrapper.cc:182-191
  c10::intrusive_ptr<c10d::Work> allreduce_coalesced(std::vector<at::Tensor>& tensors,
      const c10d::AllreduceCoalescedOptions& opts = c10d::AllreduceCoalescedOptions()) override {
    auto result = c10::make_intrusive<WorkImpl>();
    // The tensors that need no padded temporary -- element count a multiple of the group size,
    // element type that of the first such tensor -- are reduced and gathered as two collectives
    // for the whole set (moodist_pg_allreduce_many); the others take one allreduce each, as in
    // the reference, in list order.  What decides membership is the same on every rank (sizes
    // and element types, which the ranks' lists must share), never a property of one rank's
    // tensor: a tensor that is not contiguous is refused before anything is posted, on every
    // path, as the core refuses it (core/processgroup.cc:1062-1063).
    for (at::Tensor& t : tensors) {
      if (!t.is_contiguous()) {
        throw std::runtime_error("moodist: allreduce tensor must be contiguous");
      }
    }
    std::vector<at::Tensor> together;
    for (at::Tensor& t : tensors) {
      if (t.numel() > 0 && t.numel() % getSize() == 0 &&
          (together.empty() || t.scalar_type() == together[0].scalar_type())) {
        together.push_back(t);
      }
    }
    if (together.size() < 2) {
      together.clear();
    }
    if (!together.empty()) {
      std::vector<moodist_tensor> descs;
      for (at::Tensor& t : together) {
        descs.push_back(describe(t));
      }
      moodist_work* w = nullptr;
      check(extra.moodist_pg_allreduce_many(c_, descs.data(), descs.size(), static_cast<int>(reduce_op_code(opts.reduceOp)),
          stream_of(together[0]), premul_value(opts.reduceOp, together[0].scalar_type()), &w));
      result->parts.push_back(w);
      // the core owns the list from the call on and releases it exactly once, also when it fails
      check(extra.moodist_pg_keep_alive(c_, new std::vector<at::Tensor>(together), release_tensors));
    }
    for (at::Tensor& t : tensors) {
      bool done = false;
      for (const at::Tensor& u : together) {
        done = done || u.is_same(t);
      }
      if (!done) {
        allreduce_one(t, opts.reduceOp, *result);
      }
    }
    result->tensors = tensors;
    return result;
  }

  c10::intrusive_ptr<c10d::Work> barrier(const c10d::BarrierOptions& = c10d::BarrierOptions()) override {
    core->processGroupBarrier(handle_.get());
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

  api::ProcessGroup* handle() const {
    return handle_.get();
  }

  // unique among the groups of this process, as the reference's names are among its groups
  std::string moodist_name() const {
    char world[32];
    std::snprintf(world, sizeof(world), "%zx", (size_t)store_ref_.ptr());
    return "moodist-local-" + std::to_string(getRank()) + "-of-" + std::to_string(getSize()) + "-world" + world;
  }
  py::object store() const {
    return store_ref_;
  }
  int64_t get_option(const std::string& name) const {
    return core->processGroupGetOption(handle_.get(), name.c_str());
  }
  void set_option(const std::string& name, int64_t value) {
    core->processGroupSetOption(handle_.get(), name.c_str(), value);
  }
  bool get_prefer_kernel_less() const {
    return core->processGroupGetPreferKernelLess(handle_.get());
  }
  void set_prefer_kernel_less(bool value) {
    core->processGroupSetPreferKernelLess(handle_.get(), value);
  }
  void cuda_barrier() {
    core->processGroupCudaBarrier(handle_.get(), c10::hip::device_count() > 0 ? c10::hip::getCurrentHIPStream().stream() : nullptr);
  }

  // A peer that only contributes: its buffer is the staged contribution of that rank.
  c10::intrusive_ptr<c10d::Work> stage_input(const std::string& kind, at::Tensor& input, int reduce_op, float premul) {
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
    check(extra.moodist_pg_stage_input(c_, k, &i, reduce_op, stream_of(input), premul, &w));
    check(extra.moodist_pg_keep_alive(c_, new std::vector<at::Tensor>{input}, release_tensors));
    auto result = c10::make_intrusive<WorkImpl>();
    result->parts.push_back(w);
    return result;
  }

private:
  // the collective this rank has just posted through the table, as a Work
  void add_last(WorkImpl& into) {
    moodist_work* w = nullptr;
    check(extra.moodist_pg_last_work(c_, &w));
    if (w) {
      into.parts.push_back(w);
    }
  }
  c10::intrusive_ptr<c10d::Work> work(std::vector<at::Tensor> tensors) {
    auto result = c10::make_intrusive<WorkImpl>();
    add_last(*result);
    result->tensors = std::move(tensors);
    return result;
  }
  void allreduce_one(at::Tensor& t, const c10d::ReduceOp& op, WorkImpl& into) {
    Wrapped w(t);
    core->processGroupAllreduce(handle_.get(), w.ptr, reduce_op_code(op), stream_of(t), premul_value(op, t.scalar_type()));
    add_last(into);
  }

  py::object store_ref_;
  api::ProcessGroupHandle handle_;
  moodist_pg* c_;
};

// ---- compile_op_full -> CustomOp -> Future ----

struct FutureObj {
  api::FutureHandle handle;
  std::vector<at::Tensor> outputs;
  Stream stream = nullptr;
  void wait() {
    py::gil_scoped_release nogil; // wrapper/module.cc:1211-1214
    core->futureWait(handle.get(), stream);
  }
  std::vector<at::Tensor> result() {
    wait();
    return outputs;
  }
};

struct CustomOpObj {
  api::CustomOpHandle handle;
  size_t ndim = 0;
  c10::intrusive_ptr<ProcessGroup> pg; // keeps the group (and its world) alive

  std::shared_ptr<FutureObj> call(std::vector<at::Tensor> inputs, std::vector<at::Tensor> outputs) {
    std::vector<std::unique_ptr<Wrapped>> wrapped;
    std::vector<TensorPtr> in, out;
    Stream stream = nullptr;
    auto wrap = [&](const at::Tensor& t, std::vector<TensorPtr>& list) {
      wrapped.push_back(std::make_unique<Wrapped>(t));
      list.push_back(TensorPtr(wrapped.back()->ptr.get()));
      if (t.is_cuda()) {
        stream = stream_of(t);
      }
    };
    for (const at::Tensor& t : inputs) {
      wrap(t, in);
    }
    for (const at::Tensor& t : outputs) {
      wrap(t, out);
    }
    // a rank that passes no device tensor (a bystander) launches nothing, so it needs no stream
    auto fut = std::make_shared<FutureObj>();
    fut->stream = stream;
    {
      py::gil_scoped_release nogil; // wrapper/module.cc:1286-1290
      fut->handle = core->customOpCall(handle.get(), in.data(), in.size(), out.data(), out.size(), stream);
    }
    fut->outputs = std::move(outputs);
    return fut;
  }

  py::dict plan() const {
    moodist_op* op = extra.moodistOpCHandle(handle.get());
    py::dict d;
    py::list reads, sizes_in, sizes_out;
    for (int64_t i = 0, n = extra.moodist_op_plan_count(op, 0); i < n; ++i) {
      int64_t r[6];
      check(extra.moodist_op_plan_read(op, (size_t)i, r));
      reads.append(py::make_tuple(r[0], r[1], r[2], r[3], r[4], r[5]));
    }
    auto copies = [&](int which) {
      py::list l;
      for (int64_t i = 0, n = extra.moodist_op_plan_count(op, which); i < n; ++i) {
        int64_t buf[1 + 2 * 10];
        check(extra.moodist_op_plan_copy(op, which, (size_t)i, buf, 21));
        l.append(py::make_tuple(buf[0], std::vector<int64_t>(buf + 1, buf + 1 + ndim),
            std::vector<int64_t>(buf + 1 + ndim, buf + 1 + 2 * ndim)));
      }
      return l;
    };
    for (int64_t i = 0, n = extra.moodist_op_plan_count(op, 3); i < n; ++i) {
      sizes_in.append(extra.moodist_op_plan_size(op, 3, (size_t)i));
    }
    for (int64_t i = 0, n = extra.moodist_op_plan_count(op, 4); i < n; ++i) {
      sizes_out.append(extra.moodist_op_plan_size(op, 4, (size_t)i));
    }
    d["reads"] = reads;
    d["inputCopies"] = copies(1);
    d["outputCopies"] = copies(2);
    d["inputs"] = sizes_in;
    d["outputs"] = sizes_out;
    // what this rank sends each receiver during compile, in the reference's byte format
    py::list messages;
    for (int receiver = 0;; ++receiver) {
      const int64_t n = extra.moodist_op_plan_message(op, receiver, nullptr, 0);
      if (n < 0) {
        break;
      }
      std::string bytes((size_t)n, '\0');
      extra.moodist_op_plan_message(op, receiver, bytes.data(), bytes.size());
      messages.append(py::bytes(bytes));
    }
    d["messages"] = messages;
    return d;
  }
};

using Spec = std::tuple<int, std::vector<int>, std::vector<int>>;

// wrapper/processgroup_wrapper.cc:349-383: flatten to int arrays for the core
std::shared_ptr<CustomOpObj> compile_op_full(const c10::intrusive_ptr<ProcessGroup>& pg, std::vector<int> shape,
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
    obj->handle = core->compileOpFull(pg->handle(), shape.data(), ndim, static_cast<DType>(static_cast<int>(dtype)),
        ir.data(), io.data(), is.data(), ir.size(), orr.data(), oo.data(), os.data(), orr.size());
  }
  return obj;
}

} // namespace

// This side's "who drops the last reference destroys" (api/api_handle.h:168-174;
// wrapper/processgroup_wrapper.cc:100-104, :479-490): back through the table.
namespace api {
void destroy(Future* f) {
  core->futureDestroy(f);
}
void destroy(CustomOp* op) {
  core->customOpDestroy(op);
}
void destroy(ProcessGroup* pg) {
  core->processGroupDestroy(pg);
}
} // namespace api

} // namespace moodist

PYBIND11_MODULE(_C, m) {
  using namespace moodist;
  load_core();

  m.def("core_api_info", []() {
    py::dict d;
    d["path"] = core_info.path;
    d["entry"] = "moodistGetApi";
    d["version"] = core_info.version;
    d["magic"] = core_info.magic;
    d["slots"] = (sizeof(CoreApi) - sizeof(uint64_t)) / sizeof(void*);
    return d;
  });

  // A real subclass of torch.distributed.ProcessGroup: isinstance holds, torch.distributed's
  // functions accept it as `group=`, and c10d's own bindings (rank, size, _allgather_base,
  // _reduce_scatter_base, allreduce, ...) reach the overrides above through the virtual table.
  py::class_<ProcessGroup, c10d::ProcessGroup, c10::intrusive_ptr<ProcessGroup>>(m, "MoodistProcessGroup",
      py::dynamic_attr())
      .def(py::init([](py::object store, int rank, int size) {
        // A torch.distributed.Store is passed to the core as the c10d::Store it wraps (the core
        // may call back into it); any other object stands for a world by its identity.
        void* key = store.ptr();
        try {
          auto real = store.cast<c10::intrusive_ptr<c10d::Store>>();
          if (real) {
            key = real.get();
            std::lock_guard<std::mutex> l(stores_mutex);
            real_stores.insert(key);
          }
        } catch (const py::cast_error&) {
        }
        return c10::make_intrusive<ProcessGroup>(key, std::move(store), rank, size);
      }),
          py::arg("store"), py::arg("rank"), py::arg("size"))
      .def_property_readonly("_store", &ProcessGroup::store)
      .def("moodist_name", &ProcessGroup::moodist_name)
      .def("get_prefer_kernel_less", &ProcessGroup::get_prefer_kernel_less)
      .def("set_prefer_kernel_less", &ProcessGroup::set_prefer_kernel_less)
      .def("_get_option", &ProcessGroup::get_option)
      .def("_set_option", &ProcessGroup::set_option)
      .def("cuda_barrier", &ProcessGroup::cuda_barrier, py::call_guard<py::gil_scoped_release>())
      .def("compile_op_full",
          [](const c10::intrusive_ptr<ProcessGroup>& self, std::vector<int> shape, at::ScalarType dtype,
              const std::vector<Spec>& inputs, const std::vector<Spec>& outputs) {
            return compile_op_full(self, std::move(shape), dtype, inputs, outputs);
          },
          py::arg("shape"), py::arg("dtype"), py::arg("inputs"), py::arg("outputs"))
      .def("_stage_input", &ProcessGroup::stage_input, py::arg("kind"), py::arg("input"), py::arg("reduce_op") = 0,
          py::arg("premul") = 0.0f);

  py::class_<CustomOpObj, std::shared_ptr<CustomOpObj>>(m, "CustomOp")
      .def("__call__", &CustomOpObj::call, py::arg("inputs"), py::arg("outputs"))
      .def("plan", &CustomOpObj::plan);
  py::class_<FutureObj, std::shared_ptr<FutureObj>>(m, "Future")
      .def("wait", &FutureObj::wait)
      .def("result", &FutureObj::result);
}
