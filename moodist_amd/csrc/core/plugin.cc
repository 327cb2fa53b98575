// moodistGetApi and the CoreApi table (include/moodist_plugin.h): the reference's one-symbol
// boundary between the Python module and the core (api/moodist_api.h:134-271,
// core/moodist_api.cc:62-179), laid over the process groups of this build.
//
// Tensors arrive as opaque TensorPtr and are read through the WrapperApi the loader handed in,
// as the reference's core reads them (api/tensor_ptr.h:178-246).  What a collective keeps --
// its input and output tensors, a padded temporary -- is pinned with tensorAddRef until the
// launches of that collective have been enqueued.
#include "moodist_plugin.h"

#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>

#include "c_handles.h"
#include "hip_loader.h"
#include "processgroup.h"

namespace moodist {

namespace {

WrapperApi g_wrapper{};
bool g_have_wrapper = false;

const WrapperApi& wrapper() {
  if (!g_have_wrapper) {
    throw std::runtime_error("moodist: the core was not given a WrapperApi (call moodistGetApi first)");
  }
  return g_wrapper;
}

// One world per store: the ranks created with the same store pointer are each other's peers.
std::mutex g_worlds_mutex;
struct WorldEntry {
  std::weak_ptr<World> world;
  std::vector<bool> taken; // ranks that currently exist
};
std::map<void*, WorldEntry> g_worlds;

using CoreGroup = ::moodist::ProcessGroup; // inside the api:: types, "ProcessGroup" names their base

struct GroupObject : api::ProcessGroup {
  std::shared_ptr<World> world;
  CoreGroup* pg = nullptr;
  void* store = nullptr;
};

struct OpObject : api::CustomOp {
  std::shared_ptr<World> world;
  moodist_op flat{nullptr, nullptr}; // the same op as the plain C functions see it
};

struct FutureObject : api::Future {
  std::shared_ptr<Collective> collective;
  Keep held; // inputs and outputs stay alive until the future dies (core/processgroup.cc:3239-3245)
};

GroupObject* group_of(api::ProcessGroup* pg) {
  if (!pg) {
    throw std::runtime_error("moodist: null process group");
  }
  return static_cast<GroupObject*>(pg);
}

moodist_tensor describe(const TensorPtr& t, const char* what) {
  Tensor* p = t.get();
  if (!p) {
    throw std::runtime_error(std::string("moodist: ") + what + " is an undefined tensor");
  }
  const WrapperApi& w = wrapper();
  moodist_tensor d{};
  d.data = w.tensorDataPtr(p);
  d.numel = w.tensorNumel(p);
  d.itemsize = (int32_t)w.tensorItemsize(p);
  d.dtype = (int32_t)w.tensorDtype(p);
  d.device = w.tensorIsCuda(p) ? w.tensorDevice(p) : -1;
  d.contiguous = w.tensorIsContiguous(p) ? 1 : 0;
  const int64_t nd = w.tensorNdim(p);
  d.ndim = (int32_t)(nd < 10 ? nd : 10);
  for (int i = 0; i < d.ndim; ++i) {
    d.shape[i] = w.tensorSize(p, i);
  }
  return d;
}

// One more reference on the tensor, given back when the returned pointer dies.
std::shared_ptr<void> pin(const TensorPtr& t) {
  Tensor* p = t.get();
  wrapper().tensorAddRef(p);
  return std::shared_ptr<void>(p, [](void* q) { g_wrapper.tensorDecRef(static_cast<Tensor*>(q)); });
}

// Snapshot memory comes from the wrapper's caching allocator, entered on the rank's stream so
// that the block belongs to the stream that fills and reads it.
void* wrapper_alloc(size_t bytes, void** cleanup, void* stream, int device) {
  const WrapperApi& w = wrapper();
  void* guard = w.cudaStreamGuardEnter ? w.cudaStreamGuardEnter(static_cast<Stream>(stream), device) : nullptr;
  void* p = nullptr;
  try {
    p = w.cudaCachingAllocatorAlloc(bytes, cleanup);
  } catch (...) {
    if (guard) {
      w.cudaStreamGuardExit(guard);
    }
    throw;
  }
  if (guard) {
    w.cudaStreamGuardExit(guard);
  }
  return p;
}

void wrapper_free(void* cleanup) {
  g_wrapper.cudaCachingAllocatorFree(cleanup);
}

// ---- the slots of the path ----

api::ProcessGroupHandle createProcessGroup(void* store, int rank, int size) {
  std::lock_guard<std::mutex> l(g_worlds_mutex);
  WorldEntry& e = g_worlds[store];
  std::shared_ptr<World> world = e.world.lock();
  if (!world) {
    const int device = wrapper().cudaCurrentDevice ? wrapper().cudaCurrentDevice() : 0;
    world = std::make_shared<World>(size, device < 0 ? 0 : device);
    if (g_wrapper.cudaCachingAllocatorAlloc && g_wrapper.cudaCachingAllocatorFree) {
      world->allocator.alloc = wrapper_alloc;
      world->allocator.free = wrapper_free;
    }
    e.world = world;
    e.taken.assign((size_t)size, false);
  }
  if (world->size != size) {
    throw std::runtime_error("moodist: this store already serves a group of " + std::to_string(world->size) +
                             " ranks, not " + std::to_string(size));
  }
  if (rank < 0 || rank >= size) {
    throw std::runtime_error("moodist: rank " + std::to_string(rank) + " outside a group of " + std::to_string(size));
  }
  if (e.taken[(size_t)rank]) {
    throw std::runtime_error("moodist: rank " + std::to_string(rank) + " of this store's group already exists");
  }
  e.taken[(size_t)rank] = true;
  auto* g = new GroupObject;
  g->world = world;
  g->pg = world->group(rank);
  g->store = store;
  return api::ProcessGroupHandle::create(g);
}

void processGroupDestroy(api::ProcessGroup* pg) {
  GroupObject* g = static_cast<GroupObject*>(pg);
  if (!g) {
    return;
  }
  {
    std::lock_guard<std::mutex> l(g_worlds_mutex);
    auto it = g_worlds.find(g->store);
    if (it != g_worlds.end() && it->second.world.lock() == g->world) {
      std::vector<bool>& taken = it->second.taken;
      taken[(size_t)g->pg->rank] = false;
      bool any = false;
      for (bool b : taken) {
        any = any || b;
      }
      if (!any) {
        g_worlds.erase(it); // the last rank is leaving: the store may serve a new group later
      }
    }
  }
  delete g;
}

void processGroupShutdown(api::ProcessGroup*) {
  // nothing runs in the background: there is nothing to stop before the last reference goes
}

int processGroupRank(api::ProcessGroup* pg) {
  return group_of(pg)->pg->rank;
}

int processGroupSize(api::ProcessGroup* pg) {
  return group_of(pg)->pg->size;
}

bool processGroupGetPreferKernelLess(api::ProcessGroup* pg) {
  return group_of(pg)->pg->get_option("prefer_kernel_less") != 0;
}

void processGroupSetPreferKernelLess(api::ProcessGroup* pg, bool value) {
  group_of(pg)->pg->set_option("prefer_kernel_less", value ? 1 : 0);
}

int64_t processGroupGetOption(api::ProcessGroup* pg, const char* name) {
  return group_of(pg)->pg->get_option(name ? name : "");
}

void processGroupSetOption(api::ProcessGroup* pg, const char* name, int64_t value) {
  group_of(pg)->pg->set_option(name ? name : "", value);
}

void processGroupAllGather(api::ProcessGroup* pg, TensorPtr& output, const TensorPtr& input, Stream stream) {
  const moodist_tensor o = describe(output, "all_gather output"), i = describe(input, "all_gather input");
  group_of(pg)->pg->all_gather(&o, i, stream, Keep{pin(output), pin(input)});
}

void processGroupReduceScatter(api::ProcessGroup* pg, TensorPtr& output, const TensorPtr& input, ReduceOp reduceOp,
    Stream stream, float premulValue) {
  const moodist_tensor o = describe(output, "reduce_scatter output"), i = describe(input, "reduce_scatter input");
  group_of(pg)->pg->reduce_scatter(&o, i, (int)reduceOp, stream, premulValue, Keep{pin(output), pin(input)});
}

void processGroupAllreduce(api::ProcessGroup* pg, TensorPtr& tensor, ReduceOp reduceOp, Stream stream,
    float premulValue) {
  CoreGroup* g = group_of(pg)->pg;
  const moodist_tensor t = describe(tensor, "allreduce tensor");
  Keep keep{pin(tensor)};
  if (t.numel % g->size == 0) {
    g->allreduce(t, nullptr, (int)reduceOp, stream, premulValue, std::move(keep));
    return;
  }
  // the padded temporary comes from torch, as in the reference (core/processgroup.cc:1694-1697)
  const WrapperApi& w = wrapper();
  const int64_t padded = (t.numel + g->size - 1) / g->size * g->size;
  void* guard = w.cudaStreamGuardEnter ? w.cudaStreamGuardEnter(stream, t.device) : nullptr;
  TensorPtr scratch;
  try {
    scratch.reset(w.tensorEmpty(&padded, 1, (DType)t.dtype, t.device));
  } catch (...) {
    if (guard) {
      w.cudaStreamGuardExit(guard);
    }
    throw;
  }
  if (guard) {
    w.cudaStreamGuardExit(guard);
  }
  keep.push_back(pin(scratch));
  w.tensorDecRef(scratch.release()); // `keep` holds the only reference now
  const moodist_tensor s = describe(TensorPtr(static_cast<Tensor*>(keep.back().get())), "allreduce scratch");
  g->allreduce(t, &s, (int)reduceOp, stream, premulValue, std::move(keep));
}

void processGroupBarrier(api::ProcessGroup* pg) {
  group_of(pg); // every rank lives in the calling process: nobody to wait for
}

void processGroupCudaBarrier(api::ProcessGroup* pg, Stream) {
  group_of(pg); // one device: stream order is the barrier
}

void futureDestroy(api::Future* future) {
  delete static_cast<FutureObject*>(future);
}

void wait_launched(const Collective& c) {
  if (!c.launched) {
    throw std::runtime_error("moodist: a custom op was waited on before every rank of the group has called it (" +
                             std::to_string(c.arrived) + " of " + std::to_string(c.post.size()) + " have)");
  }
  if (!c.error.empty()) {
    throw std::runtime_error(c.error);
  }
}

void futureWait(api::Future* future, Stream) {
  if (!future) {
    throw std::runtime_error("moodist: null future");
  }
  // the copies were enqueued on the stream each rank passed to the call; nothing to add to `stream`
  wait_launched(*static_cast<FutureObject*>(future)->collective);
}

bool futureGetResult(api::Future*, TensorPtr*) {
  return false; // a custom op writes into the caller's outputs; only queue futures carry a result
}

void customOpDestroy(api::CustomOp* op) {
  delete static_cast<OpObject*>(op);
}

api::FutureHandle customOpCall(api::CustomOp* op, TensorPtr* inputs, size_t nInputs, TensorPtr* outputs,
    size_t nOutputs, Stream stream) {
  if (!op) {
    throw std::runtime_error("moodist: null custom op");
  }
  OpObject* o = static_cast<OpObject*>(op);
  std::vector<moodist_tensor> in, out;
  Keep launch_keep, future_keep;
  for (size_t i = 0; i < nInputs; ++i) {
    in.push_back(describe(inputs[i], "custom op input"));
    launch_keep.push_back(pin(inputs[i]));
    future_keep.push_back(pin(inputs[i]));
  }
  for (size_t i = 0; i < nOutputs; ++i) {
    out.push_back(describe(outputs[i], "custom op output"));
    launch_keep.push_back(pin(outputs[i]));
    future_keep.push_back(pin(outputs[i]));
  }
  auto* f = new FutureObject;
  api::FutureHandle handle = api::FutureHandle::create(f);
  f->held = std::move(future_keep);
  f->collective = o->flat.pg->custom_op(o->flat.op, in.data(), in.size(), out.data(), out.size(), stream,
      std::move(launch_keep));
  return handle;
}

api::CustomOpHandle compileOpFull(api::ProcessGroup* pg, const int* shape, size_t ndim, DType dtype,
    const int* inputRanks, const int* inputOffsets, const int* inputShapes, size_t nInputs, const int* outputRanks,
    const int* outputOffsets, const int* outputShapes, size_t nOutputs) {
  GroupObject* g = group_of(pg);
  auto slices = [ndim](const int* ranks, const int* offsets, const int* shapes, size_t n) {
    std::vector<SliceSpec> v(n);
    for (size_t i = 0; i < n; ++i) {
      v[i].rank = ranks[i];
      v[i].offset.assign(offsets + i * ndim, offsets + (i + 1) * ndim);
      v[i].shape.assign(shapes + i * ndim, shapes + (i + 1) * ndim);
    }
    return v;
  };
  auto* o = new OpObject;
  api::CustomOpHandle handle = api::CustomOpHandle::create(o);
  o->world = g->world;
  o->flat.pg = g->pg;
  o->flat.op = g->pg->compile_op_full(Dims(shape, shape + ndim), (int)dtype, slices(inputRanks, inputOffsets, inputShapes, nInputs),
      slices(outputRanks, outputOffsets, outputShapes, nOutputs));
  return handle;
}

// ---- every slot outside the path ----

void off_path() {
  throw std::runtime_error("moodist: this function of the core API is not supported: the build covers the "
                           "single-GPU hot path (all_gather, reduce_scatter, allreduce, compile_op) only");
}

CoreApi make_table() {
  CoreApi t;
  // every slot starts as "not supported" ...
  const OffPath refuse = off_path;
  for (size_t at = sizeof(uint64_t); at < sizeof(CoreApi); at += sizeof(OffPath)) {
    std::memcpy(reinterpret_cast<char*>(&t) + at, &refuse, sizeof(OffPath));
  }
  // ... and the path's are then filled in
  t.magic = kMoodistBuildMagic;
  t.createProcessGroup = createProcessGroup;
  t.processGroupDestroy = processGroupDestroy;
  t.processGroupShutdown = processGroupShutdown;
  t.processGroupRank = processGroupRank;
  t.processGroupSize = processGroupSize;
  t.processGroupGetPreferKernelLess = processGroupGetPreferKernelLess;
  t.processGroupSetPreferKernelLess = processGroupSetPreferKernelLess;
  t.processGroupGetOption = processGroupGetOption;
  t.processGroupSetOption = processGroupSetOption;
  t.processGroupAllGather = processGroupAllGather;
  t.processGroupReduceScatter = processGroupReduceScatter;
  t.processGroupAllreduce = processGroupAllreduce;
  t.processGroupBarrier = processGroupBarrier;
  t.processGroupCudaBarrier = processGroupCudaBarrier;
  t.futureDestroy = futureDestroy;
  t.futureWait = futureWait;
  t.futureGetResult = futureGetResult;
  t.customOpDestroy = customOpDestroy;
  t.customOpCall = customOpCall;
  t.compileOpFull = compileOpFull;
  return t;
}

CoreApi g_table = make_table();

} // namespace

// The core's side of "who drops the last reference destroys" (api/api_handle.h:168-174): a
// handle that dies inside the core, e.g. after a failed call, takes the same path as one that
// dies in the wrapper.
namespace api {
void destroy(Future* f) {
  futureDestroy(f);
}
void destroy(CustomOp* op) {
  customOpDestroy(op);
}
void destroy(ProcessGroup* pg) {
  processGroupDestroy(pg);
}
} // namespace api

} // namespace moodist

#pragma GCC visibility push(default)
extern "C" {

moodist::CoreApi* moodistGetApi(uint32_t expectedVersion, const moodist::WrapperApi* wrapperApi) {
  if (expectedVersion != moodist::kMoodistApiVersion) {
    return nullptr;
  }
  if (wrapperApi) {
    moodist::g_wrapper = *wrapperApi;
    moodist::g_have_wrapper = true;
  }
  return &moodist::g_table;
}

uint64_t moodist_build_magic(void) {
  return moodist::kMoodistBuildMagic;
}

moodist_pg* moodistGroupCHandle(moodist::api::ProcessGroup* group) {
  return group ? reinterpret_cast<moodist_pg*>(static_cast<moodist::GroupObject*>(group)->pg) : nullptr;
}

moodist_op* moodistOpCHandle(moodist::api::CustomOp* op) {
  return op ? &static_cast<moodist::OpObject*>(op)->flat : nullptr;
}

} // extern "C"
#pragma GCC visibility pop
