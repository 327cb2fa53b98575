// Drives the core through its plugin entry (include/moodist_plugin.h) the way a wrapper does,
// with a WrapperApi whose "tensors" are plain structs: the handshake, the table's layout, the
// slots of the path and of everything else, handle ownership, and -- the point of the fake
// tensors -- how long the core keeps references on what a rank posted.  No GPU is needed: a
// collective whose last rank arrives fails at the launch for want of the kernel library, which
// is one of the paths that must release every reference.
// Two builds (tests/test_sanitize_cpu.py): together with the core's sources under
// -fsanitize=address,undefined; and with -DMOODIST_DRIVER_DLOPEN against the built
// libmoodist.so (path in argv[1]), resolving moodistGetApi with dlsym as a wrapper does.
#include "moodist_plugin.h"
#include "moodist_core.h"

#ifdef MOODIST_DRIVER_DLOPEN
#include <dlfcn.h>
#endif

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace moodist {
struct Tensor : ApiRefCounted {
  void* data;
  int64_t numel;
  int itemsize;
  DType dtype;
  int device;
};
#ifdef MOODIST_DRIVER_DLOPEN
namespace api {
// this side's destroy(): back through the table, as the reference's wrapper does (linked
// together with the core's sources, the core's own definitions serve both sides)
static CoreApi* table = nullptr;
void destroy(Future* f) {
  table->futureDestroy(f);
}
void destroy(CustomOp* op) {
  table->customOpDestroy(op);
}
void destroy(ProcessGroup* pg) {
  table->processGroupDestroy(pg);
}
} // namespace api
#endif
} // namespace moodist

using namespace moodist;

static int live_tensors = 0;
static int empties_made = 0;
static int device_allocations = 0; // calls of the wrapper's caching allocator (snapshot_inputs)

static Tensor* make(int64_t numel, DType dtype = DType::Float32, int itemsize = 4, int device = 0) {
  Tensor* t = new Tensor;
  t->refcount.store(1);
  t->data = (void*)0x100000;
  t->numel = numel;
  t->itemsize = itemsize;
  t->dtype = dtype;
  t->device = device;
  ++live_tensors;
  return t;
}

static WrapperApi wrapper_table() {
  WrapperApi w{};
  w.cudaCurrentDevice = []() -> int { return 0; };
  w.tensorAddRef = [](Tensor* t) { t->refcount.fetch_add(1); };
  w.tensorDecRef = [](Tensor* t) {
    if (t->refcount.fetch_sub(1) == 1) {
      --live_tensors;
      delete t;
    }
  };
  w.tensorDataPtr = [](Tensor* t) -> void* { return t->data; };
  w.tensorNumel = [](Tensor* t) -> int64_t { return t->numel; };
  w.tensorNdim = [](Tensor*) -> int64_t { return 1; };
  w.tensorSize = [](Tensor* t, int64_t) -> int64_t { return t->numel; };
  w.tensorDtype = [](Tensor* t) -> DType { return t->dtype; };
  w.tensorDevice = [](Tensor* t) -> int { return t->device; };
  w.tensorIsContiguous = [](Tensor*) -> bool { return true; };
  w.tensorIsCuda = [](Tensor* t) -> bool { return t->device >= 0; };
  w.tensorIsCpu = [](Tensor* t) -> bool { return t->device < 0; };
  w.tensorItemsize = [](Tensor* t) -> int64_t { return t->itemsize; };
  w.tensorEmpty = [](const int64_t* sizes, int, DType dtype, int device) -> Tensor* {
    ++empties_made;
    return make(sizes[0], dtype, 4, device);
  };
  return w;
}

#define EXPECT(cond)                                              \
  do {                                                            \
    if (!(cond)) {                                                \
      std::printf("FAILED line %d: %s\n", __LINE__, #cond);       \
      return 1;                                                   \
    }                                                             \
  } while (0)

template<typename F>
static std::string thrown(F&& f) {
  try {
    f();
  } catch (const std::exception& e) {
    return e.what();
  }
  return "";
}

int main(int argc, char** argv) {
  const WrapperApi w = wrapper_table();
#ifdef MOODIST_DRIVER_DLOPEN
  // the wrapper's way in: dlopen, one symbol (wrapper/moodist_loader.cc:363-386)
  EXPECT(argc > 1);
  void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  if (!lib) {
    std::printf("dlopen: %s\n", dlerror());
    return 1;
  }
  auto moodistGetApi = reinterpret_cast<decltype(&::moodistGetApi)>(dlsym(lib, "moodistGetApi"));
  auto moodistOpCHandle = reinterpret_cast<decltype(&::moodistOpCHandle)>(dlsym(lib, "moodistOpCHandle"));
  auto moodistGroupCHandle = reinterpret_cast<decltype(&::moodistGroupCHandle)>(dlsym(lib, "moodistGroupCHandle"));
  EXPECT(moodistGetApi && moodistOpCHandle && moodistGroupCHandle);
#else
  (void)argc, (void)argv;
#endif
  // version handshake: any version but the core's own gets no table
  EXPECT(moodistGetApi(kMoodistApiVersion + 1, &w) == nullptr);
  EXPECT(moodistGetApi(0, &w) == nullptr);
  CoreApi* core = moodistGetApi(kMoodistApiVersion, &w);
  EXPECT(core != nullptr);
  EXPECT(core->magic == kMoodistBuildMagic);
#ifdef MOODIST_DRIVER_DLOPEN
  api::table = core;
#endif

  // slots outside the path refuse, whatever they would have been called with
  EXPECT(thrown([&] { core->createStore(); }).find("not supported") != std::string::npos);
  EXPECT(thrown([&] { core->processGroupBroadcast(); }).find("not supported") != std::string::npos);
  EXPECT(thrown([&] { core->queuePut(); }).find("not supported") != std::string::npos);
  EXPECT(thrown([&] { core->getProfilingEnabled(); }).find("not supported") != std::string::npos);

  int store_a = 0, store_b = 0; // their addresses stand for two stores
  {
    std::vector<api::ProcessGroupHandle> g;
    for (int r = 0; r < 4; ++r) {
      g.push_back(core->createProcessGroup(&store_a, r, 4));
    }
    for (int r = 0; r < 4; ++r) {
      EXPECT(core->processGroupRank(g[r].get()) == r && core->processGroupSize(g[r].get()) == 4);
      EXPECT(g[r].get()->refcount.load() == 1);
    }
    EXPECT(thrown([&] { core->createProcessGroup(&store_a, 1, 4); }).find("already exists") != std::string::npos);
    EXPECT(thrown([&] { core->createProcessGroup(&store_a, 0, 8); }).find("already serves a group of 4") != std::string::npos);
    EXPECT(thrown([&] { core->createProcessGroup(&store_b, 5, 4); }).find("outside a group") != std::string::npos);
    // options by name and by the dedicated pair (api/processgroup_api.h:32-40)
    EXPECT(core->processGroupGetOption(g[0].get(), "num_chunks") == -1);
    core->processGroupSetOption(g[0].get(), "num_chunks", 4);
    EXPECT(core->processGroupGetOption(g[0].get(), "num_chunks") == 4);
    EXPECT(core->processGroupGetOption(g[1].get(), "num_chunks") == -1);
    core->processGroupSetPreferKernelLess(g[2].get(), true);
    EXPECT(core->processGroupGetPreferKernelLess(g[2].get()) && core->processGroupGetOption(g[2].get(), "prefer_kernel_less") == 1);
    EXPECT(thrown([&] { core->processGroupGetOption(g[0].get(), "bogus"); }) == "Unknown option: bogus");
    EXPECT(thrown([&] { core->processGroupSetOption(g[0].get(), "snapshot_inputs", 1); }).find("needs a device allocator") !=
           std::string::npos); // this wrapper table has no allocator
    core->processGroupBarrier(g[0].get());
    core->processGroupCudaBarrier(g[0].get(), nullptr);

    // a copy of a handle shares the object; the last one to go destroys it through this side's destroy()
    {
      api::ProcessGroupHandle copy = g[3];
      EXPECT(g[3].get()->refcount.load() == 2);
    }
    EXPECT(g[3].get()->refcount.load() == 1);

    // Lifetime: rank 0 posts a reduce_scatter, then a hundred unrelated all_gathers are posted by
    // the same rank; rank 0's first tensors must still be referenced by the core when the peers
    // arrive, and must be let go once the launch has been attempted.
    TensorPtr in0(make(16)), out0(make(4));
    core->processGroupReduceScatter(g[0].get(), out0, in0, ReduceOp::SUM, nullptr, 0.0f);
    EXPECT(in0.get()->refcount.load() == 2 && out0.get()->refcount.load() == 2);
    std::vector<Tensor*> later;
    for (int k = 0; k < 100; ++k) {
      TensorPtr i(make(8)), o(make(32));
      core->processGroupAllGather(g[0].get(), o, i, nullptr);
      EXPECT(i.get()->refcount.load() == 2);
      later.push_back(i.release());
      later.push_back(o.release());
    }
    EXPECT(in0.get()->refcount.load() == 2 && out0.get()->refcount.load() == 2);
    std::vector<Tensor*> peers;
    for (int r = 1; r < 4; ++r) {
      TensorPtr i(make(16)), o(make(4));
      const std::string err = thrown([&] { core->processGroupReduceScatter(g[r].get(), o, i, ReduceOp::SUM, nullptr, 0.0f); });
      if (r < 3) {
        EXPECT(err.empty() && i.get()->refcount.load() == 2);
        EXPECT(in0.get()->refcount.load() == 2); // still waiting for rank 3
      } else {
        // the last rank triggers the launch, which fails here: no kernel library beside this binary
        EXPECT(!err.empty());
        std::printf("launch without a GPU: %s\n", err.c_str());
      }
      peers.push_back(i.release());
      peers.push_back(o.release());
    }
    // every reference the collective held is back
    EXPECT(in0.get()->refcount.load() == 1 && out0.get()->refcount.load() == 1);
    for (Tensor* t : peers) {
      EXPECT(t->refcount.load() == 1);
      w.tensorDecRef(t);
    }
    // the hundred gathers are still pending (only rank 0 posted them): still referenced
    for (Tensor* t : later) {
      EXPECT(t->refcount.load() == 2);
    }
    // mismatched collectives across ranks are reported (the reference aborts, core/cputhread.h:100-112)
    {
      TensorPtr i(make(8, DType::Float64, 8)), o(make(32, DType::Float64, 8));
      EXPECT(thrown([&] { core->processGroupAllGather(g[1].get(), o, i, nullptr); }).find("different operation, size, dtype") !=
             std::string::npos);
      w.tensorDecRef(i.release());
      w.tensorDecRef(o.release());
    }
    // validation errors carry the reference's texts
    {
      TensorPtr i(make(16, DType::Int8, 1)), o(make(4, DType::Int8, 1));
      EXPECT(thrown([&] { core->processGroupReduceScatter(g[1].get(), o, i, ReduceOp::SUM, nullptr, 0.0f); }) ==
             "Unsupported dtype for reduce operation");
      EXPECT(i.get()->refcount.load() == 1); // a refused call keeps nothing
      TensorPtr f(make(16)), fo(make(4));
      EXPECT(thrown([&] { core->processGroupReduceScatter(g[1].get(), fo, f, ReduceOp::PRODUCT, nullptr, 0.0f); }) ==
             "Unsupported reduce operation");
      TensorPtr cpu(make(16, DType::Float32, 4, -1));
      EXPECT(thrown([&] { core->processGroupAllreduce(g[1].get(), cpu, ReduceOp::SUM, nullptr, 0.0f); }).find("CPU tensor") !=
             std::string::npos);
      TensorPtr undefined;
      EXPECT(thrown([&] { core->processGroupAllreduce(g[1].get(), undefined, ReduceOp::SUM, nullptr, 0.0f); }).find("undefined tensor") !=
             std::string::npos);
      for (TensorPtr* p : {&i, &o, &f, &fo, &cpu}) {
        EXPECT(p->get()->refcount.load() == 1);
        w.tensorDecRef(p->release());
      }
    }
    // allreduce of a size the group does not divide: the padded temporary comes from tensorEmpty
    // (core/processgroup.cc:1694-1697) and lives as long as the collective is pending
    {
      const int before = empties_made, live_before = live_tensors;
      TensorPtr t(make(10));
      std::vector<api::ProcessGroupHandle> h; // a fresh world on a second store
      for (int r = 0; r < 4; ++r) {
        h.push_back(core->createProcessGroup(&store_b, r, 4));
      }
      // the copy into the temporary is enqueued at once, which needs the HIP runtime and the kernel
      // library: absent here, so the call fails -- after the temporary was made, and it must not leak
      const std::string err = thrown([&] { core->processGroupAllreduce(h[0].get(), t, ReduceOp::SUM, nullptr, 0.0f); });
      EXPECT(!err.empty());
      EXPECT(empties_made == before + 1);
      EXPECT(live_tensors == live_before + 1); // the temporary has gone again
      EXPECT(t.get()->refcount.load() == 1);
      // a size the group divides needs no temporary and stays pending; its reduce_scatter half and
      // its all_gather half share one reference on the tensor
      TensorPtr even(make(12));
      core->processGroupAllreduce(h[1].get(), even, ReduceOp::SUM, nullptr, 0.0f);
      EXPECT(empties_made == before + 1 && even.get()->refcount.load() == 2);
      h.clear(); // the world goes, with its pending collectives and their references
      EXPECT(even.get()->refcount.load() == 1);
      w.tensorDecRef(even.release());
      w.tensorDecRef(t.release());
    }

    // compile_op_full -> custom op -> future (api/moodist_api.h:244-255)
    {
      int shape[1] = {8};
      int in_ranks[1] = {0}, in_off[1] = {0}, in_shape[1] = {8};
      int out_ranks[4] = {0, 1, 2, 3}, out_off[4] = {0, 2, 4, 6}, out_shape[4] = {2, 2, 2, 2};
      std::vector<api::CustomOpHandle> ops;
      std::vector<api::ProcessGroupHandle> h;
      for (int r = 0; r < 4; ++r) {
        h.push_back(core->createProcessGroup(&store_b, r, 4));
        ops.push_back(core->compileOpFull(h[r].get(), shape, 1, DType::Float32, in_ranks, in_off, in_shape, 1, out_ranks,
            out_off, out_shape, 4));
        EXPECT(ops[r].get()->refcount.load() == 1);
      }
      EXPECT(moodistOpCHandle(ops[0].get()) != nullptr && moodistGroupCHandle(h[0].get()) != nullptr);
      TensorPtr in(make(8)), out(make(2));
      TensorPtr wrong(make(7));
      EXPECT(thrown([&] { core->customOpCall(ops[0].get(), &wrong, 1, &out, 1, nullptr); }) ==
             "moodist: custom op input has wrong size");
      EXPECT(wrong.get()->refcount.load() == 1 && out.get()->refcount.load() == 1);
      {
        api::FutureHandle fut = core->customOpCall(ops[0].get(), &in, 1, &out, 1, nullptr);
        EXPECT(in.get()->refcount.load() == 3); // the pending collective and the future
        EXPECT(thrown([&] { core->futureWait(fut.get(), nullptr); }).find("before every rank") != std::string::npos);
        TensorPtr result;
        EXPECT(!core->futureGetResult(fut.get(), &result));
      }
      EXPECT(in.get()->refcount.load() == 2); // the future has gone, the collective is still pending
      ops.clear();
      h.clear();
      EXPECT(in.get()->refcount.load() == 1 && out.get()->refcount.load() == 1);
      for (TensorPtr* p : {&in, &out, &wrong}) {
        w.tensorDecRef(p->release());
      }
    }

    g.clear(); // the world of store_a goes, with rank 0's hundred pending gathers
    for (Tensor* t : later) {
      EXPECT(t->refcount.load() == 1);
      w.tensorDecRef(t);
    }
    w.tensorDecRef(in0.release());
    w.tensorDecRef(out0.release());
  }
  EXPECT(live_tensors == 0);
  // a store whose ranks have all gone serves a new group of another size
  {
    api::ProcessGroupHandle again = core->createProcessGroup(&store_a, 0, 8);
    EXPECT(core->processGroupSize(again.get()) == 8);
  }
  // The allreduce that allocates nothing, with the one option that allocates switched on: a
  // table that HAS a device allocator (and counts its calls), a world made after it was handed
  // over, snapshot_inputs = 1.  moodist_pg_allreduce_static must not ask the allocator for
  // anything -- neither when the group size divides the element count (its reduce_scatter half
  // would snapshot the tensor) nor on the padded path (which ends early here: the fixed
  // workspace needs a device) -- while a plain reduce_scatter on the same group does ask.
  {
    WrapperApi with_allocator = wrapper_table();
    with_allocator.cudaCachingAllocatorAlloc = [](size_t bytes, void** cleanup) -> void* {
      ++device_allocations;
      void* p = std::malloc(bytes ? bytes : 1);
      *cleanup = p;
      return p;
    };
    with_allocator.cudaCachingAllocatorFree = [](void* cleanup) { std::free(cleanup); };
    EXPECT(moodistGetApi(kMoodistApiVersion, &with_allocator) == core);
    int store_c = 0;
    std::vector<api::ProcessGroupHandle> h;
    for (int r = 0; r < 4; ++r) {
      h.push_back(core->createProcessGroup(&store_c, r, 4));
    }
    core->processGroupSetOption(h[0].get(), "snapshot_inputs", 1);
    EXPECT(core->processGroupGetOption(h[0].get(), "snapshot_inputs") == 1);
    auto allreduce_static = reinterpret_cast<decltype(&moodist_pg_allreduce_static)>(
#ifdef MOODIST_DRIVER_DLOPEN
        dlsym(lib, "moodist_pg_allreduce_static")
#else
        reinterpret_cast<void*>(&moodist_pg_allreduce_static)
#endif
    );
    EXPECT(allreduce_static != nullptr);
    moodist_tensor even{};
    even.data = (void*)0x200000, even.numel = 4096, even.itemsize = 4, even.dtype = 6, even.device = 0;
    even.contiguous = 1, even.ndim = 1, even.shape[0] = 4096;
    moodist_work* work = nullptr;
    const int before = device_allocations;
    EXPECT(allreduce_static(moodistGroupCHandle(h[0].get()), &even, 0, nullptr, 0.0f, &work) == 0); // posted, pending
    EXPECT(device_allocations == before);
    moodist_tensor odd = even;
    odd.numel = 4097, odd.shape[0] = 4097;
    moodist_work* none = nullptr;
    EXPECT(allreduce_static(moodistGroupCHandle(h[1].get()), &odd, 0, nullptr, 0.0f, &none) != 0); // no device here
    EXPECT(device_allocations == before);
    // the same option on a plain reduce_scatter goes for the snapshot, which cannot be made here
    // (no kernel library or no device, depending on the build): the call fails, and whatever it
    // took from the allocator it has given back
    TensorPtr in(make(16)), out(make(4));
    EXPECT(!thrown([&] { core->processGroupReduceScatter(h[0].get(), out, in, ReduceOp::SUM, nullptr, 0.0f); }).empty());
    EXPECT(device_allocations == before || device_allocations == before + 1);
    EXPECT(in.get()->refcount.load() == 1 && out.get()->refcount.load() == 1);
    w.tensorDecRef(in.release());
    w.tensorDecRef(out.release());
#ifdef MOODIST_DRIVER_DLOPEN
    reinterpret_cast<decltype(&moodist_work_destroy)>(dlsym(lib, "moodist_work_destroy"))(work);
#else
    moodist_work_destroy(work);
#endif
  }
  EXPECT(live_tensors == 0);
  std::puts("plugin driver done");
  return 0;
}
