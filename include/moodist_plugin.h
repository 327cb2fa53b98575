/*
 * moodist_plugin.h -- the plugin entry of the host core (libmoodist.so).
 *
 * The reference's core exports ONE C-linkage symbol,
 *
 *     moodist::CoreApi* moodistGetApi(uint32_t expectedVersion, const moodist::WrapperApi*)
 *
 * (api/moodist_api.h:265-271, core/moodist_api.cc:168-179).  The Python module dlopens the
 * core, calls it with its own version number and a table of torch-backed callbacks, gets a
 * table of core functions back (NULL when the versions differ), and then checks the table's
 * `magic` against the build's (wrapper/moodist_loader.cc:363-386).  This header declares that
 * symbol and the two tables for this build, slot for slot:
 *
 *   - both tables have the reference's member order, so a slot sits at the reference's offset
 *     (magic at 0, slot k at 8 + 8k; api/moodist_api.h:64-258);
 *   - the slots of the hot path carry the reference's names and signatures, with hipStream_t
 *     (as Stream below) where the reference has CUstream (api/processgroup_api.h:29-65,
 *     api/moodist_api.h:197-216, :236-255);
 *   - the slots outside the path (store, allocators, serializer, queues, broadcast / reduce /
 *     scatter / gather / all-to-all, profiling) are typed OffPath: every one points at a
 *     function that ignores its arguments and throws std::runtime_error("... not supported").
 *
 * As in the reference this is a C++ ABI between two libraries built with the same compiler:
 * references, std::span, std::string_view and a handle returned by value cross it.  The plain
 * C functions of moodist_core.h sit underneath and stay available.
 *
 * Peers.  createProcessGroup(store, rank, size) is called once per rank.  The reference uses
 * the store to exchange addresses between processes; here the ranks created with the same
 * `store` pointer become the ranks of one in-process world on the caller's current device.
 */
#ifndef MOODIST_PLUGIN_H
#define MOODIST_PLUGIN_H

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <span>
#include <string>
#include <string_view>
#include <type_traits>
#include <vector>

struct ihipStream_t;

namespace moodist {

/* api/moodist_version.h:12.  The build magic is a random number drawn once per build and
 * compiled into both libraries, there by CMake (CMakeLists.txt:97-106), here by
 * moodist_amd/csrc/build_host.sh; the constant below only serves a translation unit compiled on
 * its own (a test driver), which then checks against a core built the same way. */
constexpr uint32_t kMoodistApiVersion = 2;
#ifndef MOODIST_BUILD_MAGIC
#define MOODIST_BUILD_MAGIC 0x4d49333535584d44ULL /* "MI355XMD" */
#endif
constexpr uint64_t kMoodistBuildMagic = MOODIST_BUILD_MAGIC;

using Stream = ihipStream_t*; /* hipStream_t */

/* torch ScalarType / c10d RedOpType numbers (api/moodist_api.h:30-55) */
enum class DType : int8_t { UInt8 = 0, Int8 = 1, Int16 = 2, Int32 = 3, Int64 = 4, Float16 = 5, Float32 = 6,
  Float64 = 7, Bool = 11, BFloat16 = 15 };
enum class ReduceOp : uint8_t { SUM = 0, AVG = 1, PRODUCT = 2, MIN = 3, MAX = 4, BAND = 5, BOR = 6, BXOR = 7,
  PREMUL_SUM = 8 };

/* Objects that cross the boundary start with their reference count (api/api_handle.h:44-46). */
struct ApiRefCounted {
  std::atomic_size_t refcount;
};

/* A torch tensor as the core sees it: opaque, owned by the wrapper, reached through the
 * WrapperApi accessors (api/moodist_api.h:26; wrapper/moodist_loader.cc:27-35). */
struct Tensor;

/* One pointer wide, like the reference's TensorPtr (api/tensor_ptr.h:73-76).  This one does
 * no reference counting of its own: the core pins what it keeps with tensorAddRef/tensorDecRef. */
class TensorPtr {
  Tensor* ptr_ = nullptr;

public:
  TensorPtr() = default;
  explicit TensorPtr(Tensor* adopted) : ptr_(adopted) {}
  Tensor* get() const {
    return ptr_;
  }
  explicit operator bool() const {
    return ptr_ != nullptr;
  }
  Tensor* release() {
    Tensor* p = ptr_;
    ptr_ = nullptr;
    return p;
  }
  void reset(Tensor* adopted = nullptr) {
    ptr_ = adopted;
  }
};
static_assert(sizeof(TensorPtr) == sizeof(void*), "TensorPtr must stay one pointer wide");

namespace api {

/* api/types.h:29-38 */
struct Store : ApiRefCounted {};
struct Queue : ApiRefCounted {};
struct Future : ApiRefCounted {};
struct CustomOp : ApiRefCounted {};
struct ProcessGroup : ApiRefCounted {};
struct Buffer : ApiRefCounted {};

/* Whoever holds the last reference calls these; each side of the boundary defines its own
 * (the wrapper's forward to the table's *Destroy slots, api/api_handle.h:168-174). */
void destroy(Future*);
void destroy(CustomOp*);
void destroy(ProcessGroup*);

/* One pointer wide and not trivially destructible, so that it is returned through a hidden
 * result slot exactly like the reference's ApiHandle<T> (api/api_handle.h:190-320). */
template<typename T>
class Handle {
  static_assert(std::is_base_of_v<ApiRefCounted, T>);
  T* ptr_ = nullptr;

public:
  Handle() = default;
  /* takes over one reference that already exists */
  static Handle adopt(T* p) {
    Handle h;
    h.ptr_ = p;
    return h;
  }
  /* a fresh object: the handle's reference is the first */
  static Handle create(T* p) {
    if (p) {
      p->refcount.store(1, std::memory_order_relaxed);
    }
    return adopt(p);
  }
  static Handle share(T* p) {
    if (p) {
      p->refcount.fetch_add(1, std::memory_order_relaxed);
    }
    return adopt(p);
  }
  Handle(const Handle& o) : ptr_(o.ptr_) {
    if (ptr_) {
      ptr_->refcount.fetch_add(1, std::memory_order_relaxed);
    }
  }
  Handle(Handle&& o) noexcept : ptr_(o.ptr_) {
    o.ptr_ = nullptr;
  }
  Handle& operator=(Handle o) noexcept {
    std::swap(ptr_, o.ptr_);
    return *this;
  }
  ~Handle() {
    drop();
  }
  void drop() {
    T* p = ptr_;
    ptr_ = nullptr;
    if (p && p->refcount.fetch_sub(1, std::memory_order_acq_rel) == 1) {
      destroy(p);
    }
  }
  T* get() const {
    return ptr_;
  }
  explicit operator bool() const {
    return ptr_ != nullptr;
  }
};

using ProcessGroupHandle = Handle<ProcessGroup>;
using FutureHandle = Handle<Future>;
using CustomOpHandle = Handle<CustomOp>;

} // namespace api

/*
 * What the core may ask of the module that loaded it (api/moodist_api.h:61-128).  The core of
 * this build calls: cudaCurrentDevice, cudaCachingAllocatorAlloc/Free (snapshot_inputs only),
 * tensorAddRef/DecRef, and the tensor accessors DataPtr, Numel, Ndim, Size, Dtype, Device,
 * IsContiguous, IsCuda, Itemsize.  The rest is declared so the table has the reference's layout.
 */
struct WrapperApi {
  int (*cudaCurrentDevice)();
  Stream (*cudaGetCurrentStream)();
  void* (*cudaStreamGuardEnter)(Stream stream, int device);
  void (*cudaStreamGuardExit)(void* guard);
  void* (*cudaCachingAllocatorAlloc)(size_t bytes, void** cleanupCtx);
  void (*cudaCachingAllocatorFree)(void* cleanupCtx);

  Tensor* (*tensorFromBlob)(void* data, const int64_t* sizes, int ndim, DType dtype, int device);
  Tensor* (*tensorEmpty)(const int64_t* sizes, int ndim, DType dtype, int device);
  Tensor* (*tensorFromBlobWithDeleter)(void* data, const int64_t* sizes, int ndim, DType dtype, int device,
      void (*deleter)(void* ctx), void* deleterCtx);
  void (*tensorAddRef)(Tensor*);
  void (*tensorDecRef)(Tensor*);

  void* (*tensorDataPtr)(Tensor*);
  int64_t (*tensorNumel)(Tensor*);
  int64_t (*tensorNdim)(Tensor*);
  int64_t (*tensorSize)(Tensor*, int64_t dim);
  int64_t (*tensorStride)(Tensor*, int64_t dim);
  DType (*tensorDtype)(Tensor*);
  int (*tensorDevice)(Tensor*);
  bool (*tensorIsContiguous)(Tensor*);
  bool (*tensorIsCuda)(Tensor*);
  bool (*tensorIsCpu)(Tensor*);
  int64_t (*tensorItemsize)(Tensor*);

  Tensor* (*tensorView)(Tensor*, const int64_t* sizes, int ndim);
  Tensor* (*tensorNarrow)(Tensor*, int dim, int64_t start, int64_t length);
  Tensor* (*tensorContiguous)(Tensor*);
  Tensor* (*tensorMulScalar)(Tensor*, double scalar);
  void (*tensorMulScalar_)(Tensor*, double scalar);
  void (*tensorRecordStream)(Tensor*, Stream stream);
  void (*tensorCopy_)(Tensor* dst, Tensor* src);
  void (*tensorSumOut)(Tensor* dst, Tensor* src, int dim);
  void (*tensorAmaxOut)(Tensor* dst, Tensor* src, int dim);
  void (*tensorAminOut)(Tensor* dst, Tensor* src, int dim);

  size_t (*dtypeSize)(DType dtype);
  void (*registerFreeMemoryCallback)();

  void (*c10dStoreSet)(void* store, std::string_view key, const std::vector<uint8_t>& value);
  std::vector<uint8_t> (*c10dStoreGet)(void* store, std::string_view key);
  void (*c10dStoreWait)(void* store, std::span<const std::string> keys);

  void (*checkSignals)();
};
static_assert(sizeof(WrapperApi) == 38 * sizeof(void*), "WrapperApi must keep the reference's 38 slots");

/* A slot outside the hot path.  Whatever the reference's signature for it, the function it
 * points at reads no argument and leaves by throwing, which is safe to call through any
 * function-pointer type under the x86-64 C++ ABI. */
using OffPath = void (*)();

/* What the core offers (api/moodist_api.h:133-258). */
struct CoreApi {
  uint64_t magic;

  /* store :137-147, internal allocator :150-152, buffers and serializer :159-167,
   * CPU allocator :172-173, device allocator :176-186 -- 29 slots */
  OffPath createStore, storeDestroy, storeClose, storeSet, storeGet, storeCheck, storeWait;
  OffPath internalAlloc, internalFree, internalAllocSize;
  OffPath bufferAllocate, serializeBufferPtr, serializeBufferSize, bufferSetSize, bufferDestroy;
  OffPath serializeObjectImpl, deserializeObjectImpl;
  OffPath cpuAllocatorAlloc, cpuAllocatorFree;
  OffPath createCudaAllocatorImpl, setCudaAllocatorImpl, cudaAllocatorImplAllocate, cudaAllocatorImplFree,
      cudaAllocatorImplRecordStream, cudaAllocatorImplGetDevice, allocatorOwns, allocatorMappedRegion,
      allocatorAddFreeCallback, allocatorRemoveFreeCallback;

  /* process group :189-197 */
  api::ProcessGroupHandle (*createProcessGroup)(void* c10dStore, int rank, int size);
  void (*processGroupDestroy)(api::ProcessGroup*);
  void (*processGroupShutdown)(api::ProcessGroup*);
  int (*processGroupRank)(api::ProcessGroup*);
  int (*processGroupSize)(api::ProcessGroup*);
  bool (*processGroupGetPreferKernelLess)(api::ProcessGroup*);
  void (*processGroupSetPreferKernelLess)(api::ProcessGroup*, bool value);
  int64_t (*processGroupGetOption)(api::ProcessGroup*, const char* name);
  void (*processGroupSetOption)(api::ProcessGroup*, const char* name, int64_t value);

  /* collectives of the path :200-204 */
  void (*processGroupAllGather)(api::ProcessGroup*, TensorPtr& output, const TensorPtr& input, Stream stream);
  void (*processGroupReduceScatter)(api::ProcessGroup*, TensorPtr& output, const TensorPtr& input, ReduceOp reduceOp,
      Stream stream, float premulValue);
  void (*processGroupAllreduce)(api::ProcessGroup*, TensorPtr& tensor, ReduceOp reduceOp, Stream stream,
      float premulValue);
  /* :205-214 */
  OffPath processGroupBroadcast, processGroupReduce;
  void (*processGroupBarrier)(api::ProcessGroup*);
  OffPath processGroupScatter, processGroupGather, processGroupAllToAll;
  void (*processGroupCudaBarrier)(api::ProcessGroup*, Stream stream);

  /* queues :217-240 -- 13 slots */
  OffPath processGroupMakeQueue, processGroupMakeQueueMulti;
  OffPath queueDestroy, queueGet, queuePut, queueQsize, queueWait, queueTransactionBegin, queueTransactionCancel,
      queueTransactionCommit, queueName;
  OffPath queueWorkDestroy, queueWorkWait;

  /* futures and compiled ops :243-255 */
  void (*futureDestroy)(api::Future*);
  void (*futureWait)(api::Future*, Stream stream);
  bool (*futureGetResult)(api::Future*, TensorPtr* outTensor);
  void (*customOpDestroy)(api::CustomOp*);
  api::FutureHandle (*customOpCall)(api::CustomOp*, TensorPtr* inputs, size_t nInputs, TensorPtr* outputs,
      size_t nOutputs, Stream stream);
  api::CustomOpHandle (*compileOpFull)(api::ProcessGroup*, const int* shape, size_t ndim, DType dtype,
      const int* inputRanks, const int* inputOffsets, const int* inputShapes, size_t nInputs, const int* outputRanks,
      const int* outputOffsets, const int* outputShapes, size_t nOutputs);

  /* profiling :257-258 */
  OffPath setProfilingEnabled, getProfilingEnabled;
};
static_assert(sizeof(CoreApi) == 8 + 69 * sizeof(void*), "CoreApi must keep the reference's 69 slots");
static_assert(offsetof(CoreApi, createProcessGroup) == 8 + 29 * sizeof(void*));
static_assert(offsetof(CoreApi, processGroupAllGather) == 8 + 38 * sizeof(void*));
static_assert(offsetof(CoreApi, futureDestroy) == 8 + 61 * sizeof(void*));
static_assert(offsetof(CoreApi, compileOpFull) == 8 + 66 * sizeof(void*));

} // namespace moodist

extern "C" {
/*
 * api/moodist_api.h:265-271.  Returns NULL unless expectedVersion == kMoodistApiVersion;
 * otherwise keeps a copy of *wrapperApi and returns the core's table, whose `magic` the caller
 * compares with its own kMoodistBuildMagic.
 */
__attribute__((visibility("default"))) moodist::CoreApi* moodistGetApi(uint32_t expectedVersion,
    const moodist::WrapperApi* wrapperApi);

/*
 * Two additions beside the reference's table, for what the single-process world adds (no
 * counterpart in the reference).  moodistGroupCHandle: the moodist_pg* (moodist_core.h) behind
 * a group made by createProcessGroup, for the plain C functions that have no slot in the table
 * (moodist_pg_stage_input, moodist_pg_all_gather_list, moodist_pg_last_work,
 * moodist_pg_keep_alive).  moodistOpCHandle: the moodist_op* behind a compiled op, for the plan
 * inspection functions (moodist_op_plan_*); borrowed, valid while the op lives.
 */
__attribute__((visibility("default"))) struct moodist_pg* moodistGroupCHandle(moodist::api::ProcessGroup* group);
__attribute__((visibility("default"))) struct moodist_op* moodistOpCHandle(moodist::api::CustomOp* op);
}

#endif /* MOODIST_PLUGIN_H */
