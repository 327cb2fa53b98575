// Host side of the hot path: per-collective validation, the in-process
// rendezvous that stands in for the reference's peer address exchange, and
// the launches through the thin C ABI of the kernel library.
//
// Follows ProcessGroupImpl in the reference (core/processgroup.cc): all_gather
// :1059-1284, reduce_scatter :1290-1668, allreduce :1674-1722, compileOpFull
// :2761-3104 / :3259-3290, customOp :3172-3256, options :334-340 / :2455-2488.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "moodist_core.h"
#include "moodist_hip.h"
#include "planner.h"

namespace moodist {

class World;

enum class Kind : int {
  all_gather = 0,
  reduce_scatter = 1,
  custom = 2,
  all_gather_many = 3,
  reduce_scatter_many = 4,
  allreduce = 5,      // input = output = the tensor (or its padded temporary); bytes = one chunk
  allreduce_many = 6, // inputs = outputs = the tensors
};

// What one rank brought to a collective.
struct Posting {
  bool arrived = false;
  bool wants_output = false;
  moodist_tensor input{};
  moodist_tensor output{};
  std::vector<moodist_tensor> inputs;  // custom op; all_gather or reduce_scatter of a list of tensors
  std::vector<moodist_tensor> outputs; // custom op; all_gather into one tensor per rank; all_gather or reduce_scatter of a list
  // reduce_scatter: the rank's chunk is reduced in pieces of this many bytes (0 = in one piece)
  size_t chunk_bytes = 0;
  bool kernel_less = false;   // this rank asked for the copy-engine form of all_gather
  bool has_copy_back = false; // allreduce through a padded temporary
  moodist_tensor copy_back{};
  void* stream = nullptr;
  // Whatever must stay alive until this rank's buffers have been read by the launches of the
  // collective (tensor references, snapshot buffers); dropped right after the launches are
  // enqueued, as the reference ties lifetime to the operation (core/processgroup.cc:3239-3245).
  std::vector<std::shared_ptr<void>> keep;
};

using Keep = std::vector<std::shared_ptr<void>>;

// Device memory for snapshots, supplied by whoever loaded the core (the reference's core
// allocates through the wrapper's caching allocator the same way, api/moodist_api.h:71-74).
struct DeviceAllocator {
  void* (*alloc)(size_t bytes, void** cleanup, void* stream, int device) = nullptr;
  void (*free)(void* cleanup) = nullptr;
};

struct Collective {
  Kind kind;
  uint64_t seq;
  int reduce_op = 0;
  float premul = 1.0f;
  size_t bytes = 0; // per-rank chunk
  int dtype = 0;
  uint32_t op_id = 0;
  int arrived = 0;
  bool launched = false;
  std::string error; // set if the launch failed; reported to every waiter
  std::vector<Posting> post;
};

struct Options { // core/processgroup.cc:334-340
  bool preferKernelLess = false;
  bool forceKernelLess = false;
  int64_t numChunks = -1;
  int64_t chunkSize = -1;
  int64_t method = -1;
  // Not in the reference: copy every posted input at the call's position in the rank's stream,
  // so that the collective reads the values of call time even though it is launched later.
  bool snapshotInputs = false;
};

// A rank's transfers as the kernel library has prepared them (mdh_copy_plan): made at the op's
// first launch, replayed by every later one with only the tensors' addresses filled in.
struct PreparedTransfers {
  mdh_copy_plan* plan = nullptr;
  // base table of the plan: first the source tensors in order of first use, then this rank's outputs
  struct Source {
    uint32_t rank, input;
  };
  std::vector<Source> sources;
  size_t n_outputs = 0;
  std::vector<const void*> bases; // scratch for a launch (launches are serialized by the world's mutex)
  ~PreparedTransfers();
};

struct CompiledOp {
  uint32_t id;
  int dtype;
  size_t itemsize;
  std::vector<RankPlan> plans; // every rank's, computed identically by every rank
  PlanWire wire;               // wire[sender][receiver]
  size_t ndim = 0;
  std::vector<std::unique_ptr<PreparedTransfers>> prepared; // per rank, filled at the first launch
};

class ProcessGroup {
public:
  ProcessGroup(World* world, int rank, int size) : world(world), rank(rank), size(size) {}

  // `keep` rides with the posting and is released once the collective's launches are enqueued.
  std::shared_ptr<Collective> all_gather(const moodist_tensor* output, const moodist_tensor& input, void* stream,
      Keep keep = {});
  std::shared_ptr<Collective> all_gather_list(const moodist_tensor* outputs, size_t n_outputs,
      const moodist_tensor& input, void* stream, Keep keep = {});
  // n all_gathers as one collective: outputs[t] receives every rank's inputs[t] (outputs may be
  // null for a rank that only contributes)
  std::shared_ptr<Collective> all_gather_many(const moodist_tensor* outputs, const moodist_tensor* inputs, size_t n,
      void* stream, Keep keep = {});
  std::shared_ptr<Collective> reduce_scatter(const moodist_tensor* output, const moodist_tensor& input, int reduce_op,
      void* stream, float premul, Keep keep = {});
  // n reduce_scatters as one collective: outputs[t] receives this rank's chunk of every rank's
  // inputs[t], reduced (outputs may be null for a rank that only contributes); one element type
  std::shared_ptr<Collective> reduce_scatter_many(const moodist_tensor* outputs, const moodist_tensor* inputs, size_t n,
      int reduce_op, void* stream, float premul, Keep keep = {});
  std::shared_ptr<Collective> allreduce(const moodist_tensor& tensor, const moodist_tensor* scratch, int reduce_op,
      void* stream, float premul, Keep keep = {});
  // n in-place allreduces of one element type whose element counts the group size divides, as
  // one collective
  std::shared_ptr<Collective> allreduce_many(const moodist_tensor* tensors, size_t n, int reduce_op, void* stream,
      float premul, Keep keep = {});
  // allreduce whose padded temporary is this rank's slice of the kernel library's fixed
  // workspace (mdh_static_workspace) instead of a tensor from the caller
  std::shared_ptr<Collective> allreduce_static(const moodist_tensor& tensor, int reduce_op, void* stream, float premul,
      Keep keep = {});
  std::shared_ptr<CompiledOp> compile_op_full(const Dims& shape, int dtype, const std::vector<SliceSpec>& inputs,
      const std::vector<SliceSpec>& outputs);
  std::shared_ptr<Collective> custom_op(const std::shared_ptr<CompiledOp>& op, const moodist_tensor* inputs,
      size_t n_inputs, const moodist_tensor* outputs, size_t n_outputs, void* stream, Keep keep = {});

  int64_t get_option(const std::string& name) const;
  void set_option(const std::string& name, int64_t value);

  World* const world;
  const int rank;
  const int size;
  Options options;
  std::shared_ptr<Collective> last; // the collective this rank posted most recently

private:
  std::shared_ptr<Collective> post_next(Kind kind, Posting p, int reduce_op, float premul, size_t bytes, int dtype,
      uint32_t op_id, const std::shared_ptr<CompiledOp>& op);
  std::shared_ptr<Collective> all_gather_impl(const moodist_tensor* output, const moodist_tensor& input, void* stream,
      const moodist_tensor* copy_back, Keep keep);
  // snapshot_inputs: replaces input.data by a copy made now on `stream`; the copy joins `keep`
  void snapshot(moodist_tensor& input, void* stream, Keep& keep);
  bool internal_input = false; // the second half of an allreduce: its input does not exist yet
  // the pieces a reduce_scatter's chunk of `bytes` is reduced in, from the options (0 = one piece)
  size_t chunk_bytes_for(size_t bytes) const;
  std::weak_ptr<Collective> static_user; // the last collective that reads this rank's workspace slice

  // "Concurrent use of process group detected" guard (core/processgroup.cc:172-183)
  struct Busy {
    explicit Busy(ProcessGroup& pg);
    ~Busy();
    ProcessGroup& pg;
  };
  std::mutex busy;
  uint64_t next_seq = 0;
  uint32_t next_op_id = 1;
};

// The node: `size` local ranks of one group sharing one device.
class World {
public:
  World(int size, int device);
  ~World();

  ProcessGroup* group(int rank) {
    return groups.at((size_t)rank).get();
  }

  // Posts `p` for (kind, seq); launches when the last rank arrives.  Throws if the ranks
  // disagree about what collective number `seq` is (the reference aborts on this,
  // core/cputhread.h:100-112).
  // `taken`, if given, is set once the posting has been accepted (before any launch).
  std::shared_ptr<Collective> post(Kind kind, uint64_t seq, int rank, Posting p, int reduce_op, float premul,
      size_t bytes, int dtype, uint32_t op_id, const std::shared_ptr<CompiledOp>& op, bool* taken = nullptr);

  // Adds `held` to what rank `rank` keeps alive for collective `c`; if the collective has
  // launched already, `held` is simply dropped.
  void attach(Collective& c, int rank, std::shared_ptr<void> held);

  const int size;
  const int device;
  DeviceAllocator allocator; // empty unless the loader supplied one
  // how many copy-engine calls the kernel-less all_gathers of this world have made so far
  uint64_t kernel_less_copies_1d = 0, kernel_less_copies_2d = 0;

private:
  void launch(Collective& c, const std::shared_ptr<CompiledOp>& op);
  // the launches of one collective of any kind but the allreduces, streams already ordered
  void run(Collective& c, const std::shared_ptr<CompiledOp>& op);
  // an allreduce: one launch for all ranks when they share a stream, else its two halves
  void run_allreduce(Collective& c);
  void order_streams_before(Collective& c);
  void order_streams_after(Collective& c);

  std::mutex mutex;
  std::vector<std::unique_ptr<ProcessGroup>> groups;
  std::map<uint64_t, std::shared_ptr<Collective>> pending;
  std::vector<void*> events; // one per rank, created on first cross-stream use
};

size_t dtype_size(int dtype);

// The copy-engine form of all_gather groups source ranks whose buffers are evenly spaced into
// one 2-D copy, as the reference groups the sources a peer holds into Copy2d{offset, length,
// pitch, num} runs for cuMemcpy2DAsync (core/processgroup.cc:114-119, :618-704, :806-820).
// A run is ranks first .. first+count-1 whose source addresses advance by src_pitch bytes
// (>= bytes); count == 1 is a plain 1-D copy.  Ranks whose source already is its place in the
// destination (in_place[j]) belong to no run.
struct GatherRun {
  size_t first;
  size_t count;
  size_t src_pitch;
};
std::vector<GatherRun> gather_runs(const std::vector<const void*>& srcs, const std::vector<bool>& in_place,
    size_t bytes);

} // namespace moodist
