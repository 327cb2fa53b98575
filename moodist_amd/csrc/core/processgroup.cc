#include "processgroup.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>

#include "hip_loader.h"

namespace moodist {

namespace {

// MOODIST_LOG_LEVEL = error | info | verbose | debug (the reference's variable and levels,
// core/logging.h:59-85); at "debug" every launch is reported on stderr.
int log_level() {
  static const int level = [] {
    const char* v = std::getenv("MOODIST_LOG_LEVEL");
    if (!v) {
      return 1;
    }
    if (!std::strcmp(v, "debug")) {
      return 4;
    }
    if (!std::strcmp(v, "verbose")) {
      return 3;
    }
    if (!std::strcmp(v, "info")) {
      return 2;
    }
    return 1;
  }();
  return level;
}

void log_debug(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void log_debug(const char* fmt, ...) {
  if (log_level() < 4) {
    return;
  }
  va_list ap;
  va_start(ap, fmt);
  std::fputs("moodist debug: ", stderr);
  std::vfprintf(stderr, fmt, ap);
  std::fputc('\n', stderr);
  va_end(ap);
}

#define MD_CHECK(cond)                                                                             \
  do {                                                                                             \
    if (!(cond)) {                                                                                 \
      throw std::runtime_error(std::string("moodist: check failed: " #cond " (") + __FILE__ + ":" + \
                               std::to_string(__LINE__) + ")");                                    \
    }                                                                                              \
  } while (0)

// dtypes the reduction kernels take: toInternalDtype (core/processgroup.cc:264-279) plus
// float16, which the reference's table lacks
void check_reduce_dtype(int dtype) {
  switch (dtype) {
  case MDH_DTYPE_FLOAT32:
  case MDH_DTYPE_FLOAT64:
  case MDH_DTYPE_INT32:
  case MDH_DTYPE_INT64:
  case MDH_DTYPE_BFLOAT16:
  case MDH_DTYPE_FLOAT16:
    return;
  default:
    throw std::runtime_error("Unsupported dtype for reduce operation");
  }
}

// toInternalReduction (core/processgroup.cc:282-296)
void check_reduce_op(int op) {
  switch (op) {
  case MDH_OP_SUM:
  case MDH_OP_PREMUL_SUM:
  case MDH_OP_AVG:
  case MDH_OP_MIN:
  case MDH_OP_MAX:
    return;
  default:
    throw std::runtime_error("Unsupported reduce operation");
  }
}

// AVG and PREMUL_SUM are defined for floating element types only (core/processgroup.cc:1315-1316,
// :1340-1344: a multiply by 1/size or by the factor)
void check_reduce_request(int dtype, int reduce_op) {
  check_reduce_dtype(dtype);
  check_reduce_op(reduce_op);
  const bool floating = dtype == MDH_DTYPE_FLOAT32 || dtype == MDH_DTYPE_FLOAT64 || dtype == MDH_DTYPE_BFLOAT16 ||
                        dtype == MDH_DTYPE_FLOAT16;
  if ((reduce_op == MDH_OP_AVG || reduce_op == MDH_OP_PREMUL_SUM) && !floating) {
    throw std::runtime_error("Unsupported reduce operation");
  }
}

void check_device_tensor(const moodist_tensor& t, int device, const char* what) {
  if (!t.contiguous) {
    throw std::runtime_error(std::string("moodist: ") + what + " must be contiguous");
  }
  if (t.device < 0) {
    throw std::runtime_error(std::string("moodist: ") + what +
                             " is a CPU tensor; this build runs the GPU path only (no CPU fallback)");
  }
  if (t.device != device) {
    throw std::runtime_error(std::string("moodist: ") + what + " is on device " + std::to_string(t.device) +
                             ", the group is on device " + std::to_string(device));
  }
  MD_CHECK(t.numel >= 0 && t.itemsize > 0);
  MD_CHECK(t.numel == 0 || t.data != nullptr);
}

size_t bytes_of(const moodist_tensor& t) {
  return (size_t)t.numel * (size_t)t.itemsize;
}

// A rank's call on a capturing stream is refused when it is made, if the runtime is loaded by
// then (it is from the first launch on); World::launch asks again for every rank's stream
// before anything is enqueued, which also covers a process whose first collective is captured.
void refuse_capture_early(void* stream, const char* what) {
  if (hip_loaded()) {
    refuse_capture(stream, what);
  }
}

} // namespace

size_t dtype_size(int dtype) {
  switch (dtype) {
  case 0:  // UInt8
  case 1:  // Int8
  case 11: // Bool
    return 1;
  case 2: // Int16
  case MDH_DTYPE_FLOAT16:
  case MDH_DTYPE_BFLOAT16:
    return 2;
  case MDH_DTYPE_INT32:
  case MDH_DTYPE_FLOAT32:
    return 4;
  case MDH_DTYPE_INT64:
  case MDH_DTYPE_FLOAT64:
    return 8;
  default:
    throw std::runtime_error("moodist: unsupported dtype " + std::to_string(dtype));
  }
}

// ---------------------------------------------------------------- ProcessGroup

ProcessGroup::Busy::Busy(ProcessGroup& pg) : pg(pg) {
  if (!pg.busy.try_lock()) {
    throw std::runtime_error("Concurrent use of process group detected - this is not supported. Moodist process "
                             "groups are not thread-safe.");
  }
}

ProcessGroup::Busy::~Busy() {
  pg.busy.unlock();
}

int64_t ProcessGroup::get_option(const std::string& name) const {
  if (name == "prefer_kernel_less") {
    return options.preferKernelLess ? 1 : 0;
  } else if (name == "force_kernel_less") {
    return options.forceKernelLess ? 1 : 0;
  } else if (name == "num_chunks") {
    return options.numChunks;
  } else if (name == "chunk_size") {
    return options.chunkSize;
  } else if (name == "method") {
    return options.method;
  } else if (name == "snapshot_inputs") {
    return options.snapshotInputs ? 1 : 0;
  } else if (name == "kernel_less_copies_1d") { // read-only counters of the world
    return (int64_t)world->kernel_less_copies_1d;
  } else if (name == "kernel_less_copies_2d") {
    return (int64_t)world->kernel_less_copies_2d;
  }
  throw std::runtime_error("Unknown option: " + name);
}

void ProcessGroup::set_option(const std::string& name, int64_t value) {
  if (name == "prefer_kernel_less") {
    options.preferKernelLess = value != 0;
  } else if (name == "force_kernel_less") {
    options.forceKernelLess = value != 0;
  } else if (name == "num_chunks") {
    if (value < -1 || value == 0 || value > 65535) {
      throw std::runtime_error("moodist: num_chunks takes -1 (auto) or 1..65535, not " + std::to_string(value));
    }
    options.numChunks = value;
  } else if (name == "chunk_size") {
    if (value < -1 || value == 0) {
      throw std::runtime_error("moodist: chunk_size takes -1 (auto) or a number of bytes, not " + std::to_string(value));
    }
    options.chunkSize = value;
  } else if (name == "method") {
    // -1 = auto, 0 = kernel, 1 = copy, 2 = direct (core/processgroup.cc:339)
    if (value == 1) {
      throw std::runtime_error("moodist: method 1 (copy) stages peers' chunks through the copy engine before reducing "
                               "them; the ranks of a local group are read in place, by method 0 (kernel) or 2 (direct)");
    }
    if (value < -1 || value > 2) {
      throw std::runtime_error("moodist: method takes -1 (auto), 0 (kernel) or 2 (direct), not " + std::to_string(value));
    }
    options.method = value;
  } else if (name == "snapshot_inputs") {
    if (value != 0 && !world->allocator.alloc) {
      throw std::runtime_error("moodist: snapshot_inputs needs a device allocator, which only a core loaded through "
                               "moodistGetApi has (the wrapper's caching allocator)");
    }
    options.snapshotInputs = value != 0;
  } else {
    throw std::runtime_error("Unknown option: " + name);
  }
}

void ProcessGroup::snapshot(moodist_tensor& input, void* stream, Keep& keep) {
  const size_t bytes = bytes_of(input);
  if (!options.snapshotInputs || internal_input || bytes == 0) {
    return;
  }
  refuse_capture(stream, "snapshot_inputs");
  void* cleanup = nullptr;
  void* copy = world->allocator.alloc(bytes, &cleanup, stream, world->device);
  if (!copy) {
    throw std::runtime_error("moodist: could not allocate " + std::to_string(bytes) + " bytes for an input snapshot");
  }
  auto release = world->allocator.free;
  keep.push_back(std::shared_ptr<void>(cleanup, [release](void* c) { release(c); }));
  check_hip(hip().MemcpyAsync(copy, input.data, bytes, kHipMemcpyDeviceToDevice, stream), "hipMemcpyAsync");
  input.data = copy;
}

// Posts `p` as this rank's next collective.  The rank's sequence advances when the world has
// taken the posting -- also when the launches this arrival triggered then failed, since every
// rank has spent that number --, and stays where it was when the posting is refused (the ranks
// disagree about the collective).
std::shared_ptr<Collective> ProcessGroup::post_next(Kind kind, Posting p, int reduce_op, float premul, size_t bytes,
    int dtype, uint32_t op_id, const std::shared_ptr<CompiledOp>& op) {
  bool taken = false;
  struct Advance {
    uint64_t& seq;
    const bool& taken;
    ~Advance() {
      if (taken) {
        ++seq;
      }
    }
  } advance{next_seq, taken};
  return last = world->post(kind, next_seq, rank, std::move(p), reduce_op, premul, bytes, dtype, op_id, op, &taken);
}

std::shared_ptr<Collective> ProcessGroup::all_gather(const moodist_tensor* output, const moodist_tensor& input,
    void* stream, Keep keep) {
  return all_gather_impl(output, input, stream, nullptr, std::move(keep));
}

std::shared_ptr<Collective> ProcessGroup::all_gather_impl(const moodist_tensor* output, const moodist_tensor& input,
    void* stream, const moodist_tensor* copy_back, Keep keep) {
  Busy guard(*this);
  refuse_capture_early(stream, "all_gather");
  check_device_tensor(input, world->device, "all_gather input");
  const size_t bytes = bytes_of(input);
  MD_CHECK(bytes > 0); // core/processgroup.cc:1078
  Posting p;
  p.input = input;
  snapshot(p.input, stream, keep);
  p.keep = std::move(keep);
  p.stream = stream;
  if (output) {
    check_device_tensor(*output, world->device, "all_gather output");
    MD_CHECK(bytes_of(*output) == bytes * (size_t)size); // :1079
    p.output = *output;
    p.wants_output = true;
    if (copy_back) {
      p.copy_back = *copy_back;
      p.has_copy_back = true;
    }
  }
  p.kernel_less = options.forceKernelLess || options.preferKernelLess;
  return post_next(Kind::all_gather, std::move(p), 0, 1.0f, bytes, input.dtype, 0, nullptr);
}

// The list form of all_gather (wrapper/processgroup_wrapper.cc:112-129).  The reference gathers
// into a flat temporary and copies each row out; here every source is copied straight into its
// destination tensor, so no temporary exists.
std::shared_ptr<Collective> ProcessGroup::all_gather_list(const moodist_tensor* outputs, size_t n_outputs,
    const moodist_tensor& input, void* stream, Keep keep) {
  Busy guard(*this);
  refuse_capture_early(stream, "all_gather");
  check_device_tensor(input, world->device, "all_gather input");
  const size_t bytes = bytes_of(input);
  MD_CHECK(bytes > 0);
  if (n_outputs != (size_t)size) {
    throw std::runtime_error("moodist: all_gather needs one output tensor per rank (" + std::to_string(size) +
                             "), got " + std::to_string(n_outputs));
  }
  Posting p;
  p.input = input;
  snapshot(p.input, stream, keep);
  p.keep = std::move(keep);
  p.stream = stream;
  p.wants_output = true;
  for (size_t i = 0; i < n_outputs; ++i) {
    check_device_tensor(outputs[i], world->device, "all_gather output");
    MD_CHECK(outputs[i].dtype == input.dtype);
    MD_CHECK(bytes_of(outputs[i]) == bytes);
    p.outputs.push_back(outputs[i]);
  }
  p.kernel_less = options.forceKernelLess || options.preferKernelLess;
  return post_next(Kind::all_gather, std::move(p), 0, 1.0f, bytes, input.dtype, 0, nullptr);
}

// allgather_into_tensor_coalesced (wrapper/processgroup_wrapper.cc:139-148).  The reference loops
// over the tensors, one collective each; here the list is one collective, and its copies --
// one contiguous segment per tensor and source rank -- go out in as few launches as the kernel's
// segment table allows (64 segments each) instead of one launch per tensor.
std::shared_ptr<Collective> ProcessGroup::all_gather_many(const moodist_tensor* outputs, const moodist_tensor* inputs,
    size_t n, void* stream, Keep keep) {
  Busy guard(*this);
  refuse_capture_early(stream, "all_gather");
  if (n == 0 || n > 0xffffu) {
    throw std::runtime_error("moodist: a coalesced all_gather takes 1..65535 tensors, not " + std::to_string(n));
  }
  Posting p;
  size_t total = 0;
  for (size_t t = 0; t < n; ++t) {
    check_device_tensor(inputs[t], world->device, "all_gather input");
    const size_t bytes = bytes_of(inputs[t]);
    MD_CHECK(bytes > 0); // core/processgroup.cc:1078
    moodist_tensor in = inputs[t];
    snapshot(in, stream, keep);
    p.inputs.push_back(in);
    total += bytes;
    if (outputs) {
      check_device_tensor(outputs[t], world->device, "all_gather output");
      MD_CHECK(bytes_of(outputs[t]) == bytes * (size_t)size); // :1079
      p.outputs.push_back(outputs[t]);
    }
  }
  p.wants_output = outputs != nullptr;
  p.keep = std::move(keep);
  p.stream = stream;
  p.kernel_less = options.forceKernelLess || options.preferKernelLess;
  return post_next(Kind::all_gather_many, std::move(p), 0, 1.0f, total, inputs[0].dtype,
             (uint32_t)n, nullptr);
}

std::shared_ptr<Collective> ProcessGroup::reduce_scatter(const moodist_tensor* output, const moodist_tensor& input,
    int reduce_op, void* stream, float premul, Keep keep) {
  Busy guard(*this);
  refuse_capture_early(stream, "reduce_scatter");
  check_device_tensor(input, world->device, "reduce_scatter input");
  check_reduce_request(input.dtype, reduce_op);
  const size_t in_bytes = bytes_of(input);
  MD_CHECK(in_bytes > 0 && in_bytes % (size_t)size == 0);
  const size_t bytes = in_bytes / (size_t)size;
  MD_CHECK(bytes % (size_t)input.itemsize == 0);
  Posting p;
  if (output) {
    check_device_tensor(*output, world->device, "reduce_scatter output");
    MD_CHECK(output->dtype == input.dtype);   // core/processgroup.cc:1312
    MD_CHECK(bytes_of(*output) == bytes);     // :1325
    p.output = *output;
    p.wants_output = true;
  }
  p.input = input;
  snapshot(p.input, stream, keep);
  p.keep = std::move(keep);
  p.stream = stream;
  p.chunk_bytes = chunk_bytes_for(bytes);
  return post_next(Kind::reduce_scatter, std::move(p), reduce_op, premul, bytes,
             input.dtype, 0, nullptr);
}

// num_chunks / chunk_size / method (core/processgroup.cc:334-340).  The reference cuts the chunk
// a rank reduces for another node into pieces (its "direct" method: per destination and piece,
// send = own (+) peers, core/reduce_scatter_direct.cc:165-177), with
//   numChunks = clamp(bytes / 131072, 1, 4);  chunkSize = roundup(ceil(bytes / numChunks), 4096);
//   numChunks = ceil(bytes / chunkSize)                                   (core/processgroup.cc:1494-1503)
// and stores the three options without reading them.  Here they are honoured: chunk_size (bytes,
// rounded up to 4096) or else num_chunks (through the arithmetic above) cut a reduce_scatter's
// reduction into pieces, and method 2 ("direct") asks for the reference's own piece count when
// neither is set.  Pieces shorter than 16 MiB share launches (mdh_reduce_many).
size_t ProcessGroup::chunk_bytes_for(size_t bytes) const {
  size_t chunk = 0;
  if (options.chunkSize > 0) {
    chunk = ((size_t)options.chunkSize + 4095u) / 4096u * 4096u;
  } else {
    size_t pieces = 0;
    if (options.numChunks > 0) {
      pieces = (size_t)options.numChunks;
    } else if (options.method == 2) {
      pieces = bytes / 131072 < 4 ? bytes / 131072 : 4;
    }
    if (pieces > 1) {
      chunk = ((bytes + pieces - 1) / pieces + 4095u) / 4096u * 4096u;
    }
  }
  return chunk >= bytes ? 0 : chunk;
}

// reduce_scatter_tensor_coalesced (wrapper/processgroup_wrapper.cc:159-170).  The reference loops
// over the tensors, one collective and one kernel launch per rank each; here the list is one
// collective and a rank's reductions share launches (mdh_reduce_many).  The whole list is
// checked before anything is posted.
std::shared_ptr<Collective> ProcessGroup::reduce_scatter_many(const moodist_tensor* outputs,
    const moodist_tensor* inputs, size_t n, int reduce_op, void* stream, float premul, Keep keep) {
  Busy guard(*this);
  refuse_capture_early(stream, "reduce_scatter");
  if (n == 0 || n > 0xffffu) {
    throw std::runtime_error("moodist: a coalesced reduce_scatter takes 1..65535 tensors, not " + std::to_string(n));
  }
  size_t total = 0;
  for (size_t t = 0; t < n; ++t) {
    check_device_tensor(inputs[t], world->device, "reduce_scatter input");
    check_reduce_request(inputs[t].dtype, reduce_op);
    if (inputs[t].dtype != inputs[0].dtype) {
      throw std::runtime_error("moodist: the tensors of a coalesced reduce_scatter must have one element type");
    }
    const size_t in_bytes = bytes_of(inputs[t]);
    MD_CHECK(in_bytes > 0 && in_bytes % (size_t)size == 0);
    const size_t bytes = in_bytes / (size_t)size;
    MD_CHECK(bytes % (size_t)inputs[t].itemsize == 0);
    if (outputs) {
      check_device_tensor(outputs[t], world->device, "reduce_scatter output");
      MD_CHECK(outputs[t].dtype == inputs[t].dtype); // core/processgroup.cc:1312
      MD_CHECK(bytes_of(outputs[t]) == bytes);       // :1325
    }
    total += bytes;
  }
  Posting p;
  for (size_t t = 0; t < n; ++t) {
    moodist_tensor in = inputs[t];
    snapshot(in, stream, keep);
    p.inputs.push_back(in);
    if (outputs) {
      p.outputs.push_back(outputs[t]);
    }
  }
  p.wants_output = outputs != nullptr;
  p.keep = std::move(keep);
  p.stream = stream;
  return post_next(Kind::reduce_scatter_many, std::move(p), reduce_op, premul, total,
             inputs[0].dtype, (uint32_t)n, nullptr);
}

// allreduce (core/processgroup.cc:1674-1722): a reduce_scatter into this rank's own chunk of the
// tensor and an all_gather of every rank's chunk; a tensor whose element count the group size
// does not divide goes through a padded temporary (:1694-1720).  One collective here: when the
// last rank arrives, the world either runs those two halves rank by rank or, when the ranks share
// a stream, one launch that reduces every chunk and stores it into every rank's tensor
// (World::run_allreduce).
std::shared_ptr<Collective> ProcessGroup::allreduce(const moodist_tensor& tensor, const moodist_tensor* scratch,
    int reduce_op, void* stream, float premul, Keep keep) {
  Busy guard(*this);
  refuse_capture_early(stream, "allreduce");
  check_device_tensor(tensor, world->device, "allreduce tensor");
  MD_CHECK(tensor.numel > 0); // core/processgroup.cc:1678
  check_reduce_request(tensor.dtype, reduce_op); // before anything is enqueued or posted
  const int64_t n = tensor.numel;
  Posting p;
  p.stream = stream;
  p.wants_output = true;
  p.kernel_less = options.forceKernelLess || options.preferKernelLess;
  size_t bytes = 0; // one chunk
  if (n % size == 0) {
    // in place (:1686-1693)
    bytes = bytes_of(tensor) / (size_t)size;
    p.input = tensor;
    snapshot(p.input, stream, keep); // the reduction then reads the copy; the result still lands in the tensor
    p.output = tensor;
  } else {
    const int64_t padded = (n + size - 1) / size * size;
    if (!scratch) {
      throw std::runtime_error("moodist: allreduce of " + std::to_string(n) + " elements over " + std::to_string(size) +
                               " ranks needs a scratch tensor of " + std::to_string(padded) + " elements");
    }
    check_device_tensor(*scratch, world->device, "allreduce scratch");
    MD_CHECK(scratch->dtype == tensor.dtype && scratch->numel >= padded);
    refuse_capture(stream, "allreduce");
    check_hip(hip().MemcpyAsync(scratch->data, tensor.data, bytes_of(tensor), kHipMemcpyDeviceToDevice, stream),
        "hipMemcpyAsync");
    // the temporary already is a copy made at the call's position in the stream: no snapshot
    moodist_tensor whole = *scratch;
    whole.numel = padded;
    whole.ndim = 1;
    whole.shape[0] = padded;
    bytes = bytes_of(whole) / (size_t)size;
    p.input = whole;
    p.output = whole;
    p.copy_back = tensor; // follows this rank's gather, wherever that gets launched
    p.has_copy_back = true;
  }
  p.chunk_bytes = chunk_bytes_for(bytes);
  p.keep = std::move(keep);
  return post_next(Kind::allreduce, std::move(p), reduce_op, premul, bytes, tensor.dtype, 0,
             nullptr);
}

// allreduce_coalesced (wrapper/processgroup_wrapper.cc:182-191), for the tensors of the list that
// need no padding: the reference runs one allreduce -- a reduce_scatter and an all_gather -- per
// tensor; here the list is one collective (World::run_allreduce).
std::shared_ptr<Collective> ProcessGroup::allreduce_many(const moodist_tensor* tensors, size_t n, int reduce_op,
    void* stream, float premul, Keep keep) {
  Busy guard(*this);
  refuse_capture_early(stream, "allreduce");
  if (n == 0 || n > 0xffffu) {
    throw std::runtime_error("moodist: a coalesced allreduce takes 1..65535 tensors, not " + std::to_string(n));
  }
  // the whole list is checked before anything is posted: a list that is refused leaves nothing
  // pending and the rank's sequence where it was
  size_t total = 0;
  for (size_t t = 0; t < n; ++t) {
    check_device_tensor(tensors[t], world->device, "allreduce tensor");
    MD_CHECK(tensors[t].numel > 0 && tensors[t].numel % size == 0);
    check_reduce_request(tensors[t].dtype, reduce_op);
    if (tensors[t].dtype != tensors[0].dtype) {
      throw std::runtime_error("moodist: the tensors of a coalesced allreduce must have one element type");
    }
    total += bytes_of(tensors[t]) / (size_t)size;
  }
  Posting p;
  for (size_t t = 0; t < n; ++t) {
    moodist_tensor in = tensors[t];
    snapshot(in, stream, keep);
    p.inputs.push_back(in);
    p.outputs.push_back(tensors[t]);
  }
  p.wants_output = true;
  p.kernel_less = options.forceKernelLess || options.preferKernelLess;
  p.keep = std::move(keep);
  p.stream = stream;
  return post_next(Kind::allreduce_many, std::move(p), reduce_op, premul, total,
             tensors[0].dtype, (uint32_t)n, nullptr);
}

std::shared_ptr<Collective> ProcessGroup::allreduce_static(const moodist_tensor& tensor, int reduce_op, void* stream,
    float premul, Keep keep) {
  check_device_tensor(tensor, world->device, "allreduce tensor");
  MD_CHECK(tensor.numel > 0);
  // No allocation of any kind in this call: the option snapshot_inputs, which copies a posted
  // input into memory from the wrapper's allocator, is not applied (the tensor is read when
  // the collective launches).
  struct NoSnapshot {
    bool& flag;
    const bool before;
    explicit NoSnapshot(bool& f) : flag(f), before(f) {
      flag = true;
    }
    ~NoSnapshot() {
      flag = before;
    }
  } no_snapshot{internal_input};
  if (tensor.numel % size == 0) {
    return allreduce(tensor, nullptr, reduce_op, stream, premul, std::move(keep)); // in place, no temporary
  }
  const HipRuntime& h = hip();
  // the workspace's address is per device: ask with the group's device current
  int current = -1;
  check_hip(h.GetDevice(&current), "hipGetDevice");
  if (current != world->device) {
    check_hip(h.SetDevice(world->device), "hipSetDevice");
  }
  void* base = nullptr;
  size_t total = 0;
  const int rc = h.static_workspace(&base, &total);
  if (current != world->device) {
    check_hip(h.SetDevice(current), "hipSetDevice");
  }
  check_mdh(rc);
  // one slice per rank: every rank's temporary is alive at the same time
  const size_t slice = total / (size_t)size / 256 * 256;
  const size_t padded = ((size_t)tensor.numel + (size_t)size - 1) / (size_t)size * (size_t)size;
  const size_t need = padded * (size_t)tensor.itemsize;
  if (need > slice) {
    throw std::runtime_error("moodist: allreduce_static needs " + std::to_string(need) +
                             " bytes for its padded temporary, the fixed workspace gives each of the " +
                             std::to_string(size) + " ranks " + std::to_string(slice) + " bytes (" +
                             std::to_string(total) + " in all)");
  }
  // This call's copy into the slice is enqueued now; a previous call's kernels read the slice
  // when ITS last rank posts.  Until then the slice is taken.
  if (auto previous = static_user.lock()) {
    if (!previous->launched && previous->error.empty()) {
      throw std::runtime_error("moodist: allreduce_static: this rank's previous allreduce_static is still waiting "
                               "for other ranks and holds the workspace");
    }
  }
  moodist_tensor scratch = tensor;
  scratch.data = (char*)base + (size_t)rank * slice;
  scratch.numel = (int64_t)padded;
  scratch.ndim = 1;
  scratch.shape[0] = (int64_t)padded;
  auto c = allreduce(tensor, &scratch, reduce_op, stream, premul, std::move(keep));
  static_user = c;
  return c;
}

std::shared_ptr<CompiledOp> ProcessGroup::compile_op_full(const Dims& shape, int dtype,
    const std::vector<SliceSpec>& inputs, const std::vector<SliceSpec>& outputs) {
  Busy guard(*this);
  if (shape.size() > MDH_MAX_DIMS) {
    // core/processgroup.cc:3138-3140
    throw std::runtime_error("moodist.compile_op_full: ndim " + std::to_string(shape.size()) +
                             " is too large and not supported!");
  }
  auto op = std::make_shared<CompiledOp>();
  op->id = next_op_id++;
  op->dtype = dtype;
  op->itemsize = dtype_size(dtype);
  op->ndim = shape.size();
  op->plans = plan_redistribution(size, shape, op->itemsize, inputs, outputs, &op->wire);
  // The reference sizes a rank's outputs largest-first (:2999-3004) but numbers its reads by
  // listing order (:2974); the two agree only when listing order is already largest-first.
  for (int r = 0; r < size; ++r) {
    size_t prev = SIZE_MAX;
    for (const SliceSpec& o : outputs) {
      if (o.rank == r) {
        const size_t n = dims_numel(o.shape);
        if (n > prev) {
          throw std::runtime_error("moodist.compile_op_full: a rank's outputs must be listed largest first");
        }
        prev = n;
      }
    }
  }
  return op;
}

std::shared_ptr<Collective> ProcessGroup::custom_op(const std::shared_ptr<CompiledOp>& op,
    const moodist_tensor* inputs, size_t n_inputs, const moodist_tensor* outputs, size_t n_outputs, void* stream,
    Keep keep) {
  Busy guard(*this);
  refuse_capture_early(stream, "custom op");
  const RankPlan& plan = op->plans[(size_t)rank];
  // core/processgroup.cc:3180-3185, :3205-3216
  if (n_inputs != plan.inputs.size()) {
    throw std::runtime_error("moodist: custom op expected different number of inputs");
  }
  if (n_outputs != plan.outputs.size()) {
    throw std::runtime_error("moodist: custom op expected different number of outputs");
  }
  Posting p;
  p.keep = std::move(keep);
  p.stream = stream;
  p.wants_output = n_outputs > 0;
  for (size_t i = 0; i < n_inputs; ++i) {
    if (!inputs[i].contiguous) {
      throw std::runtime_error("Got a non-contiguous tensor. All tensors must be contiguous.");
    }
    if (bytes_of(inputs[i]) != plan.inputs[i]) {
      throw std::runtime_error("moodist: custom op input has wrong size");
    }
    check_device_tensor(inputs[i], world->device, "custom op input");
    p.inputs.push_back(inputs[i]);
  }
  for (size_t i = 0; i < n_outputs; ++i) {
    if (!outputs[i].contiguous) {
      throw std::runtime_error("Got a non-contiguous tensor. All tensors must be contiguous.");
    }
    if (bytes_of(outputs[i]) != plan.outputs[i]) {
      throw std::runtime_error("moodist: custom op output has wrong size");
    }
    check_device_tensor(outputs[i], world->device, "custom op output");
    p.outputs.push_back(outputs[i]);
  }
  return post_next(Kind::custom, std::move(p), 0, 1.0f, 0, op->dtype, op->id, op);
}

// ---------------------------------------------------------------- kernel-less runs

std::vector<GatherRun> gather_runs(const std::vector<const void*>& srcs, const std::vector<bool>& in_place,
    size_t bytes) {
  std::vector<GatherRun> runs;
  const size_t n = srcs.size();
  // a 2-D copy's pitches are kept inside 31 bits; anything sparser goes rank by rank
  const uintptr_t max_pitch = 0x7fffffffu;
  size_t i = 0;
  while (i < n) {
    if (in_place[i]) {
      ++i;
      continue;
    }
    GatherRun run{i, 1, bytes};
    if (i + 1 < n && !in_place[i + 1]) {
      const uintptr_t a = (uintptr_t)srcs[i], b = (uintptr_t)srcs[i + 1];
      if (b > a && b - a >= bytes && b - a <= max_pitch) {
        const uintptr_t pitch = b - a;
        size_t k = i + 1;
        while (k + 1 < n && !in_place[k + 1] && (uintptr_t)srcs[k + 1] > (uintptr_t)srcs[k] &&
               (uintptr_t)srcs[k + 1] - (uintptr_t)srcs[k] == pitch) {
          ++k;
        }
        run.count = k - i + 1;
        run.src_pitch = (size_t)pitch;
      }
    }
    runs.push_back(run);
    i += run.count;
  }
  return runs;
}

// ---------------------------------------------------------------- prepared transfers

PreparedTransfers::~PreparedTransfers() {
  if (plan) {
    hip().copy_plan_destroy(plan);
  }
}

namespace {

std::unique_ptr<PreparedTransfers> prepare_transfers(const RankPlan& plan, size_t itemsize) {
  auto pt = std::make_unique<PreparedTransfers>();
  pt->n_outputs = plan.outputs.size();
  std::vector<mdh_box> boxes(plan.transfers.size());
  std::vector<int32_t> src_slots(plan.transfers.size()), dst_slots(plan.transfers.size());
  for (size_t i = 0; i < plan.transfers.size(); ++i) {
    const Transfer& t = plan.transfers[i];
    size_t slot = 0;
    for (; slot < pt->sources.size(); ++slot) {
      if (pt->sources[slot].rank == t.srcRank && pt->sources[slot].input == t.srcInput) {
        break;
      }
    }
    if (slot == pt->sources.size()) {
      pt->sources.push_back({t.srcRank, t.srcInput});
    }
    src_slots[i] = (int32_t)slot;
    MD_CHECK(t.dstOutput < pt->n_outputs);
    mdh_box& b = boxes[i];
    const size_t nd = t.shape.size();
    b.ndim = (int32_t)nd;
    b.reserved = 0;
    int64_t ss = 1, ds = 1;
    for (size_t d = nd; d-- > 0;) {
      b.shape[d] = t.shape[d];
      b.src_strides[d] = ss;
      b.dst_strides[d] = ds;
      ss *= t.srcShape[d];
      ds *= t.dstShape[d];
    }
    // byte offsets from the tensors' first bytes; the addresses come with each call
    b.src = (const void*)(uintptr_t)(linear_offset(t.srcOffset, t.srcShape) * itemsize);
    b.dst = (void*)(uintptr_t)(linear_offset(t.dstOffset, t.dstShape) * itemsize);
  }
  for (size_t i = 0; i < plan.transfers.size(); ++i) {
    dst_slots[i] = (int32_t)(pt->sources.size() + plan.transfers[i].dstOutput);
  }
  const int nbases = (int)(pt->sources.size() + pt->n_outputs);
  check_mdh(hip().copy_plan_create(boxes.data(), src_slots.data(), dst_slots.data(), (int)boxes.size(), (int)itemsize,
      nbases, &pt->plan));
  pt->bases.assign((size_t)nbases, nullptr);
  return pt;
}

} // namespace

// ---------------------------------------------------------------- World

World::World(int size, int device) : size(size), device(device) {
  if (size < 1 || size > MDH_MAX_SOURCES) {
    throw std::runtime_error("moodist: a local world holds 1.." + std::to_string(MDH_MAX_SOURCES) + " ranks, not " +
                             std::to_string(size));
  }
  for (int r = 0; r < size; ++r) {
    groups.push_back(std::make_unique<ProcessGroup>(this, r, size));
  }
  events.assign((size_t)size, nullptr);
}

World::~World() {
  for (void* e : events) {
    if (e) {
      hip().EventDestroy(e);
    }
  }
}

std::shared_ptr<Collective> World::post(Kind kind, uint64_t seq, int rank, Posting p, int reduce_op, float premul,
    size_t bytes, int dtype, uint32_t op_id, const std::shared_ptr<CompiledOp>& op, bool* taken) {
  std::lock_guard<std::mutex> l(mutex);
  std::shared_ptr<Collective>& slot = pending[seq];
  if (!slot) {
    slot = std::make_shared<Collective>();
    slot->kind = kind;
    slot->seq = seq;
    slot->reduce_op = reduce_op;
    slot->premul = premul;
    slot->bytes = bytes;
    slot->dtype = dtype;
    slot->op_id = op_id;
    slot->post.resize((size_t)size);
  }
  std::shared_ptr<Collective> c = slot;
  if (c->kind != kind || c->reduce_op != reduce_op || c->bytes != bytes || c->dtype != dtype || c->op_id != op_id ||
      c->premul != premul) {
    // the reference detects this across ranks and aborts (CHECK_DYN, core/cputhread.h:100-112)
    throw std::runtime_error("moodist: rank " + std::to_string(rank) + " issued collective #" + std::to_string(seq) +
                             " with a different operation, size, dtype or reduction than another rank did");
  }
  Posting& mine = c->post[(size_t)rank];
  MD_CHECK(!mine.arrived);
  p.arrived = true;
  mine = std::move(p);
  ++c->arrived;
  if (taken) {
    *taken = true;
  }
  if (c->arrived == size) {
    pending.erase(seq);
    // what the ranks asked to keep alive is let go once the launches are enqueued (or have
    // failed): from then on stream order protects the buffers
    struct Release {
      Collective& c;
      ~Release() {
        for (Posting& q : c.post) {
          q.keep.clear();
        }
      }
    } release{*c};
    try {
      launch(*c, op);
    } catch (const std::exception& e) {
      c->error = e.what();
      c->launched = true;
      throw;
    }
    c->launched = true;
  }
  return c;
}

void World::attach(Collective& c, int rank, std::shared_ptr<void> held) {
  std::lock_guard<std::mutex> l(mutex);
  if (!c.launched && rank >= 0 && rank < size) {
    c.post[(size_t)rank].keep.push_back(std::move(held));
  }
}

// A rank's launch reads buffers that other ranks' streams may still be producing, and later
// work on those streams may overwrite what this launch reads.  With one shared stream (the
// usual case) stream order covers both; otherwise every launch waits for an event recorded
// on each other rank's stream, and every other stream waits for the launches.
void World::order_streams_before(Collective& c) {
  bool same = true;
  for (const Posting& p : c.post) {
    same = same && p.stream == c.post[0].stream;
  }
  if (same) {
    return;
  }
  const HipRuntime& h = hip();
  for (int r = 0; r < size; ++r) {
    if (!events[(size_t)r]) {
      check_hip(h.EventCreateWithFlags(&events[(size_t)r], kHipEventDisableTiming), "hipEventCreateWithFlags");
    }
    check_hip(h.EventRecord(events[(size_t)r], c.post[(size_t)r].stream), "hipEventRecord");
  }
  for (int q = 0; q < size; ++q) {
    if (!c.post[(size_t)q].wants_output) {
      continue;
    }
    for (int r = 0; r < size; ++r) {
      if (c.post[(size_t)r].stream != c.post[(size_t)q].stream) {
        check_hip(h.StreamWaitEvent(c.post[(size_t)q].stream, events[(size_t)r], 0), "hipStreamWaitEvent");
      }
    }
  }
}

void World::order_streams_after(Collective& c) {
  bool same = true;
  for (const Posting& p : c.post) {
    same = same && p.stream == c.post[0].stream;
  }
  if (same) {
    return;
  }
  const HipRuntime& h = hip();
  for (int q = 0; q < size; ++q) {
    if (c.post[(size_t)q].wants_output) {
      check_hip(h.EventRecord(events[(size_t)q], c.post[(size_t)q].stream), "hipEventRecord");
    }
  }
  for (int r = 0; r < size; ++r) {
    for (int q = 0; q < size; ++q) {
      if (c.post[(size_t)q].wants_output && c.post[(size_t)r].stream != c.post[(size_t)q].stream) {
        check_hip(h.StreamWaitEvent(c.post[(size_t)r].stream, events[(size_t)q], 0), "hipStreamWaitEvent");
      }
    }
  }
}

namespace {

// A rank's chunk of this size and less makes a launch that is over in a few microseconds, most
// of them the launch itself; such collectives share launches among the ranks of a stream.
constexpr size_t kSharedLaunchBytes = (size_t)1 << 20;

// The ranks that asked for an output and whose reduction is not cut into pieces, grouped by the
// stream they passed, in rank order.
std::vector<std::vector<int>> ranks_by_stream(const Collective& c) {
  std::vector<std::vector<int>> groups;
  for (size_t q = 0; q < c.post.size(); ++q) {
    const Posting& pq = c.post[q];
    if (!pq.wants_output || pq.chunk_bytes != 0) {
      continue;
    }
    bool placed = false;
    for (std::vector<int>& g : groups) {
      if (c.post[(size_t)g[0]].stream == pq.stream) {
        g.push_back((int)q);
        placed = true;
        break;
      }
    }
    if (!placed) {
      groups.push_back({(int)q});
    }
  }
  return groups;
}

} // namespace

void World::launch(Collective& c, const std::shared_ptr<CompiledOp>& op) {
  if (c.kind == Kind::all_gather_many || c.kind == Kind::reduce_scatter_many || c.kind == Kind::allreduce_many) {
    // the ranks agreed on the number of tensors and their total size (post); now tensor by tensor
    const size_t n = c.post[0].inputs.size();
    for (int j = 0; j < size; ++j) {
      const Posting& pj = c.post[(size_t)j];
      bool same = pj.inputs.size() == n;
      for (size_t t = 0; same && t < n; ++t) {
        same = bytes_of(pj.inputs[t]) == bytes_of(c.post[0].inputs[t]);
      }
      if (!same) {
        throw std::runtime_error("moodist: rank " + std::to_string(j) + " brought a different list of tensors to "
                                 "collective #" + std::to_string(c.seq) + " than rank 0 did");
      }
    }
  }
  const HipRuntime& h = hip();
  int current = -1;
  check_hip(h.GetDevice(&current), "hipGetDevice");
  if (current != device) {
    check_hip(h.SetDevice(device), "hipSetDevice");
  }
  // before anything is enqueued -- an event record on a capturing stream would already be a
  // node of its graph
  for (int r = 0; r < size; ++r) {
    bool seen = false;
    for (int k = 0; k < r; ++k) {
      seen = seen || c.post[(size_t)k].stream == c.post[(size_t)r].stream;
    }
    if (!seen) {
      refuse_capture(c.post[(size_t)r].stream, "collective launch");
    }
  }
  order_streams_before(c);
  log_debug("collective #%llu: launching %s for %d ranks, %zu bytes per rank, dtype %d", (unsigned long long)c.seq,
      c.kind == Kind::reduce_scatter        ? "reduce_scatter"
      : c.kind == Kind::all_gather          ? "all_gather"
      : c.kind == Kind::all_gather_many     ? "all_gather of a list"
      : c.kind == Kind::reduce_scatter_many ? "reduce_scatter of a list"
      : c.kind == Kind::allreduce           ? "allreduce"
      : c.kind == Kind::allreduce_many      ? "allreduce of a list"
                                            : "custom op",
      size, c.bytes, c.dtype);
  if (c.kind == Kind::allreduce || c.kind == Kind::allreduce_many) {
    run_allreduce(c);
  } else {
    run(c, op);
  }
  order_streams_after(c);
  if (current != device && current >= 0) {
    check_hip(h.SetDevice(current), "hipSetDevice");
  }
}

namespace {

// The q-th of `size` equal chunks of a contiguous tensor, as a 1-D tensor.
moodist_tensor chunk_of(const moodist_tensor& t, int q, int size) {
  moodist_tensor chunk = t;
  chunk.numel = t.numel / size;
  chunk.data = (char*)t.data + (size_t)q * (size_t)chunk.numel * (size_t)t.itemsize;
  chunk.ndim = 1;
  chunk.shape[0] = chunk.numel;
  return chunk;
}

} // namespace

// allreduce and allreduce of a list.  Every rank's tensors are addressable here, so when the
// ranks share a stream ONE launch does it all: a job per chunk c (and tensor), sources = every
// rank's chunk c, folded in the order of the rank that owns the chunk (first = c), the result
// stored over every source (mdh_allreduce_many) -- every tensor is read once and written once,
// where reduce_scatter + all_gather read them once, write a chunk, and read and write all other
// chunks again.  Ranks on different streams, pieces (num_chunks / chunk_size / method), the
// copy-engine gather or snapshots of the inputs take the composition: the reduce_scatter of every
// rank, the streams ordered, the all_gather of every rank (core/processgroup.cc:1686-1693).
void World::run_allreduce(Collective& c) {
  const HipRuntime& h = hip();
  const bool list = c.kind == Kind::allreduce_many;
  const size_t n = list ? c.post[0].inputs.size() : 1;
  bool one_launch = true;
  for (const Posting& p : c.post) {
    one_launch = one_launch && p.stream == c.post[0].stream && p.chunk_bytes == 0 && !p.kernel_less;
    for (size_t t = 0; t < n; ++t) {
      one_launch = one_launch && (list ? p.inputs[t].data == p.outputs[t].data : p.input.data == p.output.data);
    }
  }
  if (one_launch) {
    const size_t itemsize = dtype_size(c.dtype);
    const float scale = c.reduce_op == MDH_OP_AVG ? 1.0f / (float)size : c.premul;
    // a job per tensor and chunk, handed over in batches of a few thousand (a long list over
    // many ranks would otherwise need size x size pointers per tensor all at once)
    constexpr size_t kBatchJobs = 4096;
    const size_t per_call = n * (size_t)size < kBatchJobs ? n * (size_t)size : kBatchJobs;
    std::vector<const void*> tables(per_call * (size_t)size);
    std::vector<mdh_reduce_job> jobs(per_call);
    void* stream = c.post[0].stream;
    size_t k = 0;
    for (size_t t = 0; t < n; ++t) {
      const size_t bytes = list ? bytes_of(c.post[0].inputs[t]) / (size_t)size : c.bytes;
      for (int q = 0; q < size; ++q) {
        for (int j = 0; j < size; ++j) {
          const moodist_tensor& in = list ? c.post[(size_t)j].inputs[t] : c.post[(size_t)j].input;
          tables[k * (size_t)size + (size_t)j] = (const char*)in.data + bytes * (size_t)q;
        }
        jobs[k].srcs = tables.data() + k * (size_t)size;
        jobs[k].nsrc = size;
        jobs[k].first = q;
        jobs[k].dst = nullptr;
        jobs[k].numel = bytes / itemsize;
        if (++k == per_call) {
          check_mdh(h.allreduce_many(jobs.data(), (int)k, c.dtype, c.reduce_op, scale, stream));
          k = 0;
        }
      }
    }
    if (k > 0) {
      check_mdh(h.allreduce_many(jobs.data(), (int)k, c.dtype, c.reduce_op, scale, stream));
    }
    for (const Posting& p : c.post) {
      if (p.has_copy_back) { // through a padded temporary (core/processgroup.cc:1716-1720)
        check_hip(h.MemcpyAsync(p.copy_back.data, p.output.data, (size_t)p.copy_back.numel * (size_t)p.copy_back.itemsize,
                      kHipMemcpyDeviceToDevice, stream),
            "hipMemcpyAsync");
      }
    }
    return;
  }
  // the two halves, as two collectives of their own kinds
  Collective rs, ag;
  rs.kind = list ? Kind::reduce_scatter_many : Kind::reduce_scatter;
  ag.kind = list ? Kind::all_gather_many : Kind::all_gather;
  rs.seq = ag.seq = c.seq;
  rs.reduce_op = c.reduce_op;
  rs.premul = c.premul;
  rs.bytes = ag.bytes = c.bytes;
  rs.dtype = ag.dtype = c.dtype;
  rs.post.resize((size_t)size);
  ag.post.resize((size_t)size);
  for (int q = 0; q < size; ++q) {
    const Posting& p = c.post[(size_t)q];
    Posting& r = rs.post[(size_t)q];
    Posting& g = ag.post[(size_t)q];
    r.arrived = g.arrived = true;
    r.wants_output = g.wants_output = true;
    r.stream = g.stream = p.stream;
    r.chunk_bytes = p.chunk_bytes;
    g.kernel_less = p.kernel_less;
    if (list) {
      for (size_t t = 0; t < n; ++t) {
        const moodist_tensor mine = chunk_of(p.outputs[t], q, size);
        r.inputs.push_back(p.inputs[t]);
        r.outputs.push_back(mine);
        g.inputs.push_back(mine);
        g.outputs.push_back(p.outputs[t]);
      }
    } else {
      const moodist_tensor mine = chunk_of(p.output, q, size);
      r.input = p.input;
      r.output = mine;
      g.input = mine;
      g.output = p.output;
      g.has_copy_back = p.has_copy_back;
      g.copy_back = p.copy_back;
    }
  }
  run(rs, nullptr);
  // every rank's gather reads what the other ranks' reductions write
  order_streams_after(rs);
  order_streams_before(ag);
  run(ag, nullptr);
}

void World::run(Collective& c, const std::shared_ptr<CompiledOp>& op) {
  const HipRuntime& h = hip();
  std::vector<const void*> srcs((size_t)size);
  if (c.kind == Kind::reduce_scatter) {
    // out_q = in_q[q] (+) in_{q+1}[q] (+) ... in rank order starting at q (core/group.cc:567-570;
    // core/reduce_scatter.cc:180-191), pitch = bytes (core/processgroup.cc:1322)
    const size_t itemsize = dtype_size(c.dtype);
    const size_t numel = c.bytes / itemsize;
    // AVG is SUM then a multiply by 1.0f/size (core/processgroup.cc:1664-1667); PREMUL_SUM
    // multiplies every input by the factor first (:1374-1378)
    const float scale = c.reduce_op == MDH_OP_AVG ? 1.0f / (float)size : c.premul;
    // Short reductions are bound by the launch, not by memory: the ranks that share a stream
    // (in one process they usually all do) share ONE launch, a job per rank (mdh_reduce_many).
    std::vector<bool> done((size_t)size, false);
    if (c.bytes <= kSharedLaunchBytes) {
      for (const std::vector<int>& ranks : ranks_by_stream(c)) {
        if (ranks.size() < 2) {
          continue;
        }
        std::vector<const void*> tables(ranks.size() * (size_t)size);
        std::vector<mdh_reduce_job> jobs(ranks.size());
        for (size_t k = 0; k < ranks.size(); ++k) {
          const int q = ranks[k];
          for (int j = 0; j < size; ++j) {
            tables[k * (size_t)size + (size_t)j] = (const char*)c.post[(size_t)j].input.data + c.bytes * (size_t)q;
          }
          jobs[k].srcs = tables.data() + k * (size_t)size;
          jobs[k].nsrc = size;
          jobs[k].first = q;
          jobs[k].dst = c.post[(size_t)q].output.data;
          jobs[k].numel = numel;
          done[(size_t)q] = true;
        }
        check_mdh(h.reduce_many(jobs.data(), (int)jobs.size(), c.dtype, c.reduce_op, scale, c.post[(size_t)ranks[0]].stream));
      }
    }
    for (int q = 0; q < size; ++q) {
      const Posting& pq = c.post[(size_t)q];
      if (!pq.wants_output || done[(size_t)q]) {
        continue;
      }
      for (int j = 0; j < size; ++j) {
        srcs[(size_t)j] = (const char*)c.post[(size_t)j].input.data + c.bytes * (size_t)q;
      }
      if (pq.chunk_bytes == 0) {
        check_mdh(h.reduce(srcs.data(), size, q, pq.output.data, numel, c.dtype, c.reduce_op, scale, pq.stream));
        continue;
      }
      // in pieces (the options num_chunks / chunk_size / method of the rank that asks): piece k
      // covers bytes [k * chunk, min(bytes, (k + 1) * chunk)) of every source and of the output
      const size_t chunk = pq.chunk_bytes / itemsize * itemsize;
      const size_t pieces = (c.bytes + chunk - 1) / chunk;
      std::vector<const void*> tables(pieces * (size_t)size);
      std::vector<mdh_reduce_job> jobs(pieces);
      for (size_t k = 0; k < pieces; ++k) {
        const size_t at = k * chunk;
        for (int j = 0; j < size; ++j) {
          tables[k * (size_t)size + (size_t)j] = (const char*)srcs[(size_t)j] + at;
        }
        jobs[k].srcs = tables.data() + k * (size_t)size;
        jobs[k].nsrc = size;
        jobs[k].first = q;
        jobs[k].dst = (char*)pq.output.data + at;
        jobs[k].numel = ((at + chunk < c.bytes ? chunk : c.bytes - at)) / itemsize;
      }
      check_mdh(h.reduce_many(jobs.data(), (int)pieces, c.dtype, c.reduce_op, scale, pq.stream));
    }
  } else if (c.kind == Kind::reduce_scatter_many) {
    // out_q[t] = in_q[t][q] (+) in_{q+1}[t][q] (+) ... for every tensor t: one job per tensor, the
    // jobs of a rank in shared launches
    const size_t itemsize = dtype_size(c.dtype);
    const size_t n = c.post[0].inputs.size();
    const float scale = c.reduce_op == MDH_OP_AVG ? 1.0f / (float)size : c.premul;
    std::vector<const void*> tables(n * (size_t)size);
    std::vector<mdh_reduce_job> jobs(n);
    for (int q = 0; q < size; ++q) {
      const Posting& pq = c.post[(size_t)q];
      if (!pq.wants_output) {
        continue;
      }
      for (size_t t = 0; t < n; ++t) {
        const size_t bytes = bytes_of(pq.inputs[t]) / (size_t)size;
        for (int j = 0; j < size; ++j) {
          tables[t * (size_t)size + (size_t)j] = (const char*)c.post[(size_t)j].inputs[t].data + bytes * (size_t)q;
        }
        jobs[t].srcs = tables.data() + t * (size_t)size;
        jobs[t].nsrc = size;
        jobs[t].first = q;
        jobs[t].dst = pq.outputs[t].data;
        jobs[t].numel = bytes / itemsize;
      }
      check_mdh(h.reduce_many(jobs.data(), (int)n, c.dtype, c.reduce_op, scale, pq.stream));
    }
  } else if (c.kind == Kind::all_gather) {
    // out_q[pitch*j .. +bytes] = in_j for every j (core/allgather.cc:381-390)
    // Short gathers, like short reductions: the ranks that share a stream share one launch, a
    // contiguous copy per destination rank and source rank.
    std::vector<bool> done((size_t)size, false);
    if (c.bytes <= kSharedLaunchBytes) {
      for (const std::vector<int>& ranks : ranks_by_stream(c)) {
        bool plain = ranks.size() >= 2;
        for (int q : ranks) {
          plain = plain && c.post[(size_t)q].outputs.empty() && !c.post[(size_t)q].kernel_less;
        }
        if (!plain) {
          continue;
        }
        std::vector<mdh_box> boxes;
        boxes.reserve(ranks.size() * (size_t)size);
        for (int q : ranks) {
          for (int j = 0; j < size; ++j) {
            mdh_box b{};
            b.src = c.post[(size_t)j].input.data;
            b.dst = (char*)c.post[(size_t)q].output.data + c.bytes * (size_t)j;
            if (b.src == b.dst) {
              continue; // already in place
            }
            b.ndim = 1;
            b.shape[0] = (int64_t)c.bytes;
            b.src_strides[0] = b.dst_strides[0] = 1;
            boxes.push_back(b);
          }
          done[(size_t)q] = true;
        }
        void* stream = c.post[(size_t)ranks[0]].stream;
        if (!boxes.empty()) {
          check_mdh(h.copy_boxes(boxes.data(), (int)boxes.size(), 1, stream));
        }
        for (int q : ranks) {
          const Posting& pq = c.post[(size_t)q];
          if (pq.has_copy_back) { // allreduce through a padded temporary (core/processgroup.cc:1716-1720)
            check_hip(h.MemcpyAsync(pq.copy_back.data, pq.output.data,
                          (size_t)pq.copy_back.numel * (size_t)pq.copy_back.itemsize, kHipMemcpyDeviceToDevice, stream),
                "hipMemcpyAsync");
          }
        }
      }
    }
    for (int q = 0; q < size; ++q) {
      const Posting& pq = c.post[(size_t)q];
      if (!pq.wants_output || done[(size_t)q]) {
        continue;
      }
      for (int j = 0; j < size; ++j) {
        srcs[(size_t)j] = c.post[(size_t)j].input.data;
      }
      if (!pq.outputs.empty()) {
        // one destination tensor per source rank
        if (pq.kernel_less) {
          for (int j = 0; j < size; ++j) {
            if (pq.outputs[(size_t)j].data != srcs[(size_t)j]) {
              check_hip(h.MemcpyAsync(pq.outputs[(size_t)j].data, srcs[(size_t)j], c.bytes, kHipMemcpyDeviceToDevice,
                            pq.stream),
                  "hipMemcpyAsync");
            }
          }
        } else {
          std::vector<mdh_box> boxes;
          boxes.reserve((size_t)size);
          for (int j = 0; j < size; ++j) {
            if (pq.outputs[(size_t)j].data == srcs[(size_t)j]) {
              continue; // already in place
            }
            mdh_box b{};
            b.src = srcs[(size_t)j];
            b.dst = pq.outputs[(size_t)j].data;
            b.ndim = 1;
            b.shape[0] = (int64_t)c.bytes;
            b.src_strides[0] = b.dst_strides[0] = 1;
            boxes.push_back(b);
          }
          if (!boxes.empty()) {
            check_mdh(h.copy_boxes(boxes.data(), (int)boxes.size(), 1, pq.stream));
          }
        }
      } else if (pq.kernel_less) {
        // copy-engine form (core/processgroup.cc:706-833): ranks whose buffers are evenly spaced
        // -- slices of one staging allocation, with or without padding between them -- move as
        // one copy: 1-D when they are adjacent, 2-D (hipMemcpy2DAsync, the reference's
        // cuMemcpy2DAsync :806-820) when there is a pitch; the others one copy per rank
        std::vector<bool> in_place((size_t)size);
        for (int j = 0; j < size; ++j) {
          in_place[(size_t)j] = (char*)pq.output.data + c.bytes * (size_t)j == srcs[(size_t)j];
        }
        for (const GatherRun& run : gather_runs(srcs, in_place, c.bytes)) {
          void* dst = (char*)pq.output.data + c.bytes * run.first;
          if (run.count == 1 || run.src_pitch == c.bytes) {
            check_hip(h.MemcpyAsync(dst, srcs[run.first], c.bytes * run.count, kHipMemcpyDeviceToDevice, pq.stream),
                "hipMemcpyAsync");
            ++kernel_less_copies_1d;
          } else {
            const int rc = h.Memcpy2DAsync(dst, c.bytes, srcs[run.first], run.src_pitch, c.bytes, run.count,
                kHipMemcpyDeviceToDevice, pq.stream);
            if (rc == kHipErrorInvalidValue) {
              // The runtime refuses some shapes when it checks its arguments, before anything is
              // enqueued (seen with rows of a few bytes at an odd pitch): rank by rank then.
              (void)h.GetLastError();
              log_debug("hipMemcpy2DAsync refused width %zu, %zu rows, pitches %zu -> %zu: one copy per rank", c.bytes,
                  run.count, run.src_pitch, c.bytes);
              for (size_t k = 0; k < run.count; ++k) {
                check_hip(h.MemcpyAsync((char*)dst + c.bytes * k, (const char*)srcs[run.first] + run.src_pitch * k, c.bytes,
                              kHipMemcpyDeviceToDevice, pq.stream),
                    "hipMemcpyAsync");
                ++kernel_less_copies_1d;
              }
            } else {
              check_hip(rc, "hipMemcpy2DAsync");
              ++kernel_less_copies_2d;
            }
          }
        }
      } else {
        check_mdh(h.gather(srcs.data(), size, pq.output.data, c.bytes, 1, c.bytes, c.bytes, c.bytes, pq.stream));
      }
      if (pq.has_copy_back) {
        // allreduce through a padded temporary: copy the result back (core/processgroup.cc:1716-1720)
        const moodist_tensor& back = pq.copy_back;
        check_hip(h.MemcpyAsync(back.data, pq.output.data, (size_t)back.numel * (size_t)back.itemsize,
                      kHipMemcpyDeviceToDevice, pq.stream),
            "hipMemcpyAsync");
      }
    }
  } else if (c.kind == Kind::all_gather_many) {
    // out_q[t][bytes_t*j .. +bytes_t] = in_j[t] for every tensor t and rank j: one table of
    // contiguous copies per destination rank
    const size_t n = c.post[0].inputs.size();
    std::vector<mdh_box> boxes;
    for (int q = 0; q < size; ++q) {
      const Posting& pq = c.post[(size_t)q];
      if (!pq.wants_output) {
        continue;
      }
      boxes.clear();
      boxes.reserve(n * (size_t)size);
      for (size_t t = 0; t < n; ++t) {
        const size_t bytes = bytes_of(pq.inputs[t]);
        for (int j = 0; j < size; ++j) {
          mdh_box b{};
          b.src = c.post[(size_t)j].inputs[t].data;
          b.dst = (char*)pq.outputs[t].data + bytes * (size_t)j;
          if (b.src == b.dst) {
            continue; // already in place
          }
          if (pq.kernel_less) { // the copy-engine form: one copy per tensor and source rank
            check_hip(h.MemcpyAsync(b.dst, b.src, bytes, kHipMemcpyDeviceToDevice, pq.stream), "hipMemcpyAsync");
            ++kernel_less_copies_1d;
            continue;
          }
          b.ndim = 1;
          b.shape[0] = (int64_t)bytes;
          b.src_strides[0] = b.dst_strides[0] = 1;
          boxes.push_back(b);
        }
      }
      if (!boxes.empty()) {
        check_mdh(h.copy_boxes(boxes.data(), (int)boxes.size(), 1, pq.stream));
      }
    }
  } else {
    // Every read of every rank, with its staging copies folded in, as strided box copies
    // straight from the source rank's tensor into the destination tensor.  The launches were
    // prepared when the op first ran (box geometry, tiles, grids, kernel arguments): a call
    // fills in the tensors' addresses and enqueues them.
    MD_CHECK(op != nullptr);
    if (op->prepared.size() != (size_t)size) {
      op->prepared.resize((size_t)size);
    }
    for (int q = 0; q < size; ++q) {
      const Posting& pq = c.post[(size_t)q];
      const RankPlan& plan = op->plans[(size_t)q];
      if (plan.transfers.empty()) {
        continue;
      }
      if (!op->prepared[(size_t)q]) {
        op->prepared[(size_t)q] = prepare_transfers(plan, op->itemsize);
      }
      PreparedTransfers& pt = *op->prepared[(size_t)q];
      MD_CHECK(pt.n_outputs == pq.outputs.size());
      size_t k = 0;
      for (const PreparedTransfers::Source& src : pt.sources) {
        const Posting& ps = c.post[src.rank];
        MD_CHECK(src.input < ps.inputs.size());
        pt.bases[k++] = ps.inputs[src.input].data;
      }
      for (const moodist_tensor& o : pq.outputs) {
        pt.bases[k++] = o.data;
      }
      check_mdh(h.copy_plan_launch(pt.plan, pt.bases.data(), (int)pt.bases.size(), pq.stream));
    }
  }
}

} // namespace moodist
