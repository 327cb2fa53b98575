// extern "C" surface of the host core (include/moodist_core.h): handle
// ownership and exception-to-return-code conversion, nothing else.
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "c_handles.h"
#include "hip_loader.h"
#include "moodist_core.h"
#include "processgroup.h"

using namespace moodist;

namespace {

thread_local std::string g_error;

template<typename F>
int guarded(F&& f) {
  try {
    f();
    return 0;
  } catch (const std::exception& e) {
    g_error = e.what();
    return 1;
  } catch (...) {
    g_error = "moodist: unknown error";
    return 1;
  }
}

ProcessGroup* as_pg(moodist_pg* pg) {
  if (!pg) {
    throw std::runtime_error("moodist: null process group");
  }
  return reinterpret_cast<ProcessGroup*>(pg);
}

void give(moodist_work** out, std::shared_ptr<Collective> c) {
  if (out) {
    *out = new moodist_work{std::move(c)};
  }
}

void wait_launched(const Collective& c, const char* what) {
  if (!c.launched) {
    throw std::runtime_error(std::string("moodist: ") + what + " waited on before every rank of the group has " +
                             "called it (" + std::to_string(c.arrived) + " of " + std::to_string(c.post.size()) +
                             " have)");
  }
  if (!c.error.empty()) {
    throw std::runtime_error(c.error);
  }
}

std::vector<SliceSpec> slices(const int* ranks, const int* offsets, const int* shapes, size_t n, size_t ndim) {
  std::vector<SliceSpec> v(n);
  for (size_t i = 0; i < n; ++i) {
    v[i].rank = ranks[i];
    v[i].offset.assign(offsets + i * ndim, offsets + (i + 1) * ndim);
    v[i].shape.assign(shapes + i * ndim, shapes + (i + 1) * ndim);
  }
  return v;
}

} // namespace

#pragma GCC visibility push(default)
extern "C" {

int moodist_core_check_version(uint32_t expected_version) {
  return expected_version == MOODIST_CORE_API_VERSION ? 1 : 0;
}

const char* moodist_last_error(void) {
  return g_error.c_str();
}

int moodist_world_create(int size, int device, moodist_world** world) {
  return guarded([&] {
    if (!world) {
      throw std::runtime_error("moodist: null out pointer");
    }
    *world = new moodist_world{std::make_shared<World>(size, device)};
  });
}

void moodist_world_destroy(moodist_world* world) {
  delete world;
}

moodist_pg* moodist_world_group(moodist_world* world, int rank) {
  if (!world || rank < 0 || rank >= world->impl->size) {
    g_error = "moodist: no such rank in this world";
    return nullptr;
  }
  return reinterpret_cast<moodist_pg*>(world->impl->group(rank));
}

int moodist_pg_rank(moodist_pg* pg) {
  return pg ? reinterpret_cast<ProcessGroup*>(pg)->rank : -1;
}

int moodist_pg_size(moodist_pg* pg) {
  return pg ? reinterpret_cast<ProcessGroup*>(pg)->size : -1;
}

int moodist_pg_get_option(moodist_pg* pg, const char* name, int64_t* value) {
  return guarded([&] { *value = as_pg(pg)->get_option(name ? name : ""); });
}

int moodist_pg_set_option(moodist_pg* pg, const char* name, int64_t value) {
  return guarded([&] { as_pg(pg)->set_option(name ? name : "", value); });
}

int moodist_pg_all_gather(moodist_pg* pg, const moodist_tensor* output, const moodist_tensor* input, void* stream,
    moodist_work** work) {
  return guarded([&] {
    if (!output || !input) {
      throw std::runtime_error("moodist: null tensor");
    }
    give(work, as_pg(pg)->all_gather(output, *input, stream));
  });
}

int moodist_pg_all_gather_list(moodist_pg* pg, const moodist_tensor* outputs, size_t n_outputs,
    const moodist_tensor* input, void* stream, moodist_work** work) {
  return guarded([&] {
    if (!outputs || !input) {
      throw std::runtime_error("moodist: null tensor");
    }
    give(work, as_pg(pg)->all_gather_list(outputs, n_outputs, *input, stream));
  });
}

int moodist_pg_all_gather_many(moodist_pg* pg, const moodist_tensor* outputs, const moodist_tensor* inputs, size_t n,
    void* stream, moodist_work** work) {
  return guarded([&] {
    if (!inputs) {
      throw std::runtime_error("moodist: null tensor");
    }
    give(work, as_pg(pg)->all_gather_many(outputs, inputs, n, stream));
  });
}

int moodist_pg_reduce_scatter_many(moodist_pg* pg, const moodist_tensor* outputs, const moodist_tensor* inputs, size_t n,
    int reduce_op, void* stream, float premul_value, moodist_work** work) {
  return guarded([&] {
    if (!inputs) {
      throw std::runtime_error("moodist: null tensor");
    }
    give(work, as_pg(pg)->reduce_scatter_many(outputs, inputs, n, reduce_op, stream, premul_value));
  });
}

int moodist_pg_allreduce_many(moodist_pg* pg, const moodist_tensor* tensors, size_t n, int reduce_op, void* stream,
    float premul_value, moodist_work** work) {
  return guarded([&] {
    if (!tensors) {
      throw std::runtime_error("moodist: null tensor");
    }
    give(work, as_pg(pg)->allreduce_many(tensors, n, reduce_op, stream, premul_value));
  });
}

int moodist_pg_reduce_scatter(moodist_pg* pg, const moodist_tensor* output, const moodist_tensor* input,
    int reduce_op, void* stream, float premul_value, moodist_work** work) {
  return guarded([&] {
    if (!output || !input) {
      throw std::runtime_error("moodist: null tensor");
    }
    give(work, as_pg(pg)->reduce_scatter(output, *input, reduce_op, stream, premul_value));
  });
}

int moodist_pg_allreduce(moodist_pg* pg, const moodist_tensor* tensor, const moodist_tensor* scratch, int reduce_op,
    void* stream, float premul_value, moodist_work** work) {
  return guarded([&] {
    if (!tensor) {
      throw std::runtime_error("moodist: null tensor");
    }
    give(work, as_pg(pg)->allreduce(*tensor, scratch, reduce_op, stream, premul_value));
  });
}

int moodist_pg_allreduce_static(moodist_pg* pg, const moodist_tensor* tensor, int reduce_op, void* stream,
    float premul_value, moodist_work** work) {
  return guarded([&] {
    if (!tensor) {
      throw std::runtime_error("moodist: null tensor");
    }
    give(work, as_pg(pg)->allreduce_static(*tensor, reduce_op, stream, premul_value));
  });
}

int moodist_pg_stage_input(moodist_pg* pg, int kind, const moodist_tensor* input, int reduce_op, void* stream,
    float premul_value, moodist_work** work) {
  return guarded([&] {
    if (!input) {
      throw std::runtime_error("moodist: null tensor");
    }
    if (kind == 0) {
      give(work, as_pg(pg)->all_gather(nullptr, *input, stream));
    } else if (kind == 1) {
      give(work, as_pg(pg)->reduce_scatter(nullptr, *input, reduce_op, stream, premul_value));
    } else {
      throw std::runtime_error("moodist: stage_input kind must be 0 (all_gather) or 1 (reduce_scatter)");
    }
  });
}

int moodist_pg_last_work(moodist_pg* pg, moodist_work** work) {
  return guarded([&] {
    if (!work) {
      throw std::runtime_error("moodist: null out pointer");
    }
    std::shared_ptr<Collective> c = as_pg(pg)->last;
    *work = c ? new moodist_work{std::move(c)} : nullptr;
  });
}

int moodist_pg_keep_alive(moodist_pg* pg, void* ctx, void (*release)(void* ctx)) {
  return guarded([&] {
    if (!release) {
      throw std::runtime_error("moodist: null release function");
    }
    std::shared_ptr<void> held(ctx, release); // from here on `ctx` is released exactly once
    ProcessGroup* g = as_pg(pg);
    if (g->last) {
      g->world->attach(*g->last, g->rank, std::move(held));
    }
  });
}

int moodist_work_is_completed(moodist_work* work) {
  return work && work->c->launched && work->c->error.empty() ? 1 : 0;
}

int moodist_work_wait(moodist_work* work) {
  return guarded([&] {
    if (!work) {
      throw std::runtime_error("moodist: null work");
    }
    wait_launched(*work->c, "a collective was");
  });
}

void moodist_work_destroy(moodist_work* work) {
  delete work;
}

int moodist_compile_op_full(moodist_pg* pg, const int* shape, size_t ndim, int dtype, const int* input_ranks,
    const int* input_offsets, const int* input_shapes, size_t n_inputs, const int* output_ranks,
    const int* output_offsets, const int* output_shapes, size_t n_outputs, moodist_op** op) {
  return guarded([&] {
    if (!op) {
      throw std::runtime_error("moodist: null out pointer");
    }
    Dims dims(shape, shape + ndim);
    auto compiled = as_pg(pg)->compile_op_full(dims, dtype, slices(input_ranks, input_offsets, input_shapes, n_inputs, ndim),
        slices(output_ranks, output_offsets, output_shapes, n_outputs, ndim));
    *op = new moodist_op{as_pg(pg), std::move(compiled)};
  });
}

void moodist_op_destroy(moodist_op* op) {
  delete op;
}

int moodist_op_call(moodist_op* op, const moodist_tensor* inputs, size_t n_inputs, const moodist_tensor* outputs,
    size_t n_outputs, void* stream, moodist_future** future) {
  return guarded([&] {
    if (!op || !future) {
      throw std::runtime_error("moodist: null custom op");
    }
    *future = new moodist_future{op->pg->custom_op(op->op, inputs, n_inputs, outputs, n_outputs, stream)};
  });
}

int moodist_future_wait(moodist_future* future, void* stream) {
  (void)stream; // the copies were enqueued on the stream the rank passed to the call; nothing to add
  return guarded([&] {
    if (!future) {
      throw std::runtime_error("moodist: null future");
    }
    wait_launched(*future->c, "a custom op was");
  });
}

void moodist_future_destroy(moodist_future* future) {
  delete future;
}

int64_t moodist_kernel_less_runs(const void* const* srcs, size_t n, size_t bytes, const void* dst, int64_t* out,
    size_t capacity) {
  if (!srcs && n) {
    return -1;
  }
  std::vector<const void*> s(srcs, srcs + n);
  std::vector<bool> in_place(n, false);
  for (size_t j = 0; dst && j < n; ++j) {
    in_place[j] = (const char*)dst + bytes * j == s[j];
  }
  const std::vector<GatherRun> runs = gather_runs(s, in_place, bytes);
  for (size_t i = 0; i < runs.size() && out && 3 * i + 2 < capacity; ++i) {
    out[3 * i] = (int64_t)runs[i].first, out[3 * i + 1] = (int64_t)runs[i].count, out[3 * i + 2] = (int64_t)runs[i].src_pitch;
  }
  return (int64_t)runs.size();
}

int64_t moodist_op_plan_count(moodist_op* op, int what) {
  if (!op) {
    return -1;
  }
  const RankPlan& p = op->op->plans[(size_t)op->pg->rank];
  switch (what) {
  case 0:
    return (int64_t)p.reads.size();
  case 1:
    return (int64_t)p.inputCopies.size();
  case 2:
    return (int64_t)p.outputCopies.size();
  case 3:
    return (int64_t)p.inputs.size();
  case 4:
    return (int64_t)p.outputs.size();
  default:
    return -1;
  }
}

int moodist_op_plan_read(moodist_op* op, size_t i, int64_t out[6]) {
  return guarded([&] {
    const RankPlan& p = op->op->plans[(size_t)op->pg->rank];
    const PlanRead& r = p.reads.at(i);
    out[0] = r.rank, out[1] = r.inputIndex, out[2] = r.outputIndex;
    out[3] = (int64_t)r.inputOffset, out[4] = (int64_t)r.outputOffset, out[5] = (int64_t)r.bytes;
  });
}

int moodist_op_plan_copy(moodist_op* op, int which, size_t i, int64_t* out, size_t out_len) {
  return guarded([&] {
    const RankPlan& p = op->op->plans[(size_t)op->pg->rank];
    const PlanCopy& c = (which == 1 ? p.inputCopies : p.outputCopies).at(i);
    if (out_len < 1 + 2 * c.offset.size()) {
      throw std::runtime_error("moodist: plan buffer too small");
    }
    size_t k = 0;
    out[k++] = c.index;
    for (int64_t v : c.offset) {
      out[k++] = v;
    }
    for (int64_t v : c.shape) {
      out[k++] = v;
    }
  });
}

int64_t moodist_op_plan_message(moodist_op* op, int receiver, void* buffer, size_t capacity) {
  if (!op || receiver < 0 || receiver >= op->pg->size) {
    return -1;
  }
  const std::vector<uint8_t>& bytes = op->op->wire[(size_t)op->pg->rank][(size_t)receiver];
  if (buffer && capacity >= bytes.size()) {
    std::memcpy(buffer, bytes.data(), bytes.size());
  }
  return (int64_t)bytes.size();
}

int moodist_plan_message_check(const void* bytes, size_t length, size_t ndim) {
  return guarded([&] {
    const uint8_t* p = (const uint8_t*)bytes;
    check_plan_message(std::vector<uint8_t>(p, p + length), ndim);
  });
}

int64_t moodist_op_plan_size(moodist_op* op, int which, size_t i) {
  if (!op) {
    return -1;
  }
  const RankPlan& p = op->op->plans[(size_t)op->pg->rank];
  const std::vector<size_t>& v = which == 3 ? p.inputs : p.outputs;
  return i < v.size() ? (int64_t)v[i] : -1;
}

} // extern "C"
#pragma GCC visibility pop
