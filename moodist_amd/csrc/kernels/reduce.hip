// C ABI entries of the K-source reduction: argument checks, fold-order rotation
// of the pointer table, dispatch on element type.
#include "reduce_kernels.h"

#include <algorithm>
#include <utility>
#include <vector>

namespace mdh {
namespace {

struct OpInfo {
  size_t itemsize;
  bool floating;
  int fold_op;
  int mode;
};

int parse_dtype_and_op(const char* who, int dtype, int op, OpInfo* out) {
  switch (dtype) {
  case MDH_DTYPE_FLOAT32:
    out->itemsize = 4, out->floating = true;
    break;
  case MDH_DTYPE_FLOAT64:
    out->itemsize = 8, out->floating = true;
    break;
  case MDH_DTYPE_INT32:
    out->itemsize = 4, out->floating = false;
    break;
  case MDH_DTYPE_INT64:
    out->itemsize = 8, out->floating = false;
    break;
  case MDH_DTYPE_BFLOAT16:
  case MDH_DTYPE_FLOAT16:
    out->itemsize = 2, out->floating = true;
    break;
  default:
    set_error("Unsupported dtype for reduce operation (%d)", dtype);
    return MDH_EDTYPE;
  }
  out->mode = kPlain;
  switch (op) {
  case MDH_OP_SUM:
    out->fold_op = kSum;
    break;
  case MDH_OP_AVG:
    out->fold_op = kSum, out->mode = kAvg;
    break;
  case MDH_OP_PREMUL_SUM:
    out->fold_op = kSum, out->mode = kPremul;
    break;
  case MDH_OP_MIN:
    out->fold_op = kMin;
    break;
  case MDH_OP_MAX:
    out->fold_op = kMax;
    break;
  default:
    set_error("Unsupported reduce operation (%d)", op);
    return MDH_EOP;
  }
  if (out->mode != kPlain && !out->floating) {
    set_error("Unsupported reduce operation (%d) for integer dtype %d", op, dtype);
    return MDH_EOP;
  }
  (void)who;
  return MDH_OK;
}

// The checks on one reduction's operands; on success ordered[0 .. nsrc-1] holds the source
// pointers in fold order (first, first+1, ..., wrapping round).  `label` names the reduction in
// messages ("" for the only one, " (job 3)" in a list).
int check_operands(const char* who, const char* label, const void* const* srcs, int nsrc, int first, const void* dst,
    size_t numel, size_t itemsize, const void** ordered) {
  if (nsrc < 1 || nsrc > MDH_MAX_SOURCES) {
    set_error("%s: nsrc %d outside 1..%d%s", who, nsrc, MDH_MAX_SOURCES, label);
    return MDH_EINVAL;
  }
  if (first < 0 || first >= nsrc) {
    set_error("%s: first %d outside 0..%d%s", who, first, nsrc - 1, label);
    return MDH_EINVAL;
  }
  if (numel == 0) {
    return MDH_OK;
  }
  if (numel > (size_t)1 << 48) {
    set_error("%s: numel %zu is not a plausible device size%s", who, numel, label);
    return MDH_EINVAL;
  }
  if (!srcs || !dst) {
    set_error("%s: null pointer%s", who, label);
    return MDH_EINVAL;
  }
  const uintptr_t bytes = (uintptr_t)numel * itemsize;
  for (int j = 0; j < nsrc; ++j) {
    const void* p = srcs[(first + j) % nsrc];
    if (!p) {
      set_error("%s: source %d is null%s", who, (first + j) % nsrc, label);
      return MDH_EINVAL;
    }
    if ((uintptr_t)p % itemsize) {
      set_error("%s: source %d is not aligned to its element size%s", who, (first + j) % nsrc, label);
      return MDH_EINVAL;
    }
    // dst may be exactly one source (in-place allreduce); partial overlap would race
    const uintptr_t s = (uintptr_t)p, d = (uintptr_t)dst;
    if (s != d && s < d + bytes && d < s + bytes) {
      set_error("%s: destination partially overlaps source %d%s", who, (first + j) % nsrc, label);
      return MDH_EINVAL;
    }
    ordered[j] = p;
  }
  if ((uintptr_t)dst % itemsize) {
    set_error("%s: destination is not aligned to its element size%s", who, label);
    return MDH_EINVAL;
  }
  return MDH_OK;
}

// The argument struct of one launch of its own.
ReduceArgs single_launch_args(const void* const* ordered, int nsrc, void* dst, size_t numel, size_t itemsize, int mode,
    float scale) {
  ReduceArgs a{}; // unused source slots stay null
  for (int j = 0; j < nsrc; ++j) {
    a.src[j] = ordered[j];
  }
  a.dst = dst;
  a.numel = numel;
  a.head = 0;
  // Stores want the destination on the 64-byte grid: a wave's 1 KiB store whose ends fall
  // inside 64-byte units costs about 6 % of a launch (22.8 us aligned or off by 64 B, 24.2 us off
  // by 4, 16 or 32 B), loads off the grid 1 %.  When the destination is off the grid and there is
  // more than a few vectors to write, the vectors start at its next 64-byte boundary and the
  // elements before it are folded one by one, like the few after the last whole vector.
  const uintptr_t bytes = (uintptr_t)numel * itemsize;
  const uintptr_t off_grid = (uintptr_t)dst & 63;
  if (off_grid != 0 && bytes >= 256) {
    const uintptr_t head_bytes = 64 - off_grid; // a multiple of the element size: dst is element-aligned
    a.head = (uint32_t)(head_bytes / itemsize);
    for (int j = 0; j < nsrc; ++j) {
      a.src[j] = (const char*)a.src[j] + head_bytes;
    }
    a.dst = (char*)dst + head_bytes;
    a.numel = numel - a.head;
  }
  a.nvec = a.numel * itemsize / 16;
  a.scale = scale;
  a.nsrc = nsrc;
  a.mode = mode;
  return a;
}

int dispatch_single(int dtype, int fold_op, const ReduceArgs& a, hipStream_t s) {
#define MDH_DISPATCH(tname)                   \
  switch (fold_op) {                          \
  case kSum:                                  \
    return reduce_launch_##tname##_sum(a, s); \
  case kMin:                                  \
    return reduce_launch_##tname##_min(a, s); \
  default:                                    \
    return reduce_launch_##tname##_max(a, s); \
  }
  switch (dtype) {
  case MDH_DTYPE_FLOAT32:
    MDH_DISPATCH(f32)
  case MDH_DTYPE_FLOAT64:
    MDH_DISPATCH(f64)
  case MDH_DTYPE_INT32:
    MDH_DISPATCH(i32)
  case MDH_DTYPE_INT64:
    MDH_DISPATCH(i64)
  case MDH_DTYPE_BFLOAT16:
    MDH_DISPATCH(bf16)
  default:
    MDH_DISPATCH(f16)
  }
#undef MDH_DISPATCH
}

int dispatch_many(int dtype, int fold_op, const ManyJob* jobs, int njobs, int mode, float scale, bool spread, hipStream_t s) {
#define MDH_DISPATCH(tname)                                             \
  switch (fold_op) {                                                    \
  case kSum:                                                            \
    return reduce_many_launch_##tname##_sum(jobs, njobs, mode, scale, spread, s); \
  case kMin:                                                            \
    return reduce_many_launch_##tname##_min(jobs, njobs, mode, scale, spread, s); \
  default:                                                              \
    return reduce_many_launch_##tname##_max(jobs, njobs, mode, scale, spread, s); \
  }
  switch (dtype) {
  case MDH_DTYPE_FLOAT32:
    MDH_DISPATCH(f32)
  case MDH_DTYPE_FLOAT64:
    MDH_DISPATCH(f64)
  case MDH_DTYPE_INT32:
    MDH_DISPATCH(i32)
  case MDH_DTYPE_INT64:
    MDH_DISPATCH(i64)
  case MDH_DTYPE_BFLOAT16:
    MDH_DISPATCH(bf16)
  default:
    MDH_DISPATCH(f16)
  }
#undef MDH_DISPATCH
}

// A job of a list with this many bytes per source and more gets a launch of its own, with the
// shape a single reduction of its size gets (and its cut into several launches when it is very
// long).  Below, sharing still pays: eight jobs of 8 x 4 MiB take 49 us in one launch and 60 us
// in eight, of 8 x 8 MiB 97.8 against 100.1 us; of 8 x 16 MiB 196.5 against 183.3 us.
constexpr size_t kOwnLaunchBytes = (size_t)16 << 20;
constexpr size_t kSpreadPieceBytes = (size_t)32 << 20;

} // namespace
} // namespace mdh

extern "C" int mdh_reduce(const void* const* srcs, int nsrc, int first, void* dst, size_t numel, int dtype, int op,
    float scale, void* stream) {
  using namespace mdh;
  // (the count and the fold's start are checked before the dtype, whatever the size)
  if (nsrc < 1 || nsrc > MDH_MAX_SOURCES) {
    set_error("mdh_reduce: nsrc %d outside 1..%d", nsrc, MDH_MAX_SOURCES);
    return MDH_EINVAL;
  }
  if (first < 0 || first >= nsrc) {
    set_error("mdh_reduce: first %d outside 0..%d", first, nsrc - 1);
    return MDH_EINVAL;
  }
  OpInfo info;
  if (const int rc = parse_dtype_and_op("mdh_reduce", dtype, op, &info)) {
    return rc;
  }
  const void* ordered[MDH_MAX_SOURCES];
  if (const int rc = check_operands("mdh_reduce", "", srcs, nsrc, first, dst, numel, info.itemsize, ordered)) {
    return rc;
  }
  if (numel == 0) {
    return MDH_OK;
  }
  if (const int rc = refuse_capture((hipStream_t)stream, "mdh_reduce")) {
    return rc;
  }
  const ReduceArgs a = single_launch_args(ordered, nsrc, dst, numel, info.itemsize, info.mode, scale);
  return dispatch_single(dtype, info.fold_op, a, (hipStream_t)stream);
}

namespace mdh {
namespace {

// mdh_reduce_many and mdh_allreduce_many: the second stores every job's result over all of the
// job's sources (`spread`) and ignores jobs[j].dst.
int reduce_list(const char* who, const mdh_reduce_job* jobs, int njobs, int dtype, int op, float scale, bool spread,
    void* stream) {
  if (njobs < 0 || njobs > 65535 || (njobs > 0 && !jobs)) {
    set_error("%s: bad job table (%d jobs)", who, njobs);
    return MDH_EINVAL;
  }
  OpInfo info;
  if (const int rc = parse_dtype_and_op(who, dtype, op, &info)) {
    return rc;
  }
  // every job is checked before anything is enqueued
  std::vector<const void*> pool;
  std::vector<size_t> pool_at((size_t)njobs);
  size_t pointers = 0;
  for (int j = 0; j < njobs; ++j) {
    pointers += jobs[j].nsrc > 0 && jobs[j].nsrc <= MDH_MAX_SOURCES ? (size_t)jobs[j].nsrc : 0;
  }
  pool.resize(pointers + MDH_MAX_SOURCES);
  size_t at = 0;
  bool any = false;
  for (int j = 0; j < njobs; ++j) {
    char label[32];
    std::snprintf(label, sizeof(label), " (job %d)", j);
    pool_at[(size_t)j] = at;
    const mdh_reduce_job& job = jobs[j];
    // (spread: the first source of the fold stands in for the destination, which it is)
    const void* dst = job.dst;
    if (spread && job.srcs && job.nsrc >= 1 && job.nsrc <= MDH_MAX_SOURCES && job.first >= 0 && job.first < job.nsrc) {
      dst = job.srcs[job.first];
    }
    if (const int rc = check_operands(who, label, job.srcs, job.nsrc, job.first, dst, job.numel, info.itemsize, pool.data() + at)) {
      return rc;
    }
    if (spread && job.numel != 0) {
      // every source is written: no two of them may share a byte
      const uintptr_t bytes = (uintptr_t)job.numel * info.itemsize;
      std::pair<uintptr_t, int> by_address[MDH_MAX_SOURCES];
      for (int x = 0; x < job.nsrc; ++x) {
        by_address[x] = {(uintptr_t)job.srcs[x], x};
      }
      std::sort(by_address, by_address + job.nsrc);
      for (int x = 0; x + 1 < job.nsrc; ++x) {
        if (by_address[x + 1].first - by_address[x].first < bytes) {
          const int lo = std::min(by_address[x].second, by_address[x + 1].second);
          const int hi = std::max(by_address[x].second, by_address[x + 1].second);
          set_error("%s: sources %d and %d overlap%s", who, lo, hi, label);
          return MDH_EINVAL;
        }
      }
    }
    at += (size_t)job.nsrc;
    any = any || job.numel != 0;
  }
  if (!any) {
    return MDH_OK;
  }
  if (const int rc = refuse_capture((hipStream_t)stream, who)) {
    return rc;
  }
  // A spread job stays in the list whatever its size (the single reduction's kernel has one
  // destination); a very long one is cut into pieces of kSpreadPieceBytes per source so that
  // launches keep their usual length.
  size_t piece_pointers = 0, piece_jobs = 0;
  for (int j = 0; spread && j < njobs; ++j) {
    const size_t bytes = jobs[j].numel * info.itemsize;
    if (bytes > kSpreadPieceBytes) {
      const size_t pieces = (bytes + kSpreadPieceBytes - 1) / kSpreadPieceBytes;
      piece_jobs += pieces;
      piece_pointers += pieces * (size_t)jobs[j].nsrc;
    }
  }
  std::vector<const void*> piece_pool(piece_pointers);
  size_t piece_at = 0;
  std::vector<ManyJob> shared;
  shared.reserve((size_t)njobs + piece_jobs);
  for (int j = 0; j < njobs; ++j) {
    const mdh_reduce_job& job = jobs[j];
    if (job.numel == 0) {
      continue;
    }
    const void* const* ordered = pool.data() + pool_at[(size_t)j];
    if (spread && job.numel * info.itemsize > kSpreadPieceBytes) {
      const size_t piece_elems = kSpreadPieceBytes / info.itemsize;
      for (size_t from = 0; from < job.numel; from += piece_elems) {
        const void** mine = piece_pool.data() + piece_at;
        for (int q = 0; q < job.nsrc; ++q) {
          mine[q] = (const char*)ordered[q] + from * info.itemsize;
        }
        piece_at += (size_t)job.nsrc;
        const size_t n = job.numel - from < piece_elems ? job.numel - from : piece_elems;
        shared.push_back(ManyJob{mine, job.nsrc, const_cast<void*>(mine[0]), (uint64_t)n});
      }
      continue;
    }
    if (!spread && job.numel * info.itemsize >= kOwnLaunchBytes) {
      const ReduceArgs a = single_launch_args(ordered, job.nsrc, job.dst, job.numel, info.itemsize, info.mode, scale);
      if (const int rc = dispatch_single(dtype, info.fold_op, a, (hipStream_t)stream)) {
        return rc;
      }
      continue;
    }
    shared.push_back(ManyJob{ordered, job.nsrc, spread ? const_cast<void*>(ordered[0]) : job.dst, (uint64_t)job.numel});
  }
  if (shared.empty()) {
    return MDH_OK;
  }
  return dispatch_many(dtype, info.fold_op, shared.data(), (int)shared.size(), info.mode, scale, spread, (hipStream_t)stream);
}

} // namespace
} // namespace mdh

extern "C" int mdh_reduce_many(const mdh_reduce_job* jobs, int njobs, int dtype, int op, float scale, void* stream) {
  return mdh::reduce_list("mdh_reduce_many", jobs, njobs, dtype, op, scale, false, stream);
}

extern "C" int mdh_allreduce_many(const mdh_reduce_job* jobs, int njobs, int dtype, int op, float scale, void* stream) {
  return mdh::reduce_list("mdh_allreduce_many", jobs, njobs, dtype, op, scale, true, stream);
}
