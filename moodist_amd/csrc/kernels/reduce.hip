// C ABI entry of the K-source reduction: argument checks, fold-order rotation
// of the pointer table, dispatch on element type.
#include "reduce_kernels.h"

extern "C" int mdh_reduce(const void* const* srcs, int nsrc, int first, void* dst, size_t numel, int dtype, int op,
    float scale, void* stream) {
  using namespace mdh;
  if (nsrc < 1 || nsrc > MDH_MAX_SOURCES) {
    set_error("mdh_reduce: nsrc %d outside 1..%d", nsrc, MDH_MAX_SOURCES);
    return MDH_EINVAL;
  }
  if (first < 0 || first >= nsrc) {
    set_error("mdh_reduce: first %d outside 0..%d", first, nsrc - 1);
    return MDH_EINVAL;
  }
  size_t itemsize;
  bool floating;
  switch (dtype) {
  case MDH_DTYPE_FLOAT32:
    itemsize = 4, floating = true;
    break;
  case MDH_DTYPE_FLOAT64:
    itemsize = 8, floating = true;
    break;
  case MDH_DTYPE_INT32:
    itemsize = 4, floating = false;
    break;
  case MDH_DTYPE_INT64:
    itemsize = 8, floating = false;
    break;
  case MDH_DTYPE_BFLOAT16:
  case MDH_DTYPE_FLOAT16:
    itemsize = 2, floating = true;
    break;
  default:
    set_error("Unsupported dtype for reduce operation (%d)", dtype);
    return MDH_EDTYPE;
  }
  int fold_op, mode = kPlain;
  switch (op) {
  case MDH_OP_SUM:
    fold_op = kSum;
    break;
  case MDH_OP_AVG:
    fold_op = kSum, mode = kAvg;
    break;
  case MDH_OP_PREMUL_SUM:
    fold_op = kSum, mode = kPremul;
    break;
  case MDH_OP_MIN:
    fold_op = kMin;
    break;
  case MDH_OP_MAX:
    fold_op = kMax;
    break;
  default:
    set_error("Unsupported reduce operation (%d)", op);
    return MDH_EOP;
  }
  if (mode != kPlain && !floating) {
    set_error("Unsupported reduce operation (%d) for integer dtype %d", op, dtype);
    return MDH_EOP;
  }
  if (numel == 0) {
    return MDH_OK;
  }
  if (numel > (size_t)1 << 48) {
    set_error("mdh_reduce: numel %zu is not a plausible device size", numel);
    return MDH_EINVAL;
  }
  if (!srcs || !dst) {
    set_error("mdh_reduce: null pointer");
    return MDH_EINVAL;
  }
  ReduceArgs a{}; // unused source slots stay null
  const uintptr_t bytes = (uintptr_t)numel * itemsize;
  for (int j = 0; j < nsrc; ++j) {
    const void* p = srcs[(first + j) % nsrc];
    if (!p) {
      set_error("mdh_reduce: source %d is null", (first + j) % nsrc);
      return MDH_EINVAL;
    }
    if ((uintptr_t)p % itemsize) {
      set_error("mdh_reduce: source %d is not aligned to its element size", (first + j) % nsrc);
      return MDH_EINVAL;
    }
    // dst may be exactly one source (in-place allreduce); partial overlap would race
    const uintptr_t s = (uintptr_t)p, d = (uintptr_t)dst;
    if (s != d && s < d + bytes && d < s + bytes) {
      set_error("mdh_reduce: destination partially overlaps source %d", (first + j) % nsrc);
      return MDH_EINVAL;
    }
    a.src[j] = p;
  }
  for (int j = nsrc; j < MDH_MAX_SOURCES; ++j) {
    a.src[j] = nullptr;
  }
  if ((uintptr_t)dst % itemsize) {
    set_error("mdh_reduce: destination is not aligned to its element size");
    return MDH_EINVAL;
  }
  a.dst = dst;
  a.numel = numel;
  a.head = 0;
  // Stores want the destination on the 64-byte grid: a wave's 1 KiB store whose ends fall
  // inside 64-byte units costs about 6 % of a launch (22.8 us aligned or off by 64 B, 24.2 us off
  // by 4, 16 or 32 B), loads off the grid 1 %.  When the destination is off the grid and there is
  // more than a few vectors to write, the vectors start at its next 64-byte boundary and the
  // elements before it are folded one by one, like the few after the last whole vector.
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
  hipStream_t s = (hipStream_t)stream;
#define MDH_DISPATCH(tname)                                  \
  switch (fold_op) {                                         \
  case kSum:                                                 \
    return reduce_launch_##tname##_sum(a, s);       \
  case kMin:                                                 \
    return reduce_launch_##tname##_min(a, s);       \
  default:                                                   \
    return reduce_launch_##tname##_max(a, s);       \
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
