// Single-pass K-source reduction for gfx950 (templates; one translation unit
// per element type instantiates them so the types compile in parallel).
//
// What the reference does in K-1 two-source passes over the destination
// (core/reduce_scatter.cc:104-142 emitting reduce_n2 calls,
// core/kernels.cc:171-413) is done here in one pass: every lane issues one
// 16-byte load per source (up to 8 sources x U tiles in flight), folds the
// values in the reference's order in registers and writes 16 bytes once.
// HBM traffic is (K+1) x bytes instead of (3K-3) x bytes.
//
// Fold order, element ops and the AVG / PREMUL_SUM rules are those of the
// reference's CPU path (core/cputhread.cc:125-148, :3571-3587, :3680-3686;
// core/processgroup.cc:1340-1344, :1364-1366, :1664-1667).  This file is built
// with -ffp-contract=off: a product followed by an add must round twice.
#pragma once
#include "device_common.h"

#include <type_traits>

namespace mdh {

enum Fold { kSum = 0, kMin = 1, kMax = 2 };
enum Mode { kPlain = 0, kAvg = 1, kPremul = 2 };

struct ReduceArgs {
  const void* src[MDH_MAX_SOURCES]; // already rotated into fold order
  void* dst;
  uint64_t nvec;  // 16-byte vectors on the vector path
  uint64_t numel; // all elements
  float scale;
  int nsrc;
  int mode;
};

struct bf16_t {
  uint16_t bits;
};
struct f16_t {
  uint16_t bits;
};

template<typename T>
struct Traits {
  // float, double, int32_t, int64_t
  using elem_t = T;
  using acc_t = T;
  static __device__ __forceinline__ acc_t widen(elem_t e) {
    return e;
  }
  static __device__ __forceinline__ acc_t premul(acc_t a, float s) {
    if constexpr (std::is_floating_point_v<T>) {
      return a * (T)s;
    } else {
      return a;
    }
  }
  template<int F>
  static __device__ __forceinline__ elem_t finish(acc_t a, int mode, float s) {
    if constexpr (F == kSum && std::is_floating_point_v<T>) {
      if (mode == kAvg) {
        a = a * (T)s;
      }
    }
    return a;
  }
};

template<>
struct Traits<bf16_t> {
  using elem_t = uint16_t;
  using acc_t = float;
  static __device__ __forceinline__ float widen(uint16_t e) {
    return __uint_as_float((uint32_t)e << 16);
  }
  // round to nearest even; NaN stays a quiet NaN
  static __device__ __forceinline__ uint16_t narrow(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
      return (uint16_t)((u >> 16) | 0x0040u);
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
  }
  static __device__ __forceinline__ float premul(float a, float s) {
    return widen(narrow(a * s));
  }
  template<int F>
  static __device__ __forceinline__ uint16_t finish(float a, int mode, float s) {
    if constexpr (F != kSum) {
      return (uint16_t)(__float_as_uint(a) >> 16); // a is still one operand's exact image
    } else {
      if (mode == kAvg) {
        return narrow(widen(narrow(a)) * s);
      }
      return narrow(a);
    }
  }
};

// Keeps an fp32 product in a register of its own.  Without it the compiler
// fuses (half)((float)h * s) into v_fma_mixlo_f16, which rounds the exact
// product once to fp16; the rule here is fp32 rounding first, then fp16.
__device__ __forceinline__ float materialise(float x) {
  asm("" : "+v"(x));
  return x;
}

template<>
struct Traits<f16_t> {
  using elem_t = uint16_t;
  using acc_t = float;
  static __device__ __forceinline__ float widen(uint16_t e) {
    _Float16 h;
    __builtin_memcpy(&h, &e, 2);
    return (float)h;
  }
  static __device__ __forceinline__ uint16_t narrow(float f) {
    _Float16 h = (_Float16)f; // v_cvt_f16_f32, round to nearest even
    uint16_t e;
    __builtin_memcpy(&e, &h, 2);
    return e;
  }
  static __device__ __forceinline__ float premul(float a, float s) {
    return widen(narrow(materialise(a * s)));
  }
  template<int F>
  static __device__ __forceinline__ uint16_t finish(float a, int mode, float s) {
    if constexpr (F == kSum) {
      if (mode == kAvg) {
        return narrow(materialise(widen(narrow(a)) * s));
      }
    }
    return narrow(a);
  }
};

// std::min(a, b) is (b < a) ? b : a and std::max(a, b) is (a < b) ? b : a with
// a the running value: ties, signed zeros and NaN sources keep the running value.
template<int F, typename A>
__device__ __forceinline__ A fold(A acc, A x) {
  if constexpr (F == kSum) {
    if constexpr (std::is_integral_v<A>) {
      using UA = std::make_unsigned_t<A>;
      return (A)((UA)acc + (UA)x);
    } else {
      return acc + x;
    }
  } else if constexpr (F == kMin) {
    return (x < acc) ? x : acc;
  } else {
    return (acc < x) ? x : acc;
  }
}

template<typename T>
constexpr int per_vec() {
  return 16 / (int)sizeof(typename Traits<T>::elem_t);
}

// Loads CNT sources' vectors for U sub-tiles (CNT*U loads in flight), then
// folds them into acc in source order.  Each source is addressed through a
// buffer descriptor whose base is the tile's first byte (wave-uniform, in
// SGPRs) and whose size is the bytes left in the tile: the lane offset is one
// VGPR, and vectors past the end read as zero instead of needing a predicate.
template<typename T, int F, int CNT, int U, int MODE>
__device__ __forceinline__ void fold_chunk(const ReduceArgs& a, int j0, uint64_t tile_byte, uint32_t tile_bytes,
    uint32_t lane_byte, typename Traits<T>::acc_t (&acc)[U][per_vec<T>()]) {
  using Tr = Traits<T>;
  using elem_t = typename Tr::elem_t;
  using acc_t = typename Tr::acc_t;
  constexpr int N = per_vec<T>();
  u32x4 v[CNT][U];
#pragma unroll
  for (int k = 0; k < CNT; ++k) {
    const __amdgpu_buffer_rsrc_t rs = tile_rsrc((const char*)a.src[j0 + k] + tile_byte, tile_bytes);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      v[k][u] = tile_load(rs, lane_byte + (uint32_t)u * (kBlock * 16));
    }
  }
  // Every load of the chunk is issued before the first add.  Without this fence the
  // instruction scheduler interleaves loads with arithmetic to save registers (about a dozen
  // loads in flight per lane instead of 8*U); on the eight-source workload both orders time the
  // same, the fence just makes the number in flight independent of scheduler heuristics.
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int k = 0; k < CNT; ++k) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      elem_t e[N];
      __builtin_memcpy(e, &v[k][u], 16);
#pragma unroll
      for (int i = 0; i < N; ++i) {
        acc_t x = Tr::widen(e[i]);
        if constexpr (MODE == kPremul) {
          x = Tr::premul(x, a.scale);
        }
        if (k == 0 && j0 == 0) {
          acc[u][i] = x;
        } else {
          acc[u][i] = fold<F>(acc[u][i], x);
        }
      }
    }
  }
}

template<typename T, int F>
__device__ __forceinline__ void reduce_one_elem(const ReduceArgs& a, int nsrc, uint64_t i) {
  using Tr = Traits<T>;
  using elem_t = typename Tr::elem_t;
  using acc_t = typename Tr::acc_t;
  acc_t acc = Tr::widen(((const elem_t*)a.src[0])[i]);
  if (a.mode == kPremul) {
    acc = Tr::premul(acc, a.scale);
  }
#pragma unroll 4
  for (int j = 1; j < nsrc; ++j) {
    acc_t x = Tr::widen(((const elem_t*)a.src[j])[i]);
    if (a.mode == kPremul) {
      x = Tr::premul(x, a.scale);
    }
    acc = fold<F>(acc, x);
  }
  ((elem_t*)a.dst)[i] = Tr::template finish<F>(acc, a.mode, a.scale);
}

template<typename T, int F, int NSRC, int U, int MODE>
__device__ __forceinline__ void reduce_tile(const ReduceArgs& a, int nsrc, uint64_t tile_byte, uint32_t tile_bytes) {
  using Tr = Traits<T>;
  using elem_t = typename Tr::elem_t;
  using acc_t = typename Tr::acc_t;
  constexpr int N = per_vec<T>();
  constexpr int CH = 8;
  const uint32_t lane_byte = threadIdx.x * 16;
  acc_t acc[U][N];
  if constexpr (NSRC != 0) {
    // compile-time source count: fully unrolled chunks
    static_assert(NSRC % CH == 0, "unrolled source counts are multiples of the chunk");
#pragma unroll
    for (int j0 = 0; j0 < NSRC; j0 += CH) {
      fold_chunk<T, F, CH, U, MODE>(a, j0, tile_byte, tile_bytes, lane_byte, acc);
    }
  } else {
    int j0 = 0;
    for (; nsrc - j0 >= CH; j0 += CH) {
      fold_chunk<T, F, CH, U, MODE>(a, j0, tile_byte, tile_bytes, lane_byte, acc);
    }
    switch (nsrc - j0) {
    case 1:
      fold_chunk<T, F, 1, U, MODE>(a, j0, tile_byte, tile_bytes, lane_byte, acc);
      break;
    case 2:
      fold_chunk<T, F, 2, U, MODE>(a, j0, tile_byte, tile_bytes, lane_byte, acc);
      break;
    case 3:
      fold_chunk<T, F, 3, U, MODE>(a, j0, tile_byte, tile_bytes, lane_byte, acc);
      break;
    case 4:
      fold_chunk<T, F, 4, U, MODE>(a, j0, tile_byte, tile_bytes, lane_byte, acc);
      break;
    case 5:
      fold_chunk<T, F, 5, U, MODE>(a, j0, tile_byte, tile_bytes, lane_byte, acc);
      break;
    case 6:
      fold_chunk<T, F, 6, U, MODE>(a, j0, tile_byte, tile_bytes, lane_byte, acc);
      break;
    case 7:
      fold_chunk<T, F, 7, U, MODE>(a, j0, tile_byte, tile_bytes, lane_byte, acc);
      break;
    default:
      break;
    }
  }
  const __amdgpu_buffer_rsrc_t rd = tile_rsrc((const char*)a.dst + tile_byte, tile_bytes);
  u32x4 out[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    elem_t e[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
      e[i] = Tr::template finish<F>(acc[u][i], MODE, a.scale);
    }
    __builtin_memcpy(&out[u], e, 16);
  }
  // results in registers of their own, then the stores back to back (a shared data register
  // would make each store wait for the one before it)
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    tile_store(rd, lane_byte + (uint32_t)u * (kBlock * 16), out[u]); // dropped by the hardware past the end
  }
}

// A tile is kBlock*U consecutive 16-byte vectors; tiles are dealt to
// workgroups round-robin.  Pointers need only element alignment: gfx950's
// 16-byte buffer accesses take any byte address.  Elements past the last whole
// vector (fewer than 16 bytes) are folded by workgroup 0.
template<typename T, int F, int NSRC, int U>
__global__ __launch_bounds__(kBlock) void reduce_vec_kernel(ReduceArgs a) {
  const int nsrc = NSRC ? NSRC : a.nsrc;
  constexpr uint64_t tile_bytes = (uint64_t)kBlock * U * 16;
  const uint64_t body_bytes = a.nvec * 16;
  const uint64_t ntiles = (body_bytes + tile_bytes - 1) / tile_bytes;
  for (uint64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    const uint64_t tile_byte = tile * tile_bytes;
    const uint64_t left = body_bytes - tile_byte;
    const uint32_t n = (uint32_t)(left < tile_bytes ? left : tile_bytes);
    // the mode is wave-uniform: one branch per tile keeps the scale multiplies out of the plain path
    if (F != kSum || a.mode == kPlain) {
      reduce_tile<T, F, NSRC, U, kPlain>(a, nsrc, tile_byte, n);
    } else if (a.mode == kAvg) {
      reduce_tile<T, F, NSRC, U, kAvg>(a, nsrc, tile_byte, n);
    } else {
      reduce_tile<T, F, NSRC, U, kPremul>(a, nsrc, tile_byte, n);
    }
  }
  if (blockIdx.x == 0) {
    const uint64_t i = a.nvec * per_vec<T>() + threadIdx.x;
    if (i < a.numel) {
      reduce_one_elem<T, F>(a, nsrc, i);
    }
  }
}

template<typename T, int F, int NSRC>
int launch_vec(const ReduceArgs& a, hipStream_t stream) {
  const Tuning& t = tuning();
  // 16-bit types widen every vector to eight fp32 accumulators: two sub-tiles at most, and one
  // when sixteen sources are unrolled (their loads alone fill the register budget; measured
  // 6.4 TB/s against 5.3 TB/s with two on the bf16 sixteen-source workload).
  int U = t.reduce_unroll ? t.reduce_unroll : auto_unroll(a.nvec, 4);
  if (sizeof(typename Traits<T>::elem_t) == 2) {
    U = U > 2 ? 2 : U;
    if (NSRC >= 16) {
      U = 1;
    }
  } else if (U > 4 && NSRC != 8) {
    U = 4; // eight sub-tiles exist only for the unrolled eight-source kernel (64 loads in flight)
  }
  const uint64_t tile_vecs = (uint64_t)kBlock * U;
  uint64_t ntiles = (a.nvec + tile_vecs - 1) / tile_vecs;
  if (ntiles == 0) {
    ntiles = 1; // tail only
  }
  uint64_t grid = ntiles;
  if (t.reduce_max_blocks > 0 && grid > (uint64_t)t.reduce_max_blocks) {
    grid = t.reduce_max_blocks;
  }
  if (grid > 0x7fffffffull) {
    grid = 0x7fffffffull;
  }
  dim3 g((unsigned)grid), b(kBlock);
  if (U == 1) {
    hipLaunchKernelGGL((reduce_vec_kernel<T, F, NSRC, 1>), g, b, 0, stream, a);
  } else if (U == 2) {
    hipLaunchKernelGGL((reduce_vec_kernel<T, F, NSRC, 2>), g, b, 0, stream, a);
  } else if (U == 4) {
    hipLaunchKernelGGL((reduce_vec_kernel<T, F, NSRC, 4>), g, b, 0, stream, a);
  } else {
    if constexpr (NSRC == 8 && sizeof(typename Traits<T>::elem_t) >= 4) {
      hipLaunchKernelGGL((reduce_vec_kernel<T, F, NSRC, 8>), g, b, 0, stream, a);
    }
  }
  return check_launch("reduce_vec_kernel");
}

template<typename T, int F>
int launch(const ReduceArgs& a, hipStream_t stream) {
  // Source counts with a fully unrolled instantiation; anything else takes
  // the run-time loop over chunks of eight.
  if constexpr (std::is_same_v<T, float> || std::is_same_v<T, bf16_t>) {
    if (a.nsrc == 8) {
      return launch_vec<T, F, 8>(a, stream);
    }
    if (a.nsrc == 16) {
      return launch_vec<T, F, 16>(a, stream);
    }
  }
  return launch_vec<T, F, 0>(a, stream);
}

// One entry per (element type, fold), each instantiated in its own object
// file (reduce_inst.hip compiled once per pair) so they build in parallel.
#define MDH_REDUCE_ENTRY(tname, fname) \
  int reduce_launch_##tname##_##fname(const ReduceArgs& a, hipStream_t stream)
#define MDH_REDUCE_ENTRIES(tname) \
  MDH_REDUCE_ENTRY(tname, sum);   \
  MDH_REDUCE_ENTRY(tname, min);   \
  MDH_REDUCE_ENTRY(tname, max);
MDH_REDUCE_ENTRIES(f32)
MDH_REDUCE_ENTRIES(f64)
MDH_REDUCE_ENTRIES(i32)
MDH_REDUCE_ENTRIES(i64)
MDH_REDUCE_ENTRIES(bf16)
MDH_REDUCE_ENTRIES(f16)

} // namespace mdh
