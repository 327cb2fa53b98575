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
    // both candidates are computed and one is selected: no divergent branch per element
    const uint32_t u = __float_as_uint(f);
    const uint32_t rounded = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    const uint32_t quiet = (u >> 16) | 0x0040u;
    return (uint16_t)((u & 0x7fffffffu) > 0x7f800000u ? quiet : rounded);
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
    if constexpr (sizeof(elem_t) == 2) {
      // One source at a time: left alone, the scheduler widens every 16-bit value of the chunk
      // to fp32 before the first add, which doubles the registers the chunk occupies.
      __builtin_amdgcn_sched_barrier(0);
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
  for (int j = 1; j < nsrc; ++j) {
    acc_t x = Tr::widen(((const elem_t*)a.src[j])[i]);
    if (a.mode == kPremul) {
      x = Tr::premul(x, a.scale);
    }
    acc = fold<F>(acc, x);
  }
  ((elem_t*)a.dst)[i] = Tr::template finish<F>(acc, a.mode, a.scale);
}

template<typename T, int F, int U, int MODE>
__device__ __forceinline__ void reduce_tile(const ReduceArgs& a, int nsrc, uint64_t tile_byte, uint32_t tile_bytes) {
  using Tr = Traits<T>;
  using elem_t = typename Tr::elem_t;
  using acc_t = typename Tr::acc_t;
  constexpr int N = per_vec<T>();
  constexpr int CH = 8;
  const uint32_t lane_byte = threadIdx.x * 16;
  acc_t acc[U][N];
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
  const __amdgpu_buffer_rsrc_t rd = tile_rsrc((const char*)a.dst + tile_byte, tile_bytes);
  u32x4 out[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    elem_t e[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
      e[i] = Tr::template finish<F>(acc[u][i], MODE == kPremul ? (int)kPremul : a.mode, a.scale);
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
template<typename T, int F, int U, bool PREMUL>
__global__ __launch_bounds__(kBlock) void reduce_vec_kernel(ReduceArgs a) {
  const int nsrc = a.nsrc;
  constexpr uint64_t tile_bytes = (uint64_t)kBlock * U * 16;
  const uint64_t body_bytes = a.nvec * 16;
  const uint64_t ntiles = (body_bytes + tile_bytes - 1) / tile_bytes;
  for (uint64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    const uint64_t tile_byte = tile * tile_bytes;
    const uint64_t left = body_bytes - tile_byte;
    const uint32_t n = (uint32_t)(left < tile_bytes ? left : tile_bytes);
    // PREMUL_SUM is a kernel of its own: for 16-bit types every source element is rounded to the
    // element type after the multiply, which takes several times the registers of the plain
    // fold, and a kernel's register budget is that of its hungriest path.  AVG is the plain
    // fold with one more multiply when the result is written (a wave-uniform test there).
    reduce_tile<T, F, U, PREMUL ? kPremul : kPlain>(a, nsrc, tile_byte, n);
  }
  if (blockIdx.x == 0) {
    const uint64_t i = a.nvec * per_vec<T>() + threadIdx.x;
    if (i < a.numel) {
      reduce_one_elem<T, F>(a, nsrc, i);
    }
  }
}

struct LaunchShape {
  int unroll;    // sub-tiles per lane: 1, 2 or 4
  int wg_per_cu; // 0 = as many as the registers allow
};

// Chosen by measurement on MI355X (TB/s of algorithmic bytes on one box; sub-tiles/workgroups
// per CU, "-" = no cap):
//   fp32  8 x 16 MiB   4/-: 6.34   2/-: 5.26   1/2: 5.36   2/2: 5.56
//   fp32  8 x 32 MiB   4/-: 6.40   1/2: 6.08        8 x 48 MiB   4/-: 6.37   1/2: 6.52
//   fp32  8 x 64 MiB   4/-: 6.34   1/2: 6.56        8 x 128 MiB  4/-: 6.30   1/2: 6.68
//   fp32 16 x 32 MiB   4/-: 6.40   1/2: 6.23       16 x 48 MiB   4/-: 6.30   1/2: 6.69
//   fp32 32 x 64 MiB   4/-: 5.97   1/2: 6.53       64 x 64 MiB   4/-: 6.42   1/2: 6.55
//   bf16 16 x 16 MiB   4/-: 6.27   1/2: 5.35       16 x 64 MiB   4/-: 6.13   1/2: 6.64
//   bf16  8 x 16 MiB   4/-: 6.10   2/2: 5.54        8 x 64 MiB   4/-: 6.32   2/2: 6.61   1/2: 6.08
//   fp16  8 x 64 MiB   4/-: 6.30   1/2: 6.47   2/2: 5.96
//   fp32  4 x 32 MiB   4/-: 6.48   1/2: 5.21   (few sources: a cap starves the CU)
// Four sub-tiles and no cap is best or equal below about 48 MiB per source and with fewer
// than eight sources.  Above that a launch spends most of its time in a steady state in
// which reads and writes interleave at the DRAM, and two workgroups per CU with eight loads
// in flight per lane do better (bf16 with eight or nine sources: sixteen).
template<typename T, bool PREMUL>
LaunchShape choose_shape(const ReduceArgs& a) {
  const Tuning& t = tuning();
  constexpr bool half = sizeof(typename Traits<T>::elem_t) == 2;
  LaunchShape s{auto_unroll(a.nvec, 4), 0};
  if (PREMUL && half) {
    s.unroll = 1; // the per-element rounding of PREMUL_SUM fills the register file on its own
  } else if (!PREMUL && a.nvec >= ((uint64_t)48 << 20) / 16 && a.nsrc >= 8) {
    s.unroll = (std::is_same_v<T, bf16_t> && a.nsrc < 10) ? 2 : 1;
    s.wg_per_cu = 2;
  }
  if (t.reduce_unroll) {
    s.unroll = t.reduce_unroll > 4 ? 4 : t.reduce_unroll;
  }
  if (t.reduce_wg_per_cu) {
    s.wg_per_cu = t.reduce_wg_per_cu > 8 ? 0 : t.reduce_wg_per_cu; // 9 = no cap
  }
  return s;
}

template<typename T, int F, bool PREMUL = false>
int launch_vec(const ReduceArgs& a, hipStream_t stream) {
  const Tuning& t = tuning();
  const LaunchShape shape = choose_shape<T, PREMUL>(a);
  const int U = shape.unroll;
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
  const size_t lds = kLdsForCap[shape.wg_per_cu];
#define MDH_LAUNCH_REDUCE(UU)                                                                            \
  do {                                                                                                   \
    auto* fn = reduce_vec_kernel<T, F, UU, PREMUL>;                                                      \
    if (lds > 65536) {                                                                                   \
      /* more than 64 KiB of dynamic LDS has to be allowed once per kernel */                            \
      static bool raised = false;                                                                        \
      if (!raised) {                                                                                     \
        if (hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) { \
          (void)hipGetLastError();                                                                       \
          set_error("reduce_vec_kernel: the device refused %zu bytes of dynamic LDS", lds);              \
          return MDH_ELAUNCH;                                                                            \
        }                                                                                                \
        raised = true;                                                                                   \
      }                                                                                                  \
    }                                                                                                    \
    hipLaunchKernelGGL(fn, g, b, lds, stream, a);                                                        \
  } while (0)
  if (U == 1) {
    MDH_LAUNCH_REDUCE(1);
  } else if (U == 2) {
    MDH_LAUNCH_REDUCE(2);
  } else {
    MDH_LAUNCH_REDUCE(4);
  }
#undef MDH_LAUNCH_REDUCE
  return check_launch("reduce_vec_kernel");
}

template<typename T, int F>
int launch(const ReduceArgs& a, hipStream_t stream) {
  if constexpr (F == kSum && (std::is_floating_point_v<T> || sizeof(typename Traits<T>::elem_t) == 2)) {
    if (a.mode == kPremul) {
      return launch_vec<T, F, true>(a, stream);
    }
  }
  return launch_vec<T, F>(a, stream);
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
