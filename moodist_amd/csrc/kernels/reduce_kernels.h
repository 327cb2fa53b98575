// Single-pass K-source reduction for gfx950 (templates; one translation unit
// per element type instantiates them so the types compile in parallel).
//
// What the reference does in K-1 two-source passes over the destination
// (core/reduce_scatter.cc:104-142 emitting reduce_n2 calls,
// core/kernels.cc:171-413) is done here in one pass: a wave takes a tile of up
// to 16 KiB, reads it from every source in the reference's order (one, two,
// four or eight sources' loads in flight at a time), folds in registers and
// writes the tile once.  HBM traffic is (K+1) x bytes instead of (3K-3) x bytes.
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
  uint64_t numel; // elements from the pointers on: the vectors' and the < 16 bytes after them
  uint32_t head;  // elements BEFORE the pointers (fewer than 64 bytes): see mdh_reduce
  float scale;
  int nsrc;
  int mode;
};

// reduce_vec_kernel's leading arguments (see there): vector count, tile workgroups, source count
// and mode, scale, then this many source pointers -- fourteen dwords with the padding in front
// of the pointers; ReduceArgs follows them in the argument segment.
constexpr int kEarlySources = 4;
constexpr size_t kArgsOffset = 8 + 4 + 4 + 4 + 4 + 8 * kEarlySources;
static_assert(alignof(ReduceArgs) == 8 && kArgsOffset % alignof(ReduceArgs) == 0, "ReduceArgs follows the leading arguments without padding");
static_assert(MDH_MAX_SOURCES < 256, "the source count travels in one byte");

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
  // Round to nearest even; a NaN keeps its sign and upper payload and gets the quiet bit.  That is
  // what gfx950's v_cvt_pk_bf16_f32 does, to which this conversion compiles: for every one of the
  // 2^32 fp32 bit patterns it returns ((u + 0x7fff + ((u >> 16) & 1)) >> 16), or (u >> 16) | 0x40
  // for a NaN (checked exhaustively on the GPU by tests/native/bf16_narrow_check.cc).
  static __device__ __forceinline__ uint16_t narrow(float f) {
    const __bf16 b = (__bf16)f;
    uint16_t e;
    __builtin_memcpy(&e, &b, 2);
    return e;
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

// A workgroup of the reduction is one wave: every wave is placed, runs and retires on its own,
// and a launch aims at about one wave per SIMD (1024 on the chip).
constexpr int kWave = 64;

// Loads CNT sources' vectors for U sub-tiles (CNT*U loads in flight), then
// folds them into acc in source order.  Each source is addressed through a
// buffer descriptor whose base is the tile's first byte (wave-uniform, in
// SGPRs) and whose size is the bytes left in the tile: the lane offset is one
// VGPR, and vectors past the end read as zero instead of needing a predicate.
template<typename T, int F, int CNT, int U, int MODE, bool FIRST, int NP>
__device__ __forceinline__ void fold_chunk(float scale, const char* const (&src)[NP], uint64_t tile_byte,
    uint32_t tile_bytes, uint32_t lane_byte, typename Traits<T>::acc_t (&acc)[U][per_vec<T>()]) {
  static_assert(CNT <= NP, "a chunk has at most NP sources");
  using Tr = Traits<T>;
  using elem_t = typename Tr::elem_t;
  using acc_t = typename Tr::acc_t;
  constexpr int N = per_vec<T>();
  u32x4 v[CNT][U];
#pragma unroll
  for (int k = 0; k < CNT; ++k) {
    const __amdgpu_buffer_rsrc_t rs = tile_rsrc(src[k] + tile_byte, tile_bytes);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      v[k][u] = tile_load(rs, lane_byte + (uint32_t)u * (kWave * 16));
    }
  }
  // Every load of the chunk is issued before the first add: the number in flight is then
  // CNT*U whatever the instruction scheduler would have preferred.
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
          x = Tr::premul(x, scale);
        }
        if (FIRST && k == 0) {
          acc[u][i] = x; // the first source initialises the accumulator (the reference's memcpy)
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

// One element, folded in source order.  The loads of eight sources are issued together: one
// after the other, every source would cost this lane a whole memory round trip.
template<typename T, int F>
__device__ __forceinline__ typename Traits<T>::elem_t reduce_one_elem_value(const void* const* src, int nsrc, int mode,
    float scale, int64_t i) {
  using Tr = Traits<T>;
  using elem_t = typename Tr::elem_t;
  using acc_t = typename Tr::acc_t;
  constexpr int kBatch = 8;
  acc_t acc{};
  for (int j0 = 0; j0 < nsrc; j0 += kBatch) {
    elem_t v[kBatch];
#pragma unroll
    for (int k = 0; k < kBatch; ++k) {
      const int j = j0 + k < nsrc ? j0 + k : nsrc - 1; // past the end: the last source once more, unused
      v[k] = ((const elem_t*)src[j])[i];
    }
#pragma unroll
    for (int k = 0; k < kBatch; ++k) {
      if (j0 + k < nsrc) {
        acc_t x = Tr::widen(v[k]);
        if (mode == kPremul) {
          x = Tr::premul(x, scale);
        }
        acc = j0 + k == 0 ? x : fold<F>(acc, x);
      }
    }
  }
  return Tr::template finish<F>(acc, mode, scale);
}

template<typename T, int F>
__device__ __forceinline__ void reduce_one_elem_from(const void* const* src, int nsrc, void* dst, int mode, float scale,
    int64_t i) {
  ((typename Traits<T>::elem_t*)dst)[i] = reduce_one_elem_value<T, F>(src, nsrc, mode, scale, i);
}

template<typename T, int F>
__device__ __forceinline__ void reduce_one_elem(const ReduceArgs& a, int nsrc, int64_t i) {
  reduce_one_elem_from<T, F>(a.src, nsrc, a.dst, a.mode, a.scale, i);
}

// The head before the pointers (indices -head .. -1, fewer than 64 bytes) and the tail after the
// last whole vector (fewer than 16 bytes), one element per lane: at most 31 + 7 lanes.  Kept out
// of line: inlined into the kernel, its scalar loads were scheduled in front of the tile
// workgroups' own and cost them a second scalar round trip (0.35 us of 23).
template<typename T, int F>
__device__ __attribute__((noinline)) void reduce_head_and_tail(const ReduceArgs* args, uint32_t lane_id) {
  const ReduceArgs& a = *args;
  const int64_t lane = lane_id, head = a.head;
  const int64_t i = lane < head ? lane - head : (int64_t)(a.nvec * per_vec<T>()) + (lane - head);
  if (i < (int64_t)a.numel) {
    reduce_one_elem<T, F>(a, a.nsrc, i);
  }
}

// The sources left over when the count is not a multiple of CH (1 .. CH-1 of them).
template<typename T, int F, int U, int CH, int MODE, bool FIRST, int R = CH - 1>
__device__ __forceinline__ void fold_rest(float scale, int rest, const char* const (&src)[CH], uint64_t tile_byte,
    uint32_t tile_bytes, uint32_t lane_byte, typename Traits<T>::acc_t (&acc)[U][per_vec<T>()]) {
  if constexpr (R >= 1) {
    if (rest == R) {
      fold_chunk<T, F, R, U, MODE, FIRST>(scale, src, tile_byte, tile_bytes, lane_byte, acc);
    } else {
      fold_rest<T, F, U, CH, MODE, FIRST, R - 1>(scale, rest, src, tile_byte, tile_bytes, lane_byte, acc);
    }
  }
}

// One tile: U KiB of every source (U sub-tiles of one wave-wide 16-byte load each), consumed CH
// sources at a time in order, so the fold stays a left fold and CH*U loads are in flight.
// Where the source pointers come from is the caller's business: early(integral_constant<int, K>,
// p) fills p with the pointers of sources K .. K+CH-1 for a K known at compile time (the first
// two groups), later(first, p) does the same for any group.  Slots past the last source may hold
// anything; they are never used.  more_stores(out, lane_byte) is called after the tile's stores with
// the tile's result still in registers (for results that go to more than one place).
template<typename T, int F, int U, int CH, int MODE, typename Early, typename Later, typename More>
__device__ __forceinline__ void reduce_tile_from(Early early_pointers, Later pointers, const char* dst, int nsrc, int mode_arg,
    float scale, uint64_t tile_byte, uint32_t tile_bytes, More more_stores) {
  using Tr = Traits<T>;
  using elem_t = typename Tr::elem_t;
  using acc_t = typename Tr::acc_t;
  constexpr int N = per_vec<T>();
  const uint32_t lane_byte = threadIdx.x * 16;
  acc_t acc[U][N];
  // The pointers of a group are read from the argument table one group AHEAD of their use: read
  // when needed, every group would start with a scalar round trip during which the wave has no
  // load in flight.
  const char* cur[CH];
  const char* nxt[CH];
  early_pointers(std::integral_constant<int, 0>{}, cur);
  early_pointers(std::integral_constant<int, CH>{}, nxt);
  // the first group is peeled so that "initialise or fold" is decided at compile time
  if (nsrc >= CH) {
    fold_chunk<T, F, CH, U, MODE, true>(scale, cur, tile_byte, tile_bytes, lane_byte, acc);
    int j0 = CH;
    for (; nsrc - j0 >= CH; j0 += CH) {
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        cur[k] = nxt[k];
      }
      pointers(j0 + CH, nxt);
      fold_chunk<T, F, CH, U, MODE, false>(scale, cur, tile_byte, tile_bytes, lane_byte, acc);
    }
    fold_rest<T, F, U, CH, MODE, false>(scale, nsrc - j0, nxt, tile_byte, tile_bytes, lane_byte, acc);
  } else {
    fold_rest<T, F, U, CH, MODE, true>(scale, nsrc, cur, tile_byte, tile_bytes, lane_byte, acc);
  }
  const __amdgpu_buffer_rsrc_t rd = tile_rsrc(dst + tile_byte, tile_bytes);
  u32x4 out[U];
  // AVG's extra multiply is decided once per tile (wave-uniform), not per element
  const int mode = MODE == kPremul ? (int)kPremul : mode_arg;
  if (mode == kAvg) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      elem_t e[N];
#pragma unroll
      for (int i = 0; i < N; ++i) {
        e[i] = Tr::template finish<F>(acc[u][i], kAvg, scale);
      }
      __builtin_memcpy(&out[u], e, 16);
    }
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      elem_t e[N];
#pragma unroll
      for (int i = 0; i < N; ++i) {
        e[i] = Tr::template finish<F>(acc[u][i], kPlain, scale);
      }
      __builtin_memcpy(&out[u], e, 16);
    }
  }
  // results in registers of their own, then the stores back to back (a shared data register
  // would make each store wait for the one before it)
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    tile_store(rd, lane_byte + (uint32_t)u * (kWave * 16), out[u]); // dropped by the hardware past the end
  }
  more_stores(out, lane_byte);
}

// The tile of a single reduction: pointers from the launch's argument struct, the first
// kEarlySources of them from the kernel's leading arguments.
template<typename T, int F, int U, int CH, int MODE>
__device__ __forceinline__ void reduce_tile(const ReduceArgs& a, const char* const (&early)[kEarlySources], int nsrc,
    int mode_arg, float scale, uint64_t tile_byte, uint32_t tile_bytes) {
  // (slots past the last source are never used; 63 is the table's last index)
  auto pointers = [&](int first, const char* (&p)[CH]) {
#pragma unroll
    for (int k = 0; k < CH; ++k) {
      const int j = first + k;
      p[k] = (const char*)a.src[j < MDH_MAX_SOURCES ? j : MDH_MAX_SOURCES - 1];
    }
  };
  // The first two groups' indices are compile-time constants: those below kEarlySources are
  // the kernel's leading arguments, in registers when the wave starts, so the first vector
  // loads wait for no scalar load at all.
  auto early_pointers = [&](auto first, const char* (&p)[CH]) {
#pragma unroll
    for (int k = 0; k < CH; ++k) {
      constexpr int kFirst = decltype(first)::value;
      const int j = kFirst + k;
      p[k] = j < kEarlySources ? early[j < kEarlySources ? j : 0] : (const char*)a.src[j < MDH_MAX_SOURCES ? j : MDH_MAX_SOURCES - 1];
    }
  };
  reduce_tile_from<T, F, U, CH, MODE>(early_pointers, pointers, (const char*)a.dst, nsrc, mode_arg, scale, tile_byte, tile_bytes,
      [](const u32x4 (&)[U], uint32_t) {});
}

// A tile is kWave*U consecutive 16-byte vectors (U KiB); tiles are dealt to
// waves round-robin.  Pointers need only element alignment: gfx950's
// 16-byte buffer accesses take any byte address.  Elements before the pointers (a.head, fewer
// than 64 bytes) and past the last whole vector (fewer than 16 bytes) are folded by workgroup 0,
// which has no tiles.
template<typename T, int F, int U, int CH, bool PREMUL>
__global__ __launch_bounds__(kWave) void reduce_vec_kernel(uint64_t nvec, uint32_t tile_waves, uint32_t nsrc_and_mode,
    float scale, const char* s0, const char* s1, const char* s2, const char* s3, ReduceArgs a) {
  // The leading arguments repeat what a tile workgroup needs before its first vector load and
  // to find its next tile -- vector count, number of tile workgroups, source count (low byte)
  // and mode, the scale, the first four source pointers: compiled with
  // -amdgpu-kernarg-preload-count they arrive in registers with the wave (fourteen dwords, all
  // that the hardware preloads), where a read from the argument segment is a scalar round trip
  // to memory the host has just written: 0.3-0.5 us of a launch that lasts 3-9 us.  (The scale
  // is not needed early, but a scalar load of it, once the compiler chose to copy its result
  // before the loop over the tiles, made the wave wait there for every load issued so far.)
  const char* const early[kEarlySources] = {s0, s1, s2, s3};
  const int nsrc = (int)(nsrc_and_mode & 0xff);
  const int mode = (int)(nsrc_and_mode >> 8);
  constexpr uint64_t tile_bytes = (uint64_t)kWave * U * 16;
  const uint64_t body_bytes = nvec * 16;
  const uint64_t ntiles = (body_bytes + tile_bytes - 1) / tile_bytes;
  // The head and tail elements have a workgroup of their own, workgroup 0 of every launch
  // (which finds nothing to do when there are none): folded by a workgroup that also has
  // tiles, their round trips would come on top of that wave's tiles and lengthen the whole
  // launch (by 1.5 us of 23 for eight sources).  That it is ALWAYS workgroup 0 lets the tile
  // workgroups know what they are from blockIdx alone: a test that needed a kernel argument
  // held their first loads up behind one more scalar round trip (0.4 us of 23).
  if (blockIdx.x == 0) {
    // ReduceArgs follows the leading arguments (kArgsOffset bytes) in the argument segment: the
    // function reads it from there.  (The address of the kernel's own parameter would make
    // every wave of the launch copy the struct to its stack first; and the segment's address has
    // to be taken here, in the kernel -- inside a called function the builtin yields null.)
    const char* segment = (const char*)__builtin_amdgcn_kernarg_segment_ptr();
    reduce_head_and_tail<T, F>((const ReduceArgs*)(segment + kArgsOffset), threadIdx.x);
    return;
  }
  // The tile workgroups never outnumber the tiles (a launch with no whole vector has one, whose
  // descriptors are then empty), so the first tile needs no test and the scalar loads of the
  // arguments are not held up behind a load-and-branch.
  uint64_t tile = blockIdx.x - 1;
  do {
    const uint64_t tile_byte = tile * tile_bytes;
    const uint64_t left = body_bytes - tile_byte;
    const uint32_t n = (uint32_t)(left < tile_bytes ? left : tile_bytes);
    // PREMUL_SUM is a kernel of its own, so that the plain fold carries neither its multiply nor,
    // for 16-bit types, the rounding of every source element to the element type after it.  AVG
    // is the plain fold with one more multiply when the result is written (a wave-uniform test
    // there).
    reduce_tile<T, F, U, CH, PREMUL ? kPremul : kPlain>(a, early, nsrc, mode, scale, tile_byte, n);
    tile += tile_waves;
  } while (tile < ntiles);
}

struct LaunchShape {
  int unroll;     // sub-tiles (KiB of each source) per tile: 1, 2, 4, 8 or 16
  int chunk;      // sources whose loads are in flight together: 1, 2, 4 or 8
  uint64_t waves; // grid size
};

// Chosen by measurement on MI355X (percent of 8 TB/s, algorithmic bytes; one-wave workgroups;
// tile KiB x sources in flight @ waves).  These rows were measured with the launches rotating
// over 0.6-1.2 GiB of buffers, where the 256 MB Infinity Cache still helps every shape by 2-4
// points; rotating over 4-8 GiB the order is the same (8 x 16 MiB: 16x1@1024 82.2, 16x2 81.0,
// 16x1@512 78.6, 8x2 76.8, 4x4 67.8; 64 x 4 MiB: 8x2 84.9, 16x2 77.5, 4x4 78.1, 16x1 61.7):
//   fp32  8 x 16 MiB   16x1@1024: 84.4   16x1@512: 80.4   16x2@1024: 83.3   8x2@2048: 77.9   4x8@1024: 72.8
//   fp32  8 x 64 MiB   16x1@512: 84.8    16x1@1024: 81.6  16x1@4096: 82.8   16x2@1024: 84.8  8x2@512: 83.8
//   fp32 16 x 32 MiB   16x1@512: 86.8    16x1@1024: 85.2  16x2@1024: 86.3   8x1@1024: 84.2
//   fp32 64 x 4 MiB    8x2@512: 87.0     16x1@256: 64.4   16x2@256: 78.1    4x4@1024: 80.0   4x2@1024: 85.9
//   fp32 16 x 8 MiB    16x1@512: 83.1    8x1@1024: 83.9   8x2@1024: 80.0
//   fp32  2 x 64 MiB   16x1@512: 84.3    8x2@512: 84.5    16x2@1024: 77.7
//   fp32  8 x 4 MiB    4x8@1024: 63.7    8x2@512: 60.3    16x1@256: 52.6
//   fp32  8 x 1 MiB    2x8@512: 31.3     4x8@256: 30.5    16x1@64: 16.1
//   bf16 16 x 64 MiB   16x1@4096: 84.0   16x1@1024: 82.5  16x1@512: 78.6    8x2@512: 80.8    16x2@1024: 82.5
//   bf16  8 x 16 MiB   16x1@1024: 79.4   16x1@512: 65.1   8x2@1024: 73.6    4x4@4096: 75.0
// against 79.4 / 80.1 / 78.6 / 82.3 / 77.8 / 72.2 / 63.0 / 24.2 (fp32) for 256-lane workgroups that keep
// eight sources x 4 KiB in flight per lane.  What the good shapes share: the longest tile that
// still leaves about 512 tiles, sixteen loads in flight per lane, one source (or two) at a time,
// and no more than about one wave per SIMD -- the chip then sweeps one source after the other
// and the writes come in a burst of their own, instead of nine streams interleaving at the DRAM.
template<typename T, bool PREMUL>
LaunchShape choose_shape(const ReduceArgs& a) {
  const Tuning& t = tuning();
  constexpr bool half = sizeof(typename Traits<T>::elem_t) == 2;
  // The longest tile that still leaves this many tiles: 512 (a wave on every other SIMD), or
  // 1024 for 16-bit types, whose arithmetic per byte needs every SIMD, and for sources of 2 MiB
  // and less, where the launch is over before a second tile per wave would have paid.
  // Measured from HBM, 8 sources, us per launch with 512 / 1024 tiles: bf16 2 MiB per source
  // 5.87 / 5.05, 8 MiB 15.4 / 14.6, 16 MiB (1024 / 2048) 24.0 / 26.3; fp32 1 MiB 3.58 / 3.35,
  // 2 MiB 5.24 / 5.00, 4 MiB 7.86 / 8.10, 8 MiB 12.7 / 13.0.
  const uint64_t min_tiles = (half || a.nvec <= ((uint64_t)2 << 20) / 16) ? 1024 : 512;
  int u = 16;
  while (u > 1 && a.nvec / ((uint64_t)kWave * u) < min_tiles) {
    u >>= 1;
  }
  int ch = u >= 16 ? 1 : 16 / u > 8 ? 8 : 16 / u;
  if (t.reduce_unroll) {
    u = t.reduce_unroll;
    ch = u >= 16 ? 1 : 16 / u > 8 ? 8 : 16 / u;
  }
  if (t.reduce_chunk) {
    ch = t.reduce_chunk;
    if (!t.reduce_unroll) {
      u = ch == 1 ? 16 : ch == 2 ? (u >= 16 ? 16 : 8) : ch == 4 ? 4 : u > 2 ? 2 : u;
    }
  }
  LaunchShape s{u, ch, 0};
  const uint64_t tile_vecs = (uint64_t)kWave * u;
  uint64_t ntiles = (a.nvec + tile_vecs - 1) / tile_vecs;
  if (ntiles == 0) {
    ntiles = 1; // tail only
  }
  // From two tiles per SIMD on, 512 waves that walk the tiles keep fewer streams open (fp32
  // 8 x 64 MiB: 84.8 % against 82.8 % with a wave per tile).  16-bit types spend more arithmetic
  // per byte (widening), which a lone wave on a SIMD overlaps less well with its own loads: they
  // go to 512 waves from 4096 tiles on and take 1024 in between (bf16 16 x 64 MiB: 86.7 % with
  // 512 waves, 83.0 % with 1024, 80.7 % with a wave per tile; 8 x 32 MiB, 2048 tiles: 78.9 / 81.2 /
  // 78.7 %).
  if (half) {
    s.waves = ntiles >= 4096 ? 512 : ntiles >= 2048 ? 1024 : ntiles;
  } else {
    s.waves = ntiles >= 2048 ? 512 : ntiles;
  }
  if (t.reduce_max_blocks > 0) {
    s.waves = ntiles < (uint64_t)t.reduce_max_blocks ? ntiles : (uint64_t)t.reduce_max_blocks;
  }
  return s;
}

template<typename T, int F, bool PREMUL = false>
int launch_one(const ReduceArgs& a, hipStream_t stream);

// Tiles of one launch at most.  While the waves of a launch walk the sources in step, the chip
// reads one source at a time and writes in bursts; over many tiles per wave they drift apart,
// reads and writes mix at the DRAM, and the rate falls towards that of a mixed stream (fp32
// 8 sources: 84.8 % at 64 MiB per source, 82.0 % at 128 MiB, 76.5 % at 256 MiB, 73.8 % at
// 512 MiB in one launch, whatever the grid).  A launch boundary lines the waves up again for the
// price of one launch gap (1.6 us per 90 us and more).
constexpr uint64_t kSplitTiles = 4096;

template<typename T, int F, bool PREMUL = false>
int launch_vec(const ReduceArgs& a, hipStream_t stream) {
  const Tuning& t = tuning();
  const LaunchShape whole = choose_shape<T, PREMUL>(a);
  const uint64_t tile_vecs = (uint64_t)kWave * whole.unroll;
  const uint64_t ntiles = (a.nvec + tile_vecs - 1) / tile_vecs;
  const uint64_t limit = t.reduce_split_tiles > 0 ? (uint64_t)t.reduce_split_tiles : kSplitTiles;
  if (ntiles <= limit + limit / 2) {
    return launch_one<T, F, PREMUL>(a, stream);
  }
  // equal parts, each a whole number of passes of 512 waves
  const uint64_t parts = (ntiles + limit - 1) / limit;
  const uint64_t part_tiles = ((ntiles + parts - 1) / parts + 511) / 512 * 512;
  const uint64_t part_vecs = part_tiles * tile_vecs;
  constexpr uint64_t kElemsPerVec = 16 / sizeof(typename Traits<T>::elem_t);
  for (uint64_t at = 0; at < a.nvec; at += part_vecs) {
    ReduceArgs part = a;
    for (int j = 0; j < a.nsrc; ++j) {
      part.src[j] = (const char*)a.src[j] + at * 16;
    }
    part.dst = (char*)a.dst + at * 16;
    part.head = at == 0 ? a.head : 0;
    const bool last = at + part_vecs >= a.nvec;
    part.nvec = last ? a.nvec - at : part_vecs;
    // the elements past the last whole vector belong to the last part
    part.numel = last ? a.numel - at * kElemsPerVec : part_vecs * kElemsPerVec;
    const int rc = launch_one<T, F, PREMUL>(part, stream);
    if (rc != MDH_OK) {
      return rc;
    }
  }
  return MDH_OK;
}

template<typename T, int F, bool PREMUL>
int launch_one(const ReduceArgs& a0, hipStream_t stream) {
  const Tuning& t = tuning();
  const LaunchShape shape = choose_shape<T, PREMUL>(a0);
  const ReduceArgs& a = a0;
  dim3 g((unsigned)shape.waves + 1), b(kWave); // workgroup 0 takes the head and tail elements
  // reduce_wg_per_cu (measurement only): an unused LDS allocation caps the waves resident on a CU
  const int cap = t.reduce_wg_per_cu >= 2 && t.reduce_wg_per_cu <= 8 ? t.reduce_wg_per_cu : 0;
  const size_t lds = kLdsForCap[cap];
  const uint32_t lead = (uint32_t)a.nsrc | (uint32_t)a.mode << 8;
  const char* e[kEarlySources];
  for (int j = 0; j < kEarlySources; ++j) {
    e[j] = (const char*)a.src[j]; // slots past the last source hold null and are never read
  }
#define MDH_LAUNCH_REDUCE(UU, CC)                                                  \
  if (shape.unroll == UU && shape.chunk == CC) {                                   \
    hipLaunchKernelGGL((reduce_vec_kernel<T, F, UU, CC, PREMUL>), g, b, lds, stream, a.nvec, (uint32_t)shape.waves, lead, a.scale, \
        e[0], e[1], e[2], e[3], a);                                                \
    return check_launch("reduce_vec_kernel");                                      \
  }
  MDH_LAUNCH_REDUCE(16, 1)
  MDH_LAUNCH_REDUCE(16, 2)
  MDH_LAUNCH_REDUCE(8, 2)
  MDH_LAUNCH_REDUCE(4, 4)
  MDH_LAUNCH_REDUCE(2, 8)
  MDH_LAUNCH_REDUCE(1, 8)
#undef MDH_LAUNCH_REDUCE
  set_error("reduce: no kernel for %d sub-tiles x %d sources in flight (compiled: 16x1, 16x2, 8x2, 4x4, 2x8, 1x8)",
      shape.unroll, shape.chunk);
  return MDH_EINVAL;
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

// ---- a list of reductions in one launch ----
//
// The coalesced collectives bring many small tensors at once (reduce_scatter_tensor_coalesced,
// allreduce_coalesced: wrapper/processgroup_wrapper.cc:159-191 loop over them, one collective and
// one kernel launch each).  Launches of a few KiB to a few MiB are bound by the 1.6 us an empty
// launch takes, so here a list of reductions -- jobs, each with its own sources, destination and
// length, all of one element type and operation -- shares launches: the jobs' tiles are numbered
// through, a wave finds its tile's job in a table of cumulative tile counts (scalar selects), and
// the fold is the same code as a single reduction's.
constexpr int kManyJobs = 40;
constexpr int kManyPointers = 320; // 40 jobs of 8 sources, 5 of 64
constexpr uint64_t kSpreadWaves = 512; // waves that walk the 16 KiB tiles of a launch that stores its results over every source
constexpr int kManyTailSlots = 8;  // lanes per job for the elements after its last whole vector (at most 7)

struct ManyArgs {
  const void* ptr[kManyPointers]; // every job's sources in fold order, job after job
  void* dst[kManyJobs];
  uint32_t nvec[kManyJobs];     // whole 16-byte vectors
  uint32_t tile_end[kManyJobs]; // cumulative tiles; unused entries are ~0
  uint16_t first_ptr[kManyJobs];
  uint8_t nsrc[kManyJobs];
  uint8_t tail[kManyJobs]; // elements after the last whole vector
  uint32_t njobs;
  uint32_t total_tiles;
  uint32_t tile_waves; // tile workgroups of the grid (the edge workgroups come first)
  uint32_t edge_wgs;
  float scale;
  int mode;
  uint32_t spread; // 1: a job's result is stored over every one of its sources (dst is its first)
};
static_assert(sizeof(ManyArgs) + 256 <= 4096, "kernel arguments are limited to 4 KiB");

// The elements after each job's last whole vector, one per lane: job = lane index / 8.
template<typename T, int F>
__device__ __attribute__((noinline)) void reduce_many_edges(const ManyArgs* args, uint32_t wg, uint32_t lane_id) {
  const ManyArgs& a = *args;
  const uint32_t idx = wg * kWave + lane_id;
  const uint32_t job = idx / kManyTailSlots, k = idx % kManyTailSlots;
  if (job < a.njobs && k < a.tail[job]) {
    using elem_t = typename Traits<T>::elem_t;
    const int64_t i = (int64_t)a.nvec[job] * per_vec<T>() + k;
    const void* const* src = a.ptr + a.first_ptr[job];
    const elem_t r = reduce_one_elem_value<T, F>(src, a.nsrc[job], a.mode, a.scale, i);
    ((elem_t*)a.dst[job])[i] = r;
    if (a.spread) {
      for (uint32_t q = 1; q < a.nsrc[job]; ++q) {
        ((elem_t*)const_cast<void*>(src[q]))[i] = r;
      }
    }
  }
}

template<typename T, int F, int U, int CH, bool PREMUL>
__global__ __launch_bounds__(kWave) void reduce_many_kernel(ManyArgs a) {
  constexpr uint32_t tile_bytes = (uint32_t)kWave * U * 16;
  if (blockIdx.x < a.edge_wgs) {
    // (the argument segment's address has to be taken here, in the kernel)
    reduce_many_edges<T, F>((const ManyArgs*)__builtin_amdgcn_kernarg_segment_ptr(), blockIdx.x, threadIdx.x);
    return;
  }
  // the tile workgroups never outnumber the tiles: the first tile is taken untested
  uint32_t tile = blockIdx.x - a.edge_wgs;
  do {
    uint32_t job = 0, start = 0;
#pragma unroll
    for (int k = 0; k < kManyJobs - 1; ++k) {
      const uint32_t e = a.tile_end[k];
      job = tile >= e ? (uint32_t)(k + 1) : job;
      start = tile >= e ? e : start;
    }
    const uint64_t tile_byte = (uint64_t)(tile - start) * tile_bytes;
    const uint64_t left = (uint64_t)a.nvec[job] * 16 - tile_byte;
    const uint32_t n = (uint32_t)(left < tile_bytes ? left : tile_bytes);
    const uint32_t base = a.first_ptr[job];
    auto pointers = [&](int first, const char* (&p)[CH]) {
#pragma unroll
      for (int k = 0; k < CH; ++k) {
        const uint32_t j = base + (uint32_t)(first + k);
        p[k] = (const char*)a.ptr[j < (uint32_t)kManyPointers ? j : (uint32_t)kManyPointers - 1]; // unused past the job's last source
      }
    };
    auto early_pointers = [&](auto first, const char* (&p)[CH]) { pointers(decltype(first)::value, p); };
    // spread: the result goes over every source.  A tile is read from all of them before its
    // first store (the result depends on every load), and no other wave touches its bytes.
    const uint32_t nsrc = a.nsrc[job];
    const bool spread = a.spread != 0;
    auto more_stores = [&](const u32x4 (&out)[U], uint32_t lane_byte) {
      if (spread) {
        for (uint32_t q = 1; q < nsrc; ++q) {
          const uint32_t j = base + q;
          const __amdgpu_buffer_rsrc_t rd = tile_rsrc((const char*)a.ptr[j < (uint32_t)kManyPointers ? j : (uint32_t)kManyPointers - 1] + tile_byte, n);
#pragma unroll
          for (int u = 0; u < U; ++u) {
            tile_store(rd, lane_byte + (uint32_t)u * (kWave * 16), out[u]);
          }
        }
      }
    };
    reduce_tile_from<T, F, U, CH, PREMUL ? kPremul : kPlain>(early_pointers, pointers, (const char*)a.dst[job], (int)nsrc,
        a.mode, a.scale, tile_byte, n, more_stores);
    tile += a.tile_waves;
  } while (tile < a.total_tiles);
}

// One job of a list, as the host hands it over: sources already in fold order.
struct ManyJob {
  const void* const* src;
  int nsrc;
  void* dst;
  uint64_t numel;
};

template<typename T, int F, bool PREMUL>
int launch_many_one(const ManyArgs& a, int unroll, hipStream_t stream) {
  const int chunk = unroll >= 16 ? 1 : 16 / unroll > 8 ? 8 : 16 / unroll;
  dim3 g(a.edge_wgs + a.tile_waves), b(kWave);
#define MDH_LAUNCH_MANY(UU, CC)                                                            \
  if (unroll == UU && chunk == CC) {                                                       \
    hipLaunchKernelGGL((reduce_many_kernel<T, F, UU, CC, PREMUL>), g, b, 0, stream, a);    \
    return check_launch("reduce_many_kernel");                                             \
  }
  MDH_LAUNCH_MANY(16, 1)
  MDH_LAUNCH_MANY(8, 2)
  MDH_LAUNCH_MANY(4, 4)
  MDH_LAUNCH_MANY(2, 8)
  MDH_LAUNCH_MANY(1, 8)
#undef MDH_LAUNCH_MANY
  set_error("reduce_many: no kernel for %d sub-tiles", unroll);
  return MDH_EINVAL;
}

// Packs the jobs into as few launches as the tables allow (kManyJobs jobs, kManyPointers source
// pointers each) and enqueues them.  The tile is the longest of 16, 8, 4, 2, 1 KiB that leaves
// the launch about a thousand tiles (a wave per SIMD), as for a single reduction.
template<typename T, int F, bool PREMUL>
int launch_many_typed(const ManyJob* jobs, int njobs, int mode, float scale, bool spread, hipStream_t stream) {
  using elem_t = typename Traits<T>::elem_t;
  constexpr uint64_t kPerVec = 16 / sizeof(elem_t);
  int at = 0;
  while (at < njobs) {
    // How many jobs this launch takes: what the tables hold, and no more than about kSplitTiles
    // tiles of 16 KiB -- over more tiles per wave the waves drift apart like those of one long
    // reduction (40 jobs of 8 x 4 MiB in one launch: 73.8 % of the HBM rate, 8 such jobs: 77.7 %).
    int end = at, pointers = 0;
    uint64_t vectors = 0;
    constexpr uint64_t kLaunchVectors = (kSplitTiles + kSplitTiles / 2) * (uint64_t)kWave * 16;
    while (end < njobs && end - at < kManyJobs && pointers + jobs[end].nsrc <= kManyPointers &&
           (end == at || vectors + jobs[end].numel / kPerVec <= kLaunchVectors)) {
      pointers += jobs[end].nsrc;
      vectors += jobs[end].numel / kPerVec;
      ++end;
    }
    int u = 16;
    while (u > 1 && vectors / ((uint64_t)kWave * u) < 1024) {
      u >>= 1;
    }
    if (tuning().reduce_unroll) {
      u = tuning().reduce_unroll;
    }
    ManyArgs a{};
    const uint64_t tile_vecs = (uint64_t)kWave * u;
    uint64_t tiles = 0;
    uint32_t p = 0;
    for (int k = 0; k < kManyJobs; ++k) {
      a.tile_end[k] = 0xffffffffu;
    }
    for (int j = at; j < end; ++j) {
      const ManyJob& job = jobs[j];
      const int k = j - at;
      const uint64_t nvec = job.numel / kPerVec;
      a.first_ptr[k] = (uint16_t)p;
      for (int q = 0; q < job.nsrc; ++q) {
        a.ptr[p++] = job.src[q];
      }
      a.dst[k] = job.dst;
      a.nvec[k] = (uint32_t)nvec;
      a.nsrc[k] = (uint8_t)job.nsrc;
      a.tail[k] = (uint8_t)(job.numel - nvec * kPerVec);
      tiles += (nvec + tile_vecs - 1) / tile_vecs;
      a.tile_end[k] = (uint32_t)tiles;
    }
    a.njobs = (uint32_t)(end - at);
    a.total_tiles = (uint32_t)tiles;
    // up to two tiles per SIMD a wave per tile, beyond that the waves walk the tiles, as many of
    // them as a single reduction of that many tiles gets (choose_shape)
    constexpr bool half = sizeof(elem_t) == 2;
    a.tile_waves = (uint32_t)(half ? (tiles >= 4096 ? 512 : tiles >= 2048 ? 1024 : tiles) : (tiles >= 2048 ? 512 : tiles));
    if (spread) {
      // Results stored over every source: as many bytes written as read.  Tiles of 16 KiB want
      // 512 walking waves (48 x 8 jobs of 512 KiB: 772 us against 809 with a wave per tile;
      // 8 jobs of 16 MiB: 383 against 401 us), smaller tiles a wave each (48 x 8 jobs of 32 KiB:
      // 77 us against 92 with 512 waves).
      a.tile_waves = (uint32_t)(u == 16 && tiles > kSpreadWaves ? kSpreadWaves : tiles);
    }
    if (tuning().reduce_max_blocks > 0 && a.tile_waves > (uint32_t)tuning().reduce_max_blocks) {
      a.tile_waves = (uint32_t)tuning().reduce_max_blocks;
    }
    a.edge_wgs = (a.njobs * kManyTailSlots + kWave - 1) / kWave;
    a.scale = scale;
    a.mode = mode;
    a.spread = spread ? 1u : 0u;
    const int rc = launch_many_one<T, F, PREMUL>(a, u, stream);
    if (rc != MDH_OK) {
      return rc;
    }
    at = end;
  }
  return MDH_OK;
}

template<typename T, int F>
int launch_many(const ManyJob* jobs, int njobs, int mode, float scale, bool spread, hipStream_t stream) {
  if constexpr (F == kSum && (std::is_floating_point_v<T> || sizeof(typename Traits<T>::elem_t) == 2)) {
    if (mode == kPremul) {
      return launch_many_typed<T, F, true>(jobs, njobs, mode, scale, spread, stream);
    }
  }
  return launch_many_typed<T, F, false>(jobs, njobs, mode, scale, spread, stream);
}

// One entry per (element type, fold), each instantiated in its own object
// file (reduce_inst.hip compiled once per pair) so they build in parallel.
#define MDH_REDUCE_ENTRY(tname, fname)                                                  \
  int reduce_launch_##tname##_##fname(const ReduceArgs& a, hipStream_t stream);         \
  int reduce_many_launch_##tname##_##fname(const ManyJob* jobs, int njobs, int mode, float scale, bool spread, hipStream_t stream)
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
