// Device-side helpers shared by the gfx950 kernels: 16-byte streaming loads
// and stores, and the host-side error plumbing of the C ABI.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "moodist_hip.h"

namespace mdh {

// One lane moves 16 bytes per instruction (global_load_dwordx4 /
// global_store_dwordx4): a wave64 instruction covers 1 KiB of contiguous HBM.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kBlock = 256; // 4 wave64 per workgroup

#ifndef MDH_NT_LOAD
#define MDH_NT_LOAD 1
#endif
#ifndef MDH_NT_STORE
#define MDH_NT_STORE 1
#endif

// Sources are read once and outputs written once, so both bypass cache
// retention (the `nt` bit) and leave L2 / Infinity Cache to other work.
template<typename V>
__device__ __forceinline__ V stream_load(const V* p) {
#if MDH_NT_LOAD
  return __builtin_nontemporal_load(p);
#else
  return *p;
#endif
}

template<typename V>
__device__ __forceinline__ void stream_store(V* p, V v) {
#if MDH_NT_STORE
  __builtin_nontemporal_store(v, p);
#else
  *p = v;
#endif
}

// Buffer addressing for tiles: the descriptor's base is wave-uniform and its
// size bounds the tile, so out-of-range lanes load zero and their stores are
// dropped by the address unit.  Cache-policy bits (gfx940 encoding of the
// intrinsic's aux operand): 2 = nt, 16 = sc1.
//   loads  nt   read-once data, evict first;
//   stores sc1  device-scope write-through: the line leaves L2 at once rather
//               than waiting as a dirty line (measurably faster than nt here).
#ifndef MDH_LOAD_AUX
#define MDH_LOAD_AUX 2
#endif
#ifndef MDH_STORE_AUX
#define MDH_STORE_AUX 16
#endif

__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (int)bytes, 0x00020000);
}

template<int AUX = MDH_LOAD_AUX>
__device__ __forceinline__ u32x4 tile_load(__amdgpu_buffer_rsrc_t rs, uint32_t byte_offset) {
  return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, (int)byte_offset, 0, AUX));
}

template<int AUX = MDH_STORE_AUX>
__device__ __forceinline__ void tile_store(__amdgpu_buffer_rsrc_t rs, uint32_t byte_offset, u32x4 v) {
  __builtin_amdgcn_raw_buffer_store_b128(v, rs, (int)byte_offset, 0, AUX);
}

// ---- host side ----

void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

int check_launch(const char* what);

// MDH_OK when launches may be enqueued on `stream`; MDH_ECAPTURE, with the message set, when the
// stream is being captured into a graph (see MDH_ECAPTURE).  Every launch function asks before
// it enqueues anything.
int refuse_capture(hipStream_t stream, const char* who);

// 0 = choose by size (the default); any other value is taken as given.
struct Tuning {
  int reduce_unroll = 0; // KiB of each source per tile: 1, 2, 4, 8, 16
  int reduce_chunk = 0;  // sources in flight together: 1, 2, 4, 8
  int reduce_max_blocks = 0;
  int reduce_split_tiles = 0; // tiles of one launch at most (longer reductions are cut into several launches)
  int reduce_wg_per_cu = 0; // cap on resident workgroups per CU (1..8; 9 = none), through an unused LDS allocation
  int copy_unroll = 0; // contiguous segments
  int box_unroll = 0;  // strided boxes
  int copy_max_blocks = 0;
  int copy_wg_per_cu = 0; // as reduce_wg_per_cu, for the copy kernels
  int box_policy = 0;     // loads of the strided-box kernel: 1 plain, 0 or 2 nt
  int box_tile_cols = 0;  // columns (16-byte vectors) of a strided-box tile, a power of two; the tile's rows follow
  int box_transpose = 0;  // 1: transposing boxes take the plain strided kernel instead of LDS-staged tiles; 2: tiles always dealt row by row; 3: always along the diagonals
  int box_transpose_wgs = 0; // workgroups that walk the tiles of a transposing launch (0 = one per tile)
  int box_transpose_tile = 0; // tile of the transposing copy with 16-byte accesses: 0 T x T, 1 T x 2T, 2 2T x T, 3 2T x 2T (A x B)
  int box_preload = 0;    // 1: never launch equal boxes of full tiles from preloaded arguments
  // measurement variants of the dense copy of up to eight equal segments (see copy_flat8_kernel)
  int copy_xcd_run = 0;    // 2, 4, 8, ...: every XCD takes runs of this many consecutive tiles
  int copy_grid_order = 0; // 1: the grid is transposed, the segments advance together
  int copy_tail_tiles = 0; // this many tiles at every segment's end are dealt as two halves each
  int copy_lds = 0;        // 1: loads go straight to LDS, stores are fed from there
  int allow_capture = 0;  // 1: launch functions accept a capturing stream (for a host-side check of what a capture records)
};
Tuning& tuning();

// An unused dynamic LDS allocation of this size lets exactly n workgroups share a CU's 160 KiB
// (index n): the only handle a launch has on how many workgroups a CU holds at once.
constexpr size_t kLdsForCap[9] = {0, 98304, 65536, 49152, 40960, 32768, 27136, 23296, 20480};

// Sub-tiles per lane, where longer tiles are wanted (short strided launches, dense copies of
// unequal segments): the widest that still leaves a workgroup for every CU -- below one per CU
// the smaller tile wins (1 MiB per source took 3.6 us with one sub-tile against 4.8 us with four).
inline int auto_unroll(uint64_t vectors, int widest) {
  int u = widest;
  while (u > 1 && vectors / ((uint64_t)kBlock * u) < 256) {
    u >>= 1;
  }
  return u;
}

} // namespace mdh
