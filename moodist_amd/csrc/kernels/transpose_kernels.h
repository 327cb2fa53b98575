// LDS-staged tiles for boxes that TRANSPOSE: the dimension along which the source is contiguous
// (A) is not the one along which the destination is (B).  Copied vector by vector along either
// side, such a box coalesces on that side only and moves one element per lane and memory
// transaction on the other (a 4096 x 4096 fp32 transpose: 107 us, 16 % of the HBM rate).  Here a
// workgroup takes a tile of TA x TB elements, reads it along A -- consecutive lanes, consecutive
// source bytes --, turns it round in LDS and writes it along B -- consecutive lanes, consecutive
// destination bytes: both sides move whole 64-byte units.
//
// The reference has no such copy: its planner gives source and destination boxes of a
// redistribution one dimension order (core/processgroup.cc:2848-2870), so a compiled custom op
// never transposes, and its Copy is an {offset, shape} box of a contiguous tensor
// (core/cputhread.h:306-310).  mdh_copy_boxes takes any strides, transposing ones included.
#pragma once
#include <type_traits>

#include "device_common.h"

namespace mdh {

#ifndef MDH_HD
#define MDH_HD __host__ __device__ __forceinline__
#endif

constexpr int kMaxTransBoxes = 16;
constexpr int kTransBatchDims = 2;

struct TransBox {
  const char* src;
  char* dst;
  int64_t src_b; // source bytes between neighbours along B (along A: the element size)
  int64_t dst_a; // destination bytes between neighbours along A (along B: the element size)
  int64_t src_o[kTransBatchDims]; // the other extents, fastest first
  int64_t dst_o[kTransBatchDims];
  uint32_t na, nb; // elements along A and B
  uint32_t no[kTransBatchDims];
  uint32_t ta, tb; // tiles along A and B
  uint32_t diagonal; // 0: the tiles run along A first, then B; 1: along the diagonals (see trans_locate)
  uint32_t reserved;
};

struct TransArgs {
  TransBox box[kMaxTransBoxes];
  uint32_t tile_end[kMaxTransBoxes]; // cumulative tiles; unused entries are ~0
  uint32_t nboxes;
  uint32_t total_tiles;
  uint32_t tile_a, tile_b; // elements along a tile's edges (the kernel's template arguments)
};
static_assert(sizeof(TransArgs) + 256 <= 4096, "kernel arguments are limited to 4 KiB");

// Elements along a tile's edges, A x B.  Square tiles of 4-16 KiB by default: 64 x 64 for elements
// of up to 4 bytes, 32 x 32 for 8 and 16.  The shapes the kernel is compiled for are listed in
// trans_shape(); `which` (the tuning knob box_transpose_tile) picks another one for measurement.
struct TransShape {
  uint32_t a, b;
};
MDH_HD constexpr TransShape trans_shape(uint32_t elem, int which) {
  const uint32_t t = elem <= 4 ? 64u : 32u;
  return which == 1 ? TransShape{t, 2 * t} : which == 2 ? TransShape{2 * t, t} : which == 3 ? TransShape{2 * t, 2 * t} : TransShape{t, t};
}

struct TransLoc {
  uint32_t box;
  uint32_t ia, ib; // the tile's first element along A and B
  int64_t src_off, dst_off; // of that element, from the box's src and dst
};

// Which box a tile belongs to and where it starts: the cumulative ends ascend, the last one at
// or below the tile names the box (scalar selects on the device); inside a box the tiles of one
// A x B plane come first, then the other extents.  Shared by the kernel and by the host-side
// check of a prepared plan.
MDH_HD TransLoc trans_locate(const TransArgs& a, uint32_t tile, uint32_t elem) {
  uint32_t b = 0, start = 0;
#pragma unroll
  for (int k = 0; k < kMaxTransBoxes - 1; ++k) {
    const uint32_t e = a.tile_end[k];
    b = tile >= e ? (uint32_t)(k + 1) : b;
    start = tile >= e ? e : start;
  }
  const TransBox& B = a.box[b];
  uint32_t local = tile - start;
  // Consecutive tiles run at the same time.  Along A first, the tiles of a moment read whole
  // strips of source rows (every piece of a row is fetched while its neighbours are) and write
  // one column of the destination's tiles: a strip TB elements wide down every destination row.
  // When the destination's pitch is a multiple of a large power of two that strip lives in a
  // few DRAM channels; such boxes go along the diagonals instead -- B advances with every tile
  // and A with it --, which spreads both sides over rows and columns alike.
  uint32_t ta_i, tb_i;
  if (B.diagonal) {
    tb_i = local % B.tb;
    local /= B.tb;
    ta_i = (local % B.ta + tb_i) % B.ta;
    local /= B.ta;
  } else {
    ta_i = local % B.ta;
    local /= B.ta;
    tb_i = local % B.tb;
    local /= B.tb;
  }
  const uint32_t o0 = local % B.no[0], o1 = local / B.no[0];
  TransLoc t;
  t.box = b;
  t.ia = ta_i * a.tile_a;
  t.ib = tb_i * a.tile_b;
  t.src_off = (int64_t)o0 * B.src_o[0] + (int64_t)o1 * B.src_o[1] + (int64_t)t.ib * B.src_b + (int64_t)t.ia * (int64_t)elem;
  t.dst_off = (int64_t)o0 * B.dst_o[0] + (int64_t)o1 * B.dst_o[1] + (int64_t)t.ia * B.dst_a + (int64_t)t.ib * (int64_t)elem;
  return t;
}

template<int E>
struct ElemType;
template<>
struct ElemType<1> {
  using type = uint8_t;
};
template<>
struct ElemType<2> {
  using type = uint16_t;
};
template<>
struct ElemType<4> {
  using type = uint32_t;
};
template<>
struct ElemType<8> {
  using type = u32x2;
};
template<>
struct ElemType<16> {
  using type = u32x4;
};

// One tile of TA x TB elements per workgroup.  LDS holds the tile TRANSPOSED: TA rows along A, each
// row TB elements along B.
//
// WIDE: every row of the box starts on the 16-byte grid on both sides and holds a whole number
// of 16-byte vectors -- the host checks addresses, strides and extents: global memory moves as
// 16-byte vectors (V = 16 / E elements); going in, a vector's elements are scattered over V
// rows of LDS, going out, a row of LDS is read 16 bytes at a time.  The rows carry no padding;
// instead the 16-byte vectors of a row are permuted: vector j of row a sits at position
// j ^ (a / V mod vectors per row).  A wave's scatter -- one element each to V-th rows, a few
// neighbouring columns -- then lands in as many banks as it has lanes (with rows padded by 16
// bytes, whatever keeps them aligned, it took 4 to 8 turns per instruction), and the 16-byte
// reads of whole rows touch every bank once either way.
//
// Otherwise every access is one element: still consecutive lanes on consecutive addresses on
// both sides, E bytes each; rows are padded by one bank (4 bytes; 8 and 16 for elements of that
// size, which must stay aligned), so that a column of the tile walks through all banks.
template<int E, bool WIDE, int TA, int TB>
__global__ __launch_bounds__(kBlock) void transpose_kernel(TransArgs a) {
  using elem_t = typename ElemType<E>::type;
  constexpr uint32_t V = 16 / E;      // elements per 16-byte vector
  constexpr uint32_t kVecsA = TA / V; // vectors along A: a source row of the tile
  constexpr uint32_t kVecsB = TB / V; // vectors along B: a destination row of the tile
  constexpr uint32_t kPitch = WIDE ? TB * E : TB * E + (E <= 4 ? 4 : E);
  constexpr uint32_t kPerLane = WIDE ? TB * kVecsA / kBlock : TA * TB / kBlock;
  static_assert(!WIDE || (TB * kVecsA % kBlock == 0 && TA * kVecsB == TB * kVecsA), "whole vectors per lane");
  static_assert(WIDE || TA * TB % kBlock == 0, "whole elements per lane");
  using reg_t = typename std::conditional<WIDE, u32x4, elem_t>::type;
  __shared__ __attribute__((aligned(16))) char tile[TA * kPitch];

  struct Where {
    const char* src;
    char* dst;
    int64_t src_b, dst_a;
    uint32_t na, nb; // what of the tile lies inside the box
  };
  auto locate = [&](uint32_t index) {
    const TransLoc t = trans_locate(a, index, E);
    const TransBox& B = a.box[t.box];
    Where w;
    w.src = B.src + t.src_off;
    w.dst = B.dst + t.dst_off;
    w.src_b = B.src_b;
    w.dst_a = B.dst_a;
    w.na = B.na - t.ia < (uint32_t)TA ? B.na - t.ia : (uint32_t)TA;
    w.nb = B.nb - t.ib < (uint32_t)TB ? B.nb - t.ib : (uint32_t)TB;
    return w;
  };

  // A workgroup takes the tiles blockIdx.x, blockIdx.x + gridDim.x, ... -- as launched by the
  // library, exactly one.  When there are more, the loads of the next tile are issued as soon as
  // the registers are free (the current tile sits in LDS by then) and are under way while the
  // current tile is read out of LDS and stored.
  reg_t v[kPerLane];
  auto load = [&](const Where& w) {
#pragma unroll
    for (uint32_t i = 0; i < kPerLane; ++i) {
      const uint32_t idx = i * kBlock + threadIdx.x;
      v[i] = reg_t{};
      if constexpr (WIDE) {
        const uint32_t row_b = idx / kVecsA, col = idx % kVecsA;
        if (row_b < w.nb && col * V < w.na) {
          v[i] = stream_load((const reg_t*)(w.src + (int64_t)row_b * w.src_b + (int64_t)col * 16));
        }
      } else {
        const uint32_t row_b = idx / TA, col_a = idx % TA;
        if (row_b < w.nb && col_a < w.na) {
          v[i] = stream_load((const reg_t*)(w.src + (int64_t)row_b * w.src_b + (int64_t)col_a * E));
        }
      }
    }
  };
  auto scatter = [&]() {
#pragma unroll
    for (uint32_t i = 0; i < kPerLane; ++i) {
      const uint32_t idx = i * kBlock + threadIdx.x;
      if constexpr (WIDE) {
        const uint32_t row_b = idx / kVecsA, col = idx % kVecsA;
        elem_t e[V];
        __builtin_memcpy(e, &v[i], 16);
        // rows col * V ... + V - 1 share one permutation: a / V = col
        const uint32_t at = ((row_b / V) ^ (col % kVecsB)) * 16 + (row_b % V) * E;
#pragma unroll
        for (uint32_t k = 0; k < V; ++k) {
          *(elem_t*)(tile + (col * V + k) * kPitch + at) = e[k];
        }
      } else {
        const uint32_t row_b = idx / TA, col_a = idx % TA;
        elem_t e;
        __builtin_memcpy(&e, &v[i], E);
        *(elem_t*)(tile + col_a * kPitch + row_b * E) = e;
      }
    }
  };
  auto store = [&](const Where& w) {
#pragma unroll
    for (uint32_t i = 0; i < kPerLane; ++i) {
      const uint32_t idx = i * kBlock + threadIdx.x;
      if constexpr (WIDE) {
        const uint32_t row_a = idx / kVecsB, col = idx % kVecsB;
        if (row_a < w.na && col * V < w.nb) {
          const u32x4 out = *(const u32x4*)(tile + row_a * kPitch + (col ^ (row_a / V % kVecsB)) * 16);
          stream_store((u32x4*)(w.dst + (int64_t)row_a * w.dst_a + (int64_t)col * 16), out);
        }
      } else {
        const uint32_t row_a = idx / TB, col_b = idx % TB;
        if (row_a < w.na && col_b < w.nb) {
          const elem_t out = *(const elem_t*)(tile + row_a * kPitch + col_b * E);
          stream_store((elem_t*)(w.dst + (int64_t)row_a * w.dst_a + (int64_t)col_b * E), out);
        }
      }
    }
  };

  uint32_t index = blockIdx.x;
  Where cur = locate(index);
  load(cur);
  for (;;) {
    scatter();
    __syncthreads();
    const uint32_t next = index + gridDim.x;
    const bool more = next < a.total_tiles;
    Where nxt = cur;
    if (more) {
      nxt = locate(next);
      load(nxt);
    }
    store(cur);
    if (!more) {
      break;
    }
    __syncthreads(); // every wave has read the tile out of LDS before the next one goes in
    cur = nxt;
    index = next;
  }
}

} // namespace mdh
