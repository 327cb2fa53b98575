// Streaming copies for gfx950: all-gather chunk assembly and the N-d box
// copies of a shard redistribution, fused into one grid per launch.
//
// Where the reference runs P sequential copy_impl calls on at most 64 blocks
// (core/allgather.cc:381-390, core/kernels.cc:28-169) or hands 2-D shapes to
// the copy engine (core/processgroup.cc:806-820), this kernel takes a table of
// up to 32 boxes in its kernel arguments and spreads their tiles over the
// whole chip.  Every box is reduced on the host to
//     rows x cols vectors,  rows decomposed over <= 3 strided outer extents,
// and a tile is kBlock*U vector slots shaped 2^a rows x 2^b columns, so the
// lane -> (row, column) mapping is shifts and masks; an integer division is
// paid once per tile, never per vector.  Runs shorter than a wave's 1 KiB still
// coalesce: consecutive lanes walk a run, then step to the next row.
#include "device_common.h"
#include "transpose_kernels.h"

#include <algorithm>
#include <cstring>
#include <memory>
#include <utility>
#include <vector>

namespace mdh {
namespace {

constexpr int kMaxBoxes = 32;
constexpr int kMaxOuter = 3;

struct BoxDesc {
  const char* src;
  char* dst;
  int64_t src_stride[kMaxOuter]; // bytes; [0] is the fastest-varying outer extent
  int64_t dst_stride[kMaxOuter];
  uint32_t outer[kMaxOuter];
  uint32_t nouter;
  uint32_t rows; // product of outer[]
  uint32_t cols; // vectors per row
  uint32_t nct;  // column tiles per row of tiles
  uint32_t log2tc;
  uint32_t src_span; // bytes from src to the end of the box, when both spans fit 32 bits (else 0)
  uint32_t dst_span;
  // Byte offset of a row's LAST vector.  (cols - 1) * vector width when the row is a whole number
  // of vectors; a row of the 16-byte kernel that is not has one vector more, and that last one
  // ends where the row ends: it overlaps the one before it, and the bytes they share are
  // copied twice, to the same effect.
  uint32_t last_off;
};

struct CopyArgs {
  BoxDesc box[kMaxBoxes];
  uint32_t tile_end[kMaxBoxes]; // tiles of boxes 0..k, cumulative; unused entries are ~0
  uint32_t nboxes;
  uint32_t total_tiles;
  uint32_t tiles_per_box; // non-zero when every box has the same tile count
};
// with fourteen leading scalars in front (copy_rows16_kernel) and the compiler's 256 bytes of
// hidden arguments behind
static_assert(sizeof(CopyArgs) + 56 + 256 <= 4096, "kernel arguments are limited to 4 KiB");

template<int VEC>
struct VecType;
template<>
struct VecType<16> {
  using type = u32x4;
};
template<>
struct VecType<8> {
  using type = u32x2;
};
template<>
struct VecType<4> {
  using type = uint32_t;
};
template<>
struct VecType<2> {
  using type = uint16_t;
};
template<>
struct VecType<1> {
  using type = uint8_t;
};

constexpr uint32_t ilog2(uint32_t x) {
  return x <= 1 ? 0 : 1 + ilog2(x >> 1);
}

// ---- index arithmetic, shared by the kernels and by the host-side verifier of a plan ----

#define MDH_HD __host__ __device__ __forceinline__

struct TileLoc {
  uint32_t box; // which box of the table
  uint32_t rt;  // row of tiles inside the box
  uint32_t ct;  // column of tiles
};

// Which box a tile belongs to.  Equal boxes (the shards of a gather or of a redistribution): one
// division.  Otherwise the cumulative ends are scanned: they ascend, so the last one at or
// below the tile names the box; written as selects of scalars so that on the device the whole
// scan stays on the scalar unit (the table sits in the kernel arguments).
template<bool MAY_DIVIDE>
MDH_HD TileLoc locate_tile(const CopyArgs& a, uint32_t tile) {
  uint32_t b = 0, start = 0;
  if (MAY_DIVIDE && a.tiles_per_box) {
    b = tile / a.tiles_per_box;
    start = b * a.tiles_per_box;
  } else {
#pragma unroll
    for (int k = 0; k < kMaxBoxes - 1; ++k) {
      const uint32_t e = a.tile_end[k];
      b = tile >= e ? (uint32_t)(k + 1) : b;
      start = tile >= e ? e : start;
    }
  }
  const uint32_t local = tile - start;
  const uint32_t rt = local / a.box[b].nct;
  return TileLoc{b, rt, local - rt * a.box[b].nct};
}

// Slot `slot` of a tile (kBlock*U slots shaped 2^(log2slots-log2tc) rows x 2^log2tc columns):
// byte offsets of its vector from the box's src and dst.  Returns false for a slot outside the
// box (the ragged right and bottom edges).
template<typename Off>
MDH_HD bool slot_offsets(const BoxDesc& B, const TileLoc& t, uint32_t slot, uint32_t log2slots, uint32_t vec, Off* so,
    Off* dof) {
  const uint32_t log2tc = B.log2tc;
  const uint32_t log2tr = log2slots - log2tc;
  const uint32_t tcmask = (1u << log2tc) - 1u;
  const uint32_t col = (t.ct << log2tc) + (slot & tcmask);
  uint32_t row = (t.rt << log2tr) + (slot >> log2tc);
  const bool ok = col < B.cols && row < B.rows;
  Off s, d;
  if (B.nouter <= 1) {
    s = (Off)row * (Off)B.src_stride[0];
    d = (Off)row * (Off)B.dst_stride[0];
  } else {
    s = 0, d = 0;
    for (uint32_t k = 0; k + 1 < B.nouter; ++k) {
      const uint32_t q = row / B.outer[k];
      const uint32_t i = row - q * B.outer[k];
      s += (Off)i * (Off)B.src_stride[k];
      d += (Off)i * (Off)B.dst_stride[k];
      row = q;
    }
    s += (Off)row * (Off)B.src_stride[B.nouter - 1];
    d += (Off)row * (Off)B.dst_stride[B.nouter - 1];
  }
  const uint32_t in_row = col * vec < B.last_off ? col * vec : B.last_off;
  *so = s + (Off)in_row;
  *dof = d + (Off)in_row;
  return ok;
}

template<int VEC, int U>
__global__ __launch_bounds__(kBlock) void copy_boxes_kernel(CopyArgs a) {
  using V = typename VecType<VEC>::type;
  constexpr uint32_t log2slots = ilog2(kBlock * U);
  // The grid never exceeds the tile count, so the first tile needs no test: the scalar loads of
  // the whole table header are then issued together instead of behind a first load-and-branch.
  uint32_t tile = blockIdx.x;
  do {
    const TileLoc t = locate_tile<false>(a, tile);
    const BoxDesc& B = a.box[t.box];
    V v[U];
    bool ok[U];
    int64_t doff[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int64_t so;
      ok[u] = slot_offsets<int64_t>(B, t, (uint32_t)u * kBlock + threadIdx.x, log2slots, VEC, &so, &doff[u]);
      if (ok[u]) {
        v[u] = stream_load((const V*)(B.src + so));
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (ok[u]) {
        stream_store((V*)(B.dst + doff[u]), v[u]);
      }
    }
    tile += gridDim.x;
  } while (tile < a.total_tiles);
}

// The same tiling for boxes whose byte span fits 32 bits on both sides (all but
// multi-GiB boxes) and whose vectors are 16 bytes: each side is addressed through
// one buffer descriptor per box (wave-uniform base) and a 32-bit lane offset, so
// a slot costs two integer multiplies instead of 64-bit address arithmetic, and
// an out-of-range slot is given the offset just past the descriptor's end -- its
// load returns zero and its store is dropped -- instead of a predicate.
//
// EQUAL: every box of the table has the same number of tiles (the shards of a gather or of a
// redistribution).  The grid is then two-dimensional -- blockIdx.y is the box, blockIdx.x the
// tile inside it -- so the address of the box's descriptor is known when the wave starts and
// all of its scalar loads go out in one batch; nothing of the table header is read.  On the
// 16 MiB redistribution, whose whole launch lasts 5 us, that is 0.5 us.
//
// PLAIN selects the cache policy of the loads: nt (the default) or plain (the tuning knob
// box_policy = 1).  Stores are nt+sc1 either way.  Measured on MI355X, us per launch, loads
// plain / nt, with every operand coming from HBM (the launches rotate over 4 GiB of buffers):
//   [64,512,1024] bf16 dim0->dim2, 16 MiB moved    4.98 /  4.71      8192^2 bf16, 32 MiB    8.56 /  8.03
//   8192^2 fp32, 64 MiB                           13.90 / 12.87      gather 8 x [4096,4096] bf16 into pitch 4160   84.6 / 80.9
// When the sources are partly still in the 256 MB Infinity Cache (the same few hundred MiB
// copied again and again) the order turns round for the redistributions, which read one block
// of columns out of every row: 3.92 / 4.60, 6.92 / 7.79 and 10.91 / 12.85 -- plain loads may then
// hit in that cache, nt loads go past it.  A caller that knows its sources to be freshly
// written and small can ask for them with the knob.
// A box's descriptor, read from the argument table in ONE batch of scalar loads: every field the
// common case needs passes through an empty asm statement, which the compiler has to have all of
// them ready for at once.  Left to itself it reads each field where it is first used, behind the
// branches of the index arithmetic: four scalar round trips in a row before the first vector
// load, in launches that last 5 us.
__device__ __forceinline__ void read_at_once(const BoxDesc& B) {
  asm volatile("" ::"s"((uint64_t)(uintptr_t)B.src), "s"((uint64_t)(uintptr_t)B.dst), "s"((uint64_t)B.src_stride[0]),
               "s"((uint64_t)B.dst_stride[0]), "s"(B.nouter), "s"(B.rows), "s"(B.cols), "s"(B.nct), "s"(B.log2tc),
               "s"(B.src_span), "s"(B.dst_span), "s"(B.last_off));
}

template<int U, bool EQUAL, bool PLAIN>
__global__ __launch_bounds__(kBlock) void copy_boxes16_kernel(CopyArgs a) {
  constexpr int kLoad = PLAIN ? 0 : 2;
  constexpr int kStore = 18;
  constexpr uint32_t log2slots = ilog2(kBlock * U);
  uint32_t tile = blockIdx.x; // first tile untested, as above
  do {
    TileLoc t;
    if (EQUAL) {
      read_at_once(a.box[blockIdx.y]);
      const uint32_t nct = a.box[blockIdx.y].nct;
      const uint32_t rt = blockIdx.x / nct;
      t = TileLoc{blockIdx.y, rt, blockIdx.x - rt * nct};
    } else {
      t = locate_tile<true>(a, tile);
    }
    const BoxDesc& B = a.box[t.box];
    const __amdgpu_buffer_rsrc_t rs = tile_rsrc(B.src, B.src_span);
    const __amdgpu_buffer_rsrc_t rd = tile_rsrc(B.dst, B.dst_span);
    u32x4 v[U];
    uint32_t doff[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      uint32_t so, dof;
      const bool ok = slot_offsets<uint32_t>(B, t, (uint32_t)u * kBlock + threadIdx.x, log2slots, 16u, &so, &dof);
      // the span itself is the first offset past the descriptor's end
      doff[u] = ok ? dof : B.dst_span;
      v[u] = tile_load<kLoad>(rs, ok ? so : B.src_span);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      tile_store<kStore>(rd, doff[u], v[u]);
    }
    if (EQUAL) {
      break; // one tile per workgroup
    }
    tile += gridDim.x;
  } while (tile < a.total_tiles);
}

// ---- the same copy for equal boxes of full tiles, started from preloaded arguments ----
//
// In the form above a wave's first vector load waits for a scalar round trip to the argument
// table, which the host has just written (0.3-0.5 us of launches that last 4-13 us).  When the
// boxes of a launch are at most eight, have the same two-dimensional shape on the source side
// and consist of full tiles only -- the shards of a redistribution or of a padded gather --
// everything the loads need fits the fourteen dwords that the hardware hands a wave in registers
// when it starts (kernels compiled with -amdgpu-kernarg-preload-count): the source row pitch,
// the tile shape, and the eight source addresses as 48 bits each.  The destination side still
// comes from the table, read while the vector loads are in flight.
constexpr int kEarlyBoxes = 8;

struct PackedSources {
  uint32_t lo[kEarlyBoxes];     // source addresses, low halves
  uint32_t hi[kEarlyBoxes / 2]; // bits 32..47 of two addresses each: box 2k low, box 2k+1 high
};

struct RowsLead {
  uint32_t src_stride; // bytes between rows of the source
  uint32_t shape;      // log2tc | column tiles per row << 5
  PackedSources from;
};
static_assert(sizeof(RowsLead) == 14 * 4, "fourteen dwords are preloaded");

// The same for copy_flat_kernel's equal segments (below).
struct FlatLead {
  uint32_t bytes; // of every segment
  uint32_t reserved;
  PackedSources from;
};
static_assert(sizeof(FlatLead) == 14 * 4, "fourteen dwords are preloaded");

MDH_HD uint32_t pick8(uint32_t i, uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3, uint32_t a4, uint32_t a5, uint32_t a6,
    uint32_t a7) {
  uint32_t r = a0;
  r = i == 1 ? a1 : r;
  r = i == 2 ? a2 : r;
  r = i == 3 ? a3 : r;
  r = i == 4 ? a4 : r;
  r = i == 5 ? a5 : r;
  r = i == 6 ? a6 : r;
  r = i == 7 ? a7 : r;
  return r;
}

// Source address of box y out of the packed halves (selects of scalars: y is wave-uniform).
MDH_HD uint64_t packed_source_address(uint32_t y, uint32_t l0, uint32_t l1, uint32_t l2, uint32_t l3, uint32_t l4, uint32_t l5,
    uint32_t l6, uint32_t l7, uint32_t h0, uint32_t h1, uint32_t h2, uint32_t h3) {
  const uint32_t lo = pick8(y, l0, l1, l2, l3, l4, l5, l6, l7);
  const uint32_t pair = pick8(y >> 1, h0, h1, h2, h3, 0, 0, 0, 0);
  const uint32_t hi = (y & 1u) ? pair >> 16 : pair & 0xffffu;
  return (uint64_t)hi << 32 | lo;
}

// Offset of a slot of a full tile on one side of the box: what slot_offsets computes for a box
// of one strided extent whose rows are a whole number of vectors.
MDH_HD uint32_t rows_offset(uint32_t stride, uint32_t log2tc, uint32_t log2slots, uint32_t rt, uint32_t ct, uint32_t slot) {
  const uint32_t col = (ct << log2tc) + (slot & ((1u << log2tc) - 1u));
  const uint32_t row = (rt << (log2slots - log2tc)) + (slot >> log2tc);
  return row * stride + col * 16u;
}

template<int U, bool PLAIN>
__global__ __launch_bounds__(kBlock) void copy_rows16_kernel(uint32_t src_stride, uint32_t shape, uint32_t l0, uint32_t l1,
    uint32_t l2, uint32_t l3, uint32_t l4, uint32_t l5, uint32_t l6, uint32_t l7, uint32_t h0, uint32_t h1, uint32_t h2,
    uint32_t h3, CopyArgs a) {
  constexpr int kLoad = PLAIN ? 0 : 2;
  constexpr int kStore = 18;
  constexpr uint32_t log2slots = ilog2(kBlock * U);
  const uint32_t y = blockIdx.y;
  const uint32_t log2tc = shape & 31u, nct = shape >> 5;
  const uint32_t rt = blockIdx.x / nct;
  const TileLoc t{y, rt, blockIdx.x - rt * nct};
  // every slot of every tile lies inside the box (the host launches this form for nothing
  // else), so the descriptor needs no end
  const char* src = (const char*)(uintptr_t)packed_source_address(y, l0, l1, l2, l3, l4, l5, l6, l7, h0, h1, h2, h3);
  const __amdgpu_buffer_rsrc_t rs = tile_rsrc(src, 0xffffffffu);
  u32x4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    v[u] = tile_load<kLoad>(rs, rows_offset(src_stride, log2tc, log2slots, t.rt, t.ct, (uint32_t)u * kBlock + threadIdx.x));
  }
  // The loads are out before anything of the table is waited for.  (The destination side is
  // straight-line code on purpose: with branches between the loads and the stores the compiler
  // sinks the loads below them, behind the wait for the table.)
  __builtin_amdgcn_sched_barrier(0);
  const BoxDesc& B = a.box[y];
  const __amdgpu_buffer_rsrc_t rd = tile_rsrc(B.dst, B.dst_span);
  const uint32_t dst_stride = (uint32_t)B.dst_stride[0];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    tile_store<kStore>(rd, rows_offset(dst_stride, log2tc, log2slots, t.rt, t.ct, (uint32_t)u * kBlock + threadIdx.x), v[u]);
  }
}

// Contiguous segments (the shards of a dense all-gather, or any box that
// collapses to one run): no per-lane index arithmetic at all.  A tile is
// kBlock*U consecutive 16-byte vectors of one segment, addressed through a
// buffer descriptor based at the tile (wave-uniform), so a lane needs one
// 32-bit offset and the ragged last tile is clipped by the address unit.
constexpr int kMaxSegments = 64;

struct FlatArgs {
  const char* src[kMaxSegments]; // first byte of the segment's whole vectors (after its head)
  char* dst[kMaxSegments];
  uint32_t tile_end[kMaxSegments]; // cumulative tiles; unused entries are ~0
  uint64_t bytes[kMaxSegments];    // of whole vectors: multiples of 16
  // The segment's first bytes, up to its destination's next 64-byte boundary, and its last
  // bytes (fewer than 16, or fewer than 80 when equal segments were given one common length of
  // whole vectors): they sit before src/dst and after src/dst + bytes, and are copied byte by
  // byte by workgroups of their own, in front of the tile workgroups.
  uint8_t head[kMaxSegments]; // 0..63
  uint8_t tail[kMaxSegments]; // 0..79
  uint32_t nsegs;
  uint32_t total_tiles;
  uint32_t tiles_per_seg; // non-zero when every segment has the same tile count
  // 0: no segment has a head or a tail.  1: some have, and the first kEdgeWgs workgroups of the
  // one-dimensional grid copy them.  2: some have, and workgroup 0 of every row of the
  // two-dimensional grid copies its segment's (the tiles are then workgroups 1, 2, ...).
  uint32_t edge_wgs;
};
static_assert(sizeof(FlatArgs) + 56 + 256 <= 4096, "kernel arguments are limited to 4 KiB");

// Edge bytes are numbered per segment: slots 0..63 are the head's bytes, 64..143 the tail's.
constexpr uint32_t kMaxTail = 80;
constexpr uint32_t kEdgeSlots = 64 + kMaxTail;
static_assert(kEdgeSlots <= (uint32_t)kBlock, "one workgroup has a lane for every edge byte of a segment");
// Workgroups that copy them in the one-dimensional form of the grid: one lane per slot of a
// full table.
constexpr uint32_t kEdgeWgs = (kMaxSegments * kEdgeSlots + 255) / 256;

// The byte a slot stands for, as an offset from the segment's src/dst (negative in the head);
// false for a slot the segment does not use.
MDH_HD bool edge_offset(const FlatArgs& a, uint32_t seg, uint32_t slot, int64_t* off) {
  if (slot < 64) {
    const uint32_t head = a.head[seg];
    *off = (int64_t)slot - (int64_t)head;
    return slot < head;
  }
  *off = (int64_t)a.bytes[seg] + (int64_t)(slot - 64);
  return slot - 64 < a.tail[seg];
}

// Which segment a tile belongs to, and the tile's first byte inside it (same two ways as for boxes).
MDH_HD uint32_t locate_segment(const FlatArgs& a, uint32_t tile, uint32_t* local) {
  uint32_t seg;
  if (a.tiles_per_seg) {
    seg = tile / a.tiles_per_seg;
    *local = tile - seg * a.tiles_per_seg;
  } else {
    seg = 0;
    uint32_t start = 0;
#pragma unroll
    for (int k = 0; k < kMaxSegments - 1; ++k) {
      const uint32_t e = a.tile_end[k];
      seg = tile >= e ? (uint32_t)(k + 1) : seg;
      start = tile >= e ? e : start;
    }
    *local = tile - start;
  }
  return seg;
}

// Workgroup `wg` of `nwg` edge workgroups: one byte per lane and round.  Out of line, reading the
// arguments from the kernel's argument segment (FlatArgs is the kernel's only argument, so it
// sits at the segment's start): inlined, its loads were scheduled in front of the tile
// workgroups' own.
__device__ __attribute__((noinline)) void copy_edges(const FlatArgs* args, uint32_t wg, uint32_t nwg, uint32_t lane) {
  const FlatArgs& a = *args;
  if (a.edge_wgs == 0) {
    return;
  }
  const uint32_t all = a.nsegs * kEdgeSlots;
  for (uint32_t idx = wg * kBlock + lane; idx < all; idx += nwg * kBlock) {
    const uint32_t seg = idx / kEdgeSlots, slot = idx - seg * kEdgeSlots;
    int64_t off;
    if (edge_offset(a, seg, slot, &off)) {
      a.dst[seg][off] = a.src[seg][off];
    }
  }
}

// The two-dimensional form: the edge bytes of one segment, one per lane, by workgroup 0 of the
// segment's row.  Out of line for the same reason.
__device__ __attribute__((noinline)) void copy_segment_edges(const FlatArgs* args, uint32_t seg, uint32_t lane) {
  const FlatArgs& a = *args;
  int64_t off;
  if (lane < kEdgeSlots && edge_offset(a, seg, lane, &off)) {
    a.dst[seg][off] = a.src[seg][off];
  }
}

// EQUAL: as for the boxes -- segments of equal tile count, blockIdx.y the segment, blockIdx.x the
// tile; when they have heads or tails (edge_wgs == 2) workgroup 0 of every row copies those and
// the tiles are workgroups 1, 2, ...  Otherwise the first kEdgeWgs workgroups of the
// grid are the edge workgroups -- ALWAYS, finding nothing to do when no segment has a head or a
// tail: a tile workgroup then knows what it is from blockIdx alone, and its first loads do not
// wait for a kernel argument to decide it.
template<int U, bool EQUAL, bool EDGES = false>
__global__ __launch_bounds__(kBlock) void copy_flat_kernel(FlatArgs a) {
  static_assert(EQUAL || !EDGES, "the edge column belongs to the two-dimensional form");
  constexpr uint32_t tile_bytes = kBlock * U * 16;
  const uint32_t lane_byte = threadIdx.x * 16;
  uint32_t first_tile = blockIdx.x, tile_wgs = 0;
  const uint32_t row = blockIdx.y;
  if (!EQUAL) {
    if (blockIdx.x < kEdgeWgs) {
      // the segment's address has to be taken here, in the kernel
      copy_edges((const FlatArgs*)__builtin_amdgcn_kernarg_segment_ptr(), blockIdx.x, kEdgeWgs, threadIdx.x);
      return;
    }
    first_tile = blockIdx.x - kEdgeWgs, tile_wgs = gridDim.x - kEdgeWgs;
  }
  uint32_t tile = first_tile; // untested, as in the box kernels
  do {
    uint32_t local;
    if (EDGES) { // (a template argument: read from the table, it would cost the tiles a scalar round trip)
      if (blockIdx.x == 0) {
        copy_segment_edges((const FlatArgs*)__builtin_amdgcn_kernarg_segment_ptr(), row, threadIdx.x);
        return;
      }
      tile = blockIdx.x - 1;
    }
    const uint32_t seg = EQUAL ? (local = tile, row) : locate_segment(a, tile, &local);
    const uint64_t off = (uint64_t)local * tile_bytes;
    const uint64_t left = a.bytes[seg] - off;
    const uint32_t n = left < tile_bytes ? (uint32_t)left : tile_bytes;
    const __amdgpu_buffer_rsrc_t rs = tile_rsrc(a.src[seg] + off, n);
    const __amdgpu_buffer_rsrc_t rd = tile_rsrc(a.dst[seg] + off, n);
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      v[u] = tile_load(rs, lane_byte + (uint32_t)u * (kBlock * 16));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      tile_store(rd, lane_byte + (uint32_t)u * (kBlock * 16), v[u]);
    }
    if (EQUAL) {
      break;
    }
    tile += tile_wgs;
  } while (tile < a.total_tiles);
}

// Equal segments again -- at most eight, all of one length (the dense all-gather of up to eight
// shards) -- started from preloaded arguments like copy_rows16_kernel: the segments' length and
// their source addresses arrive in registers, the destination's address is read from the table
// while the vector loads are in flight.
//
// EDGES: the segments have heads or tails -- shards whose length is not a whole number of
// vectors, or whose destinations are off the 64-byte grid, cut to one common length of whole
// vectors.  Workgroup 0 of every row copies its segment's edge bytes and the tiles are
// workgroups 1, 2, ...: a workgroup knows which it is from blockIdx alone.
// VARIANT (measurement only; the tuning knobs copy_xcd_run, copy_grid_order, copy_tail_tiles and
// copy_lds select it, the library by itself never does): 0 is the kernel as described above.
//   1  the second leading argument carries a different dealing of the tiles: bits 0-4, n > 0:
//      every XCD (workgroups go to the eight XCDs round-robin) takes runs of 2^(n-1) consecutive
//      tiles instead of every eighth tile; bit 5: the grid is transposed, blockIdx.x the segment
//      and blockIdx.y the tile, so that the segments advance together (and with eight segments
//      every XCD copies one of them); bits 8-31: that many tiles at every segment's end are dealt
//      as two halves each, so that the launch ends on short workgroups;
//   2  the loads go straight to LDS (buffer_load ... lds) and the stores are fed from there by
//      ds_read_b128: no vector register holds a byte in flight.
constexpr uint32_t kVariantOrderMask = 31u, kVariantTransposed = 32u, kVariantTailShift = 8;

constexpr int waitcnt_vm(int n) { // s_waitcnt vmcnt(n), other counters left alone (gfx9 encoding)
  return (n & 0xf) | ((n >> 4) << 14) | (0x7 << 4) | (0xf << 8);
}

// Sub-tile I's load has landed when at most U-1-I loads are still out (they complete in order):
// its 16 bytes per lane go from LDS to the destination while the later ones are still in flight.
template<int U, int... I>
__device__ __forceinline__ void drain_staged(std::integer_sequence<int, I...>, const char* staged, __amdgpu_buffer_rsrc_t rd,
    uint32_t lane_byte) {
  ((__builtin_amdgcn_s_waitcnt(waitcnt_vm(U - 1 - I)),
       tile_store(rd, lane_byte + (uint32_t)I * (kBlock * 16), *(const u32x4*)(staged + I * (kBlock * 16) + lane_byte))),
      ...);
}

template<int U, bool EDGES, int VARIANT = 0>
__global__ __launch_bounds__(kBlock) void copy_flat8_kernel(uint32_t bytes, uint32_t opts, uint32_t l0, uint32_t l1, uint32_t l2,
    uint32_t l3, uint32_t l4, uint32_t l5, uint32_t l6, uint32_t l7, uint32_t h0, uint32_t h1, uint32_t h2, uint32_t h3,
    FlatArgs a) {
  static_assert(VARIANT == 0 || !EDGES, "the measurement variants are for segments without edge bytes");
  constexpr uint32_t tile_bytes = kBlock * U * 16;
  const uint32_t lane_byte = threadIdx.x * 16;
  uint32_t seg = blockIdx.y;
  if (EDGES && blockIdx.x == 0) {
    // FlatArgs follows the fourteen leading dwords in the argument segment
    const char* segment = (const char*)__builtin_amdgcn_kernarg_segment_ptr();
    copy_segment_edges((const FlatArgs*)(segment + sizeof(FlatLead)), seg, threadIdx.x);
    return;
  }
  uint32_t off = (blockIdx.x - (EDGES ? 1u : 0u)) * tile_bytes; // below the segment's length, which fits 32 bits
  uint32_t reach = tile_bytes;
  if (VARIANT == 1) {
    uint32_t b = blockIdx.x;
    if (opts & kVariantTransposed) {
      seg = blockIdx.x, b = blockIdx.y;
    }
    const uint32_t order = opts & kVariantOrderMask;
    if (order) {
      const uint32_t lr = order - 1, xcd = b & 7u, idx = b >> 3;
      b = ((((idx >> lr) << 3) | xcd) << lr) | (idx & ((1u << lr) - 1u));
    }
    const uint32_t tail = opts >> kVariantTailShift;
    const uint32_t whole = (bytes + tile_bytes - 1) / tile_bytes - tail; // tiles dealt whole
    off = b * tile_bytes;
    if (b >= whole) {
      off = whole * tile_bytes + (b - whole) * (tile_bytes / 2);
      reach = tile_bytes / 2;
    }
  }
  // (Wave-uniform, and it must stay in scalar registers: it is the size of the tile's buffer
  // descriptors.  Written as a saturating subtraction it is compiled to a vector instruction,
  // and every load and store then runs inside a loop that makes its descriptor uniform again --
  // 2 us of an 80 us launch.  Only a variant's half tiles can start past the segment's end.)
  const uint32_t left = VARIANT == 1 ? bytes - (uint32_t)__builtin_amdgcn_readfirstlane((int)(off < bytes ? off : bytes)) : bytes - off;
  const uint32_t n = left < reach ? left : reach;
  const char* src = (const char*)(uintptr_t)packed_source_address(seg, l0, l1, l2, l3, l4, l5, l6, l7, h0, h1, h2, h3);
  const __amdgpu_buffer_rsrc_t rs = tile_rsrc(src + off, n);
  if (VARIANT == 2) {
    extern __shared__ __attribute__((aligned(16))) char staged[];
    const uint32_t wave_base = (threadIdx.x >> 6) * 1024u;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // a wave's 64 lanes land in 1 KiB of LDS starting at the (wave-uniform) address given
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void*)(staged + u * (kBlock * 16) + wave_base),
          16, (int)(lane_byte + (uint32_t)u * (kBlock * 16)), 0, 0, MDH_LOAD_AUX);
    }
    const __amdgpu_buffer_rsrc_t rd = tile_rsrc(a.dst[seg] + off, n);
    drain_staged<U>(std::make_integer_sequence<int, U>{}, staged, rd, lane_byte);
    return;
  }
  u32x4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    v[u] = tile_load(rs, lane_byte + (uint32_t)u * (kBlock * 16));
  }
  __builtin_amdgcn_sched_barrier(0); // the loads are out before the table is waited for
  const __amdgpu_buffer_rsrc_t rd = tile_rsrc(a.dst[seg] + off, n);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    tile_store(rd, lane_byte + (uint32_t)u * (kBlock * 16), v[u]);
  }
}

// ---- host side: reduce a box to the kernel's form ----

struct HostBox {
  const char* src;
  char* dst;
  int nd; // strided extents, slowest first; the contiguous run is separate
  int64_t shape[MDH_MAX_DIMS + 1];
  int64_t sstride[MDH_MAX_DIMS + 1]; // bytes
  int64_t dstride[MDH_MAX_DIMS + 1];
  int64_t run; // contiguous bytes per row
};

int vec_width(const HostBox& h) {
  uint64_t bits = (uint64_t)(uintptr_t)h.src | (uint64_t)(uintptr_t)h.dst | (uint64_t)h.run | 16u;
  for (int d = 0; d < h.nd; ++d) {
    bits |= (uint64_t)h.sstride[d] | (uint64_t)h.dstride[d];
  }
  return (int)(bits & (~bits + 1)); // lowest set bit: 1, 2, 4, 8 or 16
}

// One kernel launch of a copy, with everything but the base addresses decided: what a
// prepared plan replays.
struct Step {
  enum Kind { kFlat, kBoxes16, kBoxes, kTrans } kind;
  int vec;    // kBoxes: bytes per vector
  int unroll; // sub-tiles
  uint32_t grid;
  uint32_t grid_y; // > 0: the two-dimensional form for equal boxes / segments (grid x grid_y workgroups)
  bool plain_loads; // kBoxes16: plain instead of nt loads (tuning knob)
  bool preloaded = false; // equal boxes of full tiles / equal segments of one length: started from preloaded arguments
  bool edge_column = false; // kFlat, two-dimensional form: workgroup 0 of every row copies its segment's edge bytes
  int variant = 0;          // copy_flat8_kernel's measurement variants (tuning knobs only)
  uint32_t variant_opts = 0;
  uint32_t variant_grid_x = 0, variant_grid_y = 0;
  size_t lds;
  FlatArgs flat;   // kFlat
  CopyArgs boxes;  // kBoxes16, kBoxes
  TransArgs trans; // kTrans: vec is the element size, plain_loads unused
  bool wide = false; // kTrans: 16-byte global accesses
};

int launch_step(const Step& st, const FlatArgs* flat, const CopyArgs* boxes, hipStream_t stream,
    const TransArgs* trans = nullptr);

// Whether a launch of equal boxes qualifies for copy_rows16_kernel: at most eight boxes, one
// strided extent, the same shape on the source side, rows a whole number of vectors, and no
// tile with a slot outside its box.
inline bool uniform_full_rows(const CopyArgs& a, int unroll) {
  if (a.nboxes == 0 || a.nboxes > (uint32_t)kEarlyBoxes || a.tiles_per_box == 0) {
    return false;
  }
  const BoxDesc& f = a.box[0];
  const uint32_t slots = (uint32_t)kBlock * (uint32_t)unroll;
  if (f.nouter > 1 || (slots >> f.log2tc) == 0 || f.cols == 0 || f.rows == 0) {
    return false;
  }
  const uint32_t tr = slots >> f.log2tc;
  if ((uint64_t)f.nct << f.log2tc != f.cols || f.rows % tr != 0 || f.nct >= (1u << 27) ||
      (uint64_t)f.last_off != ((uint64_t)f.cols - 1) * 16) {
    return false;
  }
  if (f.src_stride[0] < 0 || f.src_stride[0] > 0xffffffffll) {
    return false;
  }
  // the end of the last vector of the last row: the largest offset the kernel forms, plus 16
  const uint64_t reach = (uint64_t)(f.rows - 1) * (uint64_t)f.src_stride[0] + (uint64_t)f.cols * 16;
  if (f.src_span == 0 || reach > f.src_span) {
    return false;
  }
  for (uint32_t k = 0; k < a.nboxes; ++k) {
    // the destination side may differ from box to box, but is addressed the same way
    const BoxDesc& b = a.box[k];
    if (b.dst_stride[0] < 0 || b.dst_stride[0] > 0xffffffffll || b.dst_span == 0 ||
        (uint64_t)(f.rows - 1) * (uint64_t)b.dst_stride[0] + (uint64_t)f.cols * 16 > b.dst_span) {
      return false;
    }
  }
  for (uint32_t k = 1; k < a.nboxes; ++k) {
    const BoxDesc& b = a.box[k];
    if (b.nouter > 1 || b.rows != f.rows || b.cols != f.cols || b.nct != f.nct || b.log2tc != f.log2tc ||
        b.last_off != f.last_off || b.src_stride[0] != f.src_stride[0] || b.src_span != f.src_span) {
      return false;
    }
  }
  return true;
}

// Packs up to eight source addresses as 48 bits each; false when one does not fit, and the
// launch then takes the table form.
inline bool pack_sources(const char* const* src, uint32_t n, PackedSources* out) {
  PackedSources P{};
  for (uint32_t k = 0; k < n; ++k) {
    const uint64_t addr = (uint64_t)(uintptr_t)src[k];
    if (addr >> 48) {
      return false;
    }
    P.lo[k] = (uint32_t)addr;
    P.hi[k / 2] |= (uint32_t)(addr >> 32) << (16 * (k & 1));
  }
  for (uint32_t k = 0; k < n; ++k) {
    // through the function the kernels unpack them with
    if (packed_source_address(k, P.lo[0], P.lo[1], P.lo[2], P.lo[3], P.lo[4], P.lo[5], P.lo[6], P.lo[7], P.hi[0], P.hi[1],
            P.hi[2], P.hi[3]) != (uint64_t)(uintptr_t)src[k]) {
      return false;
    }
  }
  *out = P;
  return true;
}

// The leading arguments of copy_rows16_kernel for these (patched) boxes.
inline bool make_rows_lead(const CopyArgs& a, RowsLead* lead) {
  const char* src[kEarlyBoxes];
  for (uint32_t k = 0; k < a.nboxes; ++k) {
    src[k] = a.box[k].src;
  }
  lead->src_stride = (uint32_t)a.box[0].src_stride[0];
  lead->shape = a.box[0].log2tc | a.box[0].nct << 5;
  return pack_sources(src, a.nboxes, &lead->from);
}

// Whether a two-dimensional launch of flat segments qualifies for copy_flat8_kernel: at most
// eight segments, all of the same length.
inline bool uniform_segments(const FlatArgs& a) {
  if (a.nsegs == 0 || a.nsegs > (uint32_t)kEarlyBoxes || a.tiles_per_seg == 0 || a.edge_wgs == 1) {
    return false;
  }
  for (uint32_t k = 0; k < a.nsegs; ++k) {
    if (a.bytes[k] != a.bytes[0] || a.bytes[k] > 0xffffffffull) {
      return false;
    }
  }
  return true;
}

inline bool make_flat_lead(const FlatArgs& a, FlatLead* lead, uint32_t opts = 0) {
  lead->bytes = (uint32_t)a.bytes[0];
  lead->reserved = opts;
  return pack_sources(a.src, a.nsegs, &lead->from);
}

// The grid a step is launched with: st.grid (x st.grid_y) tile workgroups, and in the
// one-dimensional form of a flat step the edge workgroups in front of them.
inline void launch_dims(const Step& st, uint32_t* x, uint32_t* y) {
  if (st.kind == Step::kTrans) {
    *x = st.grid, *y = 1;
  } else if (st.variant != 0) {
    *x = st.variant_grid_x, *y = st.variant_grid_y;
  } else if (st.grid_y > 0) {
    *x = st.grid + (st.edge_column ? 1u : 0u);
    *y = st.grid_y;
  } else {
    *x = st.grid + (st.kind == Step::kFlat ? kEdgeWgs : 0u);
    *y = 1;
  }
}

struct Launcher {
  hipStream_t stream;
  std::vector<Step>* record = nullptr; // when set, launches are recorded here instead of enqueued
  std::vector<BoxDesc> pending[5]; // by log2(VEC)
  std::vector<BoxDesc> pending16;  // 16-byte vectors, spans inside 32 bits: copy_boxes16_kernel
  struct Segment {
    const char* src; // of the whole vectors
    char* dst;
    uint64_t bytes; // of whole vectors
    uint8_t head, tail;
  };
  std::vector<Segment> flat; // contiguous runs: whole vectors plus head and tail bytes
  std::vector<TransBox> transposing[5][2]; // by log2(element size) and whether global accesses are 16 bytes wide
  int rc = MDH_OK;
  int unroll = 2; // sub-tiles of the box launch being assembled

  // Launch shapes, measured with every operand coming from HBM (the launches rotate over 4 GiB):
  // sub-tiles per lane x workgroups resident per CU (an unused LDS allocation holds the others
  // back; "-" = no cap), us per launch.  (Zero-filled buffers, which copy 2-3 % faster than any
  // other data; the order of the shapes is the same with random data.)
  //   dense, 8 shards of    1 MiB   4 MiB   8 MiB  16 MiB  32 MiB  64 MiB
  //     1 x -                4.06   11.72   21.61   41.70   81.87
  //     2 x -                4.18   12.30   22.35   43.02   85.67
  //     4 x -                4.20   12.12   22.53   43.40   86.46
  //     2 x 4                4.03   11.82   21.48   40.72   80.62  162.33
  //     2 x 3                4.29   11.43   20.97   40.10   78.74  154.97
  //     4 x 2                4.09   11.90   21.64   41.34   81.18  165.87
  //   strided, 8 boxes     256 B x 4096   2 KiB x 1024   4 KiB x 1024   4 KiB x 4096   8 KiB x 4096 (padded pitch)
  //     1 x -                  4.41           7.40          11.57          40.83          79.14
  //     2 x -                  4.37           7.55          12.23          42.77          84.43
  //     2 x 4                  4.34           7.64          11.76          41.06          80.24
  //     2 x 3                  4.81           7.56          11.68          40.48          79.60
  // Dense copies of equal segments (the two-dimensional form of the grid), 32 MiB and more: two
  // sub-tiles, three workgroups per CU (24 KiB in flight per CU; the same bytes as six workgroups
  // of one sub-tile, which take 41.5 us where these take 40.1); shorter ones: one sub-tile, every
  // workgroup resident.  Unequal segments (the one-dimensional form, whose workgroups scan the
  // segment table for every tile they take and do better with longer tiles): four sub-tiles,
  // from 128 MiB on two with four workgroups per CU.
  // Strided boxes: one sub-tile and no cap throughout, except launches of 8 MiB and less, which
  // are over in 4 us and do better with half as many workgroups to dispatch.
  static constexpr uint64_t kCappedCopyBytes = (uint64_t)32 << 20;
  static constexpr uint64_t kLongRaggedBytes = (uint64_t)128 << 20;
  static constexpr uint64_t kShortBoxBytes = (uint64_t)8 << 20;
  size_t lds = 0; // of the launch being assembled
  bool plain_loads = false;

  // `cap` is the library's own choice (0 = none), which the knob overrides
  void choose_cap(int cap) {
    if (tuning().copy_wg_per_cu) {
      cap = tuning().copy_wg_per_cu;
    }
    lds = cap >= 2 && cap <= 8 ? kLdsForCap[cap] : 0; // one per CU would need the LDS limit raised
  }

  // The measurement variants of copy_flat8_kernel, for launches that qualify (preloaded form, no
  // edge bytes); a knob that does not fit the launch is ignored.
  void choose_variant(Step& st, const FlatArgs& a) {
    const Tuning& t = tuning();
    if (!st.preloaded || st.edge_column || !(t.copy_xcd_run || t.copy_grid_order || t.copy_tail_tiles || t.copy_lds)) {
      return;
    }
    const uint32_t tiles = a.tiles_per_seg;
    if (t.copy_lds) {
      st.variant = 2, st.variant_opts = 0;
      st.variant_grid_x = st.grid, st.variant_grid_y = st.grid_y;
      const size_t need = (size_t)kBlock * 16 * (size_t)st.unroll;
      st.lds = st.lds > need ? st.lds : need;
      return;
    }
    uint32_t opts = 0, gx = tiles;
    const uint32_t tail = (uint32_t)t.copy_tail_tiles;
    if (tail > 0 && tail < tiles && a.bytes[0] % ((uint64_t)kBlock * 16 * (uint64_t)st.unroll) == 0) {
      opts |= tail << kVariantTailShift;
      gx = tiles + tail;
    }
    const uint32_t run = (uint32_t)t.copy_xcd_run;
    if (run >= 2 && (run & (run - 1)) == 0 && gx == tiles && tiles % (8 * run) == 0 && !t.copy_grid_order) {
      uint32_t lr = 0;
      while ((1u << lr) < run) {
        ++lr;
      }
      opts |= lr + 1;
    }
    if (t.copy_grid_order) {
      opts |= kVariantTransposed;
      st.variant_grid_x = st.grid_y, st.variant_grid_y = gx;
    } else {
      st.variant_grid_x = gx, st.variant_grid_y = st.grid_y;
    }
    st.variant = 1, st.variant_opts = opts;
  }

  void flush_flat() {
    const Tuning& t = tuning();
    uint64_t all_vectors = 0;
    for (const Segment& g : flat) {
      all_vectors += g.bytes / 16;
    }
    bool even = flat.size() > 1, same_total = flat.size() > 1;
    uint64_t shortest = flat.empty() ? 0 : flat[0].bytes;
    for (const Segment& g : flat) {
      even = even && g.bytes == flat[0].bytes && !g.head && !g.tail;
      same_total = same_total && g.head + g.bytes + g.tail == flat[0].head + flat[0].bytes + flat[0].tail;
      shortest = g.bytes < shortest ? g.bytes : shortest;
    }
    // Segments of one total length whose heads differ (shards that are not a whole number of
    // vectors, or land off the 64-byte grid): all get the shortest one's whole vectors, and the
    // longer tails (fewer than 80 bytes) go with the edge bytes.  They are then equal segments
    // and take the two-dimensional form.
    bool cut = false;
    if (!even && same_total && shortest > 0) {
      for (Segment& g : flat) {
        const uint64_t tail = g.bytes - shortest + g.tail;
        if (tail >= kMaxTail) {
          same_total = false;
        }
      }
      if (same_total) {
        for (Segment& g : flat) {
          g.tail = (uint8_t)(g.bytes - shortest + g.tail);
          g.bytes = shortest;
        }
        even = cut = true;
      }
    }
    const uint64_t all_bytes = all_vectors * 16;
    int U, cap;
    if (cut) {
      // sources off the 16-byte grid: one sub-tile and no cap at every size (8 x (32 MiB + 2)
      // 83.7 us, against 87.5 with the shape of aligned segments and 84.9 with 2 x 4)
      U = 1, cap = 0;
    } else if (even) {
      U = all_bytes >= kCappedCopyBytes ? 2 : 1;
      cap = all_bytes >= kCappedCopyBytes ? 3 : 0;
    } else {
      U = all_bytes >= kLongRaggedBytes ? 2 : auto_unroll(all_vectors, 4);
      cap = all_bytes >= kLongRaggedBytes ? 4 : 0;
    }
    if (t.copy_unroll) {
      U = t.copy_unroll;
    }
    choose_cap(cap);
    const uint64_t tile_bytes = (uint64_t)kBlock * U * 16;
    size_t i = 0;
    while (i < flat.size()) {
      FlatArgs a;
      a.nsegs = 0;
      uint64_t tiles = 0;
      uint64_t first_tiles = 0;
      bool equal = true, edges = false;
      while (i < flat.size() && a.nsegs < (uint32_t)kMaxSegments) {
        const Segment& g = flat[i];
        const uint64_t n = (g.bytes + tile_bytes - 1) / tile_bytes;
        if (tiles + n > 0x7fffffffull) {
          break; // a segment is at most 2^30 bytes, so the next launch always makes progress
        }
        if (a.nsegs == 0) {
          first_tiles = n;
        }
        equal = equal && n == first_tiles;
        tiles += n;
        a.src[a.nsegs] = g.src;
        a.dst[a.nsegs] = g.dst;
        a.bytes[a.nsegs] = g.bytes;
        a.head[a.nsegs] = g.head;
        a.tail[a.nsegs] = g.tail;
        edges = edges || g.head || g.tail;
        a.tile_end[a.nsegs] = (uint32_t)tiles;
        ++a.nsegs;
        ++i;
      }
      for (uint32_t k = a.nsegs; k < (uint32_t)kMaxSegments; ++k) {
        a.src[k] = nullptr, a.dst[k] = nullptr, a.bytes[k] = 0;
        a.head[k] = a.tail[k] = 0;
        a.tile_end[k] = 0xffffffffu;
      }
      a.total_tiles = (uint32_t)tiles;
      a.tiles_per_seg = equal ? (uint32_t)first_tiles : 0;
      a.edge_wgs = edges ? 1 : 0;
      if (tiles == 0) {
        continue;
      }
      uint32_t grid = a.total_tiles;
      if (t.copy_max_blocks > 0 && grid > (uint32_t)t.copy_max_blocks) {
        grid = (uint32_t)t.copy_max_blocks;
      }
      Step st;
      st.kind = Step::kFlat, st.vec = 16, st.unroll = U, st.grid = grid, st.grid_y = 0, st.lds = lds;
      st.plain_loads = false;
      if (a.tiles_per_seg && grid == a.total_tiles && a.nsegs > 1) {
        st.grid = a.tiles_per_seg, st.grid_y = a.nsegs;
        st.edge_column = edges;
        a.edge_wgs = edges ? 2 : 0;
        st.preloaded = t.box_preload != 1 && uniform_segments(a);
        choose_variant(st, a);
      }
      submit(st, &a, nullptr);
    }
    flat.clear();
  }

  // Enqueues the step now, or files it for a plan.
  void submit(Step& st, const FlatArgs* f, const CopyArgs* c, const TransArgs* x = nullptr) {
    if (record) {
      if (f) {
        st.flat = *f;
      } else if (c) {
        st.boxes = *c;
      } else {
        st.trans = *x;
      }
      record->push_back(st);
      return;
    }
    const int r = launch_step(st, f, c, stream, x);
    if (r != MDH_OK) {
      rc = r;
    }
  }

  void launch_boxes(CopyArgs& a, int vec, bool buffer16) {
    const Tuning& t = tuning();
    uint32_t grid = a.total_tiles;
    if (t.copy_max_blocks > 0 && grid > (uint32_t)t.copy_max_blocks) {
      grid = (uint32_t)t.copy_max_blocks;
    }
    if (grid > 0x7fffffffu) {
      grid = 0x7fffffffu;
    }
    Step st;
    st.kind = buffer16 ? Step::kBoxes16 : Step::kBoxes;
    st.vec = vec, st.unroll = unroll, st.grid = grid, st.grid_y = 0, st.lds = buffer16 ? lds : 0;
    st.plain_loads = plain_loads;
    if (buffer16 && a.tiles_per_box && grid == a.total_tiles) {
      st.grid = a.tiles_per_box, st.grid_y = a.nboxes;
      st.preloaded = t.box_preload != 1 && uniform_full_rows(a, unroll);
    }
    submit(st, nullptr, &a);
  }

  void flush_class(int lg) {
    auto& list = lg == 5 ? pending16 : pending[lg];
    uint64_t all_vectors = 0;
    for (const BoxDesc& d : list) {
      all_vectors += (uint64_t)d.rows * d.cols;
    }
    const uint64_t all_bytes = all_vectors * (lg == 5 ? 16u : 1u << lg);
    choose_cap(0); // (a cap exists for the 16-byte buffer kernel only, and only by the knob)
    plain_loads = tuning().box_policy == 1;
    const int U = tuning().box_unroll ? tuning().box_unroll : all_bytes <= kShortBoxBytes ? auto_unroll(all_vectors, 2) : 1;
    unroll = U;
    const uint32_t slots = (uint32_t)kBlock * (uint32_t)U;
    size_t i = 0;
    while (i < list.size()) {
      CopyArgs a{};
      a.nboxes = 0;
      uint64_t tiles = 0;
      uint64_t first_n = 0;
      bool equal = true;
      while (i < list.size() && a.nboxes < (uint32_t)kMaxBoxes) {
        BoxDesc d = list[i];
        // Tile width: the power of two that covers the row, up to 64 columns -- 1 KiB, what one
        // wave moves with one instruction, so that the four waves of a workgroup work on four rows
        // rather than on 4 KiB of one: rows of 2 KiB at a pitch of 16 KiB (bf16 8192^2 over 8
        // ranks) 7.45 -> 7.14 us, rows of 4 KiB at 32 KiB 11.77 -> 11.55 us, rows of 8 KiB into a
        // padded pitch level (80.7 / 81.0 us); rows of a power-of-two pitch map to few DRAM
        // channels at a time (the same rows at a pitch 256 bytes longer: 12.96 -> 12.18 us), and a
        // workgroup spread over more rows evens that out.  Unless the column tiles of that width
        // would be more than a sixteenth empty (a row of 513 vectors in tiles of 512 columns is
        // two tiles, the second with one column in use: a gather of rows of 8200 bytes took
        // 114 us, against 80 us for rows of 8192); then the widest that is not, down to 16
        // columns (256 bytes of a row per wave instruction) if the rows are many.
        constexpr uint32_t kWidestTile = 64;
        uint32_t tc = 1, log2tc = 0;
        while (tc < d.cols && tc < slots && tc < kWidestTile) {
          tc <<= 1, ++log2tc;
        }
        while (tc > 16 && (slots >> (log2tc - 1)) <= d.rows &&
               (uint64_t)((d.cols + tc - 1) / tc) * tc * 16 > (uint64_t)d.cols * 17) {
          tc >>= 1, --log2tc;
        }
        if (const uint32_t forced = (uint32_t)tuning().box_tile_cols; forced != 0 && forced <= slots) {
          tc = 1, log2tc = 0; // (measurement knob, a power of two: checked when it is set)
          while (tc < forced) {
            tc <<= 1, ++log2tc;
          }
        }
        const uint32_t tr = slots >> log2tc;
        d.log2tc = log2tc;
        d.nct = (d.cols + tc - 1) / tc;
        const uint64_t n = (uint64_t)d.nct * ((d.rows + tr - 1) / tr);
        if (tiles + n > 0x7fffffffull) {
          if (a.nboxes == 0) {
            set_error("copy: one box needs %llu tiles, more than a grid can index", (unsigned long long)n);
            rc = MDH_EINVAL;
            return;
          }
          break;
        }
        if (a.nboxes == 0) {
          first_n = n;
        }
        equal = equal && n == first_n;
        tiles += n;
        a.tile_end[a.nboxes] = (uint32_t)tiles;
        a.box[a.nboxes++] = d;
        ++i;
      }
      a.tiles_per_box = equal ? (uint32_t)first_n : 0;
      for (uint32_t k = a.nboxes; k < (uint32_t)kMaxBoxes; ++k) {
        a.tile_end[k] = 0xffffffffu;
      }
      a.total_tiles = (uint32_t)tiles;
      if (tiles == 0) {
        continue;
      }
      launch_boxes(a, lg == 5 ? 16 : 1 << lg, lg == 5);
    }
    list.clear();
  }

  void flush_transposing() {
    for (int lg = 0; lg < 5; ++lg) {
      for (int wide = 0; wide < 2; ++wide) {
        std::vector<TransBox>& list = transposing[lg][wide];
        size_t i = 0;
        while (i < list.size()) {
          TransArgs a{};
          uint64_t tiles = 0;
          for (int k = 0; k < kMaxTransBoxes; ++k) {
            a.tile_end[k] = 0xffffffffu;
          }
          while (i < list.size() && a.nboxes < (uint32_t)kMaxTransBoxes) {
            const TransBox& b = list[i];
            const uint64_t n = (uint64_t)b.ta * b.tb * b.no[0] * b.no[1];
            if (tiles + n > 0x7fffffffull) {
              if (a.nboxes == 0) {
                set_error("copy: one transposing box needs %llu tiles, more than a grid can index", (unsigned long long)n);
                rc = MDH_EINVAL;
                return;
              }
              break;
            }
            tiles += n;
            a.tile_end[a.nboxes] = (uint32_t)tiles;
            a.box[a.nboxes++] = b;
            ++i;
          }
          a.total_tiles = (uint32_t)tiles;
          const TransShape shape = trans_shape(1u << lg, wide ? tuning().box_transpose_tile : 0);
          a.tile_a = shape.a, a.tile_b = shape.b;
          Step st;
          st.kind = Step::kTrans, st.vec = 1 << lg, st.unroll = 1, st.grid_y = 0, st.lds = 0;
          // One workgroup per tile.  (The kernel can walk: with fewer workgroups each takes every
          // grid-th tile and has the next one's loads under way while it stores the current one.
          // Measured, eight resident workgroups per CU walking lose 3-14 % against a fresh
          // workgroup per tile; the knob remains for measurement.)
          const uint32_t walkers = tuning().box_transpose_wgs > 0 ? (uint32_t)tuning().box_transpose_wgs : a.total_tiles;
          st.grid = a.total_tiles < walkers ? a.total_tiles : walkers;
          st.plain_loads = false, st.wide = wide != 0;
          submit(st, nullptr, nullptr, &a);
        }
        list.clear();
      }
    }
  }

  void flush() {
    flush_flat();
    flush_transposing();
    for (int lg = 5; lg >= 0; --lg) {
      flush_class(lg);
    }
  }

  // A box whose contiguous run is one element and whose source is contiguous along one extent
  // (A), its destination along another (B): copied tile by tile through LDS (transpose_kernel),
  // so that both sides move consecutive bytes.  Both extents must be at least kMinTransExtent
  // long (below that a tile would be mostly empty, and the plain kernel, which then still
  // coalesces on one side, is no worse), and at most two other extents may remain.
  static constexpr int64_t kMinTransExtent = 16;
  // a destination pitch that is a multiple of this puts a column of tiles into few DRAM channels
  static constexpr int64_t kCrowdingPitch = 4096;

  bool try_transposing(const HostBox& h) {
    if (tuning().box_transpose == 1 || h.nd < 2 || h.nd > 2 + kTransBatchDims || h.run > 16 || (h.run & (h.run - 1)) != 0) {
      return false;
    }
    int A = -1, B = -1;
    for (int d = 0; d < h.nd; ++d) {
      if (A < 0 && h.sstride[d] == h.run && h.dstride[d] != h.run) {
        A = d;
      } else if (B < 0 && h.dstride[d] == h.run && h.sstride[d] != h.run) {
        B = d;
      }
    }
    if (A < 0 || B < 0 || h.shape[A] < kMinTransExtent || h.shape[B] < kMinTransExtent) {
      return false;
    }
    const uint32_t E = (uint32_t)h.run;
    TransBox b{};
    b.src = h.src, b.dst = h.dst;
    b.src_b = h.sstride[B], b.dst_a = h.dstride[A];
    b.na = (uint32_t)h.shape[A], b.nb = (uint32_t)h.shape[B];
    if ((int64_t)b.na != h.shape[A] || (int64_t)b.nb != h.shape[B]) {
      return false;
    }
    b.no[0] = b.no[1] = 1;
    int k = 0;
    for (int d = h.nd - 1; d >= 0; --d) { // fastest first
      if (d == A || d == B) {
        continue;
      }
      if (h.shape[d] > 0x7fffffff) {
        return false;
      }
      b.no[k] = (uint32_t)h.shape[d];
      b.src_o[k] = h.sstride[d];
      b.dst_o[k] = h.dstride[d];
      ++k;
    }
    const uint64_t align = (uint64_t)(uintptr_t)b.src | (uint64_t)(uintptr_t)b.dst | (uint64_t)b.src_b | (uint64_t)b.dst_a |
                           (uint64_t)b.src_o[0] | (uint64_t)b.src_o[1] | (uint64_t)b.dst_o[0] | (uint64_t)b.dst_o[1] |
                           (uint64_t)b.na * E | (uint64_t)b.nb * E;
    const bool wide = (align & 15) == 0 && E < 16;
    const TransShape shape = trans_shape(E, wide ? tuning().box_transpose_tile : 0);
    b.ta = (b.na + shape.a - 1) / shape.a, b.tb = (b.nb + shape.b - 1) / shape.b;
    // the order of the tiles: see trans_locate
    b.diagonal = tuning().box_transpose == 2 ? 0u : tuning().box_transpose == 3 ? 1u : b.dst_a % kCrowdingPitch == 0 ? 1u : 0u;
    if (!count_piece()) {
      return true;
    }
    int lg = 0;
    while ((1u << lg) < E) {
      ++lg;
    }
    // (an element of 16 bytes is a vector already: the element-wise form moves 16 bytes per lane)
    transposing[lg][wide ? 1 : 0].push_back(b);
    return true;
  }

  // A box the kernels cannot index (more than kMaxOuter strided extents, or more than 2^31
  // rows) is cut into pieces on the host.  The number of pieces of one call is bounded, so that
  // an absurd box is refused instead of occupying the host for hours.
  static constexpr size_t kMaxPieces = (size_t)1 << 20;
  size_t pieces = 0;

  bool count_piece() {
    if (++pieces > kMaxPieces) {
      set_error("copy: the boxes of this call break into more than %zu pieces; split the call", kMaxPieces);
      rc = MDH_EINVAL;
      return false;
    }
    return true;
  }

  // rows x run with <= kMaxOuter strided extents
  void emit(const HostBox& h) {
    if (!count_piece()) {
      return;
    }
    const int vec = vec_width(h);
    int lg = 0;
    while ((1 << lg) < vec) {
      ++lg;
    }
    BoxDesc d;
    d.src = h.src;
    d.dst = h.dst;
    d.nouter = h.nd > 0 ? (uint32_t)h.nd : 1u;
    uint64_t rows = 1;
    for (int k = 0; k < kMaxOuter; ++k) {
      d.outer[k] = 1;
      d.src_stride[k] = 0;
      d.dst_stride[k] = 0;
    }
    for (int k = 0; k < h.nd; ++k) {
      const int dim = h.nd - 1 - k; // fastest first
      d.outer[k] = (uint32_t)h.shape[dim];
      d.src_stride[k] = h.sstride[dim];
      d.dst_stride[k] = h.dstride[dim];
      rows *= (uint64_t)h.shape[dim];
    }
    d.rows = (uint32_t)rows;
    d.cols = (uint32_t)(h.run / vec);
    d.last_off = (d.cols - 1) * (uint32_t)vec;
    d.nct = d.log2tc = 0;
    d.src_span = d.dst_span = 0;
    uint64_t sspan = (uint64_t)h.run, dspan = (uint64_t)h.run;
    for (int k = 0; k < h.nd; ++k) {
      sspan += (uint64_t)(h.shape[k] - 1) * (uint64_t)h.sstride[k];
      dspan += (uint64_t)(h.shape[k] - 1) * (uint64_t)h.dstride[k];
    }
    // (any byte alignment of bases and strides: the buffer path does not need it)
    if (h.run >= 16 && sspan < 0xffffff00ull && dspan < 0xffffff00ull) {
      d.cols = (uint32_t)((h.run + 15) / 16);
      d.last_off = (uint32_t)(h.run - 16);
      d.src_span = (uint32_t)sspan;
      d.dst_span = (uint32_t)dspan;
      pending16.push_back(d);
      return;
    }
    pending[lg].push_back(d);
  }

  static constexpr int64_t kAlignDestinationFrom = 4096;

  // Splits what the kernel's 32-bit extents or kMaxOuter cannot hold.
  void add(HostBox h) {
    if (rc != MDH_OK) {
      return;
    }
    if (h.nd == 0) {
      // One contiguous run.  16-byte buffer loads and stores take any byte alignment on gfx950,
      // so the run moves as whole vectors wherever it starts, and what is not a whole vector --
      // the last < 16 bytes -- is copied byte by byte by the flat kernel's edge workgroups, in
      // the same launch.  Stores want the destination on the 64-byte grid: off it by 4, 16 or 32
      // bytes a long copy loses 12-17 % (8 x 32 MiB: 80.6 us aligned or off by 64 B, 91.8 us off by
      // 32 B, 95.5 us off by 4 B; sources off the grid: 80.8 us).  A run of 4 KiB and more whose
      // destination is off the grid therefore starts its vectors at the next 64-byte boundary
      // and leaves the bytes before it to the edge workgroups as well.
      const int64_t max_run = (int64_t)1 << 30; // keeps tile counts inside 32 bits
      if (h.run > max_run) {
        HostBox p = h;
        for (int64_t off = 0; off < h.run; off += max_run) {
          p.src = h.src + off, p.dst = h.dst + off;
          p.run = std::min(max_run, h.run - off);
          add(p);
        }
        return;
      }
      if (h.run >= 32) {
        const uintptr_t off_grid = (uintptr_t)h.dst & 63;
        const int64_t head = off_grid != 0 && h.run >= kAlignDestinationFrom ? 64 - (int64_t)off_grid : 0;
        const int64_t rest = h.run - head;
        if (count_piece()) {
          flat.push_back(Segment{h.src + head, h.dst + head, (uint64_t)(rest & ~(int64_t)15), (uint8_t)head,
              (uint8_t)(rest & 15)});
        }
        return;
      }
      emit(h);
      return;
    }
    if (try_transposing(h)) {
      return;
    }
    uint64_t rows = 1;
    for (int d = 0; d < h.nd; ++d) {
      rows *= (uint64_t)h.shape[d];
    }
    if (h.nd > kMaxOuter || rows > 0x7fffffffull || h.run > ((int64_t)1 << 30)) {
      // walk the slowest extent on the host
      HostBox p = h;
      p.nd = h.nd - 1;
      for (int d = 0; d < p.nd; ++d) {
        p.shape[d] = h.shape[d + 1];
        p.sstride[d] = h.sstride[d + 1];
        p.dstride[d] = h.dstride[d + 1];
      }
      for (int64_t i = 0; i < h.shape[0] && rc == MDH_OK; ++i) {
        p.src = h.src + i * h.sstride[0];
        p.dst = h.dst + i * h.dstride[0];
        add(p);
      }
      return;
    }
    // Rows of 16 bytes and more that are not a whole number of 16-byte vectors go to the 16-byte
    // kernel all the same, their last vector pulled back to end with the row (emit): 8 x 4096 rows
    // of 8194 bytes 94 us, 8 x 1024 rows of 4098 bytes 15.7 us, against 97 and 16.4 us with the
    // tails split off into a box for the narrow kernel.  Only tails that the narrow kernel moves
    // as 8-byte vectors are still split off: rows of 8200 bytes 85.6 us split, 91.8 us not.
    if (h.run >= 32 && (h.run & 15) == 8) {
      HostBox body = h, tail = h;
      body.run = h.run - 8;
      tail.src = h.src + body.run;
      tail.dst = h.dst + body.run;
      tail.run = 8;
      if (vec_width(tail) == 8) {
        emit(body);
        emit(tail);
        return;
      }
    }
    emit(h);
  }
};

// Drops unit extents, merges extents that are contiguous with each other on
// both sides, and splits off the innermost extent as the byte run when it is
// dense on both sides.  Returns false for an empty box.
bool canonicalise(const char* src, char* dst, int ndim, const int64_t* shape, const int64_t* sstr,
    const int64_t* dstr, int64_t itemsize, HostBox& h) {
  h.src = src;
  h.dst = dst;
  h.nd = 0;
  h.run = itemsize;
  for (int d = 0; d < ndim; ++d) {
    if (shape[d] == 0) {
      return false;
    }
  }
  for (int d = 0; d < ndim; ++d) {
    if (shape[d] == 1) {
      continue;
    }
    const int64_t ss = sstr[d] * itemsize, ds = dstr[d] * itemsize;
    h.shape[h.nd] = shape[d];
    h.sstride[h.nd] = ss;
    h.dstride[h.nd] = ds;
    ++h.nd;
  }
  // merge from the inside out
  int n = 0;
  for (int d = 0; d < h.nd; ++d) {
    if (n > 0 && h.sstride[n - 1] == h.shape[d] * h.sstride[d] && h.dstride[n - 1] == h.shape[d] * h.dstride[d]) {
      h.shape[n - 1] *= h.shape[d];
      h.sstride[n - 1] = h.sstride[d];
      h.dstride[n - 1] = h.dstride[d];
    } else {
      h.shape[n] = h.shape[d];
      h.sstride[n] = h.sstride[d];
      h.dstride[n] = h.dstride[d];
      ++n;
    }
  }
  h.nd = n;
  if (h.nd > 0 && h.sstride[h.nd - 1] == itemsize && h.dstride[h.nd - 1] == itemsize) {
    h.run = h.shape[h.nd - 1] * itemsize;
    --h.nd;
  }
  return true;
}

template<int VEC>
void launch_boxes_vec(const Step& st, const CopyArgs& a, hipStream_t stream) {
  dim3 g(st.grid), b(kBlock);
  switch (st.unroll) {
  case 1:
    hipLaunchKernelGGL((copy_boxes_kernel<VEC, 1>), g, b, 0, stream, a);
    break;
  case 2:
    hipLaunchKernelGGL((copy_boxes_kernel<VEC, 2>), g, b, 0, stream, a);
    break;
  case 4:
    hipLaunchKernelGGL((copy_boxes_kernel<VEC, 4>), g, b, 0, stream, a);
    break;
  default:
    hipLaunchKernelGGL((copy_boxes_kernel<VEC, 8>), g, b, 0, stream, a);
    break;
  }
}

template<int E>
void launch_transposing(const Step& st, const TransArgs& a, hipStream_t stream) {
  dim3 g(st.grid), b(kBlock);
  constexpr uint32_t T = trans_shape(E, 0).a;
  if (!st.wide) {
    hipLaunchKernelGGL((transpose_kernel<E, false, T, T>), g, b, 0, stream, a);
    return;
  }
  if constexpr (E < 16) {
    // (the shapes other than T x T are measurement variants: the knob box_transpose_tile)
    if (a.tile_a == T && a.tile_b == 2 * T) {
      hipLaunchKernelGGL((transpose_kernel<E, true, T, 2 * T>), g, b, 0, stream, a);
    } else if (a.tile_a == 2 * T && a.tile_b == T) {
      hipLaunchKernelGGL((transpose_kernel<E, true, 2 * T, T>), g, b, 0, stream, a);
    } else if (a.tile_a == 2 * T && a.tile_b == 2 * T) {
      hipLaunchKernelGGL((transpose_kernel<E, true, 2 * T, 2 * T>), g, b, 0, stream, a);
    } else {
      hipLaunchKernelGGL((transpose_kernel<E, true, T, T>), g, b, 0, stream, a);
    }
  }
}

int launch_step(const Step& st, const FlatArgs* flat, const CopyArgs* boxes, hipStream_t stream, const TransArgs* trans) {
  if (st.kind == Step::kTrans) {
    switch (st.vec) {
    case 1:
      launch_transposing<1>(st, *trans, stream);
      break;
    case 2:
      launch_transposing<2>(st, *trans, stream);
      break;
    case 4:
      launch_transposing<4>(st, *trans, stream);
      break;
    case 8:
      launch_transposing<8>(st, *trans, stream);
      break;
    default:
      launch_transposing<16>(st, *trans, stream);
      break;
    }
    return check_launch("transpose_kernel");
  }
  const bool equal = st.grid_y > 0;
  uint32_t gx, gy;
  launch_dims(st, &gx, &gy);
  dim3 g(gx, gy), b(kBlock);
#define MDH_COMMA ,
#define MDH_PACKED(P) \
  P.lo[0], P.lo[1], P.lo[2], P.lo[3], P.lo[4], P.lo[5], P.lo[6], P.lo[7], P.hi[0], P.hi[1], P.hi[2], P.hi[3]
#define MDH_LAUNCH_COPY(kernel, more, args)                                                  \
  switch (st.unroll) {                                                                 \
  case 1:                                                                              \
    if (equal) {                                                                       \
      hipLaunchKernelGGL((kernel<1, true more>), g, b, st.lds, stream, args);               \
    } else {                                                                           \
      hipLaunchKernelGGL((kernel<1, false more>), g, b, st.lds, stream, args);              \
    }                                                                                  \
    break;                                                                             \
  case 2:                                                                              \
    if (equal) {                                                                       \
      hipLaunchKernelGGL((kernel<2, true more>), g, b, st.lds, stream, args);               \
    } else {                                                                           \
      hipLaunchKernelGGL((kernel<2, false more>), g, b, st.lds, stream, args);              \
    }                                                                                  \
    break;                                                                             \
  case 4:                                                                              \
    if (equal) {                                                                       \
      hipLaunchKernelGGL((kernel<4, true more>), g, b, st.lds, stream, args);               \
    } else {                                                                           \
      hipLaunchKernelGGL((kernel<4, false more>), g, b, st.lds, stream, args);              \
    }                                                                                  \
    break;                                                                             \
  default:                                                                             \
    if (equal) {                                                                       \
      hipLaunchKernelGGL((kernel<8, true more>), g, b, st.lds, stream, args);               \
    } else {                                                                           \
      hipLaunchKernelGGL((kernel<8, false more>), g, b, st.lds, stream, args);              \
    }                                                                                  \
    break;                                                                             \
  }
  switch (st.kind) {
  case Step::kFlat: {
    FlatLead L;
    if (st.preloaded && st.variant != 0 && make_flat_lead(*flat, &L, st.variant_opts)) {
#define MDH_LAUNCH_VARIANT(UU)                                                                                               \
  if (st.variant == 1) {                                                                                                     \
    hipLaunchKernelGGL((copy_flat8_kernel<UU, false, 1>), g, b, st.lds, stream, L.bytes, L.reserved, MDH_PACKED(L.from), *flat); \
  } else {                                                                                                                   \
    hipLaunchKernelGGL((copy_flat8_kernel<UU, false, 2>), g, b, st.lds, stream, L.bytes, L.reserved, MDH_PACKED(L.from), *flat); \
  }
      switch (st.unroll) {
      case 1:
        MDH_LAUNCH_VARIANT(1)
        break;
      case 2:
        MDH_LAUNCH_VARIANT(2)
        break;
      case 4:
        MDH_LAUNCH_VARIANT(4)
        break;
      default:
        MDH_LAUNCH_VARIANT(8)
        break;
      }
#undef MDH_LAUNCH_VARIANT
      return check_launch("copy_flat8_kernel");
    }
    if (st.preloaded && make_flat_lead(*flat, &L)) {
#define MDH_LAUNCH_FLAT8(UU)                                                                                          \
  if (st.edge_column) {                                                                                               \
    hipLaunchKernelGGL((copy_flat8_kernel<UU, true>), g, b, st.lds, stream, L.bytes, L.reserved, MDH_PACKED(L.from), *flat);  \
  } else {                                                                                                            \
    hipLaunchKernelGGL((copy_flat8_kernel<UU, false>), g, b, st.lds, stream, L.bytes, L.reserved, MDH_PACKED(L.from), *flat); \
  }
      switch (st.unroll) {
      case 1:
        MDH_LAUNCH_FLAT8(1)
        break;
      case 2:
        MDH_LAUNCH_FLAT8(2)
        break;
      case 4:
        MDH_LAUNCH_FLAT8(4)
        break;
      default:
        MDH_LAUNCH_FLAT8(8)
        break;
      }
#undef MDH_LAUNCH_FLAT8
      return check_launch("copy_flat8_kernel");
    }
    if (st.edge_column) {
      switch (st.unroll) {
      case 1:
        hipLaunchKernelGGL((copy_flat_kernel<1, true, true>), g, b, st.lds, stream, *flat);
        break;
      case 2:
        hipLaunchKernelGGL((copy_flat_kernel<2, true, true>), g, b, st.lds, stream, *flat);
        break;
      case 4:
        hipLaunchKernelGGL((copy_flat_kernel<4, true, true>), g, b, st.lds, stream, *flat);
        break;
      default:
        hipLaunchKernelGGL((copy_flat_kernel<8, true, true>), g, b, st.lds, stream, *flat);
        break;
      }
      return check_launch("copy_flat_kernel");
    }
    MDH_LAUNCH_COPY(copy_flat_kernel, , *flat)
    return check_launch("copy_flat_kernel");
  }
  case Step::kBoxes16: {
    RowsLead L;
    if (st.preloaded && make_rows_lead(*boxes, &L)) {
#define MDH_LAUNCH_ROWS(UU, PP)                                                                                  \
  hipLaunchKernelGGL((copy_rows16_kernel<UU, PP>), g, b, st.lds, stream, L.src_stride, L.shape, MDH_PACKED(L.from), *boxes)
      switch (st.unroll) {
      case 1:
        if (st.plain_loads) {
          MDH_LAUNCH_ROWS(1, true);
        } else {
          MDH_LAUNCH_ROWS(1, false);
        }
        break;
      case 2:
        if (st.plain_loads) {
          MDH_LAUNCH_ROWS(2, true);
        } else {
          MDH_LAUNCH_ROWS(2, false);
        }
        break;
      case 4:
        if (st.plain_loads) {
          MDH_LAUNCH_ROWS(4, true);
        } else {
          MDH_LAUNCH_ROWS(4, false);
        }
        break;
      default:
        if (st.plain_loads) {
          MDH_LAUNCH_ROWS(8, true);
        } else {
          MDH_LAUNCH_ROWS(8, false);
        }
        break;
      }
#undef MDH_LAUNCH_ROWS
      return check_launch("copy_rows16_kernel");
    }
    if (st.plain_loads) {
      MDH_LAUNCH_COPY(copy_boxes16_kernel, MDH_COMMA true, *boxes)
    } else {
      MDH_LAUNCH_COPY(copy_boxes16_kernel, MDH_COMMA false, *boxes)
    }
    return check_launch("copy_boxes16_kernel");
  }
#undef MDH_LAUNCH_COPY
#undef MDH_PACKED
#undef MDH_COMMA
  default:
    switch (st.vec) {
    case 16:
      launch_boxes_vec<16>(st, *boxes, stream);
      break;
    case 8:
      launch_boxes_vec<8>(st, *boxes, stream);
      break;
    case 4:
      launch_boxes_vec<4>(st, *boxes, stream);
      break;
    case 2:
      launch_boxes_vec<2>(st, *boxes, stream);
      break;
    default:
      launch_boxes_vec<1>(st, *boxes, stream);
      break;
    }
    return check_launch("copy_boxes_kernel");
  }
}

// Checks shared by mdh_copy_boxes and mdh_copy_plan_create.  Returns MDH_OK, or an error with
// the message set; *empty is set when the box moves nothing.
int check_box(const char* who, const mdh_box& b, int i, int itemsize, bool* empty) {
  *empty = false;
  if (b.ndim < 0 || b.ndim > MDH_MAX_DIMS) {
    set_error("%s: box %d has %d dimensions (0..%d allowed)", who, i, b.ndim, MDH_MAX_DIMS);
    return MDH_EINVAL;
  }
  int64_t numel = 1;
  for (int d = 0; d < b.ndim; ++d) {
    if (b.shape[d] < 0 || b.src_strides[d] < 0 || b.dst_strides[d] < 0) {
      set_error("%s: box %d has a negative extent or stride", who, i);
      return MDH_EINVAL;
    }
    if (b.shape[d] && numel > ((int64_t)1 << 48) / b.shape[d]) {
      set_error("%s: box %d is not a plausible device size", who, i);
      return MDH_EINVAL;
    }
    numel *= b.shape[d];
  }
  if (numel == 0) {
    *empty = true;
    return MDH_OK;
  }
  // the bytes a side spans must be a plausible device size too (keeps every later offset
  // computation inside 64 bits)
  unsigned __int128 sspan = 0, dspan = 0;
  for (int d = 0; d < b.ndim; ++d) {
    sspan += (unsigned __int128)(b.shape[d] - 1) * (unsigned __int128)b.src_strides[d];
    dspan += (unsigned __int128)(b.shape[d] - 1) * (unsigned __int128)b.dst_strides[d];
  }
  if (sspan > ((unsigned __int128)1 << 48) || dspan > ((unsigned __int128)1 << 48)) {
    set_error("%s: box %d spans more than a plausible device size", who, i);
    return MDH_EINVAL;
  }
  (void)itemsize;
  return MDH_OK;
}

// ---- prepared plans ----
//
// While a plan is being prepared, base address number `slot` is stood in for by a made-up
// address (slot + 1) << kSlotShift, 16-byte aligned like every real base a plan accepts; the
// boxes' offsets ride in the low bits through all the splitting and merging above.  Afterwards
// every address in the recorded kernel arguments is taken apart again into (slot, offset).
constexpr int kSlotShift = 44;
constexpr uint64_t kOffsetMask = ((uint64_t)1 << kSlotShift) - 1;

struct Patch {
  uint32_t step;
  uint32_t entry;
  int32_t src_slot, dst_slot;
  uint64_t src_off, dst_off;
};

} // namespace
} // namespace mdh

struct mdh_copy_plan {
  std::vector<mdh::Step> steps;
  std::vector<mdh::Patch> patches;
  std::vector<mdh_box> boxes; // as given (offsets in src/dst), for bases that are not 16-byte aligned
  std::vector<int32_t> src_slot, dst_slot;
  int itemsize = 0;
  int nbases = 0;
};

extern "C" int mdh_copy_plan_create(const mdh_box* boxes, const int32_t* src_slots, const int32_t* dst_slots, int nboxes,
    int itemsize, int nbases, mdh_copy_plan** plan) {
  using namespace mdh;
  if (!plan) {
    set_error("mdh_copy_plan_create: null out pointer");
    return MDH_EINVAL;
  }
  *plan = nullptr;
  if (nboxes < 0 || (nboxes > 0 && (!boxes || !src_slots || !dst_slots)) || nbases < 0 || nbases > 4096) {
    set_error("mdh_copy_plan_create: bad table");
    return MDH_EINVAL;
  }
  if (itemsize < 1 || itemsize > 16 || (itemsize & (itemsize - 1))) {
    set_error("mdh_copy_plan_create: itemsize %d is not 1, 2, 4, 8 or 16", itemsize);
    return MDH_EINVAL;
  }
  std::unique_ptr<mdh_copy_plan> p(new mdh_copy_plan);
  p->itemsize = itemsize;
  p->nbases = nbases;
  Launcher L;
  L.stream = nullptr;
  L.record = &p->steps;
  for (int i = 0; i < nboxes; ++i) {
    const mdh_box& b = boxes[i];
    if (src_slots[i] < 0 || src_slots[i] >= nbases || dst_slots[i] < 0 || dst_slots[i] >= nbases) {
      set_error("mdh_copy_plan_create: box %d names a base outside 0..%d", i, nbases - 1);
      return MDH_EINVAL;
    }
    bool empty;
    const int rc = check_box("mdh_copy_plan_create", b, i, itemsize, &empty);
    if (rc != MDH_OK) {
      return rc;
    }
    const uint64_t so = (uint64_t)(uintptr_t)b.src, dof = (uint64_t)(uintptr_t)b.dst;
    uint64_t sspan = 0, dspan = 0;
    for (int d = 0; d < b.ndim; ++d) {
      sspan += (uint64_t)(b.shape[d] ? b.shape[d] - 1 : 0) * (uint64_t)b.src_strides[d];
      dspan += (uint64_t)(b.shape[d] ? b.shape[d] - 1 : 0) * (uint64_t)b.dst_strides[d];
    }
    if (so + (sspan + 1) * (uint64_t)itemsize > kOffsetMask || dof + (dspan + 1) * (uint64_t)itemsize > kOffsetMask) {
      set_error("mdh_copy_plan_create: box %d reaches past %llu bytes from its base", i, (unsigned long long)kOffsetMask);
      return MDH_EINVAL;
    }
    if ((so | dof) % (unsigned)itemsize) {
      set_error("mdh_copy_plan_create: box %d is not aligned to its element size", i);
      return MDH_EINVAL;
    }
    p->boxes.push_back(b);
    p->src_slot.push_back(src_slots[i]);
    p->dst_slot.push_back(dst_slots[i]);
    if (empty) {
      continue;
    }
    const char* fake_src = (const char*)(uintptr_t)((((uint64_t)src_slots[i] + 1) << kSlotShift) + so);
    char* fake_dst = (char*)(uintptr_t)((((uint64_t)dst_slots[i] + 1) << kSlotShift) + dof);
    HostBox h;
    if (canonicalise(fake_src, fake_dst, b.ndim, b.shape, b.src_strides, b.dst_strides, itemsize, h)) {
      L.add(h);
    }
  }
  if (L.rc == MDH_OK) {
    L.flush();
  }
  if (L.rc != MDH_OK) {
    return L.rc;
  }
  auto split = [](const void* fake, int32_t* slot, uint64_t* off) {
    const uint64_t v = (uint64_t)(uintptr_t)fake;
    *slot = (int32_t)(v >> kSlotShift) - 1;
    *off = v & kOffsetMask;
  };
  for (size_t s = 0; s < p->steps.size(); ++s) {
    Step& st = p->steps[s];
    const uint32_t n = st.kind == Step::kFlat ? st.flat.nsegs : st.kind == Step::kTrans ? st.trans.nboxes : st.boxes.nboxes;
    for (uint32_t k = 0; k < n; ++k) {
      Patch pa;
      pa.step = (uint32_t)s, pa.entry = k;
      if (st.kind == Step::kFlat) {
        split(st.flat.src[k], &pa.src_slot, &pa.src_off);
        split(st.flat.dst[k], &pa.dst_slot, &pa.dst_off);
      } else if (st.kind == Step::kTrans) {
        split(st.trans.box[k].src, &pa.src_slot, &pa.src_off);
        split(st.trans.box[k].dst, &pa.dst_slot, &pa.dst_off);
      } else {
        split(st.boxes.box[k].src, &pa.src_slot, &pa.src_off);
        split(st.boxes.box[k].dst, &pa.dst_slot, &pa.dst_off);
      }
      p->patches.push_back(pa);
    }
  }
  *plan = p.release();
  return MDH_OK;
}

// Host-side replay of a plan's kernels: every tile and every slot goes through the same index
// functions the device code uses, against made-up bases of the given sizes.
extern "C" int mdh_copy_plan_verify(const mdh_copy_plan* plan, const uint64_t* base_bytes, int nbases) {
  using namespace mdh;
  if (!plan || nbases != plan->nbases || (nbases > 0 && !base_bytes)) {
    set_error("mdh_copy_plan_verify: the plan takes %d bases", plan ? plan->nbases : 0);
    return MDH_EINVAL;
  }
  for (int i = 0; i < nbases; ++i) {
    if (base_bytes[i] > ((uint64_t)1 << 31)) {
      set_error("mdh_copy_plan_verify: base %d is larger than the 2 GiB this check walks byte by byte", i);
      return MDH_EINVAL;
    }
  }
  // For every destination byte: 1 + (source slot << 40 | source byte), 0 = not written.
  std::vector<std::vector<uint64_t>> expect((size_t)nbases), got((size_t)nbases);
  std::vector<std::vector<uint8_t>> repeatable((size_t)nbases); // bytes a ragged row's last vector has written
  auto dest = [&](std::vector<std::vector<uint64_t>>& m, int slot) -> std::vector<uint64_t>& {
    if (m[(size_t)slot].empty()) {
      m[(size_t)slot].assign((size_t)base_bytes[slot], 0);
    }
    return m[(size_t)slot];
  };
  // what the boxes say, element by element
  for (size_t i = 0; i < plan->boxes.size(); ++i) {
    const mdh_box& b = plan->boxes[i];
    const int ss = plan->src_slot[i], ds = plan->dst_slot[i];
    int64_t idx[MDH_MAX_DIMS] = {0};
    int64_t numel = 1;
    for (int d = 0; d < b.ndim; ++d) {
      numel *= b.shape[d];
    }
    std::vector<uint64_t>& m = dest(expect, ds);
    for (int64_t e = 0; e < numel; ++e) {
      uint64_t so = (uint64_t)(uintptr_t)b.src, dof = (uint64_t)(uintptr_t)b.dst;
      for (int d = 0; d < b.ndim; ++d) {
        so += (uint64_t)(idx[d] * b.src_strides[d]) * (uint64_t)plan->itemsize;
        dof += (uint64_t)(idx[d] * b.dst_strides[d]) * (uint64_t)plan->itemsize;
      }
      if (so + (uint64_t)plan->itemsize > base_bytes[ss] || dof + (uint64_t)plan->itemsize > base_bytes[ds]) {
        set_error("mdh_copy_plan_verify: box %zu itself reaches outside its bases", i);
        return MDH_EINVAL;
      }
      for (int k = 0; k < plan->itemsize; ++k) {
        if (m[dof + k]) {
          set_error("mdh_copy_plan_verify: the boxes overlap in base %d at byte %llu", ds, (unsigned long long)(dof + k));
          return MDH_EINVAL;
        }
        m[dof + k] = 1 + (((uint64_t)ss << 40) | (so + k));
      }
      for (int d = b.ndim - 1; d >= 0; --d) {
        if (++idx[d] < b.shape[d]) {
          break;
        }
        idx[d] = 0;
      }
    }
  }
  // what the kernels would do
  auto split = [](const void* fake, int* slot, uint64_t* off) {
    const uint64_t v = (uint64_t)(uintptr_t)fake;
    *slot = (int)(v >> kSlotShift) - 1;
    *off = v & kOffsetMask;
  };
  // may_repeat: a ragged row's last vector, which overlaps the one before it -- a byte may then
  // be written a second time, with the same source byte
  auto move = [&](int ss, uint64_t so, int ds, uint64_t dof, uint32_t n, size_t step, bool may_repeat = false) -> bool {
    if (ss < 0 || ss >= nbases || ds < 0 || ds >= nbases || so + n > base_bytes[ss] || dof + n > base_bytes[ds]) {
      set_error("mdh_copy_plan_verify: step %zu moves %u bytes from base %d + %llu to base %d + %llu: outside the bases", step, n,
          ss, (unsigned long long)so, ds, (unsigned long long)dof);
      return false;
    }
    std::vector<uint64_t>& m = dest(got, ds);
    for (uint32_t k = 0; k < n; ++k) {
      const uint64_t what = 1 + (((uint64_t)ss << 40) | (so + k));
      if (m[dof + k] && !(m[dof + k] == what && (may_repeat || repeatable[(size_t)ds][dof + k]))) {
        set_error("mdh_copy_plan_verify: step %zu writes base %d byte %llu a second time", step, ds, (unsigned long long)(dof + k));
        return false;
      }
      m[dof + k] = what;
      if (may_repeat) {
        if (repeatable[(size_t)ds].empty()) {
          repeatable[(size_t)ds].assign((size_t)base_bytes[ds], 0);
        }
        repeatable[(size_t)ds][dof + k] = 1;
      }
    }
    return true;
  };
  for (size_t s = 0; s < plan->steps.size(); ++s) {
    const Step& st = plan->steps[s];
    if (st.kind == Step::kTrans) {
      // one tile per workgroup, every element of every tile through the kernel's own index function
      const TransArgs& a = st.trans;
      const uint32_t E = (uint32_t)st.vec;
      if (st.grid == 0 || st.grid > a.total_tiles || a.nboxes == 0 || a.nboxes > (uint32_t)kMaxTransBoxes || a.tile_a == 0 ||
          a.tile_b == 0) {
        set_error("mdh_copy_plan_verify: step %zu has a grid of %u workgroups for %u tiles", s, st.grid, a.total_tiles);
        return MDH_EINVAL;
      }
      for (uint32_t tile = 0; tile < a.total_tiles; ++tile) {
        const TransLoc t = trans_locate(a, tile, E);
        if (t.box >= a.nboxes) {
          set_error("mdh_copy_plan_verify: step %zu tile %u lands in box %u of %u", s, tile, t.box, a.nboxes);
          return MDH_EINVAL;
        }
        const TransBox& B = a.box[t.box];
        if (t.ia >= B.na || t.ib >= B.nb) {
          set_error("mdh_copy_plan_verify: step %zu tile %u starts outside its box", s, tile);
          return MDH_EINVAL;
        }
        int ss, ds;
        uint64_t sbase, dbase;
        split(B.src, &ss, &sbase);
        split(B.dst, &ds, &dbase);
        const uint32_t na = B.na - t.ia < a.tile_a ? B.na - t.ia : a.tile_a, nb = B.nb - t.ib < a.tile_b ? B.nb - t.ib : a.tile_b;
        if (st.wide && ((na * E) % 16 != 0 || (nb * E) % 16 != 0 || ((sbase + (uint64_t)t.src_off) & 15) != 0 ||
                           ((dbase + (uint64_t)t.dst_off) & 15) != 0 || (B.src_b & 15) != 0 || (B.dst_a & 15) != 0)) {
          set_error("mdh_copy_plan_verify: step %zu box %u: 16-byte accesses do not fit this box", s, t.box);
          return MDH_EINVAL;
        }
        for (uint32_t ib = 0; ib < nb; ++ib) {
          for (uint32_t ia = 0; ia < na; ++ia) {
            const int64_t so = t.src_off + (int64_t)ib * B.src_b + (int64_t)ia * E;
            const int64_t dof = t.dst_off + (int64_t)ia * B.dst_a + (int64_t)ib * E;
            if (!move(ss, sbase + (uint64_t)so, ds, dbase + (uint64_t)dof, E, s)) {
              return MDH_EINVAL;
            }
          }
        }
      }
      continue;
    }
    // every workgroup takes its first tile untested: the grid must not exceed the tile count
    const uint32_t step_tiles = st.kind == Step::kFlat ? st.flat.total_tiles : st.boxes.total_tiles;
    if (st.grid == 0 || st.grid > step_tiles) {
      set_error("mdh_copy_plan_verify: step %zu has a grid of %u workgroups for %u tiles", s, st.grid, step_tiles);
      return MDH_EINVAL;
    }
    if (st.grid_y) {
      // two-dimensional form: workgroup (x, y) takes tile x of entry y and no other
      const uint32_t per = st.kind == Step::kFlat ? st.flat.tiles_per_seg : st.boxes.tiles_per_box;
      const uint32_t n = st.kind == Step::kFlat ? st.flat.nsegs : st.boxes.nboxes;
      if (st.kind == Step::kBoxes || per == 0 || st.grid != per || st.grid_y != n || (uint64_t)per * n != step_tiles) {
        set_error("mdh_copy_plan_verify: step %zu: a %u x %u grid does not match %u entries of %u tiles", s, st.grid,
            st.grid_y, n, per);
        return MDH_EINVAL;
      }
    }
    if (st.variant != 0) {
      set_error("mdh_copy_plan_verify: step %zu was prepared with a measurement knob set (copy_xcd_run, copy_grid_order, "
                "copy_tail_tiles or copy_lds), which this check does not replay", s);
      return MDH_EINVAL;
    }
    if (st.kind == Step::kFlat) {
      const FlatArgs& a = st.flat;
      const uint32_t tile_bytes = (uint32_t)kBlock * (uint32_t)st.unroll * 16u;
      for (uint32_t tile = 0; tile < a.total_tiles; ++tile) {
        uint32_t local;
        const uint32_t seg = locate_segment(a, tile, &local);
        if (seg >= a.nsegs) {
          set_error("mdh_copy_plan_verify: step %zu tile %u lands in segment %u of %u", s, tile, seg, a.nsegs);
          return MDH_EINVAL;
        }
        const uint64_t off = (uint64_t)local * tile_bytes;
        if (off >= a.bytes[seg]) {
          set_error("mdh_copy_plan_verify: step %zu tile %u starts past the end of its segment", s, tile);
          return MDH_EINVAL;
        }
        const uint64_t left = a.bytes[seg] - off;
        const uint32_t n = left < tile_bytes ? (uint32_t)left : tile_bytes;
        int ss, ds;
        uint64_t so, dof;
        split(a.src[seg], &ss, &so);
        split(a.dst[seg], &ds, &dof);
        if (!move(ss, so + off, ds, dof + off, n, s)) {
          return MDH_EINVAL;
        }
      }
      if ((st.grid_y != 0 && a.edge_wgs == 1) || (st.grid_y == 0 && a.edge_wgs == 2) ||
          st.edge_column != (a.edge_wgs == 2)) {
        set_error("mdh_copy_plan_verify: step %zu: edge workgroups of the other form of the grid", s);
        return MDH_EINVAL;
      }
      // copy_flat8_kernel takes every segment's length from one leading argument
      if (st.preloaded && (!st.grid_y || !uniform_segments(a))) {
        set_error("mdh_copy_plan_verify: step %zu: the preloaded form does not fit this launch", s);
        return MDH_EINVAL;
      }
      // the edge workgroups: every slot of every segment, through the kernel's own mapping
      if ((a.edge_wgs != 0) != [&] {
            for (uint32_t seg = 0; seg < a.nsegs; ++seg) {
              if (a.head[seg] || a.tail[seg]) {
                return true;
              }
            }
            return false;
          }()) {
        set_error("mdh_copy_plan_verify: step %zu: edge workgroups do not match the segments' heads and tails", s);
        return MDH_EINVAL;
      }
      for (uint32_t seg = 0; seg < a.nsegs && a.edge_wgs; ++seg) {
        int ss, ds;
        uint64_t so, dof;
        split(a.src[seg], &ss, &so);
        split(a.dst[seg], &ds, &dof);
        for (uint32_t slot = 0; slot < kEdgeSlots; ++slot) {
          int64_t off;
          if (!edge_offset(a, seg, slot, &off)) {
            continue;
          }
          if (off < 0 && ((uint64_t)-off > so || (uint64_t)-off > dof)) {
            set_error("mdh_copy_plan_verify: step %zu segment %u: head byte before its base", s, seg);
            return MDH_EINVAL;
          }
          if (!move(ss, so + (uint64_t)off, ds, dof + (uint64_t)off, 1, s)) {
            return MDH_EINVAL;
          }
        }
      }
      continue;
    }
    const CopyArgs& a = st.boxes;
    const uint32_t slots = (uint32_t)kBlock * (uint32_t)st.unroll;
    uint32_t log2slots = 0;
    while ((1u << log2slots) < slots) {
      ++log2slots;
    }
    const bool buffer16 = st.kind == Step::kBoxes16;
    for (uint32_t tile = 0; tile < a.total_tiles; ++tile) {
      const TileLoc t = buffer16 ? locate_tile<true>(a, tile) : locate_tile<false>(a, tile);
      if (t.box >= a.nboxes) {
        set_error("mdh_copy_plan_verify: step %zu tile %u lands in box %u of %u", s, tile, t.box, a.nboxes);
        return MDH_EINVAL;
      }
      const BoxDesc& B = a.box[t.box];
      int ss, ds;
      uint64_t sbase, dbase;
      split(B.src, &ss, &sbase);
      split(B.dst, &ds, &dbase);
      for (uint32_t slot = 0; slot < slots; ++slot) {
        uint64_t so, dof;
        if (buffer16) {
          uint32_t so32, dof32;
          const bool inside = slot_offsets<uint32_t>(B, t, slot, log2slots, 16u, &so32, &dof32);
          if (st.preloaded) {
            // copy_rows16_kernel: no slot may lie outside the box, and its own arithmetic --
            // from the leading arguments alone -- must name the same source vector
            const BoxDesc& f = a.box[0];
            const uint32_t early = rows_offset((uint32_t)f.src_stride[0], f.log2tc, log2slots, t.rt, t.ct, slot);
            const uint32_t early_dst = rows_offset((uint32_t)B.dst_stride[0], f.log2tc, log2slots, t.rt, t.ct, slot);
            if (!inside || early != so32 || early_dst != dof32 || !uniform_full_rows(a, st.unroll)) {
              set_error("mdh_copy_plan_verify: step %zu box %u: the preloaded form does not fit this launch", s, t.box);
              return MDH_EINVAL;
            }
          }
          if (!inside) {
            continue; // the kernel gives this slot the offset just past the descriptor
          }
          // an access the descriptor would clip is an access the kernel silently loses
          if ((uint64_t)so32 + 16 > B.src_span || (uint64_t)dof32 + 16 > B.dst_span) {
            set_error("mdh_copy_plan_verify: step %zu box %u: a vector lies outside the box's own descriptor", s, t.box);
            return MDH_EINVAL;
          }
          so = so32, dof = dof32;
        } else {
          int64_t so64, dof64;
          if (!slot_offsets<int64_t>(B, t, slot, log2slots, (uint32_t)st.vec, &so64, &dof64)) {
            continue;
          }
          so = (uint64_t)so64, dof = (uint64_t)dof64;
        }
        // the last vector of a row that is not a whole number of vectors overlaps the one before
        const uint32_t col = (t.ct << B.log2tc) + (slot & ((1u << B.log2tc) - 1u));
        const bool pulled_back = buffer16 && (B.last_off & 15) != 0 && col == B.cols - 1;
        if (!move(ss, sbase + so, ds, dbase + dof, buffer16 ? 16u : (uint32_t)st.vec, s, pulled_back)) {
          return MDH_EINVAL;
        }
      }
    }
  }
  for (int b = 0; b < nbases; ++b) {
    const std::vector<uint64_t>&e = expect[(size_t)b], &g = got[(size_t)b];
    for (size_t i = 0; i < (size_t)base_bytes[b]; ++i) {
      const uint64_t x = e.empty() ? 0 : e[i], y = g.empty() ? 0 : g[i];
      if (x != y) {
        set_error("mdh_copy_plan_verify: base %d byte %zu: the boxes ask for source %llx, the kernels bring %llx", b, i,
            (unsigned long long)x, (unsigned long long)y);
        return MDH_EINVAL;
      }
    }
  }
  return MDH_OK;
}

extern "C" void mdh_copy_plan_destroy(mdh_copy_plan* plan) {
  delete plan;
}

extern "C" int mdh_copy_plan_launches(const mdh_copy_plan* plan) {
  return plan ? (int)plan->steps.size() : -1;
}

// Writes the caller's addresses into a copy of launch `s`'s argument block; `at` is the first
// patch of that launch, the return value the first patch of the next.
static size_t patch_step(const mdh_copy_plan& plan, size_t s, size_t at, const void* const* bases, mdh::FlatArgs* flat,
    mdh::CopyArgs* boxes, mdh::TransArgs* trans = nullptr) {
  for (; at < plan.patches.size() && plan.patches[at].step == s; ++at) {
    const mdh::Patch& pa = plan.patches[at];
    const char* src = (const char*)bases[pa.src_slot] + pa.src_off;
    char* dst = (char*)bases[pa.dst_slot] + pa.dst_off;
    if (flat) {
      flat->src[pa.entry] = src;
      flat->dst[pa.entry] = dst;
    } else if (boxes) {
      boxes->box[pa.entry].src = src;
      boxes->box[pa.entry].dst = dst;
    } else {
      trans->box[pa.entry].src = src;
      trans->box[pa.entry].dst = dst;
    }
  }
  return at;
}

extern "C" int mdh_copy_plan_launch(const mdh_copy_plan* plan, const void* const* bases, int nbases, void* stream) {
  using namespace mdh;
  if (!plan || nbases != plan->nbases || (nbases > 0 && !bases)) {
    set_error("mdh_copy_plan_launch: the plan takes %d base addresses", plan ? plan->nbases : 0);
    return MDH_EINVAL;
  }
  if (const int rc = refuse_capture((hipStream_t)stream, "mdh_copy_plan_launch")) {
    return rc;
  }
  uintptr_t low = 0;
  for (int i = 0; i < nbases; ++i) {
    low |= (uintptr_t)bases[i];
  }
  if (low & 15) {
    // prepared for 16-byte aligned bases (what decides the vector width of narrow rows): any
    // other table goes the general way, box by box
    std::vector<mdh_box> boxes(plan->boxes);
    for (size_t i = 0; i < boxes.size(); ++i) {
      boxes[i].src = (const char*)bases[plan->src_slot[i]] + (uintptr_t)plan->boxes[i].src;
      boxes[i].dst = (char*)bases[plan->dst_slot[i]] + (uintptr_t)plan->boxes[i].dst;
    }
    return mdh_copy_boxes(boxes.data(), (int)boxes.size(), plan->itemsize, stream);
  }
  // a used base must exist
  for (const Patch& pa : plan->patches) {
    if (!bases[pa.src_slot] || !bases[pa.dst_slot]) {
      set_error("mdh_copy_plan_launch: base %d is null", !bases[pa.src_slot] ? pa.src_slot : pa.dst_slot);
      return MDH_EINVAL;
    }
  }
  size_t at = 0;
  for (size_t s = 0; s < plan->steps.size(); ++s) {
    const Step& st = plan->steps[s];
    int rc;
    if (st.kind == Step::kFlat) {
      FlatArgs a = st.flat;
      at = patch_step(*plan, s, at, bases, &a, nullptr);
      rc = launch_step(st, &a, nullptr, (hipStream_t)stream);
    } else if (st.kind == Step::kTrans) {
      TransArgs a = st.trans;
      at = patch_step(*plan, s, at, bases, nullptr, nullptr, &a);
      rc = launch_step(st, nullptr, nullptr, (hipStream_t)stream, &a);
    } else {
      CopyArgs a = st.boxes;
      at = patch_step(*plan, s, at, bases, nullptr, &a);
      rc = launch_step(st, nullptr, &a, (hipStream_t)stream);
    }
    if (rc != MDH_OK) {
      return rc;
    }
  }
  return MDH_OK;
}

extern "C" int mdh_copy_plan_step_arguments(const mdh_copy_plan* plan, const void* const* bases, int nbases, int step,
    void* out, size_t capacity, size_t* size, uint32_t* leading_scalars, uint32_t* grid_x, uint32_t* grid_y,
    uint32_t* block, uint32_t* lds) {
  using namespace mdh;
  if (!plan || nbases != plan->nbases || (nbases > 0 && !bases) || step < 0 || (size_t)step >= plan->steps.size() ||
      !size) {
    set_error("mdh_copy_plan_step_arguments: bad plan, base table or launch number");
    return MDH_EINVAL;
  }
  for (int i = 0; i < nbases; ++i) {
    if ((uintptr_t)bases[i] & 15) {
      set_error("mdh_copy_plan_step_arguments: base %d is not 16-byte aligned (such a call is not served from the "
                "prepared launches)", i);
      return MDH_EINVAL;
    }
  }
  const Step& st = plan->steps[(size_t)step];
  size_t at = 0;
  while (at < plan->patches.size() && plan->patches[at].step < (size_t)step) {
    ++at;
  }
  FlatArgs flat;
  CopyArgs boxes;
  TransArgs trans;
  union {
    RowsLead rows;
    FlatLead flat;
  } lead;
  static_assert(sizeof(RowsLead) == sizeof(FlatLead), "one size of leading arguments");
  size_t lead_bytes = 0;
  const void* from;
  if (st.kind == Step::kTrans) {
    trans = st.trans;
    patch_step(*plan, (size_t)step, at, bases, nullptr, nullptr, &trans);
    from = &trans;
    *size = sizeof(TransArgs);
  } else if (st.kind == Step::kFlat) {
    flat = st.flat;
    patch_step(*plan, (size_t)step, at, bases, &flat, nullptr);
    from = &flat;
    *size = sizeof(FlatArgs);
    if (st.preloaded && make_flat_lead(flat, &lead.flat, st.variant ? st.variant_opts : 0u)) {
      lead_bytes = sizeof(FlatLead);
      *size += lead_bytes;
    }
  } else {
    boxes = st.boxes;
    patch_step(*plan, (size_t)step, at, bases, nullptr, &boxes);
    from = &boxes;
    *size = sizeof(CopyArgs);
    if (st.kind == Step::kBoxes16 && st.preloaded && make_rows_lead(boxes, &lead.rows)) {
      lead_bytes = sizeof(RowsLead);
      *size += lead_bytes;
    }
  }
  if (leading_scalars) {
    *leading_scalars = (uint32_t)(lead_bytes / 4);
  }
  uint32_t gx, gy;
  launch_dims(st, &gx, &gy);
  if (grid_x) *grid_x = gx;
  if (grid_y) *grid_y = gy;
  if (block) *block = (uint32_t)kBlock;
  if (lds) *lds = (uint32_t)st.lds;
  if (out) {
    if (capacity < *size) {
      set_error("mdh_copy_plan_step_arguments: the block is %zu bytes", *size);
      return MDH_EINVAL;
    }
    std::memcpy(out, &lead, lead_bytes);
    std::memcpy((char*)out + lead_bytes, from, *size - lead_bytes);
  }
  return MDH_OK;
}

extern "C" int mdh_copy_boxes(const mdh_box* boxes, int nboxes, int itemsize, void* stream) {
  using namespace mdh;
  if (nboxes < 0 || (nboxes > 0 && !boxes)) {
    set_error("mdh_copy_boxes: bad box table");
    return MDH_EINVAL;
  }
  if (itemsize < 1 || itemsize > 16 || (itemsize & (itemsize - 1))) {
    set_error("mdh_copy_boxes: itemsize %d is not 1, 2, 4, 8 or 16", itemsize);
    return MDH_EINVAL;
  }
  if (nboxes > 0) {
    if (const int rc = refuse_capture((hipStream_t)stream, "mdh_copy_boxes")) {
      return rc;
    }
  }
  Launcher L;
  L.stream = (hipStream_t)stream;
  for (int i = 0; i < nboxes; ++i) {
    const mdh_box& b = boxes[i];
    bool empty;
    const int rc = check_box("mdh_copy_boxes", b, i, itemsize, &empty);
    if (rc != MDH_OK) {
      return rc;
    }
    if (empty) {
      continue;
    }
    if (!b.src || !b.dst) {
      set_error("mdh_copy_boxes: box %d has a null pointer", i);
      return MDH_EINVAL;
    }
    if (((uintptr_t)b.src | (uintptr_t)b.dst) % (unsigned)itemsize) {
      set_error("mdh_copy_boxes: box %d is not aligned to its element size", i);
      return MDH_EINVAL;
    }
    HostBox h;
    if (canonicalise((const char*)b.src, (char*)b.dst, b.ndim, b.shape, b.src_strides, b.dst_strides, itemsize, h)) {
      L.add(h);
    }
  }
  if (L.rc == MDH_OK) {
    L.flush();
  }
  return L.rc;
}

extern "C" int mdh_gather(const void* const* srcs, int nsrc, void* dst, size_t width, size_t rows, size_t src_pitch,
    size_t dst_pitch, size_t dst_shard_stride, void* stream) {
  using namespace mdh;
  if (nsrc < 0 || nsrc > 65536) {
    set_error("mdh_gather: nsrc %d out of range", nsrc);
    return MDH_EINVAL;
  }
  if (nsrc == 0 || width == 0 || rows == 0) {
    return MDH_OK;
  }
  if (!srcs || !dst) {
    set_error("mdh_gather: null pointer");
    return MDH_EINVAL;
  }
  if (rows > 1 && (src_pitch < width || dst_pitch < width)) {
    set_error("mdh_gather: a row pitch is smaller than the row width");
    return MDH_EINVAL;
  }
  const unsigned __int128 limit = (unsigned __int128)1 << 48;
  if (width > limit || rows > ((size_t)1 << 40) || (unsigned __int128)rows * src_pitch > limit ||
      (unsigned __int128)rows * dst_pitch > limit || (unsigned __int128)nsrc * dst_shard_stride > limit) {
    set_error("mdh_gather: not a plausible device size");
    return MDH_EINVAL;
  }
  const size_t extent = (rows - 1) * dst_pitch + width;
  if (nsrc > 1 && dst_shard_stride < extent) {
    set_error("mdh_gather: shards would overlap in the destination");
    return MDH_EINVAL;
  }
  if (const int rc = refuse_capture((hipStream_t)stream, "mdh_gather")) {
    return rc;
  }
  Launcher L;
  L.stream = (hipStream_t)stream;
  for (int s = 0; s < nsrc; ++s) {
    if (!srcs[s]) {
      set_error("mdh_gather: source %d is null", s);
      return MDH_EINVAL;
    }
    char* out = (char*)dst + (size_t)s * dst_shard_stride;
    if ((const char*)srcs[s] == out && (rows == 1 || src_pitch == dst_pitch)) {
      continue; // shard already in place
    }
    const int64_t shape[2] = {(int64_t)rows, (int64_t)width};
    const int64_t ss[2] = {(int64_t)src_pitch, 1};
    const int64_t ds[2] = {(int64_t)dst_pitch, 1};
    HostBox h;
    if (canonicalise((const char*)srcs[s], out, 2, shape, ss, ds, 1, h)) {
      L.add(h);
    }
  }
  if (L.rc == MDH_OK) {
    L.flush();
  }
  return L.rc;
}
