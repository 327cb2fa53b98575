/*
 * moodist_hip.h -- thin C ABI between the C++ host side and the hand-written
 * HIP kernels for gfx950 (MI355X).
 *
 * The reference has no such seam: its host code launches run-time generated
 * kernels directly with cuLaunchKernel (core/processgroup.cc:1240-1242 for
 * allgather_local, :1651-1657 for reduce_scatter_local, :1556-1557 for
 * reduce_scatter_direct) after filling AllGatherParameters /
 * ReduceScatterParameters (core/allgather.h:14-24, core/reduce_scatter.h:14-26).
 * Each entry point below replaces one of those launches (named per function)
 * and takes the same facts as plain pointers and sizes.
 *
 * Contract shared by every launch function:
 *   - returns 0 on success, an MDH_E* code otherwise (never throws, never
 *     aborts); mdh_error_string() names a code, mdh_last_error() holds detail
 *     for the calling thread;
 *   - allocates nothing, frees nothing, never synchronises: work is enqueued
 *     on `stream` (a hipStream_t; NULL is the default stream) and the caller
 *     owns every buffer until that work has finished.  Long copies ask for
 *     40 KiB of dynamic LDS per workgroup that the kernels never touch: it
 *     limits how many workgroups a CU holds at once;
 *   - `stream` must not be capturing (hipStreamBeginCapture): a launch function that finds it
 *     capturing enqueues and records nothing and returns MDH_ECAPTURE.  Graph replay of these
 *     launches is not supported;
 *   - all data pointers are device pointers on the current device; pointer
 *     TABLES (srcs, boxes) are host memory and are consumed before return;
 *   - dtype codes are torch ScalarType numbers and op codes are c10d RedOpType
 *     numbers, the same numbers the reference's API carries
 *     (api/moodist_api.h:30-55).
 */
#ifndef MOODIST_HIP_H
#define MOODIST_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MDH_ABI_VERSION 2

/* error codes */
#define MDH_OK 0
#define MDH_EINVAL 1      /* bad argument (null pointer, count or size out of range) */
#define MDH_EDTYPE 2      /* "Unsupported dtype for reduce operation" (core/processgroup.cc:277) */
#define MDH_EOP 3         /* "Unsupported reduce operation" (core/processgroup.cc:294) */
#define MDH_ELAUNCH 4     /* the HIP runtime refused the launch; see mdh_last_error() */
#define MDH_ENODEVICE 5   /* no usable gfx950 device */
#define MDH_ECAPTURE 6    /* `stream` is being captured into a graph: nothing was enqueued or recorded.
                             Replaying a graph that holds these launches is not supported (the one replay
                             ever made of them raised an illegal-address fault whose cause was not found),
                             so every launch function refuses a capturing stream. */

/* api/moodist_api.h:30-42 */
#define MDH_DTYPE_INT32 3
#define MDH_DTYPE_INT64 4
#define MDH_DTYPE_FLOAT16 5
#define MDH_DTYPE_FLOAT32 6
#define MDH_DTYPE_FLOAT64 7
#define MDH_DTYPE_BFLOAT16 15

/* api/moodist_api.h:45-55 */
#define MDH_OP_SUM 0
#define MDH_OP_AVG 1
#define MDH_OP_MIN 3
#define MDH_OP_MAX 4
#define MDH_OP_PREMUL_SUM 8

#define MDH_MAX_SOURCES 64 /* the reference stops at 8 peer slots (core/reduce_scatter.h:22-23) */
#define MDH_MAX_DIMS 10    /* compile_op accepts up to 10 dimensions (core/processgroup.cc:3110-3141) */

int mdh_abi_version(void);
const char* mdh_error_string(int code);
const char* mdh_last_error(void);

/*
 * Local multi-source reduction: dst[i] = srcs[first][i] (+) srcs[first+1][i]
 * (+) ... wrapping round to srcs[first-1][i], a left fold in exactly that
 * order, in one pass over memory.
 *
 * Replaces: the reduce_scatter_local kernel launch (core/processgroup.cc:1651-1653;
 * fold built by core/reduce_scatter.cc:104-142, :180-191 as K-1 two-source
 * passes), the per-destination reduction of reduce_scatter_direct
 * (core/reduce_scatter_direct.cc:165-177) and the final sum_out/amax_out/amin_out
 * over K rows (core/processgroup.cc:1599-1616).  `first` expresses the
 * reference's peer order: own chunk, then ranks rank+1..P-1, 0..rank-1
 * (core/group.cc:567-570).
 *
 * srcs[j] points at source j's chunk (the caller has already added
 * pitch*rank); dst may equal srcs[first] exactly (allreduce reduces in place,
 * core/processgroup.cc:1689-1692) but must not otherwise overlap a source.
 *
 * op / scale:
 *   SUM, MIN, MAX  scale ignored.  MIN/MAX follow std::min/std::max on
 *                  (running value, next source): ties and NaN keep the
 *                  running value (core/cputhread.cc:131-143).
 *   AVG            SUM, then one multiply by `scale` with its own rounding
 *                  (the caller passes 1.0f/size; core/processgroup.cc:1664-1667).
 *   PREMUL_SUM     each source times `scale` with its own rounding, then SUM
 *                  (core/processgroup.cc:1374-1378).
 *   AVG and PREMUL_SUM need a floating dtype.
 * float32/float64: IEEE adds in fold order, bit-exact.  int32/int64: wrapping
 * adds, signed min/max.  bfloat16/float16: sources widened to fp32, folded in
 * fp32, rounded to nearest even once.
 *
 * Pointers need element alignment only, sizes none: no staging copy is ever
 * made (the reference stages through an aligned buffer when bytes % 16 or
 * address % 16 is non-zero, core/processgroup.cc:1409-1431).  numel == 0 is a
 * no-op.
 */
int mdh_reduce(const void* const* srcs, int nsrc, int first, void* dst, size_t numel, int dtype, int op,
    float scale, void* stream);

/*
 * A list of such reductions, all of one element type and operation, in as few launches as
 * possible: job j is mdh_reduce(jobs[j].srcs, jobs[j].nsrc, jobs[j].first, jobs[j].dst,
 * jobs[j].numel, dtype, op, scale, stream), with the same results bit for bit.
 *
 * Replaces: the loops of the coalesced collectives, which run one reduce_scatter (and so one
 * kernel launch per rank) per tensor (wrapper/processgroup_wrapper.cc:159-170 for
 * reduce_scatter_tensor_coalesced, :182-191 for allreduce_coalesced; the fold of each is
 * core/reduce_scatter.cc:104-142).  Launches of a few KiB to a few MiB are bound by the launch
 * itself, so the jobs share launches: up to 40 jobs and 320 source pointers per launch, their
 * tiles numbered through, about 96 MiB of every source at most.  A job of 16 MiB per source and
 * more gets a launch of its own, shaped as mdh_reduce shapes it.  Jobs with numel == 0 are skipped.
 *
 * The jobs must be independent: no job's destination may overlap another job's sources or
 * destination (within a job, dst may equal srcs[first], as for mdh_reduce).  Every job is
 * checked before anything is enqueued: on an error nothing has been launched.
 */
typedef struct mdh_reduce_job {
  const void* const* srcs; /* nsrc device pointers (the table itself is host memory) */
  int32_t nsrc;            /* 1..MDH_MAX_SOURCES */
  int32_t first;           /* the fold starts at srcs[first] */
  void* dst;
  size_t numel;
} mdh_reduce_job;
int mdh_reduce_many(const mdh_reduce_job* jobs, int njobs, int dtype, int op, float scale, void* stream);

/*
 * The same list of reductions with every job's result stored over ALL of the job's sources:
 * afterwards each of jobs[j].srcs[0 .. nsrc-1] holds, in its first numel elements, what
 * mdh_reduce(jobs[j].srcs, nsrc, jobs[j].first, ...) yields, bit for bit.  jobs[j].dst is ignored.
 *
 * Replaces: the allreduce of ranks whose tensors one GPU can address (all local ranks of a
 * process here; with mapped peer memory, the ranks of a node), which the reference composes of
 * a reduce_scatter into the rank's own chunk and an all_gather of the chunks
 * (core/processgroup.cc:1674-1722): one job per chunk c, srcs[r] = rank r's tensor + c * chunk,
 * first = c (the fold order of the rank that owns the chunk, core/group.cc:567-570).  One launch
 * reads every tensor once and writes every tensor once -- 2 * P * bytes where the composition
 * moves (3 * P - 1) * bytes in two launches per rank.
 *
 * A tile is read from every source before its first store and belongs to one wave, so the
 * sources are read and overwritten in place.  The sources of a job must not overlap one
 * another, and the jobs must be independent.  Jobs of any length stay in shared launches
 * (pieces of 32 MiB per source).  Every job is checked before anything is enqueued.
 */
int mdh_allreduce_many(const mdh_reduce_job* jobs, int njobs, int dtype, int op, float scale, void* stream);

/*
 * All-gather chunk assembly: for every shard s < nsrc and row r < rows,
 * copy `width` bytes from srcs[s] + r*src_pitch to
 * dst + s*dst_shard_stride + r*dst_pitch.
 *
 * Replaces: the allgather_local kernel launch (core/processgroup.cc:1240-1242;
 * P sequential copy_impl calls, core/allgather.cc:381-390) with rows = 1,
 * width = bytes, dst_shard_stride = pitch; and the copy-engine form
 * (Copy2d + cuMemcpy2DAsync, core/processgroup.cc:806-820) and the padded
 * staging copies (:1130-1136, :1273-1283) with rows > 1.
 *
 * srcs[s] == dst + s*dst_shard_stride is allowed (a shard already in place is
 * skipped); other overlap is not.  Any alignment; width == 0 or rows == 0 is a
 * no-op.
 */
int mdh_gather(const void* const* srcs, int nsrc, void* dst, size_t width, size_t rows, size_t src_pitch,
    size_t dst_pitch, size_t dst_shard_stride, void* stream);

/*
 * One N-d box to move: shape[d] elements along dimension d, element strides on
 * each side.  src/dst point at the box's first element (offset already added).
 */
typedef struct mdh_box {
  const void* src;
  void* dst;
  int32_t ndim; /* 0..MDH_MAX_DIMS */
  int32_t reserved;
  int64_t shape[MDH_MAX_DIMS];
  int64_t src_strides[MDH_MAX_DIMS]; /* in elements, >= 0 */
  int64_t dst_strides[MDH_MAX_DIMS]; /* in elements, >= 0 */
} mdh_box;

/*
 * Shard redistribution: copy every box, strided on either side, in as few
 * launches as the table allows (boxes are fused into one grid).
 *
 * Replaces: the execution of a compiled custom op -- each Read is a byte-exact
 * move (core/cputhread.cc:5628-5672) and each Copy an {offset, shape} box of a
 * tensor to or from contiguous staging (core/cputhread.h:306-310).  A box with
 * both sides strided is the fused form Copy -> Read -> Copy, so no staging
 * buffer exists.  Destination boxes must not overlap each other or any source.
 *
 * A box may transpose: its source contiguous along one dimension, its destination along
 * another (out[c][r] = in[r][c]).  The reference's planner never produces one (source and
 * destination boxes of a redistribution share a dimension order,
 * core/processgroup.cc:2848-2870); here such a box, when both dimensions are at least 16
 * elements long, is copied in tiles of 64 x 64 (32 x 32 for 8- and 16-byte elements) that are
 * read along the source's contiguous dimension, turned round in LDS and written along the
 * destination's, so that both sides move whole cache lines.
 */
int mdh_copy_boxes(const mdh_box* boxes, int nboxes, int itemsize, void* stream);

/*
 * The same copies, prepared once and replayed: what a compiled custom op runs on every call.
 *
 * Replaces: the split the reference makes between compileOpFull, which computes the reads and
 * copies of an op once (core/processgroup.cc:2761-3104), and customOp, which on every call only
 * checks sizes and enqueues them (core/processgroup.cc:3172-3256).  Here everything about the
 * launches except the tensors' addresses is decided at create time -- boxes merged and split,
 * vector widths, tiles, grids, the kernels' argument blocks -- and a launch patches addresses
 * into a copy of those blocks and enqueues the kernels.
 *
 * create: boxes[i].src / boxes[i].dst hold BYTE OFFSETS from base number src_slots[i] /
 * dst_slots[i] of a table of `nbases` base addresses that is supplied at launch (a custom op's
 * input and output tensors).  Shapes and strides as in mdh_copy_boxes.  Needs no device.
 * launch: bases[] are device addresses; the result is that of mdh_copy_boxes on the boxes with
 * the offsets added to the bases.  Plans are prepared for 16-byte aligned bases (torch
 * allocations are); a table with a less aligned base is served through mdh_copy_boxes.
 * A plan is immutable after create: launches of one plan may run concurrently.
 * launches: how many kernels one launch of the plan enqueues (-1 for NULL).
 * verify: replays the plan's kernels ON THE HOST -- every tile, every slot, through the very
 * index functions the device code is built from -- against bases of the given byte sizes, and
 * checks that no access leaves its base or is clipped by a box's buffer descriptor, that every
 * destination byte the boxes name is written exactly once, and that it receives the source byte
 * the boxes name.  Needs no device; walks byte by byte (bases up to 2 GiB).  No counterpart in
 * the reference (its coverage check is on the plan, core/processgroup.cc:3079-3081).
 */
typedef struct mdh_copy_plan mdh_copy_plan;
int mdh_copy_plan_create(const mdh_box* boxes, const int32_t* src_slots, const int32_t* dst_slots, int nboxes,
    int itemsize, int nbases, mdh_copy_plan** plan);
int mdh_copy_plan_launch(const mdh_copy_plan* plan, const void* const* bases, int nbases, void* stream);
int mdh_copy_plan_launches(const mdh_copy_plan* plan);
int mdh_copy_plan_verify(const mdh_copy_plan* plan, const uint64_t* base_bytes, int nbases);
/*
 * Introspection, no reference counterpart: the kernel-argument block and the launch shape
 * that launch number `step` (0 .. mdh_copy_plan_launches-1) passes for these 16-byte aligned
 * bases.  `*size` receives the block's size; `out` may be NULL to ask for the size only.  The
 * block begins with `*leading_scalars` 4-byte scalars, each a kernel parameter of its own
 * (0 for most launches, 14 for one started from preloaded arguments); the rest is one struct
 * parameter.  Enqueues nothing.  For host-side checks of a launch's argument block (for one, against
 * the kernel node a stream capture recorded, read back and never replayed).
 */
int mdh_copy_plan_step_arguments(const mdh_copy_plan* plan, const void* const* bases, int nbases, int step, void* out,
    size_t capacity, size_t* size, uint32_t* leading_scalars, uint32_t* grid_x, uint32_t* grid_y, uint32_t* block,
    uint32_t* lds);
void mdh_copy_plan_destroy(mdh_copy_plan* plan);

/*
 * Set-up call of the library's fixed workspace, no reference counterpart: a device array of
 * MDH_STATIC_WORKSPACE_BYTES that belongs to the library (every GPU the library runs on
 * holds one from the moment the library's code is loaded there until the process ends).
 * Returns the array's address on the CURRENT device and its size; the first call on a
 * device looks the address up (hipGetSymbolAddress), later calls return the kept value.
 * Allocates nothing.  The memory keeps whatever its last user left in it, and all users on
 * one GPU share it: moodist_pg_allreduce_static (moodist_core.h) is the one user.
 */
#define MDH_STATIC_WORKSPACE_BYTES (64u << 20)
int mdh_static_workspace(void** address, size_t* bytes);

/*
 * Launch-shape knobs, for measurement; 0 (the default) lets the library choose
 * by size.  Names: "reduce_unroll" (KiB of every source per tile: 1, 2, 4, 8, 16),
 * "reduce_chunk" (sources whose loads are in flight together: 1, 2, 4, 8; the pairs
 * compiled are 16x1, 16x2, 8x2, 4x4, 2x8, 1x8 and a call that forces another pair fails),
 * "reduce_max_blocks" (waves of the grid; 0 = chosen by size), "reduce_split_tiles" (tiles
 * of one launch at most: longer reductions are cut into several launches; 0 = 4096),
 * "reduce_wg_per_cu" (2..8
 * caps the workgroups resident on a CU, 9 = never cap), "copy_unroll" (1, 2,
 * 4, 8; contiguous segments), "box_unroll" (1, 2, 4, 8; strided boxes),
 * "copy_max_blocks", "copy_wg_per_cu" (2..8, 9 = never cap), "box_policy" (loads of the
 * strided-box kernel: 1 = plain, which pays when the sources are still in the Infinity Cache;
 * 0 or 2 = nt, the default), "box_preload" (1 = never start equal boxes of full tiles from
 * preloaded kernel arguments), "box_transpose" (1 = boxes that transpose take the plain strided
 * kernel instead of LDS-staged tiles; 2 = tiles, always dealt row by row; 3 = always along the
 * diagonals; by default the destination's pitch decides), "box_transpose_wgs" (workgroups that walk the tiles of a transposing
 * launch, each taking every grid-th tile; 0 = one workgroup per tile), "box_transpose_tile" (0..3: the tile
 * of the transposing copy, T x T, T x 2T, 2T x T or 2T x 2T elements, for measurement), "box_tile_cols" (a power of two: the columns, in 16-byte vectors, of
 * a strided-box tile; its rows follow from the tile's 256 x box_unroll slots), four variants of the dense copy of up to eight equal segments that
 * exist for measurement and that the library never chooses by itself -- "copy_xcd_run" (2, 4, 8, ...:
 * each of the eight XCDs takes runs of that many consecutive tiles, where by default adjacent tiles
 * go to different XCDs), "copy_grid_order" (1: the segments advance together instead of one after
 * the other), "copy_tail_tiles" (that many tiles at every segment's end are dealt as two halves
 * each, so the launch ends on short workgroups), "copy_lds" (1: loads go straight to LDS and the
 * stores are fed from there) --, "allow_capture" (1 = the launch functions accept a capturing
 * stream; only for a host-side comparison of what a capture records with what an eager launch
 * passes, by a program that destroys the graph without instantiating it).  Returns MDH_EINVAL
 * for an unknown name or value.
 * No counterpart in the reference, whose grid is fixed at 4/16/64 blocks
 * (core/kernels.cc:547-556).
 */
int mdh_set_tuning(const char* name, int value);
int mdh_get_tuning(const char* name, int* value);

#ifdef __cplusplus
}
#endif
#endif /* MOODIST_HIP_H */
