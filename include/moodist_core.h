/*
 * moodist_core.h -- C ABI of the host core (libmoodist.so): the process-group
 * operator surface for the single-GPU hot path, with the local peers of a
 * group emulated inside one process.
 *
 * The reference exposes this surface as a table of C++ function pointers
 * obtained through its one extern "C" symbol, moodistGetApi
 * (api/moodist_api.h:134-271, core/moodist_api.cc:168-179); the functions
 * below are the members of that table that belong to the path, by the same
 * names and argument order (api/processgroup_api.h:29-65,
 * api/moodist_api.h:197-216, :244-255), with
 *   - TensorPtr (an opaque torch tensor reached through callbacks,
 *     api/tensor_ptr.h:73-315) replaced by the plain moodist_tensor below,
 *   - CUstream replaced by a hipStream_t passed as void*,
 *   - C++ exceptions replaced by a return code (0 = success) plus
 *     moodist_last_error() for the calling thread; messages are the
 *     reference's where it has one.
 *
 * Peers.  The reference runs one process per rank and obtains its peers'
 * buffer addresses through shared memory and CUDA IPC
 * (core/processgroup.cc:1150-1169, :1448-1470).  Here a moodist_world stands
 * for the node: it owns `size` process groups (ranks 0..size-1) on one
 * device.  A collective call posts the caller's addresses; when every rank of
 * the world has posted the same collective, the kernels of all ranks that
 * asked for an output are launched, each on the stream its rank passed.  A
 * rank that only contributes (its buffer is a staged peer contribution) posts
 * with moodist_pg_stage_input().  The returned work is complete once that
 * launch has happened; as in the reference (wrapper/processgroup_wrapper.cc:63-85)
 * ordering with later work is by stream, not by the host.
 *
 * Nothing here synchronises the host with the device.
 *
 * Every rank numbers its collectives; call k of one rank meets call k of the others, and calls
 * that differ (operation, size, element type, reduction) are an error for the rank that arrives
 * with the difference -- the reference aborts there (core/cputhread.h:100-112).  A call that
 * is refused, for this or for its arguments, has posted nothing and leaves the rank's numbering
 * where it was.
 *
 * A stream that is being captured into a graph (hipStreamBeginCapture) is refused by every
 * collective, with an error and nothing recorded: replaying a graph that holds this library's
 * launches is not supported.
 */
#ifndef MOODIST_CORE_H
#define MOODIST_CORE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* api/moodist_version.h:12 (kMoodistApiVersion) */
#define MOODIST_CORE_API_VERSION 2

/* The number this library's build drew (build_host.sh), the same one its API table carries in
 * `magic` (api/moodist_api.h:265-271): readable before the table is asked for.  No counterpart
 * in the reference, where only the table holds it. */
uint64_t moodist_build_magic(void);

typedef struct moodist_tensor {
  void* data;         /* device pointer */
  int64_t numel;
  int32_t itemsize;
  int32_t dtype;      /* torch ScalarType number (api/moodist_api.h:30-42) */
  int32_t device;     /* device index, -1 for host memory */
  int32_t contiguous; /* non-zero if dense row-major */
  int32_t ndim;
  int32_t reserved;
  int64_t shape[10];
} moodist_tensor;

typedef struct moodist_world moodist_world;
typedef struct moodist_pg moodist_pg;
typedef struct moodist_work moodist_work;
typedef struct moodist_op moodist_op;
typedef struct moodist_future moodist_future;

/* moodistGetApi's handshake (api/moodist_api.h:265-271): returns 0 unless
 * expected_version == MOODIST_CORE_API_VERSION. */
int moodist_core_check_version(uint32_t expected_version);
const char* moodist_last_error(void);

/* createProcessGroup (api/processgroup_api.h:21) for every local rank at once. */
int moodist_world_create(int size, int device, moodist_world** world);
void moodist_world_destroy(moodist_world* world);
/* Borrowed pointer, valid until the world is destroyed. */
moodist_pg* moodist_world_group(moodist_world* world, int rank);

/* processGroupRank / processGroupSize (api/processgroup_api.h:30-31) */
int moodist_pg_rank(moodist_pg* pg);
int moodist_pg_size(moodist_pg* pg);
/* processGroupGetOption / processGroupSetOption (api/processgroup_api.h:39-40).
 * Names as in the reference (core/processgroup.cc:2455-2488): prefer_kernel_less,
 * force_kernel_less, num_chunks, chunk_size, method; and, not in the reference,
 * snapshot_inputs (needs a core loaded through moodistGetApi) and the read-only counters
 * kernel_less_copies_1d / kernel_less_copies_2d (copy-engine calls the world's kernel-less
 * all_gathers have made).  Unknown name -> error. */
int moodist_pg_get_option(moodist_pg* pg, const char* name, int64_t* value);
int moodist_pg_set_option(moodist_pg* pg, const char* name, int64_t value);

/* processGroupAllGather (api/processgroup_api.h:43; core/processgroup.cc:1059-1284) */
int moodist_pg_all_gather(moodist_pg* pg, const moodist_tensor* output, const moodist_tensor* input, void* stream,
    moodist_work** work);
/* c10d's list form, allgather(output_lists, inputs) (wrapper/processgroup_wrapper.cc:112-129):
 * outputs[j] receives rank j's input.  The reference gathers into a flat temporary and copies
 * each row out; here the sources are copied straight into the outputs.  Outputs must be
 * dense, of the input's dtype and size; n_outputs must equal the group size. */
int moodist_pg_all_gather_list(moodist_pg* pg, const moodist_tensor* outputs, size_t n_outputs,
    const moodist_tensor* input, void* stream, moodist_work** work);
/* c10d's allgather_into_tensor_coalesced (wrapper/processgroup_wrapper.cc:139-148), which the
 * reference serves with one all_gather per tensor: here the n tensors are ONE collective --
 * outputs[t] (group size times inputs[t]'s bytes) receives every rank's inputs[t] -- and its
 * copies go out in as few launches as the segment table of the copy kernel allows.  Every
 * rank must bring lists of the same length and sizes.  `outputs` may be NULL for a rank that
 * only contributes. */
int moodist_pg_all_gather_many(moodist_pg* pg, const moodist_tensor* outputs, const moodist_tensor* inputs, size_t n,
    void* stream, moodist_work** work);
/* processGroupReduceScatter (api/processgroup_api.h:45-46; core/processgroup.cc:1290-1668).
 * reduce_op is a c10d RedOpType number; premul_value is used by PREMUL_SUM only. */
int moodist_pg_reduce_scatter(moodist_pg* pg, const moodist_tensor* output, const moodist_tensor* input,
    int reduce_op, void* stream, float premul_value, moodist_work** work);
/* c10d's reduce_scatter_tensor_coalesced, which the reference serves with one reduce_scatter per
 * tensor (wrapper/processgroup_wrapper.cc:159-170), as ONE collective: outputs[t] receives this
 * rank's chunk of every rank's inputs[t], reduced; a rank's reductions share kernel launches
 * (mdh_reduce_many).  All tensors must have one element type; every rank must bring lists of the
 * same length and sizes.  `outputs` may be NULL for a rank that only contributes.  The whole
 * list is checked before anything is posted. */
int moodist_pg_reduce_scatter_many(moodist_pg* pg, const moodist_tensor* outputs, const moodist_tensor* inputs, size_t n,
    int reduce_op, void* stream, float premul_value, moodist_work** work);
/* processGroupAllreduce (api/processgroup_api.h:48-49; core/processgroup.cc:1674-1722): a
 * reduce-scatter into the rank's own chunk followed by an all-gather, in place.  When numel
 * is not a multiple of the group size the reference allocates a padded temporary through
 * torch (:1694-1697); here the caller passes it as `scratch` (>= roundup(numel, size)
 * elements, same dtype), or NULL when numel divides evenly.
 * The call is ONE collective (one sequence number; every rank must call allreduce).  Ranks that
 * passed the same stream get one kernel launch for all of them, which reduces every chunk in
 * its owner's fold order and stores it into every rank's tensor (mdh_allreduce_many); ranks on
 * different streams, the chunk options, the copy-engine gather and snapshot_inputs get the
 * reduce_scatter and the all_gather, rank by rank.  The results are the same bit for bit. */
int moodist_pg_allreduce(moodist_pg* pg, const moodist_tensor* tensor, const moodist_tensor* scratch, int reduce_op,
    void* stream, float premul_value, moodist_work** work);
/* c10d's allreduce_coalesced (wrapper/processgroup_wrapper.cc:182-191), which the reference serves
 * with one allreduce per tensor, for tensors of one element type whose element counts the group
 * size divides (the others go through moodist_pg_allreduce one by one): ONE collective, served
 * like moodist_pg_allreduce -- by shared launches that reduce every chunk of every tensor and
 * store it into every rank's tensor when the ranks passed the same stream, else by the
 * reduce_scatter of the list into the rank's own chunks and the all_gather of every tensor's
 * chunks.  A list that is refused (mixed element types, an operation the type does not support)
 * leaves nothing posted. */
int moodist_pg_allreduce_many(moodist_pg* pg, const moodist_tensor* tensors, size_t n, int reduce_op, void* stream,
    float premul_value, moodist_work** work);
/* No counterpart in the reference.  moodist_pg_allreduce for callers that cannot allocate
 * device memory and have no temporary to pass (tight serving loops, harnesses that forbid
 * hipMalloc): the padded temporary is this rank's slice of the
 * kernel library's fixed workspace (mdh_static_workspace in moodist_hip.h, 64 MiB per GPU,
 * split evenly over the group's ranks and rounded down to 256 bytes).  Allocates and frees no
 * device memory.  Same results as moodist_pg_allreduce.  Limits:
 *  - roundup(numel, size) * itemsize must fit the rank's slice (8 MiB for 8 ranks), else error;
 *  - a rank's next call is refused while its previous one still waits for other ranks;
 *  - all calls on one GPU share the workspace: a rank's calls must be ordered on the GPU (one
 *    stream, or the caller's own events), and two worlds on one GPU must not use it at the
 *    same time -- calls that overlap race;
 *  - the padding elements hold what the last call left there; they are reduced and thrown
 *    away, nothing needs to start at zero.
 * When numel is a multiple of the group size no temporary is used at all.  The first call on
 * a device looks the workspace's address up (and may load the kernel library's code there).
 * The group option snapshot_inputs, which copies a posted input into memory from an allocator,
 * is not applied to this call: the tensor is read when the collective launches.
 * Like every collective here it refuses a stream that is being captured into a graph. */
int moodist_pg_allreduce_static(moodist_pg* pg, const moodist_tensor* tensor, int reduce_op, void* stream,
    float premul_value, moodist_work** work);
/* No counterpart in the reference, where a peer's contribution is whatever that peer's own
 * collective call passes: posts this rank's input for the next collective without asking
 * for an output.  kind: 0 = all_gather, 1 = reduce_scatter. */
int moodist_pg_stage_input(moodist_pg* pg, int kind, const moodist_tensor* input, int reduce_op, void* stream,
    float premul_value, moodist_work** work);

/* The work of the collective this rank posted most recently (a new reference; NULL into *work
 * if it has posted none).  For callers of the CoreApi table, whose collectives return nothing
 * (api/processgroup_api.h:43-49) -- there a call has done its part when it returns, here the
 * launch may still be waiting for other ranks.  No counterpart in the reference. */
int moodist_pg_last_work(moodist_pg* pg, moodist_work** work);

/* Ties `ctx` to the collective this rank posted most recently: release(ctx) is called exactly
 * once, when that collective's launches have been enqueued (at once if they already have, or
 * if the rank has posted nothing).  For the buffers of the calls above, which the core reads
 * when the LAST rank posts: the caller keeps them alive at least that long.  The reference
 * holds tensor references inside the operation instead (core/processgroup.cc:3239-3245), as
 * the CoreApi table of moodist_plugin.h does here. */
int moodist_pg_keep_alive(moodist_pg* pg, void* ctx, void (*release)(void* ctx));

/* Work: wait() fails if not every rank has posted yet (the launch has not happened). */
int moodist_work_is_completed(moodist_work* work);
int moodist_work_wait(moodist_work* work);
void moodist_work_destroy(moodist_work* work);

/* compileOpFull (api/moodist_api.h:244-248; core/processgroup.cc:2761-3104, :3259-3290):
 * every rank passes the same full lists; offsets and shapes are ndim ints per slice. */
int moodist_compile_op_full(moodist_pg* pg, const int* shape, size_t ndim, int dtype, const int* input_ranks,
    const int* input_offsets, const int* input_shapes, size_t n_inputs, const int* output_ranks,
    const int* output_offsets, const int* output_shapes, size_t n_outputs, moodist_op** op);
void moodist_op_destroy(moodist_op* op);
/* customOpCall (api/moodist_api.h:250-252; core/processgroup.cc:3172-3256) */
int moodist_op_call(moodist_op* op, const moodist_tensor* inputs, size_t n_inputs, const moodist_tensor* outputs,
    size_t n_outputs, void* stream, moodist_future** future);
/* futureWait (api/moodist_api.h:253-255; core/processgroup.cc:2650-2661) */
int moodist_future_wait(moodist_future* future, void* stream);
void moodist_future_destroy(moodist_future* future);

/* How the kernel-less all_gather would group `n` source buffers of `bytes` bytes each into
 * copy-engine calls: ranks whose buffers are evenly spaced form one run, as the reference
 * groups the sources a peer holds into Copy2d{offset, length, pitch, num}
 * (core/processgroup.cc:114-119, :618-704).  Writes first, count, src_pitch per run into out
 * (3 values each, as far as capacity allows) and returns the number of runs.  A rank whose
 * source is dst + rank*bytes is in place and belongs to no run (dst may be NULL). */
int64_t moodist_kernel_less_runs(const void* const* srcs, size_t n, size_t bytes, const void* dst, int64_t* out,
    size_t capacity);

/* The plan of the calling rank, as the reference's CustomOpDescriptor holds it
 * (core/cputhread.h:296-322), for inspection.  what: 0 reads, 1 inputCopies, 2 outputCopies,
 * 3 inputs, 4 outputs.  moodist_op_plan_count returns the number of entries. */
int64_t moodist_op_plan_count(moodist_op* op, int what);
/* reads: out[6] = rank, inputIndex, outputIndex, inputOffset, outputOffset, bytes. */
int moodist_op_plan_read(moodist_op* op, size_t i, int64_t out[6]);
/* copies: index, then ndim offsets, then ndim shapes into out (1 + 2*ndim values). */
int moodist_op_plan_copy(moodist_op* op, int which, size_t i, int64_t* out, size_t out_len);
/* inputs / outputs: byte size of entry i. */
int64_t moodist_op_plan_size(moodist_op* op, int which, size_t i);
/* The serialized list this rank would put on `receiver`'s queue during compile
 * (core/processgroup.cc:3022-3033): a 64-bit count, then per piece, packed, little-endian:
 *   u8 contiguous (always 0); i32 offset[ndim]; i32 shape[ndim]; u32 inputRank, outputRank,
 *   inputIndex, outputIndex; u64 inputOffset, outputOffset (elements); u8 outputContiguous
 * (TInput, :2735-2753, written by core/serialization.h's raw-byte serializer).  Returns the
 * length; copies the bytes when buffer is non-NULL and capacity suffices; -1 on a bad argument. */
int64_t moodist_op_plan_message(moodist_op* op, int receiver, void* buffer, size_t capacity);
/* Parses such a list for `ndim` dimensions: 0, or an error with the reference deserializer's
 * message ("Deserializer: reached end of data", "deserializeBuffer: N trailing bytes"). */
int moodist_plan_message_check(const void* bytes, size_t length, size_t ndim);

#ifdef __cplusplus
}
#endif
#endif /* MOODIST_CORE_H */
