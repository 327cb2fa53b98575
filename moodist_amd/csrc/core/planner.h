// compile_op planner: integer box geometry that turns "every rank holds these
// slices, every rank wants those slices" into per-rank lists of reads and
// staging copies, and into the fused strided transfers the GPU path executes.
//
// Behaviour follows the reference's compileOpFullImpl
// (core/processgroup.cc:2761-3104) and its descriptor (core/cputhread.h:296-322).
// The reference runs one planner per rank process and exchanges the
// per-destination lists through queues as serialized bytes (:3005-3077); here
// all ranks live in one process, so one call plans every rank, but the lists
// still pass through the reference's byte format between the sender half and
// the receiver half.
#pragma once

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <vector>

namespace moodist {

using Dims = std::vector<int64_t>;

struct SliceSpec { // one input or output slice in global coordinates
  int rank;
  Dims offset;
  Dims shape;
};

// core/cputhread.h:298-305
struct PlanRead {
  uint32_t rank;
  uint32_t inputIndex;
  uint32_t outputIndex;
  size_t inputOffset; // bytes
  size_t outputOffset;
  size_t bytes;
};

// core/cputhread.h:306-310: an {offset, shape} box inside tensor `index`
// <-> a contiguous staging tensor
struct PlanCopy {
  uint32_t index;
  Dims offset;
  Dims shape;
};

// One read with its staging copies folded in: the box `shape` found at
// `srcOffset` inside source tensor (srcRank, srcInput) lands at `dstOffset`
// inside destination tensor dstOutput of the planning rank.  Both tensors are
// contiguous with the given shapes.
struct Transfer {
  uint32_t srcRank;
  uint32_t srcInput;
  uint32_t dstOutput;
  Dims shape;
  Dims srcOffset, srcShape;
  Dims dstOffset, dstShape;
};

struct RankPlan {
  std::vector<PlanRead> reads;
  std::vector<PlanCopy> inputCopies;
  std::vector<PlanCopy> outputCopies;
  std::vector<size_t> inputs; // byte sizes the rank must pass, in this order
  std::vector<size_t> outputs;
  std::vector<Dims> inputShapes;
  std::vector<Dims> outputShapes;
  std::vector<Transfer> transfers;
};

// wire[sender][receiver]: the serialized list the sender puts on the receiver's queue
// (core/processgroup.cc:3022-3033, format of core/serialization.h).
using PlanWire = std::vector<std::vector<std::vector<uint8_t>>>;

// Throws std::runtime_error("moodist.compile_op_full: could not find input for
// all output elements") when some output element has no source
// (core/processgroup.cc:3079-3081).
std::vector<RankPlan> plan_redistribution(int size, const Dims& shape, size_t itemsize,
    const std::vector<SliceSpec>& inputs, const std::vector<SliceSpec>& outputs, PlanWire* wire = nullptr);

// Parses a serialized list for `ndim` dimensions; throws the reference's deserializer errors
// on a short buffer or trailing bytes.
void check_plan_message(const std::vector<uint8_t>& bytes, size_t ndim);

size_t dims_numel(const Dims& d);
size_t linear_offset(const Dims& offset, const Dims& shape);

} // namespace moodist
