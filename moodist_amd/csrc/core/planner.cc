#include "planner.h"

#include <algorithm>
#include <cstring>
#include <string>

namespace moodist {

size_t dims_numel(const Dims& d) {
  size_t n = 1;
  for (int64_t x : d) {
    n *= (size_t)x;
  }
  return n;
}

// row-major element offset of `offset` inside a tensor of `shape` (core/processgroup.cc:2788-2796)
size_t linear_offset(const Dims& offset, const Dims& shape) {
  size_t result = 0, stride = 1;
  for (size_t i = shape.size(); i-- > 0;) {
    result += (size_t)offset[i] * stride;
    stride *= (size_t)shape[i];
  }
  return result;
}

namespace {

struct Slice {
  uint32_t rank;
  uint32_t index; // position among the rank's slices as the caller listed them
  Dims offset, shape;
  size_t numel;
};

struct Hit { // intersection of a destination with entry `index` of some list
  Dims offset, shape;
  size_t index;
};

bool overlaps(const Dims& ao, const Dims& as, const Dims& bo, const Dims& bs) {
  for (size_t i = 0; i < ao.size(); ++i) {
    if (ao[i] >= bo[i] + bs[i] || bo[i] >= ao[i] + as[i]) {
      return false;
    }
  }
  return true;
}

bool inside(const Dims& ao, const Dims& as, const Dims& bo, const Dims& bs) {
  for (size_t i = 0; i < ao.size(); ++i) {
    if (ao[i] < bo[i] || ao[i] + as[i] > bo[i] + bs[i]) {
      return false;
    }
  }
  return true;
}

// a slab that spans every dimension but the first is one contiguous range (:2863-2870)
bool whole_rows(const Dims& part, const Dims& whole) {
  for (size_t i = 1; i < part.size(); ++i) {
    if (part[i] != whole[i]) {
      return false;
    }
  }
  return true;
}

Dims minus(const Dims& a, const Dims& b) {
  Dims r(a.size());
  for (size_t i = 0; i < a.size(); ++i) {
    r[i] = a[i] - b[i];
  }
  return r;
}

template<typename List, typename Get>
std::vector<Hit> intersect(const Dims& doff, const Dims& dshape, const List& list, Get get) {
  std::vector<Hit> hits;
  for (size_t i = 0; i < list.size(); ++i) {
    const auto& [so, ss] = get(list[i]);
    if (!overlaps(so, ss, doff, dshape)) {
      continue;
    }
    Hit h;
    h.index = i;
    h.offset.resize(doff.size());
    h.shape.resize(doff.size());
    for (size_t j = 0; j < doff.size(); ++j) {
      const int64_t lo = std::max(so[j], doff[j]);
      const int64_t hi = std::min(so[j] + ss[j], doff[j] + dshape[j]);
      h.offset[j] = lo;
      h.shape[j] = hi - lo;
    }
    hits.push_back(std::move(h));
  }
  return hits;
}

struct Message { // what a sender tells a receiver about one piece (TInput, :2735-2753)
  Dims offset, shape;
  uint32_t inputRank, outputRank, inputIndex, outputIndex;
  size_t inputOffset, outputOffset; // elements
  bool outputContiguous;
};

// The bytes a sender puts on a receiver's queue (core/processgroup.cc:3022-3033).  The
// reference's serializer writes a vector as its 64-bit length followed by the elements, and
// every trivially copyable member as its raw bytes with no padding (core/serialization.h:148-154,
// :263-267); TInput lists its members as contiguous, offset, shape, inputRank, outputRank,
// inputIndex, outputIndex, inputOffset, outputOffset, outputContiguous (:2748-2751), offset and
// shape being std::array<int, ndim>.  `contiguous` is never set and travels as 0.  One record
// is 34 + 8*ndim bytes; the number of dimensions is not on the wire.
template<typename T>
void put(std::vector<uint8_t>& out, T v) {
  const uint8_t* p = reinterpret_cast<const uint8_t*>(&v);
  out.insert(out.end(), p, p + sizeof(T));
}

std::vector<uint8_t> encode(const std::vector<Message>& list, size_t ndim) {
  std::vector<uint8_t> out;
  out.reserve(8 + list.size() * (34 + 8 * ndim));
  put<uint64_t>(out, list.size());
  for (const Message& m : list) {
    put<uint8_t>(out, 0);
    for (int64_t v : m.offset) {
      put<int32_t>(out, (int32_t)v);
    }
    for (int64_t v : m.shape) {
      put<int32_t>(out, (int32_t)v);
    }
    put<uint32_t>(out, m.inputRank);
    put<uint32_t>(out, m.outputRank);
    put<uint32_t>(out, m.inputIndex);
    put<uint32_t>(out, m.outputIndex);
    put<uint64_t>(out, m.inputOffset);
    put<uint64_t>(out, m.outputOffset);
    put<uint8_t>(out, m.outputContiguous ? 1 : 0);
  }
  return out;
}

struct Reader {
  const uint8_t* p;
  size_t left;
  template<typename T>
  T get() {
    if (left < sizeof(T)) {
      throw std::runtime_error("Deserializer: reached end of data"); // core/serialization.h:287
    }
    T v;
    std::memcpy(&v, p, sizeof(T));
    p += sizeof(T);
    left -= sizeof(T);
    return v;
  }
};

std::vector<Message> decode(const std::vector<uint8_t>& bytes, size_t ndim) {
  Reader r{bytes.data(), bytes.size()};
  const uint64_t n = r.get<uint64_t>();
  if (n > r.left / (34 + 8 * ndim)) {
    throw std::runtime_error("Deserializer: reached end of data");
  }
  std::vector<Message> list((size_t)n);
  for (Message& m : list) {
    (void)r.get<uint8_t>();
    m.offset.resize(ndim);
    m.shape.resize(ndim);
    for (int64_t& v : m.offset) {
      v = r.get<int32_t>();
    }
    for (int64_t& v : m.shape) {
      v = r.get<int32_t>();
    }
    m.inputRank = r.get<uint32_t>();
    m.outputRank = r.get<uint32_t>();
    m.inputIndex = r.get<uint32_t>();
    m.outputIndex = r.get<uint32_t>();
    m.inputOffset = (size_t)r.get<uint64_t>();
    m.outputOffset = (size_t)r.get<uint64_t>();
    m.outputContiguous = r.get<uint8_t>() != 0;
  }
  if (r.left != 0) { // core/serialization.h:677-679
    throw std::runtime_error("deserializeBuffer: " + std::to_string(r.left) + " trailing bytes");
  }
  return list;
}

std::vector<Slice> number_slices(const std::vector<SliceSpec>& specs, int size, size_t ndim, const char* what) {
  std::vector<uint32_t> counter((size_t)size, 0);
  std::vector<Slice> out;
  out.reserve(specs.size());
  for (const SliceSpec& s : specs) {
    if (s.rank < 0 || s.rank >= size) {
      throw std::runtime_error(std::string("moodist.compile_op_full: ") + what + " names rank " +
                               std::to_string(s.rank) + " outside the group");
    }
    if (s.offset.size() != ndim || s.shape.size() != ndim) {
      throw std::runtime_error(std::string("moodist.compile_op_full: ") + what +
                               " offset/shape do not have the tensor's number of dimensions");
    }
    for (size_t i = 0; i < ndim; ++i) {
      if (s.offset[i] < 0 || s.shape[i] < 0) {
        throw std::runtime_error(std::string("moodist.compile_op_full: ") + what + " has a negative offset or shape");
      }
      if (s.offset[i] > INT32_MAX || s.shape[i] > INT32_MAX) { // `int` in the reference and on the wire
        throw std::runtime_error(std::string("moodist.compile_op_full: ") + what +
                                 " has an offset or shape that does not fit a 32-bit int");
      }
    }
    Slice d;
    d.rank = (uint32_t)s.rank;
    d.index = counter[(size_t)s.rank]++;
    d.offset = s.offset;
    d.shape = s.shape;
    d.numel = dims_numel(s.shape);
    out.push_back(std::move(d));
  }
  return out;
}

} // namespace

std::vector<RankPlan> plan_redistribution(int size, const Dims& shape, size_t itemsize,
    const std::vector<SliceSpec>& inputs_arg, const std::vector<SliceSpec>& outputs_arg, PlanWire* wire_out) {
  const size_t ndim = shape.size();
  for (int64_t v : shape) {
    if (v < 0 || v > INT32_MAX) { // dimensions are `int` in the reference and on the wire
      throw std::runtime_error("moodist.compile_op_full: a dimension does not fit a 32-bit int");
    }
  }
  std::vector<Slice> inputs = number_slices(inputs_arg, size, ndim, "an input");
  std::vector<Slice> outputs = number_slices(outputs_arg, size, ndim, "an output");

  // a rank's outputs as the caller listed them
  std::vector<std::vector<Slice>> outputsOf((size_t)size);
  for (const Slice& o : outputs) {
    outputsOf[o.rank].push_back(o);
  }

  // largest first, ties in listing order (:2848-2849)
  auto bigger = [](const Slice& a, const Slice& b) { return a.numel > b.numel; };
  std::stable_sort(inputs.begin(), inputs.end(), bigger);
  std::stable_sort(outputs.begin(), outputs.end(), bigger);

  std::vector<RankPlan> plans((size_t)size);
  std::vector<std::vector<std::vector<Message>>> mail((size_t)size,
      std::vector<std::vector<Message>>((size_t)size)); // mail[receiver][sender]

  auto slice_box = [](const Slice* s) { return std::pair<const Dims&, const Dims&>(s->offset, s->shape); };
  auto hit_box = [](const Hit& h) { return std::pair<const Dims&, const Dims&>(h.offset, h.shape); };

  for (int rank = 0; rank < size; ++rank) {
    std::vector<const Slice*> mine;
    for (const Slice& s : inputs) {
      if ((int)s.rank == rank) {
        mine.push_back(&s);
      }
    }
    std::vector<Hit> staged; // pieces this rank must copy out of a tensor into contiguous staging
    RankPlan& plan = plans[(size_t)rank];

    for (const Slice& dst : outputs) {
      if (dst.numel == 0) {
        continue;
      }
      for (const Hit& x : intersect(dst.offset, dst.shape, mine, slice_box)) {
        const Slice& src = *mine[x.index];
        const bool inputContiguous = whole_rows(x.shape, src.shape);
        if (!inputContiguous) {
          // Does staging made for an earlier destination already hold these elements as
          // at most three contiguous ranges? (:2931-2962)
          std::vector<Hit> again = intersect(dst.offset, dst.shape, staged, hit_box);
          if (!again.empty() && again.size() < 4) {
            size_t n = 0;
            bool rows = true;
            for (const Hit& y : again) {
              n += dims_numel(y.shape);
              rows = rows && whole_rows(y.shape, staged[y.index].shape);
              if (!rows) {
                break;
              }
            }
            // The reference accepts the staged pieces when their element counts add up to the
            // piece wanted (:2945-2946).  Staging can hold the same elements twice, and pieces of
            // another tensor of this rank, so equal counts do not mean the piece is covered: the
            // reference then reads one element twice and leaves another unwritten.  Here the
            // pieces must also lie inside the piece wanted and not overlap each other.
            for (size_t p = 0; rows && p < again.size(); ++p) {
              rows = inside(again[p].offset, again[p].shape, x.offset, x.shape);
              for (size_t q = 0; rows && q < p; ++q) {
                rows = !overlaps(again[p].offset, again[p].shape, again[q].offset, again[q].shape);
              }
            }
            if (rows && n == dims_numel(x.shape)) {
              for (const Hit& y : again) {
                const Hit& st = staged[y.index];
                Message m;
                m.offset = y.offset;
                m.shape = y.shape;
                m.inputRank = (uint32_t)rank;
                m.outputRank = dst.rank;
                m.inputIndex = (uint32_t)(mine.size() + y.index);
                m.outputIndex = dst.index;
                m.inputOffset = linear_offset(minus(y.offset, st.offset), st.shape);
                m.outputOffset = linear_offset(minus(y.offset, dst.offset), dst.shape);
                m.outputContiguous = whole_rows(y.shape, dst.shape);
                mail[dst.rank][(size_t)rank].push_back(std::move(m));
              }
              continue;
            }
          }
        }
        Message m;
        m.offset = x.offset;
        m.shape = x.shape;
        m.inputRank = (uint32_t)rank;
        m.outputRank = dst.rank;
        m.inputIndex = (uint32_t)x.index;
        m.outputIndex = dst.index;
        m.inputOffset = linear_offset(minus(x.offset, src.offset), src.shape);
        m.outputOffset = linear_offset(minus(x.offset, dst.offset), dst.shape);
        if (!inputContiguous) {
          m.inputIndex = (uint32_t)(mine.size() + staged.size());
          m.inputOffset = 0;
          staged.push_back(x);
        }
        m.outputContiguous = whole_rows(x.shape, dst.shape);
        mail[dst.rank][(size_t)rank].push_back(std::move(m));
      }
    }

    for (const Slice* s : mine) {
      plan.inputs.push_back(itemsize * s->numel);
      plan.inputShapes.push_back(s->shape);
    }
    for (const Slice& o : outputs) {
      if ((int)o.rank == rank) {
        plan.outputs.push_back(itemsize * o.numel);
        plan.outputShapes.push_back(o.shape);
      }
    }
    for (const Hit& h : staged) {
      PlanCopy c;
      c.index = (uint32_t)h.index;
      c.offset = minus(h.offset, mine[h.index]->offset);
      c.shape = h.shape;
      plan.inputCopies.push_back(std::move(c));
    }
  }

  // sorted positions of every rank's inputs, to resolve a transfer's source tensor
  std::vector<std::vector<const Slice*>> inputsOf((size_t)size);
  for (const Slice& s : inputs) {
    inputsOf[s.rank].push_back(&s);
  }

  // What travels: one byte string per (sender, receiver).  The receivers below work from the
  // decoded bytes, as a receiver in another process would.
  PlanWire wire((size_t)size, std::vector<std::vector<uint8_t>>((size_t)size));
  for (int receiver = 0; receiver < size; ++receiver) {
    for (int sender = 0; sender < size; ++sender) {
      wire[(size_t)sender][(size_t)receiver] = encode(mail[(size_t)receiver][(size_t)sender], ndim);
    }
  }
  mail.clear();

  for (int rank = 0; rank < size; ++rank) {
    RankPlan& plan = plans[(size_t)rank];
    size_t want = 0;
    for (const Slice& o : outputsOf[(size_t)rank]) {
      want += o.numel;
    }
    size_t have = 0;
    for (int sender = 0; sender < size; ++sender) {
      for (const Message& m : decode(wire[(size_t)sender][(size_t)rank], ndim)) {
        if (m.outputRank != (uint32_t)rank || m.inputRank != (uint32_t)sender ||
            m.outputIndex >= outputsOf[(size_t)rank].size()) { // :3052
          throw std::runtime_error("moodist.compile_op_full: a plan message does not belong to this rank");
        }
        const Slice& dst = outputsOf[(size_t)rank][m.outputIndex];
        PlanRead r;
        r.rank = m.inputRank;
        r.inputIndex = m.inputIndex;
        r.outputIndex = m.outputIndex;
        r.inputOffset = itemsize * m.inputOffset;
        r.outputOffset = itemsize * m.outputOffset;
        const size_t n = dims_numel(m.shape);
        r.bytes = itemsize * n;
        have += n;
        if (!m.outputContiguous) {
          PlanCopy c;
          c.index = r.outputIndex;
          c.offset = minus(m.offset, dst.offset);
          c.shape = m.shape;
          r.outputIndex = (uint32_t)(plan.outputs.size() + plan.outputCopies.size());
          r.outputOffset = 0;
          plan.outputCopies.push_back(std::move(c));
        }
        plan.reads.push_back(r);

        // An index past the sender's tensors names one of its staging copies; the fused
        // transfer reads the tensor that copy would have been taken from.
        const RankPlan& theirs = plans[m.inputRank];
        const size_t tensors = theirs.inputs.size();
        if (m.inputIndex >= tensors + theirs.inputCopies.size()) {
          throw std::runtime_error("moodist.compile_op_full: a plan message names an input the sender does not have");
        }
        const uint32_t origin =
            m.inputIndex < tensors ? m.inputIndex : theirs.inputCopies[m.inputIndex - tensors].index;
        const Slice& src = *inputsOf[m.inputRank][origin];
        Transfer t;
        t.srcRank = m.inputRank;
        t.srcInput = origin;
        t.dstOutput = m.outputIndex;
        t.shape = m.shape;
        t.srcOffset = minus(m.offset, src.offset);
        t.srcShape = src.shape;
        t.dstOffset = minus(m.offset, dst.offset);
        t.dstShape = dst.shape;
        plan.transfers.push_back(std::move(t));
      }
    }
    if (have != want) {
      throw std::runtime_error("moodist.compile_op_full: could not find input for all output elements");
    }
  }
  if (wire_out) {
    *wire_out = std::move(wire);
  }
  return plans;
}

void check_plan_message(const std::vector<uint8_t>& bytes, size_t ndim) {
  (void)decode(bytes, ndim);
}

} // namespace moodist
