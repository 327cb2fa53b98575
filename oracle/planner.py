"""TEST INFRASTRUCTURE -- not part of the product.

Restatement of the reference's compile_op planner and of what executing its
plan means, for every rank of a group at once (the reference runs one copy per
rank process and exchanges the per-destination lists through queues,
core/processgroup.cc:3005-3033; here the exchange is a Python list).

  plan()      follows compileOpFullImpl, core/processgroup.cc:2761-3104.
  execute()   follows the descriptor semantics: a Copy is an {offset, shape} box
              of tensor `index` <-> a contiguous staging tensor
              (core/cputhread.h:306-310); a Read moves `bytes` bytes from
              (rank, inputIndex, inputOffset) to (outputIndex, outputOffset)
              unchanged (core/cputhread.cc:5628-5672).
  shard_box() follows py/moodist/compile.py:21-59 (DTensor Shard placement ->
              offset/shape).
  wire()      the serialized per-destination lists the ranks exchange while compiling
              (TInput, core/processgroup.cc:2735-2753, through core/serialization.h).

Pinned by: the hand-derived plan for a 4x4 row->column reshard over 2 ranks,
the 1-D all-gather plan (reference tests/test_compile_op.py:191-222), numpy
slicing of the global tensor for every executed plan (identity
out[global idx] = in[global idx]), and the invariants sum(read bytes) ==
sum(output bytes) with no output byte written twice.  wire() is pinned by a byte string
written out by hand for the 4x4 example, by the record length 34 + 8*ndim and by
unpack(pack(x)) == x; no reference test holds serialized plans.

Pure-Python loops: small cases only.
"""

import struct
from dataclasses import dataclass, field
from typing import List

import numpy as np


@dataclass
class Read:
    rank: int
    inputIndex: int
    outputIndex: int
    inputOffset: int  # bytes
    outputOffset: int  # bytes
    bytes: int


@dataclass
class Copy:
    index: int
    offset: List[int]
    shape: List[int]


@dataclass
class Descriptor:
    reads: List[Read] = field(default_factory=list)
    inputCopies: List[Copy] = field(default_factory=list)
    outputCopies: List[Copy] = field(default_factory=list)
    inputs: List[int] = field(default_factory=list)  # byte sizes
    outputs: List[int] = field(default_factory=list)
    inputShapes: List[List[int]] = field(default_factory=list)
    outputShapes: List[List[int]] = field(default_factory=list)


class PlanError(RuntimeError):
    pass


def _numel(shape):
    n = 1
    for x in shape:
        n *= x
    return n


def _linear_offset(offset, shape):  # :2788-2796
    result, stride = 0, 1
    for i in range(len(shape) - 1, -1, -1):
        result += offset[i] * stride
        stride *= shape[i]
    return result


def _intersecting(a_off, a_shape, b_off, b_shape):  # :2851-2861
    for i in range(len(a_off)):
        if a_off[i] >= b_off[i] + b_shape[i]:
            return False
        if b_off[i] >= a_off[i] + a_shape[i]:
            return False
    return True


def _contiguous(a, b):  # :2863-2870 -- every dimension but the first is whole
    return all(a[i] == b[i] for i in range(1, len(a)))


def _sub(a, b):
    return [x - y for x, y in zip(a, b)]


def _find(dst, lst):  # :2878-2900; entries are dicts with offset/shape
    rv = []
    for index, src in enumerate(lst):
        if not _intersecting(src["offset"], src["shape"], dst["offset"], dst["shape"]):
            continue
        low = [max(s, d) for s, d in zip(src["offset"], dst["offset"])]
        high = [min(so + ss, do + ds) for so, ss, do, ds in
                zip(src["offset"], src["shape"], dst["offset"], dst["shape"])]
        rv.append({"offset": low, "shape": [h - l for h, l in zip(high, low)], "index": index})
    return rv


def _descrs(args, size):
    counter = [0] * size
    out = []
    for r, off, shp in args:
        out.append({"rank": r, "index": counter[r], "offset": list(off), "shape": list(shp),
                    "numel": _numel(shp)})
        counter[r] += 1
    return out, counter


def plan(size, shape, itemsize, inputs_arg, outputs_arg, strict_reuse=True):
    """inputs_arg/outputs_arg: lists of (rank, offset, shape) in global coordinates.

    Returns one Descriptor per rank.  Reads arrive sender by sender in rank
    order (the reference's arrival order is unspecified).

    strict_reuse=False is the reference to the letter: staged pieces found inside a
    destination are reused when their element counts add up to the piece wanted
    (core/processgroup.cc:2931-2962).  Staging can hold an element twice (and pieces of the
    rank's other tensors), so the counts can match while one element is read twice and another
    never: the plan then passes the coverage check (:3079-3081) and executes to a wrong
    result (tests/test_oracle_copy.py holds such a case).  strict_reuse=True, the default and
    what the product does, also requires the pieces to lie inside the piece wanted and to be
    pairwise disjoint; plans are the same wherever the reference's are right.
    """
    return _plan(size, shape, itemsize, inputs_arg, outputs_arg, strict_reuse)[0]


def wire(size, shape, itemsize, inputs_arg, outputs_arg):
    """wire[sender][receiver]: the bytes `sender` puts on `receiver`'s queue while compiling
    (core/processgroup.cc:3015-3033)."""
    sent = _plan(size, shape, itemsize, inputs_arg, outputs_arg, True)[1]
    return [[pack_messages(sent[s][r], len(shape)) for r in range(size)] for s in range(size)]


def pack_messages(messages, ndim):
    """serializeToBuffer(IVector<TInput<std::array<int, ndim>>>): the vector is its size() as a
    size_t followed by the elements (core/serialization.h:148-154); an element writes its members
    in the order TInput::serialize lists them (core/processgroup.cc:2748-2751), each trivially
    copyable member as its raw object bytes, nothing between them (core/serialization.h:263-267;
    the header says of itself "not a cross platform serializer": x86-64, little-endian, bool = 1
    byte, int = 4, size_t = 8).  `contiguous` keeps its initialiser, false (:2737)."""
    out = [struct.pack("<Q", len(messages))]
    for m in messages:
        assert len(m["offset"]) == ndim and len(m["shape"]) == ndim
        out.append(struct.pack("<?", False))
        out.append(struct.pack("<%di" % ndim, *m["offset"]))
        out.append(struct.pack("<%di" % ndim, *m["shape"]))
        out.append(struct.pack("<IIII", m["inputRank"], m["outputRank"], m["inputIndex"], m["outputIndex"]))
        out.append(struct.pack("<QQ", m["inputOffset"], m["outputOffset"]))
        out.append(struct.pack("<?", m["outputContiguous"]))
    return b"".join(out)


def unpack_messages(data, ndim):
    """deserializeBuffer into IVector<TInput> (core/serialization.h:156-170, :671-680)."""
    (n,), pos = struct.unpack_from("<Q", data, 0), 8
    fmt = "<?%di%diIIIIQQ?" % (ndim, ndim)
    assert struct.calcsize(fmt) == 34 + 8 * ndim
    out = []
    for _ in range(n):
        v = struct.unpack_from(fmt, data, pos)
        pos += struct.calcsize(fmt)
        out.append({"offset": list(v[1:1 + ndim]), "shape": list(v[1 + ndim:1 + 2 * ndim]),
                    "inputRank": v[-7], "outputRank": v[-6], "inputIndex": v[-5], "outputIndex": v[-4],
                    "inputOffset": v[-3], "outputOffset": v[-2], "outputContiguous": v[-1]})
    if pos != len(data):
        raise PlanError("deserializeBuffer: %d trailing bytes" % (len(data) - pos))
    return out


def _inside(a, b):
    return all(ao >= bo and ao + ash <= bo + bsh
               for ao, ash, bo, bsh in zip(a["offset"], a["shape"], b["offset"], b["shape"]))


def _plan(size, shape, itemsize, inputs_arg, outputs_arg, strict_reuse=True):
    ndim = len(shape)
    for _, off, shp in list(inputs_arg) + list(outputs_arg):
        assert len(off) == ndim and len(shp) == ndim
    inputs, _ = _descrs(inputs_arg, size)
    outputs, out_count = _descrs(outputs_arg, size)

    outputsPerRank = [[] for _ in range(size)]
    for d in outputs:
        assert d["index"] == len(outputsPerRank[d["rank"]])
        outputsPerRank[d["rank"]].append(d)

    # stable sort by numel, largest first (:2848-2849)
    inputs = sorted(inputs, key=lambda d: -d["numel"])
    outputs = sorted(outputs, key=lambda d: -d["numel"])

    descs = [Descriptor() for _ in range(size)]
    sent = [[[] for _ in range(size)] for _ in range(size)]  # sent[sender][receiver]

    for rank in range(size):
        myInputs = [d for d in inputs if d["rank"] == rank]
        distInputs = []
        copyInputs = []
        for dst in outputs:  # sender loop, :2921-2984
            if dst["numel"] == 0:
                continue
            for x in _find(dst, myInputs):
                src = myInputs[x["index"]]
                inputContiguous = _contiguous(x["shape"], src["shape"])
                if not inputContiguous:
                    rr = _find(dst, copyInputs)
                    if rr and len(rr) < 4:
                        n = 0
                        cc = True
                        for x2 in rr:
                            n += _numel(x2["shape"])
                            cc = cc and _contiguous(x2["shape"], copyInputs[x2["index"]]["shape"])
                            if not cc:
                                break
                        if strict_reuse:
                            # deviation from the reference, see plan(): the pieces must lie inside
                            # the piece wanted and be pairwise disjoint
                            for p, y in enumerate(rr):
                                cc = cc and _inside(y, x) and not any(
                                    _intersecting(y["offset"], y["shape"], z["offset"], z["shape"]) for z in rr[:p])
                        if cc and n == _numel(x["shape"]):
                            for x2 in rr:
                                ci = copyInputs[x2["index"]]
                                distInputs.append({
                                    "offset": x2["offset"], "shape": x2["shape"],
                                    "inputRank": rank, "outputRank": dst["rank"],
                                    "inputIndex": len(myInputs) + x2["index"], "outputIndex": dst["index"],
                                    "inputOffset": _linear_offset(_sub(x2["offset"], ci["offset"]), ci["shape"]),
                                    "outputOffset": _linear_offset(_sub(x2["offset"], dst["offset"]), dst["shape"]),
                                    "outputContiguous": _contiguous(x2["shape"], dst["shape"]),
                                })
                            continue
                inp = {
                    "offset": x["offset"], "shape": x["shape"],
                    "inputRank": rank, "outputRank": dst["rank"],
                    "inputIndex": x["index"], "outputIndex": dst["index"],
                    "inputOffset": _linear_offset(_sub(x["offset"], src["offset"]), src["shape"]),
                    "outputOffset": _linear_offset(_sub(x["offset"], dst["offset"]), dst["shape"]),
                }
                if not inputContiguous:
                    inp["inputIndex"] = len(myInputs) + len(copyInputs)
                    inp["inputOffset"] = 0
                    copyInputs.append(x)
                inp["outputContiguous"] = _contiguous(x["shape"], dst["shape"])
                distInputs.append(inp)

        op = descs[rank]
        for x in inputs:  # :2993-2998 (sorted order)
            if x["rank"] == rank:
                op.inputs.append(itemsize * _numel(x["shape"]))
                op.inputShapes.append(list(x["shape"]))
        for x in outputs:  # :2999-3004 (sorted order)
            if x["rank"] == rank:
                op.outputs.append(itemsize * _numel(x["shape"]))
                op.outputShapes.append(list(x["shape"]))
        for x in distInputs:
            sent[rank][x["outputRank"]].append(x)
        for x in copyInputs:  # :3086-3093
            op.inputCopies.append(Copy(x["index"], _sub(x["offset"], myInputs[x["index"]]["offset"]),
                                       list(x["shape"])))

    for rank in range(size):  # receiver loop, :3043-3077
        op = descs[rank]
        total = sum(_numel(x["shape"]) for x in outputs if x["rank"] == rank)
        readNumel = 0
        for sender in range(size):
            for x in sent[sender][rank]:
                r = Read(x["inputRank"], x["inputIndex"], x["outputIndex"], itemsize * x["inputOffset"],
                         itemsize * x["outputOffset"], itemsize * _numel(x["shape"]))
                readNumel += _numel(x["shape"])
                if not x["outputContiguous"]:
                    c = Copy(r.outputIndex, _sub(x["offset"], outputsPerRank[rank][x["outputIndex"]]["offset"]),
                             list(x["shape"]))
                    r.outputIndex = len(op.outputs) + len(op.outputCopies)
                    op.outputCopies.append(c)
                    r.outputOffset = 0
                op.reads.append(r)
        if readNumel != total:  # :3079-3081
            raise PlanError("moodist.compile_op_full: could not find input for all output elements")
    return descs, sent


def _box_view(flat_bytes, tensor_shape, itemsize, offset, shape):
    """numpy view of an N-d box inside a contiguous tensor held as flat bytes."""
    a = flat_bytes.view(np.uint8).reshape(list(tensor_shape) + [itemsize])
    sl = tuple(slice(o, o + s) for o, s in zip(offset, shape))
    return a[sl]


def execute(descs, itemsize, inputs_per_rank, outputs_per_rank):
    """Run every rank's plan.  inputs_per_rank[r] / outputs_per_rank[r] are lists of
    flat uint8 arrays in the order the rank's descriptor lists them."""
    size = len(descs)
    staged_inputs = []
    for r in range(size):
        op = descs[r]
        bufs = list(inputs_per_rank[r])
        assert [b.size for b in bufs] == op.inputs, "custom op input has wrong size"
        for c in op.inputCopies:  # box of input `index` -> contiguous staging
            box = _box_view(bufs[c.index], op.inputShapes[c.index], itemsize, c.offset, c.shape)
            bufs.append(np.ascontiguousarray(box).reshape(-1))
        staged_inputs.append(bufs)
    for r in range(size):
        op = descs[r]
        outs = list(outputs_per_rank[r])
        assert [b.size for b in outs] == op.outputs, "custom op output has wrong size"
        for c in op.outputCopies:
            outs.append(np.zeros(_numel(c.shape) * itemsize, dtype=np.uint8))
        for rd in op.reads:
            src = staged_inputs[rd.rank][rd.inputIndex]
            outs[rd.outputIndex][rd.outputOffset:rd.outputOffset + rd.bytes] = \
                src[rd.inputOffset:rd.inputOffset + rd.bytes]
        for k, c in enumerate(op.outputCopies):  # contiguous staging -> box of output `index`
            box = _box_view(outs[c.index], op.outputShapes[c.index], itemsize, c.offset, c.shape)
            box[...] = outs[len(op.outputs) + k].reshape(list(c.shape) + [itemsize])


def shard_box(global_shape, mesh_sizes, coord, placements):
    """py/moodist/compile.py:21-59.  placements[i] is None (replicate) or the sharded
    tensor dim for mesh dim i; coord[i] this rank's coordinate.  Returns (offset, shape)."""
    offsets = [0] * len(global_shape)
    local = list(global_shape)
    if coord is None:
        return offsets, [0] * len(global_shape)
    for mesh_dim, dim in enumerate(placements):
        if dim is None:
            continue
        global_size = global_shape[dim]
        chunks = mesh_sizes[mesh_dim]
        chunk = (global_size + chunks - 1) // chunks
        start = chunk * coord[mesh_dim]
        if global_size < start:
            offsets[dim] = global_size
            local[dim] = 0
        else:
            offsets[dim] = start
            local[dim] = min(global_size, start + chunk) - start
    return offsets, local
