"""compile_op: front end of the redistribution planner.

Same calling convention and checks as the reference's py/moodist/compile.py:104-264: each rank
names the slices of a global tensor it holds (inputs) and wants (outputs), as dicts with
'offset' and 'shape' or as DTensors; all ranks' specifications are gathered and handed to
``compile_op_full``.  The reference gathers them through a distributed queue (:200-262); the
ranks of a LocalWorld share a process, so the gathering is a list on the world, and the
operation a rank gets back becomes callable once the last rank has called compile_op.
"""

import weakref

import torch


def _is_dtensor(x):
    return hasattr(x, "placements") and hasattr(x, "device_mesh") and hasattr(x, "to_local")


def shard_box(global_shape, mesh_sizes, coordinate, placements):
    """Offset and local shape of a Shard placement (py/moodist/compile.py:21-59): chunks of
    ceil(n / k) along the sharded dimension, the last ones possibly short or empty.
    placements[i] is the tensor dimension mesh dimension i shards, or None."""
    offsets = [0] * len(global_shape)
    local = list(global_shape)
    if coordinate is None:
        return offsets, [0] * len(global_shape)
    for mesh_dim, dim in enumerate(placements):
        if dim is None:
            continue
        n = global_shape[dim]
        k = mesh_sizes[mesh_dim]
        chunk = (n + k - 1) // k
        start = chunk * coordinate[mesh_dim]
        if n < start:
            offsets[dim], local[dim] = n, 0
        else:
            offsets[dim], local[dim] = start, min(n, start + chunk) - start
    return offsets, local


def _dtensor_box(t):
    from torch.distributed.tensor import Shard

    mesh = t.device_mesh
    dims = [p.dim if isinstance(p, Shard) else None for p in t.placements]
    off, shp = shard_box(list(t.shape), [mesh.size(i) for i in range(len(dims))], mesh.get_coordinate(), dims)
    return {"offset": off, "shape": shp}


def _normalise(specs, holder):
    if specs is None:
        return None
    out = []
    for x in specs:
        if _is_dtensor(x):
            shape, dtype = tuple(x.shape), x.dtype
            if holder["shape"] is None:
                holder["shape"], holder["dtype"] = shape, dtype
            elif holder["shape"] != shape:
                raise ValueError("All DTensors must have the same global shape, got %s and %s"
                                 % (holder["shape"], shape))
            elif holder["dtype"] != dtype:
                raise ValueError("All DTensors must have the same dtype, got %s and %s" % (holder["dtype"], dtype))
            out.append(_dtensor_box(x))
        else:
            out.append(x)
    return out


def _check(specs, ndim):
    if not isinstance(specs, (tuple, list)):
        raise TypeError("inputs/outputs must be a tuple or list, got %s" % type(specs).__name__)
    for x in specs:
        if not isinstance(x, dict):
            raise TypeError("each input/output spec must be a dict, got %s" % type(x).__name__)
        for key in ("offset", "shape"):
            if key not in x:
                raise ValueError("'%s' is missing for an input or output" % key)
            v = x[key]
            if not isinstance(v, (tuple, list)):
                raise TypeError("'%s' must be a tuple or list, got %s" % (key, type(v).__name__))
            if len(v) != ndim:
                raise ValueError("expected '%s' with %d dimensions, but got %d" % (key, ndim, len(v)))
            for i, z in enumerate(v):
                if not isinstance(z, int):
                    raise TypeError("%s[%d] must be an int, got %s" % (key, i, type(z).__name__))
    return tuple((tuple(x["offset"]), tuple(x["shape"])) for x in specs)


class _Round:
    """One collective compile_op call: what every rank of the world has said so far."""

    def __init__(self, size, first_group):
        self.size = size
        self.info = {}
        # the group that opened the round: once it is gone the round is stale (the store's id may
        # by then name another object)
        self.first = weakref.ref(first_group)

    def complete(self):
        return len(self.info) == self.size


_rounds = {}  # id(store) -> the round the ranks of that store's world are filling


class CompiledOp:
    """What compile_op returns.  Calling it runs the redistribution for this rank and returns a
    future (wrapper/module.cc:1270-1305); every rank of the world must call it."""

    def __init__(self, group, round_):
        self._group = group
        self._round = round_
        self._op = None

    def _resolve(self):
        if self._op is None:
            rnd = self._round
            if not rnd.complete():
                raise RuntimeError("moodist.compile_op: %d of %d ranks have called compile_op; the operation "
                                   "cannot run before all have" % (len(rnd.info), rnd.size))
            shape, dtype = None, None
            all_inputs, all_outputs = [], []
            for rank in sorted(rnd.info):
                nshape, ndtype, ninputs, noutputs = rnd.info[rank]
                if shape is None:
                    shape, dtype = nshape, ndtype
                if nshape != shape:
                    raise ValueError("moodist.compile_op: Ranks specified different shapes: %s vs %s"
                                     % (shape, nshape))
                if ndtype != dtype:
                    raise ValueError("moodist.compile_op: Ranks specified different dtypes: %s vs %s"
                                     % (dtype, ndtype))
                for o, s in ninputs or ():
                    all_inputs.append((rank, o, s))
                for o, s in noutputs or ():
                    all_outputs.append((rank, o, s))
            self._op = self._group.compile_op_full(shape, dtype, all_inputs, all_outputs)
        return self._op

    def __call__(self, inputs, outputs):
        return self._resolve()(list(inputs), list(outputs))

    def plan(self):
        return self._resolve().plan()


def compile_op(group, shape=None, dtype=None, inputs=None, outputs=None):
    holder = {"shape": tuple(shape) if shape is not None else None, "dtype": dtype}
    inputs = _normalise(inputs, holder)
    outputs = _normalise(outputs, holder)
    shape, dtype = holder["shape"], holder["dtype"]
    if shape is None:
        raise ValueError("shape must be provided or derivable from DTensors")
    if dtype is None:
        raise ValueError("dtype must be provided or derivable from DTensors")
    if not isinstance(dtype, torch.dtype):
        raise TypeError("dtype must be a torch.dtype, got %s" % type(dtype).__name__)
    shape = tuple(shape)
    for i, x in enumerate(shape):
        if not isinstance(x, int):
            raise TypeError("shape[%d] must be an int, got %s" % (i, type(x).__name__))
    if inputs is not None:
        inputs = _check(inputs, len(shape))
    if outputs is not None:
        outputs = _check(outputs, len(shape))

    # the ranks of a world share a store object: its identity names the round being gathered
    key = id(group._store)
    rnd = _rounds.get(key)
    if rnd is None or rnd.first() is None or rnd.complete() or group.rank() in rnd.info:
        rnd = _rounds[key] = _Round(group.size(), group)
    rnd.info[group.rank()] = (shape, dtype, inputs, outputs)
    return CompiledOp(group, rnd)
