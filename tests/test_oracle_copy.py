"""Pins oracle.c's orc_gather / orc_copy_box and oracle/planner.py.  No GPU."""

import itertools

import numpy as np
import pytest
import torch

import oracle
from oracle import planner


def _u8(a):
    return np.ascontiguousarray(a).view(np.uint8).reshape(-1)


def test_reference_known_answer_allgather_constants():
    # reference tests/test_processgroup.py:21-48
    P, chunk = 8, 4
    shards = [np.full(chunk, float(r), dtype=np.float32) for r in range(P)]
    out = oracle.all_gather(shards).view(np.float32)
    assert np.array_equal(out, np.repeat(np.arange(P, dtype=np.float32), chunk))


def test_reference_known_answer_allgather_aranges():
    # reference tests/test_processgroup.py:82-109
    P, chunk = 8, 8
    shards = [np.arange(r * 100, r * 100 + chunk, dtype=np.float32) for r in range(P)]
    out = oracle.all_gather(shards).view(np.float32)
    for r in range(P):
        assert np.array_equal(out[r * chunk:(r + 1) * chunk], shards[r])


def test_reference_known_answer_allgather_randn():
    # reference tests/test_processgroup.py:112-146: seed rank+42, 256 Ki elements, torch.equal
    P, chunk = 8, 256 * 1024
    shards = []
    for r in range(P):
        torch.manual_seed(r + 42)
        shards.append(torch.randn(chunk, dtype=torch.float32))
    out = torch.from_numpy(oracle.all_gather([s.numpy() for s in shards]).view(np.float32))
    assert torch.equal(out, torch.cat(shards))


@pytest.mark.parametrize("size", [1, 7, 64, 255, 1024, 4096, 65536])
def test_reference_known_answer_allgather_ragged(size):
    # reference tests/test_stress.py:235-280
    P = 8
    out = oracle.all_gather([np.full(size, float(r), dtype=np.float32) for r in range(P)]).view(np.float32)
    for r in range(P):
        assert (out[r * size:(r + 1) * size] == float(r)).all()


def test_gather_2d_against_numpy():
    rng = np.random.RandomState(1)
    P, rows, width, sp, dp = 5, 37, 200, 256, 300
    stride = rows * dp + 64
    shards = [rng.randint(0, 256, rows * sp).astype(np.uint8) for _ in range(P)]
    out = np.full(P * stride, 7, dtype=np.uint8)
    oracle.gather(shards, out, width, rows, sp, dp, stride)
    want = np.full(P * stride, 7, dtype=np.uint8)
    for s in range(P):
        src = shards[s].reshape(rows, sp)[:, :width]
        want[s * stride:s * stride + rows * dp].reshape(rows, dp)[:, :width] = src
    assert np.array_equal(out, want)


@pytest.mark.parametrize("itemsize", [1, 2, 4, 8])
def test_copy_box_against_numpy_slicing(itemsize):
    rng = np.random.RandomState(itemsize)
    dt = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[itemsize]
    G = rng.randint(0, 255, (6, 5, 7, 4)).astype(dt)
    out = np.zeros((3, 5, 2, 4), dtype=dt)
    off = (2, 0, 3, 0)
    shape = (3, 5, 2, 4)
    es = lambda a: [s // itemsize for s in a.strides]
    src_off = sum(o * s for o, s in zip(off, es(G)))
    oracle.copy_box(_u8(G), src_off, _u8(out), 0, shape, es(G), es(out), itemsize)
    assert np.array_equal(out, G[2:5, :, 3:5, :])
    # and back into a strided destination, including a transposing stride order
    back = np.zeros_like(G)
    oracle.copy_box(_u8(out), 0, _u8(back), src_off, shape, es(out), es(back), itemsize)
    assert np.array_equal(back[2:5, :, 3:5, :], out) and back.sum() == out.sum()
    T = np.zeros((4, 2, 5, 3), dtype=dt)
    oracle.copy_box(_u8(out), 0, _u8(T), 0, shape, es(out), [es(T)[3 - i] for i in range(4)], itemsize)
    assert np.array_equal(T, out.transpose(3, 2, 1, 0))


# ---------------- planner ----------------

def _run_plan(size, shape, np_dtype, inputs_arg, outputs_arg, G):
    """Plan, execute with the oracle and return per-rank output arrays (original arg order kept
    only when sizes are equal, which is all these tests use)."""
    itemsize = np.dtype(np_dtype).itemsize
    descs = planner.plan(size, shape, itemsize, inputs_arg, outputs_arg)
    ins = [[] for _ in range(size)]
    for r, off, shp in inputs_arg:
        sl = tuple(slice(o, o + s) for o, s in zip(off, shp))
        ins[r].append(_u8(G[sl]).copy())
    outs = [[np.zeros(n, dtype=np.uint8) for n in d.outputs] for d in descs]
    planner.execute(descs, itemsize, ins, outs)
    return descs, outs


def _check_outputs(outputs_arg, outs, G, np_dtype):
    counter = {}
    for r, off, shp in outputs_arg:
        i = counter.get(r, 0)
        counter[r] = i + 1
        sl = tuple(slice(o, o + s) for o, s in zip(off, shp))
        got = outs[r][i].view(np_dtype).reshape(shp)
        assert np.array_equal(got, G[sl]), (r, off, shp)


def test_planner_hand_derived_4x4_row_to_column():
    # 4x4 fp32 over 2 ranks, row-sharded -> column-sharded, derived by hand from
    # core/processgroup.cc:2761-3104
    inputs = [(0, [0, 0], [2, 4]), (1, [2, 0], [2, 4])]
    outputs = [(0, [0, 0], [4, 2]), (1, [0, 2], [4, 2])]
    d = planner.plan(2, [4, 4], 4, inputs, outputs)
    r0, r1 = d
    assert r0.inputs == [32] and r0.outputs == [32]
    assert [(c.index, c.offset, c.shape) for c in r0.inputCopies] == [(0, [0, 0], [2, 2]), (0, [0, 2], [2, 2])]
    assert [(c.index, c.offset, c.shape) for c in r1.inputCopies] == [(0, [0, 0], [2, 2]), (0, [0, 2], [2, 2])]
    rd = [(x.rank, x.inputIndex, x.outputIndex, x.inputOffset, x.outputOffset, x.bytes) for x in r0.reads]
    assert rd == [(0, 1, 0, 0, 0, 16), (1, 1, 0, 0, 16, 16)]
    rd = [(x.rank, x.inputIndex, x.outputIndex, x.inputOffset, x.outputOffset, x.bytes) for x in r1.reads]
    assert rd == [(0, 2, 0, 0, 0, 16), (1, 2, 0, 0, 16, 16)]
    assert r0.outputCopies == [] and r1.outputCopies == []
    G = np.arange(16, dtype=np.float32).reshape(4, 4)
    _, outs = _run_plan(2, [4, 4], np.float32, inputs, outputs, G)
    _check_outputs(outputs, outs, G, np.float32)


# Written out by hand from the member order of TInput (core/processgroup.cc:2735-2753) and the
# raw-byte serializer (core/serialization.h:148-154, :263-267): u64 count, then u8 contiguous,
# i32 offset[2], i32 shape[2], u32 inputRank, outputRank, inputIndex, outputIndex,
# u64 inputOffset, outputOffset, u8 outputContiguous.
WIRE_4X4_R1_TO_R0 = bytes.fromhex(
    "0100000000000000"          # one piece
    "00"                        # contiguous: never set
    "02000000" "00000000"       # offset [2, 0] (global coordinates)
    "02000000" "02000000"       # shape [2, 2]
    "01000000" "00000000"       # inputRank 1, outputRank 0
    "01000000" "00000000"       # inputIndex 1 (the sender's first staging copy), outputIndex 0
    "0000000000000000"          # inputOffset 0 elements
    "0400000000000000"          # outputOffset linearOffset([2,0],[4,2]) = 4 elements
    "01")                       # outputContiguous
WIRE_4X4_R0_TO_R1 = bytes.fromhex(
    "0100000000000000" "00" "00000000" "02000000" "02000000" "02000000"
    "00000000" "01000000" "02000000" "00000000" "0000000000000000" "0000000000000000" "01")
# column -> row, sender 0 to receiver 1: piece [2,0]+[2,2] is contiguous in the sender's [4,2]
# tensor at element 4 and not contiguous in the receiver's [2,4] tensor
WIRE_4X4_COL_TO_ROW_R0_TO_R1 = bytes.fromhex(
    "0100000000000000" "00" "02000000" "00000000" "02000000" "02000000"
    "00000000" "01000000" "00000000" "00000000" "0400000000000000" "0000000000000000" "00")


def test_plan_wire_bytes_hand_derived():
    inputs = [(0, [0, 0], [2, 4]), (1, [2, 0], [2, 4])]
    outputs = [(0, [0, 0], [4, 2]), (1, [0, 2], [4, 2])]
    w = planner.wire(2, [4, 4], 4, inputs, outputs)
    assert w[1][0] == WIRE_4X4_R1_TO_R0 and len(w[1][0]) == 8 + 34 + 8 * 2
    assert w[0][1] == WIRE_4X4_R0_TO_R1
    w = planner.wire(2, [4, 4], 4, outputs, inputs)
    assert w[0][1] == WIRE_4X4_COL_TO_ROW_R0_TO_R1
    # a rank with nothing for a receiver still sends an empty list: just the count
    w = planner.wire(2, [8], 4, [(0, [0], [8])], [(1, [0], [8])])
    assert w[1][0] == w[1][1] == w[0][0] == bytes(8) and len(w[0][1]) == 8 + 34 + 8


def test_plan_wire_round_trip_and_record_length():
    rng = np.random.RandomState(3)
    for ndim in (1, 2, 3, 10):
        msgs = [{"offset": [int(v) for v in rng.randint(0, 2**31 - 1, ndim)],
                 "shape": [int(v) for v in rng.randint(0, 2**31 - 1, ndim)],
                 "inputRank": int(rng.randint(0, 2**31)), "outputRank": int(rng.randint(0, 64)),
                 "inputIndex": int(rng.randint(0, 9)), "outputIndex": int(rng.randint(0, 9)),
                 "inputOffset": int(rng.randint(0, 2**62)), "outputOffset": int(rng.randint(0, 2**62)),
                 "outputContiguous": bool(rng.randint(0, 2))} for _ in range(5)]
        data = planner.pack_messages(msgs, ndim)
        assert len(data) == 8 + 5 * (34 + 8 * ndim)
        assert planner.unpack_messages(data, ndim) == msgs
        with pytest.raises(planner.PlanError, match="1 trailing bytes"):
            planner.unpack_messages(data + b"\0", ndim)


def _random_redistribution(rng, size):
    """Non-overlapping inputs (slabs along one dimension or a grid over two) dealt to random ranks,
    up to two random output boxes per rank; every rank lists its slices largest first."""
    ndim = int(rng.randint(1, 5))
    shape = [int(rng.randint(1, 12)) for _ in range(ndim)]
    d1, d2 = int(rng.randint(0, ndim)), int(rng.randint(0, ndim))
    c1 = sorted(set([0, shape[d1]] + [int(x) for x in rng.randint(0, shape[d1] + 1, 4)]))
    c2 = sorted(set([0, shape[d2]] + [int(x) for x in rng.randint(0, shape[d2] + 1, 3)])) \
        if d2 != d1 and rng.rand() < 0.5 else [0, shape[d2]]
    inputs = []
    for a, b in zip(c1[:-1], c1[1:]):
        for c, e in zip(c2[:-1], c2[1:]):
            off, shp = [0] * ndim, list(shape)
            off[d1], shp[d1] = a, b - a
            if len(c2) > 2:
                off[d2], shp[d2] = c, e - c
            inputs.append((int(rng.randint(0, size)), off, shp))
    outputs = []
    for r in range(size):
        for _ in range(int(rng.randint(0, 3))):
            lo = [int(rng.randint(0, n)) for n in shape]
            hi = [int(rng.randint(l + 1, n + 1)) for l, n in zip(lo, shape)]
            outputs.append((r, lo, [h - l for l, h in zip(lo, hi)]))
    inputs.sort(key=lambda x: (x[0], -int(np.prod(x[2]))))
    outputs.sort(key=lambda x: (x[0], -int(np.prod(x[2]))))
    return shape, inputs, outputs


def _executes_correctly(size, shape, inputs, outputs, G, **kw):
    descs = planner.plan(size, shape, 4, inputs, outputs, **kw)
    ins = [[_u8(G[tuple(slice(o, o + s) for o, s in zip(off, shp))]).copy() for r, off, shp in inputs if r == q]
           for q in range(size)]
    outs = [[np.zeros(n, dtype=np.uint8) for n in d.outputs] for d in descs]
    planner.execute(descs, 4, ins, outs)
    counter = {}
    for r, off, shp in outputs:
        i = counter.get(r, 0)
        counter[r] = i + 1
        if not np.array_equal(outs[r][i].view(np.int32).reshape(shp), G[tuple(slice(o, o + s) for o, s in zip(off, shp))]):
            return False
    return True


def test_planner_random_redistributions_execute_to_numpy_slicing():
    # pins the planner restatement (with the sound staging-reuse rule) on 600 random cases
    for seed in range(600):
        rng = np.random.RandomState(seed)
        size = int(rng.randint(1, 6))
        shape, inputs, outputs = _random_redistribution(rng, size)
        G = rng.randint(-50, 50, shape).astype(np.int32)
        assert _executes_correctly(size, shape, inputs, outputs, G), (seed, shape, inputs, outputs)


def test_reference_staging_reuse_rule_can_leave_an_element_unwritten():
    # core/processgroup.cc:2931-2962 reuses staged pieces when their element counts add up to the
    # piece wanted.  Rank 1 holds rows 11-12 and row 9 of a [15, 3] tensor; earlier destinations
    # make it stage element [9, 2] twice; rank 5 then wants [9, 1:3], finds the two staged copies
    # of [9, 2] (1 + 1 = 2 elements) and reads [9, 2] twice instead of [9, 1] and [9, 2].  The
    # plan passes the reference's coverage check (:3079-3081).  The sound rule gets it right.
    shape = [15, 3]
    inputs = [(1, [11, 0], [2, 3]), (1, [9, 0], [1, 3]), (3, [10, 0], [1, 3]), (6, [5, 0], [4, 3]),
              (7, [0, 0], [5, 3]), (7, [13, 0], [2, 3])]
    outputs = [(0, [4, 2], [8, 1]), (1, [10, 2], [5, 1]), (2, [13, 2], [2, 1]), (3, [11, 0], [3, 1]),
               (4, [3, 2], [11, 1]), (5, [9, 1], [1, 2]), (6, [12, 1], [3, 2]), (7, [11, 2], [2, 1])]
    G = np.arange(45, dtype=np.int32).reshape(15, 3)
    assert not _executes_correctly(8, shape, inputs, outputs, G, strict_reuse=False)
    assert _executes_correctly(8, shape, inputs, outputs, G)
    # where the reference's plan is right the two rules give the same plan
    for seed in range(200):
        rng = np.random.RandomState(seed)
        size = int(rng.randint(1, 6))
        shp, ins, outs = _random_redistribution(rng, size)
        Gr = rng.randint(-50, 50, shp).astype(np.int32)
        if _executes_correctly(size, shp, ins, outs, Gr, strict_reuse=False):
            assert planner.plan(size, shp, 4, ins, outs, strict_reuse=False) == planner.plan(size, shp, 4, ins, outs)


def test_planner_column_to_row_uses_output_copies():
    inputs = [(0, [0, 0], [4, 2]), (1, [0, 2], [4, 2])]
    outputs = [(0, [0, 0], [2, 4]), (1, [2, 0], [2, 4])]
    d = planner.plan(2, [4, 4], 4, inputs, outputs)
    assert all(len(x.outputCopies) == 2 and x.inputCopies == [] for x in d)
    G = np.arange(16, dtype=np.float32).reshape(4, 4)
    _, outs = _run_plan(2, [4, 4], np.float32, inputs, outputs, G)
    _check_outputs(outputs, outs, G, np.float32)


def test_planner_allgather_1d_plan():
    # reference tests/test_compile_op.py:190-222
    P, chunk = 8, 4
    inputs = [(r, [r * chunk], [chunk]) for r in range(P)]
    outputs = [(r, [0], [chunk * P]) for r in range(P)]
    d = planner.plan(P, [chunk * P], 4, inputs, outputs)
    for r in range(P):
        assert d[r].inputCopies == [] and d[r].outputCopies == []
        rd = [(x.rank, x.inputIndex, x.outputIndex, x.inputOffset, x.outputOffset, x.bytes) for x in d[r].reads]
        assert rd == [(s, 0, 0, 0, s * chunk * 4, chunk * 4) for s in range(P)]


def _cases():
    P = 8
    yield "p2p", P, [4], np.float32, [(0, [0], [4])], [(1, [0], [4])]  # test_compile_op.py:21-61
    yield "broadcast", P, [8], np.float32, [(0, [0], [8])], [(r, [0], [8]) for r in range(P)]  # :64-99
    yield "gather", P, [4 * P], np.float32, [(r, [4 * r], [4]) for r in range(P)], [(0, [0], [4 * P])]  # :102-144
    yield "scatter", P, [4 * P], np.float32, [(0, [0], [4 * P])], [(r, [4 * r], [4]) for r in range(P)]  # :147-187
    yield "allgather", P, [4 * P], np.float32, [(r, [4 * r], [4]) for r in range(P)], \
        [(r, [0], [4 * P]) for r in range(P)]  # :190-222
    yield "rows2d", P, [P, 4], np.float32, [(r, [r, 0], [1, 4]) for r in range(P)], \
        [(r, [0, 0], [P, 4]) for r in range(P)]  # :225-258
    yield "multi_in", P, [4], np.float32, [(0, [0], [2]), (0, [2], [2])], [(1, [0], [4])]  # :261-309
    for dt in (np.float32, np.float64, np.int32, np.int64):  # :312-343
        yield "dtype_%s" % np.dtype(dt).name, P, [4], dt, [(0, [0], [4])], [(r, [0], [4]) for r in range(P)]
    yield "bystanders", P, [4], np.float32, [(0, [0], [4])], [(1, [0], [4])]  # :382-423
    # beyond the reference's tests: strided slices on either side
    yield "row_to_col", P, [16, 24], np.float32, [(r, [2 * r, 0], [2, 24]) for r in range(P)], \
        [(r, [0, 3 * r], [16, 3]) for r in range(P)]
    yield "col_to_row", P, [16, 24], np.int16, [(r, [0, 3 * r], [16, 3]) for r in range(P)], \
        [(r, [2 * r, 0], [2, 24]) for r in range(P)]
    yield "dim0_to_dim2", P, [8, 6, 16], np.uint16, [(r, [r, 0, 0], [1, 6, 16]) for r in range(P)], \
        [(r, [0, 0, 2 * r], [8, 6, 2]) for r in range(P)]
    yield "overlapping_outputs", 4, [6, 6], np.float32, [(r % 2, [3 * (r % 2), 0], [3, 6]) for r in range(2)], \
        [(0, [1, 1], [4, 4]), (1, [0, 0], [6, 6]), (2, [2, 0], [2, 6]), (3, [0, 4], [6, 2])]


@pytest.mark.parametrize("case", list(_cases()), ids=lambda c: c[0])
def test_planner_executes_to_the_global_slice(case):
    _, size, shape, dt, inputs, outputs = case
    rng = np.random.RandomState(3)
    G = rng.randint(-1000, 1000, shape).astype(dt)
    descs, outs = _run_plan(size, shape, dt, inputs, outputs, G)
    _check_outputs(outputs, outs, G, dt)
    itemsize = np.dtype(dt).itemsize
    for r, d in enumerate(descs):
        # invariants: the reads cover the outputs exactly once
        assert sum(x.bytes for x in d.reads) == sum(d.outputs)
        written = {}
        for x in d.reads:
            if x.outputIndex < len(d.outputs):
                key = x.outputIndex
                seg = written.setdefault(key, np.zeros(d.outputs[key], dtype=np.int32))
                seg[x.outputOffset:x.outputOffset + x.bytes] += 1
        for seg in written.values():
            assert seg.max() <= 1
        assert all(x.bytes % itemsize == 0 for x in d.reads)


def test_planner_reports_uncovered_outputs():
    with pytest.raises(planner.PlanError, match="could not find input for all output elements"):
        planner.plan(2, [8], 4, [(0, [0], [4])], [(1, [0], [8])])


def test_shard_box_matches_torch_chunking():
    # py/moodist/compile.py:21-59 says it matches Shard.local_shard_size_and_offset: check against
    # torch.chunk-style ceil division on uneven sizes
    for n, k in itertools.product([1, 7, 8, 9, 64, 65], [1, 2, 3, 8]):
        chunk = (n + k - 1) // k
        for c in range(k):
            off, shp = planner.shard_box([n, 5], [k], [c], [0])
            start = min(n, chunk * c)
            stop = min(n, chunk * (c + 1))
            assert off == [start, 0] or (shp[0] == 0 and off[0] == n)
            assert shp == [stop - start, 5]
    assert planner.shard_box([8, 8], [2, 4], [1, 3], [0, 1]) == ([4, 6], [4, 2])
    assert planner.shard_box([8, 8], [2], None, [0]) == ([0, 0], [0, 0])
