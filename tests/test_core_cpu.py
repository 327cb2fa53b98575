"""Host core without a GPU: the C ABI of libmoodist.so, the planner against the oracle's
restatement, argument checks and the rendezvous rules.  Nothing here launches a kernel."""

import ctypes
import os
import re

import numpy as np
import pytest
import torch

import moodist_amd
from oracle import planner
from test_oracle_copy import _cases

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "moodist_amd", "libmoodist.so")


class Tensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("numel", ctypes.c_int64), ("itemsize", ctypes.c_int32),
                ("dtype", ctypes.c_int32), ("device", ctypes.c_int32), ("contiguous", ctypes.c_int32),
                ("ndim", ctypes.c_int32), ("reserved", ctypes.c_int32), ("shape", ctypes.c_int64 * 10)]


def fake(numel, dtype=6, itemsize=4, device=0, data=0x10000, contiguous=1):
    t = Tensor()
    t.data, t.numel, t.itemsize, t.dtype, t.device, t.contiguous, t.ndim = data, numel, itemsize, dtype, device, \
        contiguous, 1
    t.shape[0] = numel
    return t


@pytest.fixture(scope="module")
def core():
    L = ctypes.CDLL(LIB)
    L.moodist_last_error.restype = ctypes.c_char_p
    L.moodist_world_group.restype = ctypes.c_void_p
    L.moodist_world_group.argtypes = [ctypes.c_void_p, ctypes.c_int]
    L.moodist_world_destroy.argtypes = [ctypes.c_void_p]
    L.moodist_pg_rank.argtypes = [ctypes.c_void_p]
    L.moodist_pg_size.argtypes = [ctypes.c_void_p]
    L.moodist_pg_reduce_scatter.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                            ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p]
    L.moodist_pg_all_gather.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                        ctypes.c_void_p]
    L.moodist_pg_all_gather_list.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p,
                                             ctypes.c_void_p, ctypes.c_void_p]
    L.moodist_pg_all_gather_many.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                                             ctypes.c_void_p, ctypes.c_void_p]
    L.moodist_pg_allreduce_many.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int,
                                            ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p]
    L.moodist_pg_reduce_scatter_many.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                                                 ctypes.c_int, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p]
    L.moodist_pg_allreduce.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                       ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p]
    L.moodist_work_wait.argtypes = [ctypes.c_void_p]
    L.moodist_work_is_completed.argtypes = [ctypes.c_void_p]
    L.moodist_work_destroy.argtypes = [ctypes.c_void_p]
    L.moodist_pg_get_option.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_int64)]
    L.moodist_pg_set_option.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int64]
    return L


def make_world(core, size):
    w = ctypes.c_void_p()
    assert core.moodist_world_create(size, 0, ctypes.byref(w)) == 0, core.moodist_last_error()
    return w


def test_every_declared_symbol_is_exported(core):
    text = open(os.path.join(ROOT, "include", "moodist_core.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(moodist_[a-z_0-9]+)\s*\(", text)))
    assert len(names) >= 25
    for n in names:
        assert getattr(core, n) is not None


def test_version_handshake(core):
    # api/moodist_version.h:12: version 2; any other number is refused (api/moodist_api.h:265-271)
    assert core.moodist_core_check_version(2) == 1
    assert core.moodist_core_check_version(1) == 0
    assert core.moodist_core_check_version(3) == 0


def test_world_ranks_sizes_and_limits(core):
    w = make_world(core, 8)
    for r in range(8):
        pg = core.moodist_world_group(w, r)
        assert core.moodist_pg_rank(pg) == r and core.moodist_pg_size(pg) == 8
    assert core.moodist_world_group(w, 8) is None
    core.moodist_world_destroy(w)
    bad = ctypes.c_void_p()
    assert core.moodist_world_create(0, 0, ctypes.byref(bad)) != 0
    assert core.moodist_world_create(65, 0, ctypes.byref(bad)) != 0
    assert b"1..64 ranks" in core.moodist_last_error()


def test_options_by_name(core):
    w = make_world(core, 2)
    pg = core.moodist_world_group(w, 0)
    v = ctypes.c_int64()
    for name, default in ((b"prefer_kernel_less", 0), (b"force_kernel_less", 0), (b"num_chunks", -1),
                          (b"chunk_size", -1), (b"method", -1)):
        assert core.moodist_pg_get_option(pg, name, ctypes.byref(v)) == 0 and v.value == default
    assert core.moodist_pg_set_option(pg, b"chunk_size", 4096) == 0
    core.moodist_pg_get_option(pg, b"chunk_size", ctypes.byref(v))
    assert v.value == 4096
    assert core.moodist_pg_set_option(pg, b"bogus", 1) != 0
    assert core.moodist_last_error() == b"Unknown option: bogus"  # core/processgroup.cc:2469
    # num_chunks / chunk_size / method are honoured (they cut a reduce_scatter's reduction into
    # pieces), so values that mean nothing are refused instead of stored
    for name, bad in ((b"num_chunks", 0), (b"num_chunks", -2), (b"chunk_size", 0), (b"method", 3), (b"method", -2)):
        assert core.moodist_pg_set_option(pg, name, bad) != 0, (name, bad)
    assert core.moodist_pg_set_option(pg, b"method", 1) != 0  # copy: no counterpart among local ranks
    assert b"method 1 (copy)" in core.moodist_last_error()
    for name, good in ((b"num_chunks", 4), (b"num_chunks", -1), (b"method", 0), (b"method", 2), (b"method", -1),
                       (b"chunk_size", -1)):
        assert core.moodist_pg_set_option(pg, name, good) == 0, (name, good)
        core.moodist_pg_get_option(pg, name, ctypes.byref(v))
        assert v.value == good
    core.moodist_world_destroy(w)


def test_a_refused_list_leaves_nothing_posted(core):
    # a coalesced allreduce or reduce_scatter whose list is refused (mixed element types, an
    # operation one of the types does not support) has posted none of its tensors: the rank's next
    # collective still is its collective number 0, which the other rank's number 0 then meets
    T = type(fake(4))
    for attempt in ("allreduce_many", "reduce_scatter_many"):
        w = make_world(core, 2)
        a, b = core.moodist_world_group(w, 0), core.moodist_world_group(w, 1)
        work = ctypes.c_void_p()
        mixed = (T * 3)(fake(16), fake(8), fake(24, dtype=3))  # fp32, fp32, int32
        if attempt == "allreduce_many":
            assert core.moodist_pg_allreduce_many(a, mixed, 3, 1, None, 0.0, ctypes.byref(work)) != 0  # AVG
            assert core.moodist_pg_allreduce_many(a, mixed, 3, 0, None, 0.0, ctypes.byref(work)) != 0  # SUM
            assert b"one element type" in core.moodist_last_error()
        else:
            outs = (T * 3)(fake(8), fake(4), fake(12, dtype=3))
            assert core.moodist_pg_reduce_scatter_many(a, outs, mixed, 3, 1, None, 0.0, ctypes.byref(work)) != 0
            assert core.moodist_pg_reduce_scatter_many(a, outs, mixed, 3, 0, None, 0.0, ctypes.byref(work)) != 0
            assert b"one element type" in core.moodist_last_error()
            outs[1] = fake(5)
            same = (T * 3)(fake(16), fake(8), fake(24))
            assert core.moodist_pg_reduce_scatter_many(a, outs, same, 3, 0, None, 0.0, ctypes.byref(work)) != 0
        # rank 0's collective number 0 is this all_gather ...
        assert core.moodist_pg_all_gather(a, ctypes.byref(fake(8)), ctypes.byref(fake(4)), None, ctypes.byref(work)) == 0
        core.moodist_work_destroy(work)
        # ... so a reduce_scatter as rank 1's number 0 is a mismatch, and the same all_gather is not
        assert core.moodist_pg_reduce_scatter(b, ctypes.byref(fake(4)), ctypes.byref(fake(8)), 0, None, 0.0,
                                              ctypes.byref(work)) != 0
        assert b"different operation" in core.moodist_last_error()
        core.moodist_world_destroy(w)


def test_a_list_of_reduce_scatters_is_checked_like_one(core):
    T = type(fake(4))
    w = make_world(core, 4)
    pg = core.moodist_world_group(w, 0)
    work = ctypes.c_void_p()
    ins = (T * 2)(fake(16), fake(24))
    outs = (T * 2)(fake(4), fake(6))
    assert core.moodist_pg_reduce_scatter_many(pg, outs, ins, 0, 0, None, 0.0, ctypes.byref(work)) != 0
    assert b"1..65535 tensors" in core.moodist_last_error()
    assert core.moodist_pg_reduce_scatter_many(pg, outs, None, 2, 0, None, 0.0, ctypes.byref(work)) != 0
    assert core.moodist_pg_reduce_scatter_many(pg, outs, ins, 2, 2, None, 0.0, ctypes.byref(work)) != 0  # PRODUCT
    assert core.moodist_last_error() == b"Unsupported reduce operation"
    ins[1] = fake(25)  # not a multiple of the group size
    assert core.moodist_pg_reduce_scatter_many(pg, outs, ins, 2, 0, None, 0.0, ctypes.byref(work)) != 0
    ins[1] = fake(24, contiguous=0)
    assert core.moodist_pg_reduce_scatter_many(pg, outs, ins, 2, 0, None, 0.0, ctypes.byref(work)) != 0
    assert b"must be contiguous" in core.moodist_last_error()
    ins[1] = fake(24)
    assert core.moodist_pg_reduce_scatter_many(pg, outs, ins, 2, 0, None, 0.0, ctypes.byref(work)) == 0  # posted
    core.moodist_work_destroy(work)
    # another rank with a list of other sizes: the same total, caught before the launch
    other = core.moodist_world_group(w, 1)
    assert core.moodist_pg_reduce_scatter_many(other, None, (T * 2)(fake(20), fake(20)), 2, 0, None, 0.0,
                                               ctypes.byref(work)) == 0
    core.moodist_work_destroy(work)
    core.moodist_world_destroy(w)


def test_argument_checks_use_the_reference_messages(core):
    w = make_world(core, 4)
    pg = core.moodist_world_group(w, 0)
    work = ctypes.c_void_p()

    def rs(out, inp, op=0):
        return core.moodist_pg_reduce_scatter(pg, ctypes.byref(out), ctypes.byref(inp), op, None, 0.0,
                                              ctypes.byref(work))

    assert rs(fake(4, dtype=0, itemsize=1), fake(16, dtype=0, itemsize=1)) != 0
    assert core.moodist_last_error() == b"Unsupported dtype for reduce operation"  # core/processgroup.cc:277
    assert rs(fake(4), fake(16), op=2) != 0
    assert core.moodist_last_error() == b"Unsupported reduce operation"  # :294
    assert rs(fake(4, dtype=3), fake(16, dtype=3), op=1) != 0  # AVG of int32
    assert rs(fake(4), fake(16, contiguous=0)) != 0 and b"must be contiguous" in core.moodist_last_error()
    assert rs(fake(4), fake(16, device=-1)) != 0 and b"no CPU fallback" in core.moodist_last_error()
    assert rs(fake(4), fake(16, device=1)) != 0 and b"is on device 1" in core.moodist_last_error()
    assert rs(fake(5), fake(16)) != 0  # output is not input / size
    assert rs(fake(4, dtype=7, itemsize=8), fake(16)) != 0  # dtype mismatch
    assert core.moodist_pg_all_gather(pg, ctypes.byref(fake(15)), ctypes.byref(fake(4)), None,
                                      ctypes.byref(work)) != 0
    assert core.moodist_pg_allreduce(pg, ctypes.byref(fake(7)), None, 0, None, 0.0, ctypes.byref(work)) != 0
    assert b"needs a scratch tensor of 8 elements" in core.moodist_last_error()
    # list form of all_gather: one dense output of the input's size and dtype per rank
    four = (type(fake(4)) * 4)(*[fake(4) for _ in range(4)])
    three = (type(fake(4)) * 3)(*[fake(4) for _ in range(3)])
    assert core.moodist_pg_all_gather_list(pg, three, 3, ctypes.byref(fake(4)), None, ctypes.byref(work)) != 0
    assert b"one output tensor per rank (4), got 3" in core.moodist_last_error()
    four[2] = fake(5)
    assert core.moodist_pg_all_gather_list(pg, four, 4, ctypes.byref(fake(4)), None, ctypes.byref(work)) != 0
    four[2] = fake(4, dtype=7, itemsize=8)
    assert core.moodist_pg_all_gather_list(pg, four, 4, ctypes.byref(fake(4)), None, ctypes.byref(work)) != 0
    four[2] = fake(4, contiguous=0)
    assert core.moodist_pg_all_gather_list(pg, four, 4, ctypes.byref(fake(4)), None, ctypes.byref(work)) != 0
    assert b"must be contiguous" in core.moodist_last_error()
    # a list of all_gathers as one collective: outputs[t] is group size times inputs[t]
    T = type(fake(4))
    ins = (T * 2)(fake(4), fake(6))
    outs = (T * 2)(fake(16), fake(24))
    assert core.moodist_pg_all_gather_many(pg, outs, ins, 0, None, ctypes.byref(work)) != 0
    assert b"1..65535 tensors" in core.moodist_last_error()
    assert core.moodist_pg_all_gather_many(pg, outs, None, 2, None, ctypes.byref(work)) != 0
    outs[1] = fake(23)
    assert core.moodist_pg_all_gather_many(pg, outs, ins, 2, None, ctypes.byref(work)) != 0
    outs[1] = fake(24, contiguous=0)
    assert core.moodist_pg_all_gather_many(pg, outs, ins, 2, None, ctypes.byref(work)) != 0
    assert b"must be contiguous" in core.moodist_last_error()
    ins[0] = fake(4, device=-1)
    assert core.moodist_pg_all_gather_many(pg, None, ins, 2, None, ctypes.byref(work)) != 0
    assert b"no CPU fallback" in core.moodist_last_error()
    # a list of allreduces: every element count a multiple of the group size, a reduce dtype;
    # nothing of the list is posted when one tensor is refused
    ts = (T * 2)(fake(16), fake(24))
    assert core.moodist_pg_allreduce_many(pg, ts, 0, 0, None, 0.0, ctypes.byref(work)) != 0
    assert core.moodist_pg_allreduce_many(pg, None, 2, 0, None, 0.0, ctypes.byref(work)) != 0
    ts[1] = fake(25)
    assert core.moodist_pg_allreduce_many(pg, ts, 2, 0, None, 0.0, ctypes.byref(work)) != 0
    ts[1] = fake(24, dtype=0, itemsize=1)
    assert core.moodist_pg_allreduce_many(pg, ts, 2, 0, None, 0.0, ctypes.byref(work)) != 0
    assert core.moodist_last_error() == b"Unsupported dtype for reduce operation"
    ok = (T * 2)(fake(16), fake(24))
    assert core.moodist_pg_allreduce_many(pg, ok, 2, 0, None, 0.0, ctypes.byref(work)) == 0  # first rank of four: posted
    core.moodist_work_destroy(work)
    core.moodist_world_destroy(w)


def test_a_list_of_all_gathers_must_be_the_same_list_on_every_rank(core):
    # lists of different lengths are different collectives (caught when the second rank posts);
    # lists of the same length and total size but other tensor sizes are caught before the launch
    T = type(fake(4))
    w = make_world(core, 2)
    work = ctypes.c_void_p()
    a, b = core.moodist_world_group(w, 0), core.moodist_world_group(w, 1)
    assert core.moodist_pg_all_gather_many(a, None, (T * 2)(fake(4), fake(6)), 2, None, ctypes.byref(work)) == 0
    core.moodist_work_destroy(work)
    assert core.moodist_pg_all_gather_many(b, None, (T * 1)(fake(10)), 1, None, ctypes.byref(work)) != 0
    assert b"different operation, size, dtype or reduction" in core.moodist_last_error()
    core.moodist_world_destroy(w)
    w = make_world(core, 2)
    a, b = core.moodist_world_group(w, 0), core.moodist_world_group(w, 1)
    assert core.moodist_pg_all_gather_many(a, None, (T * 2)(fake(4), fake(6)), 2, None, ctypes.byref(work)) == 0
    core.moodist_work_destroy(work)
    assert core.moodist_pg_all_gather_many(b, None, (T * 2)(fake(5), fake(5)), 2, None, ctypes.byref(work)) != 0
    assert b"a different list of tensors" in core.moodist_last_error()
    core.moodist_world_destroy(w)


def test_work_is_incomplete_until_every_rank_has_posted(core):
    w = make_world(core, 4)
    works = []
    for r in range(3):  # the fourth rank never calls: nothing is launched, so no GPU is needed
        pg = core.moodist_world_group(w, r)
        work = ctypes.c_void_p()
        assert core.moodist_pg_reduce_scatter(pg, ctypes.byref(fake(4)), ctypes.byref(fake(16)), 0, None, 0.0,
                                              ctypes.byref(work)) == 0, core.moodist_last_error()
        works.append(work)
    for work in works:
        assert core.moodist_work_is_completed(work) == 0
        assert core.moodist_work_wait(work) != 0
        assert b"3 of 4 have" in core.moodist_last_error()
        core.moodist_work_destroy(work)
    core.moodist_world_destroy(w)


def test_mismatched_collectives_are_detected(core):
    # the reference aborts when ranks disagree about a collective (CHECK_DYN, core/cputhread.h:100-112)
    w = make_world(core, 4)
    work = ctypes.c_void_p()
    pg0, pg1 = core.moodist_world_group(w, 0), core.moodist_world_group(w, 1)
    assert core.moodist_pg_reduce_scatter(pg0, ctypes.byref(fake(4)), ctypes.byref(fake(16)), 0, None, 0.0,
                                          ctypes.byref(work)) == 0
    assert core.moodist_pg_all_gather(pg1, ctypes.byref(fake(16)), ctypes.byref(fake(4)), None,
                                      ctypes.byref(work)) != 0
    assert b"different operation" in core.moodist_last_error()
    pg2 = core.moodist_world_group(w, 2)
    assert core.moodist_pg_reduce_scatter(pg2, ctypes.byref(fake(8)), ctypes.byref(fake(32)), 0, None, 0.0,
                                          ctypes.byref(work)) != 0  # other size
    pg3 = core.moodist_world_group(w, 3)
    assert core.moodist_pg_reduce_scatter(pg3, ctypes.byref(fake(4)), ctypes.byref(fake(16)), 4, None, 0.0,
                                          ctypes.byref(work)) != 0  # other reduction
    core.moodist_world_destroy(w)


def test_allreduce_is_one_collective(core):
    # an allreduce takes ONE collective number: after it, the rank's next call is its number 1,
    # and a rank that spells the two halves out does not pair with ranks that call allreduce
    w = make_world(core, 2)
    a, b = core.moodist_world_group(w, 0), core.moodist_world_group(w, 1)
    work = ctypes.c_void_p()
    t = fake(8)
    assert core.moodist_pg_allreduce(a, ctypes.byref(t), None, 0, None, 0.0, ctypes.byref(work)) == 0, core.moodist_last_error()
    assert core.moodist_work_is_completed(work) == 0  # rank 1 has not called
    core.moodist_work_destroy(work)
    # rank 0's number 1 is an all_gather; rank 1's number 0 must be the allreduce, not a reduce_scatter
    assert core.moodist_pg_all_gather(a, ctypes.byref(fake(8)), ctypes.byref(fake(4)), None, ctypes.byref(work)) == 0
    core.moodist_work_destroy(work)
    assert core.moodist_pg_reduce_scatter(b, ctypes.byref(fake(4)), ctypes.byref(fake(8)), 0, None, 0.0,
                                          ctypes.byref(work)) != 0
    assert b"different operation" in core.moodist_last_error()
    # an allreduce of another size or with another reduction is a mismatch as well
    assert core.moodist_pg_allreduce(b, ctypes.byref(fake(16)), None, 0, None, 0.0, ctypes.byref(work)) != 0
    assert core.moodist_pg_allreduce(b, ctypes.byref(fake(8)), None, 4, None, 0.0, ctypes.byref(work)) != 0
    # refused before anything is posted: an operation the type does not take, a missing temporary
    assert core.moodist_pg_allreduce(b, ctypes.byref(fake(8, dtype=3)), None, 1, None, 0.0, ctypes.byref(work)) != 0
    assert b"Unsupported reduce operation" in core.moodist_last_error()
    assert core.moodist_pg_allreduce(b, ctypes.byref(fake(7)), None, 0, None, 0.0, ctypes.byref(work)) != 0
    assert b"needs a scratch tensor of 8 elements" in core.moodist_last_error()
    core.moodist_world_destroy(w)


# ---------------- planner: C++ against the oracle's restatement ----------------

@pytest.mark.parametrize("case", list(_cases()), ids=lambda c: c[0])
def test_cpp_planner_matches_oracle_planner(case):
    _, size, shape, dt, inputs, outputs = case
    tdt = {np.dtype(np.float32): torch.float32, np.dtype(np.float64): torch.float64, np.dtype(np.int32): torch.int32,
           np.dtype(np.int64): torch.int64, np.dtype(np.int16): torch.int16,
           np.dtype(np.uint16): torch.bfloat16}[np.dtype(dt)]
    want = planner.plan(size, shape, np.dtype(dt).itemsize, inputs, outputs)
    world = moodist_amd.LocalWorld(size, 0)
    for r, pg in enumerate(world):
        got = pg.compile_op_full(shape, tdt, inputs, outputs).plan()
        d = want[r]
        assert got["reads"] == [(x.rank, x.inputIndex, x.outputIndex, x.inputOffset, x.outputOffset, x.bytes)
                                for x in d.reads]
        assert got["inputCopies"] == [(c.index, c.offset, c.shape) for c in d.inputCopies]
        assert got["outputCopies"] == [(c.index, c.offset, c.shape) for c in d.outputCopies]
        assert got["inputs"] == d.inputs and got["outputs"] == d.outputs
        # what rank r sends every receiver, byte for byte
        assert got["messages"] == planner.wire(size, shape, np.dtype(dt).itemsize, inputs, outputs)[r]


def test_cpp_planner_random_boxes_match_oracle():
    rng = np.random.RandomState(7)
    for trial in range(60):
        ndim = rng.randint(1, 4)
        shape = [int(rng.randint(2, 9)) for _ in range(ndim)]
        size = int(rng.randint(2, 5))
        # inputs: split one random dimension into `size` slabs (covers the tensor); outputs: random boxes
        d = int(rng.randint(0, ndim))
        cuts = sorted(set([0, shape[d]] + [int(x) for x in rng.randint(0, shape[d] + 1, size - 1)]))
        inputs = []
        for i in range(len(cuts) - 1):
            off = [0] * ndim
            shp = list(shape)
            off[d], shp[d] = cuts[i], cuts[i + 1] - cuts[i]
            inputs.append((i % size, off, shp))
        outputs = []
        for r in range(size):
            off = [int(rng.randint(0, s)) for s in shape]
            shp = [int(rng.randint(1, s - o + 1)) for s, o in zip(shape, off)]
            outputs.append((r, off, shp))
        want = planner.plan(size, shape, 2, inputs, outputs)
        wire = planner.wire(size, shape, 2, inputs, outputs)
        world = moodist_amd.LocalWorld(size, 0)
        for r, pg in enumerate(world):
            got = pg.compile_op_full(shape, torch.bfloat16, inputs, outputs).plan()
            assert got["reads"] == [(x.rank, x.inputIndex, x.outputIndex, x.inputOffset, x.outputOffset, x.bytes)
                                    for x in want[r].reads], (trial, r)
            assert got["inputCopies"] == [(c.index, c.offset, c.shape) for c in want[r].inputCopies]
            assert got["outputCopies"] == [(c.index, c.offset, c.shape) for c in want[r].outputCopies]
            assert got["messages"] == wire[r], (trial, r)


def test_cpp_planner_random_multi_slice_cases_match_oracle():
    # several slices per rank, grids, overlapping outputs: the cases in which staging is reused
    from test_oracle_copy import _random_redistribution

    for seed in range(150):
        rng = np.random.RandomState(seed)
        size = int(rng.randint(1, 6))
        shape, inputs, outputs = _random_redistribution(rng, size)
        want = planner.plan(size, shape, 4, inputs, outputs)
        wire = planner.wire(size, shape, 4, inputs, outputs)
        world = moodist_amd.LocalWorld(size, 0)
        for r, pg in enumerate(world):
            got = pg.compile_op_full(shape, torch.int32, inputs, outputs).plan()
            assert got["reads"] == [(x.rank, x.inputIndex, x.outputIndex, x.inputOffset, x.outputOffset, x.bytes)
                                    for x in want[r].reads], (seed, r)
            assert got["inputCopies"] == [(c.index, c.offset, c.shape) for c in want[r].inputCopies], (seed, r)
            assert got["outputCopies"] == [(c.index, c.offset, c.shape) for c in want[r].outputCopies], (seed, r)
            assert got["messages"] == wire[r], (seed, r)


def test_plan_messages_hand_derived_bytes_and_deserializer_errors(core):
    from test_oracle_copy import WIRE_4X4_COL_TO_ROW_R0_TO_R1, WIRE_4X4_R0_TO_R1, WIRE_4X4_R1_TO_R0

    rows = [(0, [0, 0], [2, 4]), (1, [2, 0], [2, 4])]
    cols = [(0, [0, 0], [4, 2]), (1, [0, 2], [4, 2])]
    world = moodist_amd.LocalWorld(2, 0)
    ops = [pg.compile_op_full([4, 4], torch.float32, rows, cols) for pg in world]
    assert ops[1].plan()["messages"][0] == WIRE_4X4_R1_TO_R0
    assert ops[0].plan()["messages"][1] == WIRE_4X4_R0_TO_R1
    ops = [pg.compile_op_full([4, 4], torch.float32, cols, rows) for pg in world]
    assert ops[0].plan()["messages"][1] == WIRE_4X4_COL_TO_ROW_R0_TO_R1

    core.moodist_plan_message_check.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.c_size_t]
    m = WIRE_4X4_R1_TO_R0
    assert core.moodist_plan_message_check(m, len(m), 2) == 0
    assert core.moodist_plan_message_check(m + b"\0", len(m) + 1, 2) != 0
    assert core.moodist_last_error() == b"deserializeBuffer: 1 trailing bytes"  # core/serialization.h:677-679
    assert core.moodist_plan_message_check(m, len(m) - 1, 2) != 0
    assert core.moodist_last_error() == b"Deserializer: reached end of data"  # :287
    assert core.moodist_plan_message_check(m, len(m), 3) != 0  # the dimension count is not on the wire
    assert core.moodist_plan_message_check(m, 4, 2) != 0
    huge = (2**63).to_bytes(8, "little")
    assert core.moodist_plan_message_check(huge, 8, 2) != 0


def test_planner_errors():
    world = moodist_amd.LocalWorld(2, 0)
    pg = world.groups[0]
    with pytest.raises(RuntimeError, match="could not find input for all output elements"):
        pg.compile_op_full([8], torch.float32, [(0, [0], [4])], [(1, [0], [8])])
    with pytest.raises(RuntimeError, match="ndim 11 is too large and not supported"):
        pg.compile_op_full([1] * 11, torch.float32, [], [])
    with pytest.raises(RuntimeError, match="outside the group"):
        pg.compile_op_full([8], torch.float32, [(2, [0], [8])], [])
    with pytest.raises(RuntimeError, match="listed largest first"):
        pg.compile_op_full([8], torch.float32, [(0, [0], [8])], [(1, [0], [2]), (1, [2], [6])])


def test_custom_op_argument_checks():
    world = moodist_amd.LocalWorld(2, 0)
    op = world.groups[0].compile_op_full([4], torch.float32, [(0, [0], [4])], [(1, [0], [4])])
    x = torch.zeros(4)
    with pytest.raises(RuntimeError, match="custom op expected different number of inputs"):
        op([], [])
    with pytest.raises(RuntimeError, match="custom op expected different number of outputs"):
        op([x], [x])
    with pytest.raises(RuntimeError, match="custom op input has wrong size"):
        op([torch.zeros(5)], [])
    with pytest.raises(RuntimeError, match="Got a non-contiguous tensor"):
        op([torch.zeros(4, 2)[:, 0]], [])
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        op([x], [])


# ---------------- compile_op front end (py/moodist/compile.py:104-264) ----------------

def test_compile_op_validation_messages():
    world = moodist_amd.LocalWorld(2, 0)
    g = world.groups[0]
    f32 = torch.float32
    with pytest.raises(ValueError, match="shape must be provided"):
        moodist_amd.compile_op(g, dtype=f32)
    with pytest.raises(ValueError, match="dtype must be provided"):
        moodist_amd.compile_op(g, shape=[4])
    with pytest.raises(TypeError, match="dtype must be a torch.dtype"):
        moodist_amd.compile_op(g, shape=[4], dtype="float32")
    with pytest.raises(TypeError, match=r"shape\[0\] must be an int"):
        moodist_amd.compile_op(g, shape=[4.0], dtype=f32)
    with pytest.raises(TypeError, match="'offset' must be a tuple or list"):
        moodist_amd.compile_op(g, shape=[4], dtype=f32, inputs=[{"offset": 0, "shape": [4]}])
    with pytest.raises(TypeError, match="must be a dict"):
        moodist_amd.compile_op(g, shape=[4], dtype=f32, inputs=[[0, 4]])
    with pytest.raises(ValueError, match="'shape' is missing"):
        moodist_amd.compile_op(g, shape=[4], dtype=f32, inputs=[{"offset": [0]}])
    with pytest.raises(ValueError, match="expected 'offset' with 1 dimensions, but got 2"):
        moodist_amd.compile_op(g, shape=[4], dtype=f32, inputs=[{"offset": [0, 0], "shape": [4]}])
    with pytest.raises(TypeError, match=r"shape\[0\] must be an int"):
        moodist_amd.compile_op(g, shape=[4], dtype=f32, inputs=[{"offset": [0], "shape": [4.0]}])


def test_compile_op_waits_for_every_rank_and_checks_agreement():
    world = moodist_amd.LocalWorld(2, 0)
    op0 = moodist_amd.compile_op(world.groups[0], shape=[4], dtype=torch.float32,
                                 inputs=[{"offset": [0], "shape": [4]}])
    with pytest.raises(RuntimeError, match="1 of 2 ranks have called compile_op"):
        op0.plan()
    moodist_amd.compile_op(world.groups[1], shape=[4], dtype=torch.float32, outputs=[{"offset": [0], "shape": [4]}])
    assert op0.plan()["inputs"] == [16]
    a = moodist_amd.compile_op(world.groups[0], shape=[4], dtype=torch.float32)
    moodist_amd.compile_op(world.groups[1], shape=[8], dtype=torch.float32)
    with pytest.raises(ValueError, match="Ranks specified different shapes"):
        a.plan()
    a = moodist_amd.compile_op(world.groups[0], shape=[4], dtype=torch.float32)
    moodist_amd.compile_op(world.groups[1], shape=[4], dtype=torch.float64)
    with pytest.raises(ValueError, match="Ranks specified different dtypes"):
        a.plan()


def test_shard_box_matches_oracle_restatement():
    from moodist_amd.compile import shard_box

    for n in (1, 7, 8, 9, 65):
        for k in (1, 2, 3, 8):
            for c in range(k):
                assert shard_box([n, 5], [k], [c], [0]) == planner.shard_box([n, 5], [k], [c], [0])
    assert shard_box([8, 8], [2, 4], [1, 3], [0, 1]) == ([4, 6], [4, 2])
    assert shard_box([8, 8], [2], None, [0]) == ([0, 0], [0, 0])


def test_options_object():
    world = moodist_amd.LocalWorld(2, 0)
    pg = world.groups[1]
    assert pg.options().prefer_kernel_less is False and pg.options().num_chunks is None
    pg.options().prefer_kernel_less = True
    pg.options().num_chunks = 4
    assert pg.get_prefer_kernel_less() and pg.options().num_chunks == 4
    with pg.options(num_chunks=2, force_kernel_less=True) as same:
        assert same is pg and pg.options().num_chunks == 2 and pg.options().force_kernel_less
    assert pg.options().num_chunks == 4 and not pg.options().force_kernel_less
    pg.options().num_chunks = None
    assert pg._get_option("num_chunks") == -1
    with pytest.raises(AttributeError):
        pg.options().bogus
    with pytest.raises(ValueError):
        pg.options(bogus=1)


def test_process_group_is_a_c10d_process_group():
    # reference: the Python type IS a torch.distributed.ProcessGroup (wrapper/module.cc:851-865)
    import torch.distributed as dist

    world = moodist_amd.LocalWorld(3, 0)
    for r, pg in enumerate(world):
        assert isinstance(pg, dist.ProcessGroup) and isinstance(pg, moodist_amd.MoodistProcessGroup)
        assert pg.rank() == r and pg.size() == 3
        assert pg.moodist_name().startswith("moodist-local-%d-of-3-world" % r)
        assert moodist_amd.find_process_group(pg.moodist_name()) is pg
        assert pg.world is world
    assert len({pg.moodist_name() for pg in world}) == 3
    with pytest.raises(RuntimeError, match="send is not supported"):
        world.groups[0].send([torch.zeros(1)], 1, 0)


def test_torch_distributed_functions_take_the_group():
    # torch.distributed's own functions accept the object as group= and reach the overrides; with
    # CPU tensors the core then refuses (this build has no CPU path), which shows where the call went
    import torch.distributed as dist

    pg = moodist_amd.LocalWorld(2, 0).groups[0]
    with pytest.raises(RuntimeError, match="all_gather input is a CPU tensor"):
        dist.all_gather_into_tensor(torch.zeros(4), torch.zeros(2), group=pg)
    with pytest.raises(RuntimeError, match="reduce_scatter input is a CPU tensor"):
        dist.reduce_scatter_tensor(torch.zeros(2), torch.zeros(4), group=pg)
    with pytest.raises(RuntimeError, match="allreduce tensor is a CPU tensor"):
        dist.all_reduce(torch.zeros(4), group=pg)


def test_reference_constructor_joins_ranks_through_the_store():
    # reference: moodist.MoodistProcessGroup(store, rank, size) (wrapper/module.cc:547-566); the ranks that
    # share a store object are the ranks of one group
    import torch.distributed as dist

    store = dist.HashStore()
    pgs = [moodist_amd.MoodistProcessGroup(store, r, 4) for r in range(4)]
    assert [pg.rank() for pg in pgs] == [0, 1, 2, 3] and all(pg.size() == 4 for pg in pgs)
    assert all(pg._store is store for pg in pgs)
    with pytest.raises(RuntimeError, match="rank 2 of this store's group already exists"):
        moodist_amd.MoodistProcessGroup(store, 2, 4)
    other = moodist_amd.MoodistProcessGroup(dist.HashStore(), 0, 4)
    assert other._store is not store
    with pytest.raises(RuntimeError, match="already serves a group of 4 ranks"):
        moodist_amd.MoodistProcessGroup(store, 0, 8)
    with pytest.raises(RuntimeError, match="outside a group"):
        moodist_amd.MoodistProcessGroup(store, 4, 4)
    # a rank that has gone can be made again; a store whose ranks have all gone serves a new group
    del pgs[2]
    pgs.insert(2, moodist_amd.MoodistProcessGroup(store, 2, 4))
    assert pgs[2].rank() == 2
    del pgs, other
    again = moodist_amd.MoodistProcessGroup(store, 0, 8)
    assert again.size() == 8
    pgs = [moodist_amd.MoodistProcessGroup(dist.HashStore(), 0, 4)]
    # prefer_kernel_less as setter and as context manager (py/moodist/backend.py:17-43)
    pg = pgs[0]
    pg.prefer_kernel_less(True)
    assert pg.get_prefer_kernel_less() is True
    with pg.prefer_kernel_less(False):
        assert pg.get_prefer_kernel_less() is False
    assert pg.get_prefer_kernel_less() is True


def test_backend_is_registered_with_torch_distributed():
    # py/moodist/backend.py:71-78, :112-116: "moodist" is a torch.distributed backend whose creator
    # builds the group the reference's way and enters it into the name registry
    import subprocess
    import sys
    from datetime import timedelta

    import torch.distributed as dist

    assert dist.Backend("moodist") == "moodist" and dist.Backend.MOODIST == "moodist"
    assert "MOODIST" in dist.Backend._plugins
    assert dist.Backend.backend_capability["moodist"] == ["cuda"] or tuple(dist.Backend.backend_capability["moodist"]) == ("cuda",)
    creator = dist.Backend._plugins["MOODIST"].creator_fn
    assert creator is moodist_amd.create_moodist_backend
    store = dist.HashStore()
    groups = [creator(store, r, 2, timedelta(seconds=30)) for r in range(2)]
    for r, g in enumerate(groups):
        assert isinstance(g, dist.ProcessGroup) and g.rank() == r and g.size() == 2
        assert moodist_amd.find_process_group(g.moodist_name()) is g
    moodist_amd.register_backend()  # a second call changes nothing
    # init_process_group finds it by name (its own process: the default group is process-wide state)
    code = ("import torch.distributed as dist, moodist_amd\n"
            "dist.init_process_group('moodist', store=dist.HashStore(), rank=0, world_size=1)\n"
            "pg = dist.group.WORLD\n"
            "assert dist.get_backend() == 'moodist' and pg.size() == 1\n"
            "assert moodist_amd.find_process_group(pg.moodist_name()) is pg\n"
            "dist.destroy_process_group()\nprint('ok')\n")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300,
                       cwd=ROOT)
    assert r.returncode == 0 and "ok" in r.stdout, r.stderr[-2000:]


def test_compile_op_accepts_dtensor_like_specs():
    # py/moodist/compile.py:14-59: anything with placements / device_mesh / to_local is read as a
    # DTensor; Shard(dim) placements turn into offset/shape by ceil-division chunks
    from torch.distributed.tensor import Replicate, Shard

    class Mesh:
        def __init__(self, sizes, coord):
            self.sizes, self.coord = sizes, coord

        def size(self, i):
            return self.sizes[i]

        def get_coordinate(self):
            return self.coord

    class FakeDTensor:
        def __init__(self, shape, dtype, placements, mesh):
            self.shape, self.dtype, self.placements, self.device_mesh = torch.Size(shape), dtype, placements, mesh

        def to_local(self):
            raise NotImplementedError

    world = moodist_amd.LocalWorld(2, 0)
    ops = []
    for r, pg in enumerate(world):
        mesh = Mesh([2], [r])
        src = FakeDTensor([5, 4], torch.float32, [Shard(0)], mesh)  # rows 0-2 on rank 0, rows 3-4 on rank 1
        dst = FakeDTensor([5, 4], torch.float32, [Shard(1)], mesh)  # columns 0-1 / 2-3
        ops.append(moodist_amd.compile_op(pg, inputs=[src], outputs=[dst]))
    p0, p1 = ops[0].plan(), ops[1].plan()
    assert p0["inputs"] == [3 * 4 * 4] and p1["inputs"] == [2 * 4 * 4]
    assert p0["outputs"] == [5 * 2 * 4] and p1["outputs"] == [5 * 2 * 4]
    assert sum(rd[5] for rd in p0["reads"]) == 40 and sum(rd[5] for rd in p1["reads"]) == 40
    # replicated placement keeps the whole tensor; mismatching global shapes are refused
    rep = FakeDTensor([5, 4], torch.float32, [Replicate()], Mesh([2], [0]))
    from moodist_amd.compile import _dtensor_box

    assert _dtensor_box(rep) == {"offset": [0, 0], "shape": [5, 4]}
    other = FakeDTensor([6, 4], torch.float32, [Shard(0)], Mesh([2], [0]))
    with pytest.raises(ValueError, match="same global shape"):
        moodist_amd.compile_op(world.groups[0], inputs=[rep], outputs=[other])
    with pytest.raises(ValueError, match="same dtype"):
        moodist_amd.compile_op(world.groups[0], inputs=[rep],
                               outputs=[FakeDTensor([5, 4], torch.float64, [Shard(0)], Mesh([2], [0]))])


def _runs(core, srcs, nbytes, dst=None):
    core.moodist_kernel_less_runs.restype = ctypes.c_int64
    core.moodist_kernel_less_runs.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t, ctypes.c_size_t,
                                              ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64), ctypes.c_size_t]
    tab = (ctypes.c_void_p * len(srcs))(*srcs)
    out = (ctypes.c_int64 * (3 * len(srcs) + 3))()
    n = core.moodist_kernel_less_runs(tab, len(srcs), nbytes, dst, out, len(out))
    return [tuple(out[3 * i:3 * i + 3]) for i in range(n)]


def test_kernel_less_runs_group_evenly_spaced_sources(core):
    # The reference groups the sources a peer holds into Copy2d{offset, length, pitch, num} runs for
    # cuMemcpy2DAsync (core/processgroup.cc:618-704); here the sources are the ranks' own buffers and a
    # run is a stretch of ranks whose buffers are evenly spaced.  (first rank, count, source pitch):
    b, n = 0x7f0000000000, 4096
    # slices of one dense staging buffer: one run whose pitch equals the width (a single 1-D copy)
    assert _runs(core, [b + j * n for j in range(8)], n) == [(0, 8, n)]
    # rows of a padded staging buffer: one 2-D copy
    assert _runs(core, [b + j * (n + 64) for j in range(8)], n) == [(0, 8, n + 64)]
    # two staging buffers of four rows each, with different pitches
    two = [b + j * (n + 64) for j in range(4)] + [b + (1 << 30) + j * (2 * n) for j in range(4)]
    assert _runs(core, two, n) == [(0, 4, n + 64), (4, 4, 2 * n)]
    # unrelated allocations, some closer together than a row is long or in descending order: rank by rank
    odd = [b, b + 100, b + 50, b + (1 << 33), b + (1 << 32)]
    assert _runs(core, odd, n) == [(j, 1, n) for j in range(5)]
    # a pitch that changes mid-way ends the run; the leftover pair forms its own
    bend = [b, b + 2 * n, b + 4 * n, b + 7 * n, b + 10 * n]
    assert _runs(core, bend, n) == [(0, 3, 2 * n), (3, 2, 3 * n)]
    # pitches beyond 31 bits are not handed to a 2-D copy
    assert _runs(core, [b, b + (1 << 31), b + (1 << 32)], n) == [(0, 1, n), (1, 1, n), (2, 1, n)]
    # in-place allreduce: rank 3's chunk already sits in the destination and splits the run
    dst = b + (1 << 34)
    srcs = [b + j * (n + 64) for j in range(8)]
    srcs[3] = dst + 3 * n
    assert _runs(core, srcs, n, dst) == [(0, 3, n + 64), (4, 4, n + 64)]
    assert _runs(core, [], n) == []
