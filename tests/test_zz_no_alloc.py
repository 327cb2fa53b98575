"""moodist_pg_allreduce_static, the allreduce that takes its padded temporary from the kernel
library's fixed workspace instead of the caller, against moodist_pg_allreduce given a caller's
temporary: same bits on two calls in a row, the second with a smaller input; its limits.
Called through the C functions of include/moodist_core.h with ctypes.
"""

import ctypes
import os

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "moodist_amd", "libmoodist.so")
KERNEL_LIB = os.path.join(ROOT, "moodist_amd", "libmoodist_hip.so")
WORKSPACE_BYTES = 64 << 20

pytestmark = pytest.mark.gpu

DTYPE = {torch.float32: 6, torch.bfloat16: 15, torch.int32: 3, torch.float64: 7}
SUM, AVG, MAX = 0, 1, 4


class Tensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("numel", ctypes.c_int64), ("itemsize", ctypes.c_int32),
                ("dtype", ctypes.c_int32), ("device", ctypes.c_int32), ("contiguous", ctypes.c_int32),
                ("ndim", ctypes.c_int32), ("reserved", ctypes.c_int32), ("shape", ctypes.c_int64 * 10)]


def describe(t):
    d = Tensor()
    d.data, d.numel, d.itemsize, d.dtype = t.data_ptr(), t.numel(), t.element_size(), DTYPE[t.dtype]
    d.device, d.contiguous, d.ndim = t.device.index, 1, 1
    d.shape[0] = t.numel()
    return d


@pytest.fixture(scope="module")
def core():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    torch.cuda.set_device(0)
    L = ctypes.CDLL(LIB)
    L.moodist_last_error.restype = ctypes.c_char_p
    L.moodist_world_create.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    L.moodist_world_group.restype = ctypes.c_void_p
    L.moodist_world_group.argtypes = [ctypes.c_void_p, ctypes.c_int]
    L.moodist_world_destroy.argtypes = [ctypes.c_void_p]
    L.moodist_pg_allreduce.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                       ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p]
    L.moodist_pg_allreduce_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                              ctypes.c_float, ctypes.c_void_p]
    L.moodist_work_wait.argtypes = [ctypes.c_void_p]
    L.moodist_work_destroy.argtypes = [ctypes.c_void_p]
    return L


class World:
    def __init__(self, core, size):
        self.core, self.size = core, size
        self.handle = ctypes.c_void_p()
        assert core.moodist_world_create(size, 0, ctypes.byref(self.handle)) == 0, core.moodist_last_error()
        self.groups = [core.moodist_world_group(self.handle, r) for r in range(size)]
        self.stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def close(self):
        self.core.moodist_world_destroy(self.handle)

    def with_temporary(self, rank, tensor, temporary, op):
        work = ctypes.c_void_p()
        rc = self.core.moodist_pg_allreduce(self.groups[rank], ctypes.byref(describe(tensor)),
                                            ctypes.byref(describe(temporary)) if temporary is not None else None, op,
                                            self.stream, 0.0, ctypes.byref(work))
        return rc, work

    def static(self, rank, tensor, op):
        work = ctypes.c_void_p()
        rc = self.core.moodist_pg_allreduce_static(self.groups[rank], ctypes.byref(describe(tensor)), op, self.stream,
                                                   0.0, ctypes.byref(work))
        return rc, work

    def finish(self, works):
        for w in works:
            assert self.core.moodist_work_wait(w) == 0, self.core.moodist_last_error()
            self.core.moodist_work_destroy(w)
        torch.cuda.synchronize()


def inputs(size, numel, dtype, seed):
    out = []
    for r in range(size):
        g = torch.Generator().manual_seed(seed * 1000 + r)
        if dtype == torch.int32:
            t = torch.randint(-1000, 1000, (numel,), generator=g, dtype=torch.int32)
        else:
            t = torch.randn(numel, generator=g, dtype=torch.float32).to(dtype)
        out.append(t)
    return out


def bits(t):
    return t.view(torch.int16) if t.dtype == torch.bfloat16 else t.view(torch.int32) if t.element_size() == 4 \
        else t.view(torch.int64)


def both_ways(core, world, numel, dtype, op, seed):
    """The same inputs through moodist_pg_allreduce with a caller's temporary and through
    moodist_pg_allreduce_static; returns the two lists of per-rank results (on the host)."""
    size = world.size
    host = inputs(size, numel, dtype, seed)
    padded = (numel + size - 1) // size * size
    a = [t.cuda() for t in host]
    b = [t.cuda() for t in host]
    temporaries = [torch.empty(padded, dtype=dtype, device="cuda") for _ in range(size)]
    torch.cuda.synchronize()
    works = []
    for r in range(size):
        rc, w = world.with_temporary(r, a[r], temporaries[r] if numel % size else None, op)
        assert rc == 0, core.moodist_last_error()
        works.append(w)
    world.finish(works)
    works = []
    for r in range(size):
        rc, w = world.static(r, b[r], op)
        assert rc == 0, core.moodist_last_error()
        works.append(w)
    world.finish(works)
    return [t.cpu() for t in a], [t.cpu() for t in b], host


def test_two_calls_in_a_row_the_second_smaller_equal_the_allreduce_with_a_callers_temporary(core):
    world = World(core, 8)
    try:
        # 1,000,003 fp32 elements pad to 1,000,008: 4 MB of each rank's 8 MiB slice; then a smaller
        # one, which leaves most of the first call's bytes in the slice
        for call, (numel, seed) in enumerate(((1_000_003, 1), (12_345, 2))):
            print("call", call, "numel", numel, flush=True)
            with_temporary, static, host = both_ways(core, world, numel, torch.float32, SUM, seed)
            for r in range(8):
                assert torch.equal(bits(with_temporary[r]), bits(static[r])), (call, r)
                assert torch.equal(bits(static[r]), bits(static[0]))
            # and the value itself: chunk c is folded in the order c, c+1, ... (rank order from the
            # chunk's owner), checked on the first and the last chunk
            per = (numel + 7) // 8
            for c in (0, 7):
                lo, hi = c * per, min(numel, (c + 1) * per)
                acc = host[c][lo:hi].clone()
                for k in range(1, 8):
                    acc += host[(c + k) % 8][lo:hi]
                assert torch.equal(bits(static[3][lo:hi]), bits(acc)), (call, c)
    finally:
        world.close()


@pytest.mark.parametrize("size,numel,dtype,op", [(3, 100_001, torch.bfloat16, SUM), (5, 77_777, torch.float32, MAX),
                                                 (7, 10, torch.float32, AVG), (4, 999, torch.int32, SUM),
                                                 (8, 4096, torch.float32, SUM), (16, 1_000_001, torch.bfloat16, AVG)])
def test_other_types_operations_and_group_sizes(core, size, numel, dtype, op):
    world = World(core, size)
    try:
        print("size", size, "numel", numel, dtype, "op", op, flush=True)
        with_temporary, static, _ = both_ways(core, world, numel, dtype, op, seed=size)
        for r in range(size):
            assert torch.equal(bits(with_temporary[r]), bits(static[r])), r
    finally:
        world.close()


def test_device_memory_in_use_does_not_change_over_a_call(core):
    world = World(core, 8)
    try:
        numel = 1_500_001  # a 6 MB temporary per rank if one were allocated
        host = inputs(8, numel, torch.float32, 9)
        tensors = [t.cuda() for t in host]

        def run():
            works = []
            for r in range(8):
                rc, w = world.static(r, tensors[r], SUM)
                assert rc == 0, core.moodist_last_error()
                works.append(w)
            world.finish(works)

        run()  # the first call on a device may load the library's code there
        free_before, _ = torch.cuda.mem_get_info()
        for _ in range(3):
            run()
        free_after, _ = torch.cuda.mem_get_info()
        assert free_before - free_after < (2 << 20), (free_before, free_after)
    finally:
        world.close()


def test_back_to_back_calls_with_every_rank_on_its_own_stream(core):
    # Four ranks, each on a stream of its own, two padded allreduces in a row with different
    # data and nothing waited for in between: rank r's second copy into its workspace slice must
    # wait for the other ranks' first reductions, which read that slice on THEIR streams.  With
    # one shared stream that order is the stream's; here it is the events the world places.
    size, numel = 4, 999_999  # pads to 1,000,000: 4 MB of a rank's 16 MiB slice
    world = World(core, size)
    try:
        streams = [torch.cuda.Stream() for _ in range(size)]
        rounds = [inputs(size, numel, torch.float32, seed) for seed in (21, 22)]
        # the answer: moodist_pg_allreduce with a caller's temporary, one round at a time
        want = []
        padded = (numel + size - 1) // size * size
        for host in rounds:
            a = [t.cuda() for t in host]
            temporaries = [torch.empty(padded, dtype=torch.float32, device="cuda") for _ in range(size)]
            torch.cuda.synchronize()
            works = []
            for r in range(size):
                rc, w = world.with_temporary(r, a[r], temporaries[r], SUM)
                assert rc == 0, core.moodist_last_error()
                works.append(w)
            world.finish(works)
            want.append([t.cpu() for t in a])
        tensors = [[t.cuda() for t in host] for host in rounds]
        torch.cuda.synchronize()
        works = []
        for k in range(2):
            print("round", k, flush=True)
            for r in range(size):
                work = ctypes.c_void_p()
                rc = core.moodist_pg_allreduce_static(world.groups[r], ctypes.byref(describe(tensors[k][r])), SUM,
                                                      ctypes.c_void_p(streams[r].cuda_stream), 0.0, ctypes.byref(work))
                assert rc == 0, core.moodist_last_error()
                works.append(work)
        world.finish(works)
        for k in range(2):
            for r in range(size):
                assert torch.equal(bits(tensors[k][r].cpu()), bits(want[k][r])), (k, r)
    finally:
        world.close()


def test_limits(core):
    world = World(core, 8)
    try:
        # each of 8 ranks has 8 MiB: 2,097,152 fp32 elements fit (after padding), one more group of 8 does not
        slice_bytes = WORKSPACE_BYTES // 8
        too_big = torch.zeros(slice_bytes // 4 + 1, dtype=torch.float32, device="cuda")
        rc, _ = world.static(0, too_big, SUM)
        assert rc != 0
        message = core.moodist_last_error()
        assert b"fixed workspace" in message and str(slice_bytes).encode() in message, message
        # a multiple of the group size needs no temporary and is not limited by the workspace
        even = [torch.full((slice_bytes // 4 + 8,), float(r), device="cuda") for r in range(8)]
        works = []
        for r in range(8):
            rc, w = world.static(r, even[r], SUM)
            assert rc == 0, core.moodist_last_error()
            works.append(w)
        world.finish(works)
        assert all(bool((t == 28.0).all()) for t in even)

        # a rank's second call while its first still waits for the other ranks is refused ...
        first = [torch.full((1001,), float(r + 1), device="cuda") for r in range(8)]
        second = torch.ones(1001, device="cuda")
        rc, w0 = world.static(0, first[0], SUM)
        assert rc == 0
        rc, _ = world.static(0, second, SUM)
        assert rc != 0 and b"still waiting" in core.moodist_last_error()
        # ... and changes nothing: the first one completes when the others arrive
        works = [w0]
        for r in range(1, 8):
            rc, w = world.static(r, first[r], SUM)
            assert rc == 0, core.moodist_last_error()
            works.append(w)
        world.finish(works)
        assert all(bool((t == 36.0).all()) for t in first)
        assert bool((second == 1.0).all())
    finally:
        world.close()


def test_workspace_set_up_call(core):
    kernels = ctypes.CDLL(KERNEL_LIB)
    address, size = ctypes.c_void_p(), ctypes.c_size_t()
    assert kernels.mdh_static_workspace(ctypes.byref(address), ctypes.byref(size)) == 0
    assert address.value and address.value % 256 == 0 and size.value == WORKSPACE_BYTES
    again = ctypes.c_void_p()
    assert kernels.mdh_static_workspace(ctypes.byref(again), ctypes.byref(size)) == 0
    assert again.value == address.value
    assert kernels.mdh_static_workspace(None, None) != 0
