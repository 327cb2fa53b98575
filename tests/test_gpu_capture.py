"""A stream that is being captured into a graph is refused by every launch function of the kernel
library and by every collective of the process group: nothing is enqueued, nothing is recorded,
the capture itself goes on and ends with an empty graph.  The graph is destroyed; it is never
instantiated and nothing is ever replayed."""

import ctypes

import pytest
import torch

import moodist_amd
from moodist_amd import _abi as abi

pytestmark = pytest.mark.gpu

RELAXED = 2  # hipStreamCaptureModeRelaxed: torch's own calls on other streams are left alone


class Capture:
    """hipStreamBeginCapture / hipStreamEndCapture on a torch stream, through the runtime torch
    has loaded.  Leaving the block ends the capture, counts the graph's nodes and destroys it."""

    def __init__(self, stream):
        # the copy of the runtime this process has mapped already (torch's), not a second one
        path = "libamdhip64.so"
        for line in open("/proc/self/maps"):
            if "libamdhip64.so" in line:
                path = line.split()[-1]
                break
        self.hip = ctypes.CDLL(path)
        self.hip.hipStreamBeginCapture.argtypes = [ctypes.c_void_p, ctypes.c_int]
        self.hip.hipStreamEndCapture.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipGraphGetNodes.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_size_t)]
        self.hip.hipGraphDestroy.argtypes = [ctypes.c_void_p]
        self.stream = stream.cuda_stream
        self.nodes = None

    def __enter__(self):
        assert self.hip.hipStreamBeginCapture(self.stream, RELAXED) == 0
        return self

    def __exit__(self, *exc):
        graph = ctypes.c_void_p()
        assert self.hip.hipStreamEndCapture(self.stream, ctypes.byref(graph)) == 0
        n = ctypes.c_size_t(0)
        assert self.hip.hipGraphGetNodes(graph, None, ctypes.byref(n)) == 0
        self.nodes = n.value
        assert self.hip.hipGraphDestroy(graph) == 0
        return False


def test_kernel_library_refuses_a_capturing_stream(dev):
    n = 1 << 16
    srcs = [torch.randn(n, device=dev) for _ in range(4)]
    out = torch.zeros(n, device=dev)
    gathered = torch.zeros(4 * n, device=dev)
    before = out.clone()
    s = torch.cuda.Stream()
    torch.cuda.synchronize()
    ptrs = [x.data_ptr() for x in srcs]
    plan = abi.CopyPlan([abi.make_box(0, 0, [n], [1], [1])], [0], [1], 4, 2)
    with Capture(s) as cap:
        with pytest.raises(abi.MoodistError, match="being captured"):
            abi.reduce(ptrs, 0, out.data_ptr(), n, abi.DTYPE_FLOAT32, abi.OP_SUM, 1.0, s.cuda_stream)
        with pytest.raises(abi.MoodistError, match="being captured"):
            abi.gather(ptrs, gathered.data_ptr(), n * 4, 1, n * 4, n * 4, n * 4, s.cuda_stream)
        with pytest.raises(abi.MoodistError, match="being captured"):
            abi.copy_boxes([abi.make_box(ptrs[0], out.data_ptr(), [n], [1], [1])], 4, s.cuda_stream)
        with pytest.raises(abi.MoodistError, match="being captured"):
            plan.launch([ptrs[0], out.data_ptr()], s.cuda_stream)
        assert abi.lib().mdh_reduce(abi.ptr_table(ptrs), 4, 0, out.data_ptr(), n, abi.DTYPE_FLOAT32, abi.OP_SUM, 1.0,
                                    s.cuda_stream) == 6  # MDH_ECAPTURE
    assert cap.nodes == 0
    torch.cuda.synchronize()
    assert torch.equal(out, before)
    # the same calls on the same stream, now that it is not capturing
    abi.reduce(ptrs, 0, out.data_ptr(), n, abi.DTYPE_FLOAT32, abi.OP_SUM, 1.0, s.cuda_stream)
    s.synchronize()
    want = srcs[0].clone()
    for x in srcs[1:]:
        want += x
    assert torch.equal(out, want)


def test_process_group_refuses_a_capturing_stream(dev):
    P = 4
    world = moodist_amd.LocalWorld(P, dev)
    ins = [torch.full((P * 256,), float(r + 1), device=dev) for r in range(P)]
    outs = [torch.zeros(256, device=dev) for _ in range(P)]
    # one collective outside any capture first: the runtime is loaded from here on
    works = [pg._reduce_scatter_base(outs[r], ins[r]) for r, pg in enumerate(world)]
    for w in works:
        w.wait()
    torch.cuda.synchronize()
    assert torch.equal(outs[0], torch.full((256,), 10.0, device=dev))
    s = torch.cuda.Stream()
    odd = torch.ones(P * 64 + 1, device=dev)
    for o in outs:
        o.zero_()
    torch.cuda.synchronize()
    with Capture(s) as cap:
        with torch.cuda.stream(s):
            with pytest.raises(RuntimeError, match="being captured"):
                world.groups[0]._reduce_scatter_base(outs[0], ins[0])
            with pytest.raises(RuntimeError, match="being captured"):
                world.groups[0]._allgather_base(ins[0], outs[0])
            with pytest.raises(RuntimeError, match="being captured"):
                world.groups[0].allreduce([odd])
    assert cap.nodes == 0
    # nothing of the refused calls is pending: the group goes on as if they had not been made
    works = [pg._reduce_scatter_base(outs[r], ins[r]) for r, pg in enumerate(world)]
    for w in works:
        w.wait()
    torch.cuda.synchronize()
    for r in range(P):
        assert torch.equal(outs[r], torch.full((256,), 10.0, device=dev))
