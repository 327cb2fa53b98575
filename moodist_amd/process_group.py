"""Process groups of a local world: every rank of the group lives in this process and on one GPU.

``LocalWorld(size)`` stands for the node.  ``world.groups[r]`` is rank r's
``MoodistProcessGroup``; its collectives are the c10d ones (``_allgather_base``,
``_reduce_scatter_base``, ``allreduce``, the coalesced variants), implemented by the C++ module on
top of the host core.  A collective is launched when the last rank of the world has called it; the
work a rank gets back completes at that moment (``wait()`` before then raises).
"""

import torch

from .options import MoodistOptions


def _C():
    from . import _C as module  # the pybind11 module; importing it loads libmoodist.so

    return module


class MoodistProcessGroup:
    """Rank `rank` of a LocalWorld.  Attribute access falls through to the underlying
    torch.distributed.ProcessGroup (``.c10d``), whose virtuals the C++ module overrides.

    Extra methods follow the reference's Python type (wrapper/module.cc:836-848).
    """

    def __init__(self, world, rank):
        self.world = world
        self.c10d = _C().create_process_group(world._handle, rank)
        self._rank = rank

    def __getattr__(self, name):
        return getattr(self.c10d, name)

    def moodist_name(self):
        return _C().moodist_name(self.c10d)

    def _get_option(self, name):
        return _C().get_option(self.c10d, name)

    def _set_option(self, name, value):
        _C().set_option(self.c10d, name, int(value))

    def get_prefer_kernel_less(self):
        return self._get_option("prefer_kernel_less") != 0

    def set_prefer_kernel_less(self, value):
        self._set_option("prefer_kernel_less", 1 if value else 0)

    def options(self, **kwargs):
        o = MoodistOptions(self)
        return o(**kwargs) if kwargs else o

    def compile_op_full(self, shape, dtype, inputs, outputs):
        """inputs/outputs: every rank's (rank, offset, shape) triples (wrapper/module.cc:689-804)."""
        if not isinstance(dtype, torch.dtype):
            raise TypeError("dtype must be a torch.dtype")
        return _C().compile_op_full(self.c10d, [int(x) for x in shape], dtype,
                                    [(int(r), list(o), list(s)) for r, o, s in inputs],
                                    [(int(r), list(o), list(s)) for r, o, s in outputs])

    def stage_input(self, kind, tensor, op=None, premul=0.0):
        """Post this rank's contribution to the next collective without asking for an output:
        the tensor is the staged buffer of a peer whose own result nobody needs here."""
        code = 0 if op is None else int(getattr(op, "value", op))
        return _C().stage_input(self.c10d, kind, tensor, code, float(premul))

    def cuda_barrier(self):
        return None  # one process, one device: stream order is the barrier


class LocalWorld:
    def __init__(self, size, device=None):
        if device is None:
            device = torch.cuda.current_device() if torch.cuda.is_available() else 0
        if isinstance(device, torch.device):
            device = device.index or 0
        self.size = int(size)
        self.device = int(device)
        self._handle = _C().World(self.size, self.device)
        self._compile_round = None
        self.groups = [MoodistProcessGroup(self, r) for r in range(self.size)]

    def __len__(self):
        return self.size

    def __iter__(self):
        return iter(self.groups)
