"""Process groups of a local world: every rank of the group lives in this process and on one GPU.

``LocalWorld(size)`` stands for the node.  ``world.groups[r]`` is rank r's
``MoodistProcessGroup``; its collectives are the c10d ones (``_allgather_base``,
``_reduce_scatter_base``, ``allreduce``, the coalesced variants), implemented by the C++ module on
top of the host core.  A collective is launched when the last rank of the world has called it; the
work a rank gets back completes at that moment (``wait()`` before then raises).
"""

import weakref

import torch

from .options import MoodistOptions

_name_to_group = weakref.WeakValueDictionary()  # py/moodist/backend.py:14
_store_worlds = {}  # id(store) -> (store, weak reference to its LocalWorld)


def find_process_group(name):
    """The group whose ``moodist_name()`` is `name`, or None (py/moodist/backend.py:66-68)."""
    return _name_to_group.get(name, None)


class PreferKernelLessContext:
    """Sets prefer_kernel_less at once; restores the old value when used as a context manager
    (py/moodist/backend.py:17-43)."""

    def __init__(self, pg, value):
        self.pg = pg
        self.old_value = pg.get_prefer_kernel_less()
        pg.set_prefer_kernel_less(value)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.pg.set_prefer_kernel_less(self.old_value)
        return False


def _C():
    from . import _C as module  # the pybind11 module; importing it loads libmoodist.so

    return module


class MoodistProcessGroup:
    """Rank `rank` of a LocalWorld.  Attribute access falls through to the underlying
    torch.distributed.ProcessGroup (``.c10d``), whose virtuals the C++ module overrides.

    Extra methods follow the reference's Python type (wrapper/module.cc:836-848).

    Two ways to get one: ``LocalWorld(size).groups[rank]``, or the reference's constructor
    ``MoodistProcessGroup(store, rank, size)`` (wrapper/module.cc:547-566) -- ranks built with the
    same store object are the ranks of one local world, which stands in for the address exchange
    the reference runs through the store.
    """

    def __new__(cls, world_or_store, rank, size=None):
        if isinstance(world_or_store, LocalWorld):
            return super().__new__(cls)
        if size is None:
            raise TypeError("MoodistProcessGroup(store, rank, size): size is required")
        world = _world_of_store(world_or_store, int(size))
        if not 0 <= int(rank) < world.size:
            raise ValueError("rank %d outside a group of %d" % (rank, world.size))
        return world.groups[int(rank)]

    def __init__(self, world_or_store, rank, size=None):
        if not isinstance(world_or_store, LocalWorld):
            return  # built by its world in __new__
        world = world_or_store
        self.world = world
        self.c10d = _C().create_process_group(world._handle, rank)
        self._rank = rank
        _name_to_group[self.moodist_name()] = self

    def prefer_kernel_less(self, value):
        return PreferKernelLessContext(self, value)

    def __getattr__(self, name):
        return getattr(self.c10d, name)

    def moodist_name(self):
        # unique among the groups of this process, as the reference's names are among its groups
        return "%s-world%d" % (_C().moodist_name(self.c10d), self.world.serial)

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


def _world_of_store(store, size):
    entry = _store_worlds.get(id(store))
    world = entry[1]() if entry else None
    if world is None:
        world = LocalWorld(size)
        key = id(store)
        # the store is kept alive with the entry so that its id cannot be reused meanwhile
        _store_worlds[key] = (store, weakref.ref(world, lambda _: _store_worlds.pop(key, None)))
    if world.size != size:
        raise ValueError("this store already serves a group of %d ranks, not %d" % (world.size, size))
    return world


class LocalWorld:
    _count = 0

    def __init__(self, size, device=None):
        if device is None:
            device = torch.cuda.current_device() if torch.cuda.is_available() else 0
        if isinstance(device, torch.device):
            device = device.index or 0
        self.size = int(size)
        self.device = int(device)
        LocalWorld._count += 1
        self.serial = LocalWorld._count
        self._handle = _C().World(self.size, self.device)
        self._compile_round = None
        self.groups = [MoodistProcessGroup(self, r) for r in range(self.size)]

    def __len__(self):
        return self.size

    def __iter__(self):
        return iter(self.groups)
