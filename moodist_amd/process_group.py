"""Process groups of a local world: every rank of the group lives in this process and on one GPU.

``MoodistProcessGroup(store, rank, size)`` is the reference's constructor
(wrapper/module.cc:547-566) and the type is a real ``torch.distributed.ProcessGroup`` subclass,
defined by the C++ module: ``isinstance`` holds and ``torch.distributed`` functions take it as
``group=``.  Ranks built with the same store object are the ranks of one local world -- that
stands in for the address exchange the reference runs through the store.  ``LocalWorld(size)``
builds all ranks of a world at once: ``world.groups[r]`` is rank r's group.

A collective is launched when the last rank of the world has called it; the work a rank gets
back completes at that moment (``wait()`` before then raises).  Until then the core only holds
the posted tensors alive: it does not read them.  What a rank enqueues on its stream between its
own call and the last rank's call therefore runs BEFORE the collective, unlike in c10d; a caller
that modifies an input in that window sets ``pg.options().snapshot_inputs = True``, which copies
every posted input at the call's position in the stream.
"""

import weakref

import torch

from .options import MoodistOptions

_name_to_group = weakref.WeakValueDictionary()  # py/moodist/backend.py:14


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


def _methods(cls):
    """Python-level methods of the C++ type (the reference defines these in its module too,
    wrapper/module.cc:836-848)."""

    def options(self, **kwargs):
        o = MoodistOptions(self)
        return o(**kwargs) if kwargs else o

    def prefer_kernel_less(self, value):
        return PreferKernelLessContext(self, value)

    def stage_input(self, kind, tensor, op=None, premul=0.0):
        """Post this rank's contribution to the next collective without asking for an output:
        the tensor is the staged buffer of a peer whose own result nobody needs here."""
        code = 0 if op is None else int(getattr(op, "value", op))
        return self._stage_input(kind, tensor, code, float(premul))

    cls.options = options
    cls.prefer_kernel_less = prefer_kernel_less
    cls.stage_input = stage_input
    return cls


_type = None


def _group_type():
    """The C++ type, given its Python-level methods and a constructor hook that enters every new
    group into the name registry."""
    global _type
    if _type is None:
        cls = _methods(_C().MoodistProcessGroup)
        make = cls.__init__

        def __init__(self, store, rank, size):
            make(self, store, rank, size)
            _name_to_group[self.moodist_name()] = self

        cls.__init__ = __init__
        _type = cls
    return _type


def create_moodist_backend(store, rank, size, timeout):
    """What ``torch.distributed`` calls to make a group of the "moodist" backend
    (py/moodist/backend.py:71-78): the group is built the reference's way and entered into the
    name registry.  The ranks of one local world are the groups built on one store object."""
    return _group_type()(store, rank, size)


def register_backend():
    """Registers "moodist" with torch.distributed (py/moodist/backend.py:112-116), for GPU tensors
    only: this build has no CPU path.  Importing the package does this once."""
    import torch.distributed as dist

    if not dist.is_available() or "MOODIST" in getattr(dist.Backend, "_plugins", {}):
        return
    dist.Backend.register_backend("moodist", create_moodist_backend, devices=("cuda",))


def __getattr__(name):
    # the type lives in the C++ module, which is only loaded when first needed
    if name == "MoodistProcessGroup":
        return _group_type()
    raise AttributeError(name)


class _WorldKey:
    """Stands for a store when a world is built directly: the groups hold it, its identity names
    the world inside the core."""


class LocalWorld:
    def __init__(self, size, device=None):
        if device is None:
            device = torch.cuda.current_device() if torch.cuda.is_available() else 0
        if isinstance(device, torch.device):
            device = device.index or 0
        self.size = int(size)
        self.device = int(device)
        self._key = _WorldKey()
        cls = _group_type()
        if torch.cuda.is_available() and torch.cuda.current_device() != self.device:
            with torch.cuda.device(self.device):  # the core puts a new world on the current device
                self.groups = [cls(self._key, r, self.size) for r in range(self.size)]
        else:
            self.groups = [cls(self._key, r, self.size) for r in range(self.size)]
        for g in self.groups:
            g.world = self

    def __len__(self):
        return self.size

    def __iter__(self):
        return iter(self.groups)
