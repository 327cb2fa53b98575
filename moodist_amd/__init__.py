"""MI355X-native single-GPU core of Moodist's data-parallel collectives.

  LocalWorld / MoodistProcessGroup   the process-group operator surface (reduce_scatter,
                                     all_gather, allreduce) with local peers in one process
  compile_op                         shard redistribution
  _abi                               ctypes binding of the thin C ABI of the kernel library

The GPU kernels live in libmoodist_hip.so; nothing here computes on the CPU.
"""

from . import _abi  # noqa: F401
from ._abi import MoodistError  # noqa: F401
from .compile import compile_op  # noqa: F401
from .options import MoodistOptions, MoodistOptionsContext  # noqa: F401
from .process_group import (LocalWorld, MoodistProcessGroup, PreferKernelLessContext,  # noqa: F401
                            create_moodist_backend, find_process_group, register_backend)

register_backend()  # torch.distributed.init_process_group(backend="moodist", ...) from here on

__version__ = "0.1.0"
