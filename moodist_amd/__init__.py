"""MI355X-native single-GPU core of Moodist's data-parallel collectives."""

from . import _abi  # noqa: F401
from ._abi import MoodistError  # noqa: F401

__version__ = "0.1.0"
