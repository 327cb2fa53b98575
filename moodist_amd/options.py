"""Per-process-group options with attribute access and a context manager.

Same surface as the reference's py/moodist/options.py:55-113: ``pg.options().name`` reads,
``pg.options().name = v`` writes, ``with pg.options(name=v):`` overrides for a block.  Booleans
travel as 0/1 and "auto" as -1 (api/processgroup_api.h:35-40).  ``snapshot_inputs`` is this
build's addition.
"""

import contextlib

_BOOL = ("prefer_kernel_less", "force_kernel_less", "snapshot_inputs")
_INT = ("num_chunks", "chunk_size", "method")


def _encode(name, value):
    if name in _BOOL:
        return 1 if value else 0
    if name in _INT:
        return -1 if value is None else int(value)
    raise ValueError("Unknown option: %s" % name)


def _decode(name, raw):
    if name in _BOOL:
        return raw != 0
    return None if raw == -1 else raw


@contextlib.contextmanager
def _override(pg, raw_values):
    """Applies the raw values for the duration of a with-block, then puts back what was there
    before, last change first."""
    undo = contextlib.ExitStack()
    with undo:
        for name, raw in raw_values:
            undo.callback(pg._set_option, name, pg._get_option(name))
            pg._set_option(name, raw)
        yield pg


def MoodistOptionsContext(pg, overrides):
    """The context manager ``pg.options(name=value, ...)`` returns; `overrides` maps names to raw
    (encoded) values."""
    return _override(pg, list(overrides.items()))


class MoodistOptions:
    def __init__(self, pg):
        object.__setattr__(self, "_pg", pg)

    def __call__(self, **kwargs):
        return MoodistOptionsContext(self._pg, {k: _encode(k, v) for k, v in kwargs.items()})

    def __getattr__(self, name):
        if name.startswith("_") or name not in _BOOL + _INT:
            raise AttributeError("Unknown option: %s" % name)
        return _decode(name, self._pg._get_option(name))

    def __setattr__(self, name, value):
        if name not in _BOOL + _INT:
            raise AttributeError("Unknown option: %s" % name)
        self._pg._set_option(name, _encode(name, value))
