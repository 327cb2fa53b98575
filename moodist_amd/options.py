"""Per-process-group options with attribute access and a context manager.

Same surface as the reference's py/moodist/options.py:55-113: ``pg.options().name`` reads,
``pg.options().name = v`` writes, ``with pg.options(name=v):`` overrides for a block.  Booleans
travel as 0/1 and "auto" as -1 (api/processgroup_api.h:35-40).
"""

_BOOL = ("prefer_kernel_less", "force_kernel_less")
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


class MoodistOptionsContext:
    def __init__(self, pg, overrides):
        self._pg = pg
        self._overrides = overrides
        self._saved = {}

    def __enter__(self):
        for name, raw in self._overrides.items():
            self._saved[name] = self._pg._get_option(name)
            self._pg._set_option(name, raw)
        return self._pg

    def __exit__(self, *exc):
        for name, raw in self._saved.items():
            self._pg._set_option(name, raw)
        return False


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
