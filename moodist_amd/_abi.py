"""ctypes binding of the thin C ABI (include/moodist_hip.h) of libmoodist_hip.so.

The library holds the hand-written gfx950 kernels.  There is no fallback: if
it is missing, loading raises, and every call that fails raises MoodistError
with the library's own message.
"""

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmoodist_hip.so")

# torch ScalarType / c10d RedOpType numbers (include/moodist_hip.h)
DTYPE_INT32, DTYPE_INT64, DTYPE_FLOAT16, DTYPE_FLOAT32, DTYPE_FLOAT64, DTYPE_BFLOAT16 = 3, 4, 5, 6, 7, 15
OP_SUM, OP_AVG, OP_MIN, OP_MAX, OP_PREMUL_SUM = 0, 1, 3, 4, 8
MAX_SOURCES = 64
MAX_DIMS = 10
ABI_VERSION = 2

SYMBOLS = (
    "mdh_abi_version", "mdh_error_string", "mdh_last_error", "mdh_reduce", "mdh_reduce_many", "mdh_allreduce_many", "mdh_gather", "mdh_copy_boxes",
    "mdh_set_tuning", "mdh_get_tuning", "mdh_copy_plan_create", "mdh_copy_plan_launch", "mdh_copy_plan_launches",
    "mdh_copy_plan_verify", "mdh_copy_plan_destroy", "mdh_copy_plan_step_arguments", "mdh_static_workspace",
)


class MoodistError(RuntimeError):
    pass


class Box(ctypes.Structure):
    _fields_ = [
        ("src", ctypes.c_void_p),
        ("dst", ctypes.c_void_p),
        ("ndim", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("shape", ctypes.c_int64 * MAX_DIMS),
        ("src_strides", ctypes.c_int64 * MAX_DIMS),
        ("dst_strides", ctypes.c_int64 * MAX_DIMS),
    ]


class ReduceJob(ctypes.Structure):
    _fields_ = [
        ("srcs", ctypes.POINTER(ctypes.c_void_p)),
        ("nsrc", ctypes.c_int32),
        ("first", ctypes.c_int32),
        ("dst", ctypes.c_void_p),
        ("numel", ctypes.c_size_t),
    ]


_lib = None


def lib():
    """Load libmoodist_hip.so (once). Raises MoodistError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MoodistError(
            "libmoodist_hip.so is not built (%s); run `python -c 'import __graft_entry__ as g; g.build()'` "
            "or moodist_amd/csrc/build.sh" % LIB_PATH)
    L = ctypes.CDLL(LIB_PATH)
    vpp = ctypes.POINTER(ctypes.c_void_p)
    L.mdh_abi_version.restype = ctypes.c_int
    L.mdh_error_string.argtypes = [ctypes.c_int]
    L.mdh_error_string.restype = ctypes.c_char_p
    L.mdh_last_error.restype = ctypes.c_char_p
    L.mdh_reduce.argtypes = [vpp, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int,
                             ctypes.c_int, ctypes.c_float, ctypes.c_void_p]
    L.mdh_reduce.restype = ctypes.c_int
    L.mdh_reduce_many.argtypes = [ctypes.POINTER(ReduceJob), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_float,
                                  ctypes.c_void_p]
    L.mdh_reduce_many.restype = ctypes.c_int
    L.mdh_allreduce_many.argtypes = [ctypes.POINTER(ReduceJob), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_float,
                                  ctypes.c_void_p]
    L.mdh_allreduce_many.restype = ctypes.c_int
    L.mdh_gather.argtypes = [vpp, ctypes.c_int, ctypes.c_void_p] + [ctypes.c_size_t] * 5 + [ctypes.c_void_p]
    L.mdh_gather.restype = ctypes.c_int
    L.mdh_copy_boxes.argtypes = [ctypes.POINTER(Box), ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    L.mdh_copy_boxes.restype = ctypes.c_int
    L.mdh_copy_plan_create.argtypes = [ctypes.POINTER(Box), ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32),
                                       ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_void_p)]
    L.mdh_copy_plan_create.restype = ctypes.c_int
    L.mdh_copy_plan_launch.argtypes = [ctypes.c_void_p, vpp, ctypes.c_int, ctypes.c_void_p]
    L.mdh_copy_plan_launch.restype = ctypes.c_int
    L.mdh_copy_plan_launches.argtypes = [ctypes.c_void_p]
    L.mdh_copy_plan_launches.restype = ctypes.c_int
    L.mdh_copy_plan_verify.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64), ctypes.c_int]
    L.mdh_copy_plan_verify.restype = ctypes.c_int
    L.mdh_copy_plan_destroy.argtypes = [ctypes.c_void_p]
    L.mdh_copy_plan_destroy.restype = None
    u32p = ctypes.POINTER(ctypes.c_uint32)
    L.mdh_copy_plan_step_arguments.argtypes = [ctypes.c_void_p, vpp, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                               ctypes.c_size_t, ctypes.POINTER(ctypes.c_size_t), u32p, u32p, u32p, u32p, u32p]
    L.mdh_copy_plan_step_arguments.restype = ctypes.c_int
    L.mdh_set_tuning.argtypes = [ctypes.c_char_p, ctypes.c_int]
    L.mdh_set_tuning.restype = ctypes.c_int
    L.mdh_get_tuning.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_int)]
    L.mdh_get_tuning.restype = ctypes.c_int
    if L.mdh_abi_version() != ABI_VERSION:
        raise MoodistError("libmoodist_hip.so has ABI version %d, expected %d" % (L.mdh_abi_version(), ABI_VERSION))
    _lib = L
    return L


def check(rc):
    if rc != 0:
        L = lib()
        detail = L.mdh_last_error().decode()
        raise MoodistError(detail or L.mdh_error_string(rc).decode())


def ptr_table(ptrs):
    tab = (ctypes.c_void_p * max(len(ptrs), 1))()
    for i, p in enumerate(ptrs):
        tab[i] = p
    return tab


def reduce(src_ptrs, first, dst_ptr, numel, dtype, op, scale=1.0, stream=0):
    check(lib().mdh_reduce(ptr_table(src_ptrs), len(src_ptrs), first, dst_ptr, numel, dtype, op, scale, stream))


def reduce_jobs(jobs):
    """A ctypes job table for mdh_reduce_many from (src_ptrs, first, dst_ptr, numel) tuples; the
    second value returned keeps the pointer tables alive."""
    arr = (ReduceJob * max(len(jobs), 1))()
    tables = []
    for k, (src_ptrs, first, dst_ptr, numel) in enumerate(jobs):
        tab = ptr_table(src_ptrs)
        tables.append(tab)
        arr[k].srcs = ctypes.cast(tab, ctypes.POINTER(ctypes.c_void_p))
        arr[k].nsrc, arr[k].first, arr[k].dst, arr[k].numel = len(src_ptrs), first, dst_ptr, numel
    return arr, tables


def reduce_many(jobs, dtype, op, scale=1.0, stream=0):
    """jobs: (src_ptrs, first, dst_ptr, numel) tuples, all of one element type and operation."""
    arr, tables = reduce_jobs(jobs)
    check(lib().mdh_reduce_many(arr, len(jobs), dtype, op, scale, stream))
    del tables


def allreduce_many(jobs, dtype, op, scale=1.0, stream=0):
    """The same list with every job's result stored over all of the job's sources (dst_ptr is
    ignored)."""
    arr, tables = reduce_jobs(jobs)
    check(lib().mdh_allreduce_many(arr, len(jobs), dtype, op, scale, stream))
    del tables


def gather(src_ptrs, dst_ptr, width, rows, src_pitch, dst_pitch, dst_shard_stride, stream=0):
    check(lib().mdh_gather(ptr_table(src_ptrs), len(src_ptrs), dst_ptr, width, rows, src_pitch, dst_pitch,
                           dst_shard_stride, stream))


def make_box(src_ptr, dst_ptr, shape, src_strides, dst_strides):
    b = Box()
    b.src, b.dst, b.ndim = src_ptr, dst_ptr, len(shape)
    for d in range(len(shape)):
        b.shape[d], b.src_strides[d], b.dst_strides[d] = shape[d], src_strides[d], dst_strides[d]
    return b


def copy_boxes(boxes, itemsize, stream=0):
    arr = (Box * max(len(boxes), 1))(*boxes)
    check(lib().mdh_copy_boxes(arr, len(boxes), itemsize, stream))


class CopyPlan:
    """A prepared set of box copies (mdh_copy_plan): `boxes` carry byte offsets in src/dst, relative to
    bases[src_slots[i]] / bases[dst_slots[i]] of the table given to launch()."""

    def __init__(self, boxes, src_slots, dst_slots, itemsize, nbases):
        n = len(boxes)
        arr = (Box * max(n, 1))(*boxes)
        ss = (ctypes.c_int32 * max(n, 1))(*src_slots)
        ds = (ctypes.c_int32 * max(n, 1))(*dst_slots)
        self._plan = ctypes.c_void_p()
        self.nbases = nbases
        check(lib().mdh_copy_plan_create(arr, ss, ds, n, itemsize, nbases, ctypes.byref(self._plan)))

    def launch(self, bases, stream=0):
        check(lib().mdh_copy_plan_launch(self._plan, ptr_table(bases), len(bases), stream))

    def verify(self, base_bytes):
        """Host-side replay of the plan's kernels against bases of these sizes (no GPU needed)."""
        arr = (ctypes.c_uint64 * max(len(base_bytes), 1))(*base_bytes)
        check(lib().mdh_copy_plan_verify(self._plan, arr, len(base_bytes)))

    @property
    def launches(self):
        return lib().mdh_copy_plan_launches(self._plan)

    def step_arguments(self, bases, step):
        """What launch number `step` passes for these bases, without enqueuing anything: (argument
        bytes, leading 4-byte scalar parameters among them, grid x, grid y, block, LDS bytes)."""
        buf = ctypes.create_string_buffer(4096)
        size = ctypes.c_size_t()
        lead, gx, gy, block, lds = (ctypes.c_uint32() for _ in range(5))
        check(lib().mdh_copy_plan_step_arguments(self._plan, ptr_table(bases), len(bases), step, buf, len(buf),
                                                 ctypes.byref(size), ctypes.byref(lead), ctypes.byref(gx),
                                                 ctypes.byref(gy), ctypes.byref(block), ctypes.byref(lds)))
        return buf.raw[:size.value], lead.value, gx.value, gy.value, block.value, lds.value

    def __del__(self):
        if getattr(self, "_plan", None):
            lib().mdh_copy_plan_destroy(self._plan)
            self._plan = None


def set_tuning(name, value):
    check(lib().mdh_set_tuning(name.encode(), value))


def get_tuning(name):
    v = ctypes.c_int()
    check(lib().mdh_get_tuning(name.encode(), ctypes.byref(v)))
    return v.value
