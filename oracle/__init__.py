"""TEST INFRASTRUCTURE -- not part of the product.

ctypes/numpy front-end of ``oracle.c`` (the CPU restatement of the reference's
CPU collective path) and of ``planner.py`` (the restatement of the compile_op
planner).  Only tests, the smoke check and the benchmark's cpu_baseline leg may
import this package; the shipped code under ``moodist_amd/`` never does.
"""

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

# torch ScalarType numbers (reference: api/moodist_api.h:30-42)
DT_I32, DT_I64, DT_F16, DT_F32, DT_F64, DT_BF16 = 3, 4, 5, 6, 7, 15
# c10d RedOpType numbers (reference: api/moodist_api.h:45-55)
OP_SUM, OP_AVG, OP_MIN, OP_MAX, OP_PREMUL_SUM = 0, 1, 3, 4, 8

ITEMSIZE = {DT_I32: 4, DT_I64: 8, DT_F16: 2, DT_F32: 4, DT_F64: 8, DT_BF16: 2}
# 16-bit floats travel as raw uint16 bit patterns on the numpy side
NP_DTYPE = {
    DT_I32: np.int32,
    DT_I64: np.int64,
    DT_F16: np.uint16,
    DT_F32: np.float32,
    DT_F64: np.float64,
    DT_BF16: np.uint16,
}


def build(force=False):
    """Compile liboracle.so with the Makefile beside this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vpp = ctypes.POINTER(ctypes.c_void_p)
        L.orc_reduce.argtypes = [vpp, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
                                 ctypes.c_int, ctypes.c_int, ctypes.c_float]
        L.orc_reduce.restype = ctypes.c_int
        L.orc_gather.argtypes = [vpp, ctypes.c_int, ctypes.c_void_p] + [ctypes.c_size_t] * 5
        L.orc_gather.restype = ctypes.c_int
        i64p = ctypes.POINTER(ctypes.c_int64)
        L.orc_copy_box.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, i64p, i64p, i64p, ctypes.c_int]
        L.orc_copy_box.restype = ctypes.c_int
        L.orc_cpu_reduce_scatter_ranks.argtypes = [vpp, vpp, ctypes.c_int, ctypes.c_int, ctypes.c_size_t,
                                                   ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                                   ctypes.POINTER(ctypes.c_double)]
        L.orc_cpu_reduce_scatter_ranks.restype = ctypes.c_double
        L.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_bf16_to_f32.restype = ctypes.c_float
        L.orc_f32_to_f16.argtypes = [ctypes.c_float]
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f16_to_f32.restype = ctypes.c_float
        _lib = L
    return _lib


def _ptr_table(arrays):
    tab = (ctypes.c_void_p * max(len(arrays), 1))()
    for i, a in enumerate(arrays):
        tab[i] = a.ctypes.data
    return tab


def reduce(srcs, first, dtype, op, scale=1.0):
    """srcs: list of equal-length 1-D numpy arrays of NP_DTYPE[dtype]. Returns the folded array."""
    srcs = [np.ascontiguousarray(s, dtype=NP_DTYPE[dtype]) for s in srcs]
    n = srcs[0].size
    assert all(s.size == n for s in srcs)
    out = np.empty(n, dtype=NP_DTYPE[dtype])
    rc = lib().orc_reduce(_ptr_table(srcs), len(srcs), first, out.ctypes.data, n, dtype, op, scale)
    if rc != 0:
        raise ValueError("orc_reduce rejected its arguments (code %d)" % rc)
    return out


def gather(srcs, out, width, rows, src_pitch, dst_pitch, dst_shard_stride):
    """Byte-level 2-D gather into `out` (a writable uint8 numpy array), in place."""
    srcs = [np.ascontiguousarray(s).view(np.uint8).reshape(-1) for s in srcs]
    assert out.dtype == np.uint8 and out.flags.c_contiguous
    rc = lib().orc_gather(_ptr_table(srcs), len(srcs), out.ctypes.data, width, rows, src_pitch, dst_pitch,
                          dst_shard_stride)
    if rc != 0:
        raise ValueError("orc_gather rejected its arguments (code %d)" % rc)
    return out


def all_gather(srcs):
    """Contiguous all-gather of equal-size shards (any dtype), returns uint8 bytes."""
    srcs = [np.ascontiguousarray(s).view(np.uint8).reshape(-1) for s in srcs]
    b = srcs[0].size
    out = np.empty(b * len(srcs), dtype=np.uint8)
    return gather(srcs, out, b, 1, b, b, b)


def copy_box(src, src_off, dst, dst_off, shape, src_strides, dst_strides, itemsize):
    """Element box copy between flat byte buffers; offsets and strides in elements."""
    assert src.dtype == np.uint8 and dst.dtype == np.uint8
    nd = len(shape)
    arr = lambda v: (ctypes.c_int64 * max(nd, 1))(*v)
    rc = lib().orc_copy_box(src.ctypes.data + src_off * itemsize, dst.ctypes.data + dst_off * itemsize, nd,
                            arr(shape), arr(src_strides), arr(dst_strides), itemsize)
    if rc != 0:
        raise ValueError("orc_copy_box rejected its arguments (code %d)" % rc)
    return dst


def cpu_reduce_scatter_seconds(inputs, outputs, nthreads, numel, dtype, op=OP_SUM, reps=3):
    """Time the restated CPU reduce-scatter with `nthreads` rank-threads that live through all
    `reps` repetitions; returns (median seconds, best seconds) per repetition; see oracle.c."""
    best = ctypes.c_double()
    t = lib().orc_cpu_reduce_scatter_ranks(_ptr_table(inputs), _ptr_table(outputs), len(inputs), nthreads, numel,
                                           dtype, op, reps, ctypes.byref(best))
    if t < 0:
        raise ValueError("orc_cpu_reduce_scatter_ranks rejected its arguments")
    return t, best.value
