"""Helpers shared by the tests: dtype tables and torch <-> numpy bit views."""

import numpy as np
import torch

import oracle

TORCH_TO_CODE = {
    torch.float32: oracle.DT_F32,
    torch.float64: oracle.DT_F64,
    torch.int32: oracle.DT_I32,
    torch.int64: oracle.DT_I64,
    torch.bfloat16: oracle.DT_BF16,
    torch.float16: oracle.DT_F16,
}
ALL_DTYPES = list(TORCH_TO_CODE)
OPS = {"SUM": oracle.OP_SUM, "AVG": oracle.OP_AVG, "MIN": oracle.OP_MIN, "MAX": oracle.OP_MAX,
       "PREMUL_SUM": oracle.OP_PREMUL_SUM}


def bits(t):
    """CPU numpy array holding the tensor's bit pattern (16-bit floats as uint16)."""
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def from_bits(a, dtype):
    """Inverse of bits()."""
    if dtype in (torch.bfloat16, torch.float16):
        return torch.from_numpy(a.view(np.int16).copy()).view(dtype)
    return torch.from_numpy(a.copy())


def same_bits(a, b):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype.itemsize == b.dtype.itemsize and \
        np.array_equal(a.view(np.uint8), b.view(np.uint8))


def random_sources(P, n, dtype, seed, scale=3.0):
    g = torch.Generator().manual_seed(seed)
    if dtype.is_floating_point:
        return [(torch.randn(n, generator=g) * scale).to(dtype) for _ in range(P)]
    hi = 2 ** 30
    return [(torch.randint(-hi, hi, (n,), generator=g) * 3).to(dtype) for _ in range(P)]


def fold_order(P, first):
    return [(first + j) % P for j in range(P)]
