"""Writes tests/golden/*.npz: seeded inputs and the outputs expected from the hot path.

The reference cannot be imported or built here (its process group needs libcuda and NVML
at construction, core/group.cc:68-70, :102-105), so the expected outputs are produced by
the CPU oracle after the oracle itself has been pinned by tests/test_oracle_*.py, plus the
hand-derived known answers below.  Inputs come from numpy's legacy RandomState, whose
streams are frozen across numpy versions.  16-bit floats are stored as uint16 bit patterns.

Run from the repository root:  python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402


def f32_to_bf16_bits(x):
    u = x.astype(np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def make_sources(rng, P, n, dtype):
    if dtype == oracle.DT_F32:
        return [rng.standard_normal(n).astype(np.float32) for _ in range(P)]
    if dtype == oracle.DT_F64:
        return [rng.standard_normal(n) for _ in range(P)]
    if dtype == oracle.DT_I32:
        return [rng.randint(-2 ** 31, 2 ** 31 - 1, n).astype(np.int32) for _ in range(P)]
    if dtype == oracle.DT_I64:
        return [rng.randint(-2 ** 62, 2 ** 62, n).astype(np.int64) * 3 for _ in range(P)]
    if dtype == oracle.DT_BF16:
        return [f32_to_bf16_bits(rng.standard_normal(n).astype(np.float32) * 1e-3) for _ in range(P)]
    if dtype == oracle.DT_F16:
        return [rng.standard_normal(n).astype(np.float16).view(np.uint16) for _ in range(P)]
    raise ValueError(dtype)


def main():
    rng = np.random.RandomState(20240607)
    cases = {}
    meta = []
    k = 0
    g = 0
    for dtype, n in ((oracle.DT_F32, 1031), (oracle.DT_BF16, 1031), (oracle.DT_F64, 257), (oracle.DT_I32, 257),
                     (oracle.DT_I64, 257), (oracle.DT_F16, 257)):
        for P, first in ((8, 0), (8, 5), (3, 2)):
            floating = dtype in (oracle.DT_F32, oracle.DT_F64, oracle.DT_BF16, oracle.DT_F16)
            ops = [oracle.OP_SUM, oracle.OP_MIN, oracle.OP_MAX] + ([oracle.OP_AVG, oracle.OP_PREMUL_SUM] if floating else [])
            srcs = make_sources(rng, P, n, dtype)
            for op in ops:
                scale = float(np.float32(1.0) / np.float32(P)) if op == oracle.OP_AVG else float(np.float32(0.37))
                out = oracle.reduce(srcs, first, dtype, op, scale)
                cases["c%d_out" % k] = out
                meta.append((k, g, dtype, P, first, op, scale))
                k += 1
            cases["g%d_src" % g] = np.stack(srcs)
            g += 1
    cases["meta"] = np.array(meta, dtype=np.float64)
    np.savez_compressed(os.path.join(HERE, "reduce_cases.npz"), **cases)

    # hand-derived known answers (no oracle involved)
    known = {
        # ((1e8 + 1) + -1e8) + 1 = 1 in fp32, natural order; rotations 1 and 3 give 0
        "order_src": np.array([[1e8], [1.0], [-1e8], [1.0]], dtype=np.float32),
        "order_out_by_first": np.array([1.0, 0.0, 1.0, 0.0], dtype=np.float32),
        # bf16 1 + 2^-8 + 2^-8 -> 1 + 2^-7 (0x3F81) with fp32 accumulation
        "bf16_src": np.array([[0x3F80], [0x3B80], [0x3B80]], dtype=np.uint16),
        "bf16_out": np.array([0x3F81], dtype=np.uint16),
        # reference tests/test_processgroup.py:51-79: ranks contribute rank+1, sum = 36 for P = 8
        "rs_src": np.stack([np.full(4, r + 1, dtype=np.float32) for r in range(8)]),
        "rs_out": np.full(4, 36.0, dtype=np.float32),
    }
    np.savez_compressed(os.path.join(HERE, "known_answers.npz"), **known)
    print("wrote", k, "reduce cases")


if __name__ == "__main__":
    main()
