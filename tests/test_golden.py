"""The committed golden vectors still match the oracle, and the hand-derived answers hold.  No GPU."""

import os

import numpy as np

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))


def load_cases():
    z = np.load(os.path.join(HERE, "golden", "reduce_cases.npz"))
    for k, g, dtype, P, first, op, scale in z["meta"]:
        yield z["g%d_src" % int(g)], z["c%d_out" % int(k)], int(dtype), int(P), int(first), int(op), float(scale)


def test_oracle_reproduces_golden_reduce_cases():
    n = 0
    for srcs, want, dtype, P, first, op, scale in load_cases():
        got = oracle.reduce(list(srcs), first, dtype, op, scale)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (dtype, P, first, op)
        n += 1
    assert n == 78


def test_hand_derived_known_answers():
    z = np.load(os.path.join(HERE, "golden", "known_answers.npz"))
    for first in range(4):
        out = oracle.reduce(list(z["order_src"]), first, oracle.DT_F32, oracle.OP_SUM)
        assert out[0] == z["order_out_by_first"][first]
    assert np.array_equal(oracle.reduce(list(z["bf16_src"]), 0, oracle.DT_BF16, oracle.OP_SUM), z["bf16_out"])
    for first in range(8):
        assert np.array_equal(oracle.reduce(list(z["rs_src"]), first, oracle.DT_F32, oracle.OP_SUM), z["rs_out"])
