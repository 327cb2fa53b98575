"""Pins oracle.c's orc_reduce: reference tests' known answers, closed forms and an
independent torch-CPU fold.  No GPU."""

import numpy as np
import pytest
import torch

import oracle
from util import ALL_DTYPES, TORCH_TO_CODE, bits, fold_order, from_bits, random_sources, same_bits

F32 = oracle.DT_F32


def test_reference_known_answer_sum_of_rank_plus_one():
    # reference tests/test_processgroup.py:51-79: every rank contributes rank+1, P(P+1)/2 comes out
    P, chunk = 8, 4
    for rank in range(P):
        srcs = [np.full(chunk, r + 1, dtype=np.float32) for r in range(P)]
        out = oracle.reduce(srcs, rank, F32, oracle.OP_SUM)
        assert np.array_equal(out, np.full(chunk, P * (P + 1) / 2, dtype=np.float32))


@pytest.mark.parametrize("size", [1, 7, 64, 255, 1024, 4096, 65536])
def test_reference_known_answer_ragged_sizes(size):
    # reference tests/test_stress.py:235-280
    P = 8
    srcs = [np.full(size, r + 1, dtype=np.float32) for r in range(P)]
    out = oracle.reduce(srcs, 3, F32, oracle.OP_SUM)
    assert np.array_equal(out, np.full(size, 36.0, dtype=np.float32))


def test_fold_order_witness_fp32():
    # ((1e8 + 1) + -1e8) + 1 == 1 in fp32; any tree or other order gives 0 or 2
    srcs = [np.array([v], dtype=np.float32) for v in (1e8, 1.0, -1e8, 1.0)]
    assert oracle.reduce(srcs, 0, F32, oracle.OP_SUM)[0] == 1.0
    # rank 2 of 4 folds 2,3,0,1 (core/group.cc:567-570): ((-1e8 + 1) + 1e8) + 1 -> 1 as well,
    # rank 1 folds 1,2,3,0: ((1 + -1e8) + 1) + 1e8 -> 0
    assert oracle.reduce(srcs, 2, F32, oracle.OP_SUM)[0] == 1.0
    assert oracle.reduce(srcs, 1, F32, oracle.OP_SUM)[0] == 0.0
    # rank 3 folds 3,0,1,2: ((1 + 1e8) + 1) + -1e8 -> 0
    assert oracle.reduce(srcs, 3, F32, oracle.OP_SUM)[0] == 0.0


def test_rotation_is_rank_then_higher_then_lower():
    # values chosen so that each of the P rotations gives a different fp32 result
    P = 4
    vals = [3e7, 1.0, -3e7, 0.5]
    srcs = [np.array([v], dtype=np.float32) for v in vals]
    for first in range(P):
        acc = np.float32(vals[first])
        for j in fold_order(P, first)[1:]:
            acc = np.float32(acc + np.float32(vals[j]))
        assert oracle.reduce(srcs, first, F32, oracle.OP_SUM)[0] == acc


def test_bf16_accumulates_in_fp32_and_rounds_once():
    # 1 + 2^-8 + 2^-8: rounding after every add gives 1.0, one rounding gives 1 + 2^-7
    vals = torch.tensor([1.0, 2.0 ** -8, 2.0 ** -8]).bfloat16()
    srcs = [bits(vals[i:i + 1]) for i in range(3)]
    out = from_bits(oracle.reduce(srcs, 0, oracle.DT_BF16, oracle.OP_SUM), torch.bfloat16)
    assert out.item() == 1.0 + 2.0 ** -7
    # the same in fp16 with its 10-bit mantissa: 1 + 2^-11 + 2^-11 -> 1 + 2^-10
    vals = torch.tensor([1.0, 2.0 ** -11, 2.0 ** -11]).half()
    srcs = [bits(vals[i:i + 1]) for i in range(3)]
    out = from_bits(oracle.reduce(srcs, 0, oracle.DT_F16, oracle.OP_SUM), torch.float16)
    assert out.item() == 1.0 + 2.0 ** -10


def test_avg_is_sum_then_one_multiply():
    g = torch.Generator().manual_seed(5)
    for P in (3, 64):
        srcs = [torch.randn(257, generator=g) for _ in range(P)]
        acc = srcs[0].clone()
        for s in srcs[1:]:
            acc.add_(s)
        scale = np.float32(1.0) / np.float32(P)
        want = acc * float(scale)  # torch mul by a Python float on an fp32 tensor multiplies in fp32
        got = oracle.reduce([s.numpy() for s in srcs], 0, F32, oracle.OP_AVG, float(scale))
        assert same_bits(got, want.numpy())
        if P == 64:  # power of two: multiplying by 2^-6 is division
            assert same_bits(got, (acc / 64).numpy())
        else:  # 1/3 is inexact: the product differs from a true division somewhere
            assert not same_bits(got, (acc / 3).numpy())


def test_premul_rounds_each_product_first():
    g = torch.Generator().manual_seed(6)
    srcs = [torch.randn(300, generator=g) for _ in range(5)]
    f = float(np.float32(0.37))
    acc = srcs[2] * f
    for j in fold_order(5, 2)[1:]:
        acc = acc + srcs[j] * f
    got = oracle.reduce([s.numpy() for s in srcs], 2, F32, oracle.OP_PREMUL_SUM, f)
    assert same_bits(got, acc.numpy())


def test_min_max_follow_std_min_max_on_running_value():
    nan = float("nan")
    a = np.array([+0.0, -0.0, nan, 1.0, 2.0], dtype=np.float32)
    b = np.array([-0.0, +0.0, 1.0, nan, 2.0], dtype=np.float32)
    # std::max(a,b) = (a<b)?b:a and std::min(a,b) = (b<a)?b:a keep the running value on ties and NaN
    mx = oracle.reduce([a, b], 0, F32, oracle.OP_MAX)
    mn = oracle.reduce([a, b], 0, F32, oracle.OP_MIN)
    for out in (mx, mn):
        assert np.signbit(out[0]) == False and out[0] == 0  # noqa: E712  +0 came first
        assert np.signbit(out[1]) == True and out[1] == 0  # noqa: E712   -0 came first
        assert np.isnan(out[2])  # NaN running value sticks
        assert out[3] == 1.0  # NaN source is ignored
        assert out[4] == 2.0
    # and with the operands swapped the other one is kept
    mx = oracle.reduce([a, b], 1, F32, oracle.OP_MAX)
    assert np.signbit(mx[0]) and not np.signbit(mx[1]) and mx[2] == 1.0 and np.isnan(mx[3])


def test_integer_sum_wraps_and_minmax_are_signed():
    big = np.array([2 ** 31 - 1, -2 ** 31, 5], dtype=np.int32)
    one = np.array([1, -1, -7], dtype=np.int32)
    assert np.array_equal(oracle.reduce([big, one], 0, oracle.DT_I32, oracle.OP_SUM),
                          np.array([-2 ** 31, 2 ** 31 - 1, -2], dtype=np.int32))
    assert np.array_equal(oracle.reduce([big, one], 0, oracle.DT_I32, oracle.OP_MIN),
                          np.array([1, -2 ** 31, -7], dtype=np.int32))
    assert np.array_equal(oracle.reduce([big, one], 0, oracle.DT_I32, oracle.OP_MAX),
                          np.array([2 ** 31 - 1, -1, 5], dtype=np.int32))
    big = np.array([2 ** 63 - 1], dtype=np.int64)
    assert oracle.reduce([big, np.array([1], dtype=np.int64)], 0, oracle.DT_I64, oracle.OP_SUM)[0] == -2 ** 63


def _torch_fold(srcs, first, dtype, op, scale):
    """Independent witness built from torch-CPU element-wise ops only."""
    order = fold_order(len(srcs), first)
    wide = dtype in (torch.bfloat16, torch.float16)

    def prep(t):
        if op == oracle.OP_PREMUL_SUM:
            t = t * scale  # 16-bit: product rounded to the 16-bit type, as torch does
        return t.float() if wide else t

    acc = prep(srcs[order[0]]).clone()
    for j in order[1:]:
        x = prep(srcs[j])
        if op == oracle.OP_MIN:
            acc = torch.where(x < acc, x, acc)
        elif op == oracle.OP_MAX:
            acc = torch.where(acc < x, x, acc)
        else:
            acc = acc + x
    if wide:
        acc = acc.to(dtype)
    if op == oracle.OP_AVG:
        acc = acc * scale
    return acc


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=str)
@pytest.mark.parametrize("P,first", [(1, 0), (2, 1), (8, 0), (8, 5), (16, 9), (64, 63)])
def test_against_torch_elementwise_fold(dtype, P, first):
    n = 1031
    srcs = random_sources(P, n, dtype, seed=P * 31 + first)
    for name, op in (("SUM", oracle.OP_SUM), ("MIN", oracle.OP_MIN), ("MAX", oracle.OP_MAX),
                     ("AVG", oracle.OP_AVG), ("PREMUL_SUM", oracle.OP_PREMUL_SUM)):
        if op in (oracle.OP_AVG, oracle.OP_PREMUL_SUM) and not dtype.is_floating_point:
            with pytest.raises(ValueError):
                oracle.reduce([bits(s) for s in srcs], first, TORCH_TO_CODE[dtype], op, 0.5)
            continue
        # the reference API carries the factor as a C float (api/processgroup_api.h:45-46)
        scale = float(np.float32(1.0) / np.float32(P)) if op == oracle.OP_AVG else float(np.float32(0.37))
        got = oracle.reduce([bits(s) for s in srcs], first, TORCH_TO_CODE[dtype], op, scale)
        want = _torch_fold(srcs, first, dtype, op, scale)
        assert same_bits(got, bits(want)), (name, dtype)


def test_16bit_conversions_match_torch():
    L = oracle.lib()
    # every bf16 / fp16 pattern widens exactly as torch does
    allbits = np.arange(65536, dtype=np.uint16)
    for dt, up in ((torch.bfloat16, L.orc_bf16_to_f32), (torch.float16, L.orc_f16_to_f32)):
        want = from_bits(allbits, dt).float().numpy()
        got = np.array([up(int(b)) for b in allbits], dtype=np.float32)
        assert same_bits(got[~np.isnan(want)], want[~np.isnan(want)])
        assert np.isnan(got[np.isnan(want)]).all()
    # narrowing: random floats over the whole exponent range plus exact ties
    rng = np.random.RandomState(0)
    f = rng.standard_normal(20000).astype(np.float32) * np.exp2(rng.randint(-30, 20, 20000)).astype(np.float32)
    ties = (np.arange(1, 2000, dtype=np.float32) * np.float32(2.0 ** -9)) + np.float32(1.0)
    f = np.concatenate([f, ties, np.array([0.0, -0.0, np.inf, -np.inf, 65504.0, 65519.9, 65520.0, 1e-8, 6e-8,
                                           3.3e38, 3.4e38], dtype=np.float32)])
    for dt, down in ((torch.bfloat16, L.orc_f32_to_bf16), (torch.float16, L.orc_f32_to_f16)):
        want = bits(torch.from_numpy(f).to(dt))
        got = np.array([down(float(x)) for x in f], dtype=np.uint16)
        assert np.array_equal(got, want)


def test_rejects_bad_arguments():
    x = np.zeros(4, dtype=np.float32)
    with pytest.raises(ValueError):
        oracle.reduce([x], 1, F32, oracle.OP_SUM)  # first out of range
    with pytest.raises(ValueError):
        oracle.reduce([x], 0, F32, 2)  # PRODUCT is not a reduce-scatter op in the reference
    with pytest.raises(KeyError):
        oracle.reduce([x], 0, 0, oracle.OP_SUM)  # uint8 is not a reduce dtype
