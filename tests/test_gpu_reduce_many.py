"""Parity of a LIST of reductions in shared launches (mdh_reduce_many) against the CPU oracle, job
by job, through the C ABI.  Same bar as for a single reduction: bit-exact with the oracle for
every dtype and op (the oracle's 16-bit rule is fp32 accumulation, one rounding)."""

import numpy as np
import pytest
import torch

import oracle
from moodist_amd import _abi as abi
from util import ALL_DTYPES, TORCH_TO_CODE, bits, random_sources, same_bits

pytestmark = pytest.mark.gpu


def scale_for(op, P):
    return float(np.float32(1.0) / np.float32(P)) if op == oracle.OP_AVG else float(np.float32(0.37))


def run_jobs(dev, dtype, op, specs, scale, offsets=None):
    """specs: (P, n, first) per job.  Builds seeded sources, runs all jobs in one call and returns
    [(out bits, oracle bits, spec)].  offsets: per job, element offset of every operand inside a
    larger allocation (misalignment)."""
    st = torch.cuda.current_stream().cuda_stream
    jobs, keep, results = [], [], []
    for k, (P, n, first) in enumerate(specs):
        off = 0 if offsets is None else offsets[k]
        srcs = random_sources(P, n, dtype, seed=1000 * k + 31 * P + n)
        dev_full = [torch.zeros(n + off + 64, dtype=dtype, device=dev) for _ in range(P)]
        for f, s in zip(dev_full, srcs):
            f[off:off + n].copy_(s)
        out_full = torch.full((n + off + 64,), 77, dtype=dtype, device=dev)
        keep.append((dev_full, out_full))
        isz = out_full.element_size()
        jobs.append(([f.data_ptr() + off * isz for f in dev_full], first, out_full.data_ptr() + off * isz, n))
        want = oracle.reduce([bits(s) for s in srcs], first, TORCH_TO_CODE[dtype], op, scale) if n else None
        results.append((out_full, off, n, want, (P, n, first)))
    abi.reduce_many(jobs, TORCH_TO_CODE[dtype], op, scale, st)
    torch.cuda.synchronize()
    for out_full, off, n, want, spec in results:
        if n:
            assert same_bits(bits(out_full[off:off + n]), want), (dtype, op, spec)
        # nothing outside the job's elements was written
        guard = torch.full((1,), 77, dtype=dtype)
        assert torch.equal(out_full[:off].cpu(), guard.expand(off)), spec
        assert torch.equal(out_full[off + n:].cpu(), guard.expand(64)), spec


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=str)
def test_ragged_sizes_mixed_source_counts_all_ops(dev, dtype):
    # sizes of the reference's stress test (tests/test_stress.py:241) plus tails, one element, an
    # empty job; 1 to 64 sources in one list (more than one launch's pointer table holds)
    specs = [(8, 1, 3), (3, 7, 0), (8, 64, 7), (1, 255, 0), (16, 1031, 5), (8, 4096 + 5, 2), (64, 70001, 63), (2, 0, 1),
             (7, 65536, 6), (33, 12345, 17), (8, 300000 + 3, 1), (9, 2, 8), (64, 513, 0), (64, 31, 40), (64, 8, 1),
             (17, 100000, 16)]
    for op in (oracle.OP_SUM, oracle.OP_MIN, oracle.OP_MAX, oracle.OP_AVG, oracle.OP_PREMUL_SUM):
        if op in (oracle.OP_AVG, oracle.OP_PREMUL_SUM) and not dtype.is_floating_point:
            continue
        run_jobs(dev, dtype, op, specs, scale_for(op, 8))


def test_more_jobs_than_one_launch_holds(dev):
    # 130 jobs of 8 sources: four launches of at most 40 jobs
    rng = np.random.RandomState(5)
    specs = [(8, int(rng.randint(1, 9000)), int(rng.randint(0, 8))) for _ in range(130)]
    run_jobs(dev, torch.float32, oracle.OP_SUM, specs, 1.0)
    run_jobs(dev, torch.bfloat16, oracle.OP_AVG, specs, scale_for(oracle.OP_AVG, 8))


def test_operands_off_every_grid(dev):
    # element offsets 0..15 of every operand inside its allocation: vectors start wherever the job starts
    specs = [(8, 5000 + k, k % 8) for k in range(16)]
    for dtype in (torch.float32, torch.bfloat16, torch.float64):
        run_jobs(dev, dtype, oracle.OP_SUM, specs, 1.0, offsets=list(range(16)))


def test_a_long_job_in_the_list_gets_its_own_launch(dev):
    # 16 MiB per source and more leaves the shared launches; results are the same either way.  The
    # 12 and 15 MiB jobs stay in them and, with the 4 MiB one, fill more than one launch's share of tiles.
    n_big = (16 << 20) // 4 + 3
    specs = [(4, 1000, 1), (4, n_big, 2), (4, 77, 0), (4, (1 << 20) + 1, 3), (8, (3 << 20) + 5, 7), (8, (15 << 20) // 4, 0)]
    run_jobs(dev, torch.float32, oracle.OP_SUM, specs, 1.0)
    run_jobs(dev, torch.float32, oracle.OP_MAX, specs, 1.0)


@pytest.mark.parametrize("unroll", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("max_blocks", [0, 3])
def test_every_tile_length_and_a_grid_that_walks(dev, unroll, max_blocks):
    old = abi.get_tuning("reduce_unroll"), abi.get_tuning("reduce_max_blocks")
    try:
        abi.set_tuning("reduce_unroll", unroll)
        abi.set_tuning("reduce_max_blocks", max_blocks)
        specs = [(8, 40000 + 3, 1), (5, 12345, 4), (16, 65536, 0), (2, 17, 1), (8, 4096, 7)]
        for dtype in (torch.float32, torch.bfloat16, torch.int64):
            run_jobs(dev, dtype, oracle.OP_SUM, specs, 1.0)
    finally:
        abi.set_tuning("reduce_unroll", old[0])
        abi.set_tuning("reduce_max_blocks", old[1])


def test_in_place_jobs_and_equality_with_single_launches(dev):
    # dst == srcs[first] (what an in-place allreduce passes), and the same bits as mdh_reduce job by job
    st = torch.cuda.current_stream().cuda_stream
    P = 8
    sizes = [257, 4096, 100003, 1]
    for dtype in (torch.float32, torch.float16):
        sets = [[s.to(dev) for s in random_sources(P, n, dtype, seed=n)] for n in sizes]
        singles = []
        for k, srcs in enumerate(sets):
            out = torch.zeros(sizes[k], dtype=dtype, device=dev)
            abi.reduce([s.data_ptr() for s in srcs], k % P, out.data_ptr(), sizes[k], TORCH_TO_CODE[dtype], oracle.OP_SUM, 1.0, st)
            singles.append(out)
        jobs = [([s.data_ptr() for s in srcs], k % P, srcs[k % P].data_ptr(), sizes[k]) for k, srcs in enumerate(sets)]
        abi.reduce_many(jobs, TORCH_TO_CODE[dtype], oracle.OP_SUM, 1.0, st)
        torch.cuda.synchronize()
        for k, srcs in enumerate(sets):
            assert same_bits(bits(srcs[k % P]), bits(singles[k])), (dtype, k)


# ---------------------------------------------------------------- results stored over every source


def run_spread_jobs(dev, dtype, op, specs, scale, offsets=None):
    """mdh_allreduce_many: specs as for run_jobs.  Afterwards EVERY source of a job must hold the
    oracle's result of that job in its first n elements, and nothing else may have changed."""
    st = torch.cuda.current_stream().cuda_stream
    jobs, results = [], []
    for k, (P, n, first) in enumerate(specs):
        off = 0 if offsets is None else offsets[k]
        srcs = random_sources(P, n, dtype, seed=2000 * k + 17 * P + n)
        dev_full = [torch.full((n + off + 64,), 55, dtype=dtype, device=dev) for _ in range(P)]
        for f, s in zip(dev_full, srcs):
            f[off:off + n].copy_(s)
        isz = dev_full[0].element_size()
        jobs.append(([f.data_ptr() + off * isz for f in dev_full], first, 0, n))
        want = oracle.reduce([bits(s) for s in srcs], first, TORCH_TO_CODE[dtype], op, scale) if n else None
        results.append((dev_full, off, n, want, (P, n, first)))
    abi.allreduce_many(jobs, TORCH_TO_CODE[dtype], op, scale, st)
    torch.cuda.synchronize()
    guard = torch.full((1,), 55, dtype=dtype)
    for dev_full, off, n, want, spec in results:
        for r, f in enumerate(dev_full):
            if n:
                assert same_bits(bits(f[off:off + n]), want), (dtype, op, spec, r)
            assert torch.equal(f[:off].cpu(), guard.expand(off)), (spec, r)
            assert torch.equal(f[off + n:].cpu(), guard.expand(64)), (spec, r)


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=str)
def test_spread_ragged_sizes_mixed_source_counts_all_ops(dev, dtype):
    specs = [(8, 1, 3), (3, 7, 0), (8, 64, 7), (1, 255, 0), (16, 1031, 5), (8, 4096 + 5, 2), (64, 70001, 63), (2, 0, 1),
             (7, 65536, 6), (33, 12345, 17), (8, 300000 + 3, 1), (9, 2, 8), (64, 513, 0), (64, 31, 40), (64, 8, 1),
             (17, 100000, 16)]
    for op in (oracle.OP_SUM, oracle.OP_MIN, oracle.OP_MAX, oracle.OP_AVG, oracle.OP_PREMUL_SUM):
        if op in (oracle.OP_AVG, oracle.OP_PREMUL_SUM) and not dtype.is_floating_point:
            continue
        run_spread_jobs(dev, dtype, op, specs, scale_for(op, 8))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.int64], ids=str)
def test_spread_operands_off_the_vector_grid(dev, dtype):
    # every operand of a job starts `off` elements into its allocation: vectors off the 16-byte grid
    specs = [(8, 5000 + k, k % 8) for k in range(9)]
    run_spread_jobs(dev, dtype, oracle.OP_SUM, specs, 1.0, offsets=[0, 1, 2, 3, 5, 7, 9, 11, 13])


def test_spread_is_the_allreduce_of_local_ranks(dev):
    # eight ranks' tensors of 8 x 3001 fp32, one job per chunk c with first = c: every tensor ends up
    # holding what reduce_scatter (chunk c folded in rank c's order) and all_gather would leave
    P, n = 8, 3001
    tensors = random_sources(P, P * n, torch.float32, seed=5)
    d = [t.to(dev) for t in tensors]
    jobs = [([x.data_ptr() + c * n * 4 for x in d], c, 0, n) for c in range(P)]
    abi.allreduce_many(jobs, abi.DTYPE_FLOAT32, abi.OP_SUM, 1.0, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    want = np.concatenate([oracle.reduce([bits(t[c * n:(c + 1) * n]) for t in tensors], c, abi.DTYPE_FLOAT32, oracle.OP_SUM, 1.0)
                           for c in range(P)])
    for x in d:
        assert same_bits(bits(x), want)


def test_spread_long_jobs_are_cut_into_pieces(dev):
    # 40 MiB per source (more than one 32 MiB piece), three sources, element-wise known answer
    n = (40 << 20) // 4 + 3
    g = torch.Generator().manual_seed(9)
    srcs = [torch.randint(-1000, 1000, (n,), dtype=torch.int32, generator=g) for _ in range(3)]
    d = [s.to(dev) for s in srcs]
    abi.allreduce_many([([x.data_ptr() for x in d], 1, 0, n)], abi.DTYPE_INT32, abi.OP_SUM, 1.0,
                       torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    want = srcs[0] + srcs[1] + srcs[2]
    for x in d:
        assert torch.equal(x.cpu(), want)
