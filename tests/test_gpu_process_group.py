"""The process-group operator surface on the GPU, written the way the reference's own tests
are (tests/test_processgroup.py, tests/test_stress.py): every rank of an 8-rank group makes the
call, here from one process.  Results are also checked against the CPU oracle, rank by rank, with
the fold starting at the rank itself."""

import numpy as np
import pytest
import torch
import torch.distributed as dist

import moodist_amd
import oracle
from util import TORCH_TO_CODE, bits, random_sources, same_bits

pytestmark = pytest.mark.gpu
P = 8


@pytest.fixture()
def world(dev):
    return moodist_amd.LocalWorld(P, dev)


def each_rank(world, fn):
    """Runs fn(rank, pg) for every rank (the body of an SPMD test), then waits on all works."""
    works = [fn(r, pg) for r, pg in enumerate(world)]
    for w in works:
        if w is not None:
            w.wait()
    torch.cuda.synchronize()


def test_pg_creation(world):
    # reference tests/test_processgroup.py:13-18
    for r, pg in enumerate(world):
        assert pg.rank() == r and pg.size() == P


def test_groups_built_the_reference_way(dev):
    # reference tests/framework.py builds each rank's group as MoodistProcessGroup(store, rank, size)
    store = dist.HashStore()
    pgs = [moodist_amd.MoodistProcessGroup(store, r, P) for r in range(P)]
    ins = [torch.full((1024,), float(r + 1), device=dev) for r in range(P)]
    outs = [torch.zeros(128, device=dev) for _ in range(P)]
    works = [pg._reduce_scatter_base(outs[r], ins[r]) for r, pg in enumerate(pgs)]
    for w in works:
        w.wait()
    torch.cuda.synchronize()
    for r in range(P):
        assert torch.equal(outs[r], torch.full((128,), 36.0, device=dev))


@pytest.mark.parametrize("kernel_less", [False, True])
def test_pg_allgather_base(world, dev, kernel_less):
    # reference tests/test_processgroup.py:21-48 (kernel and kernel-less modes)
    chunk = 4
    ins = [torch.full((chunk,), float(r), device=dev) for r in range(P)]
    outs = [torch.zeros(chunk * P, device=dev) for _ in range(P)]
    for pg in world:
        pg.options().force_kernel_less = kernel_less
    each_rank(world, lambda r, pg: pg._allgather_base(outs[r], ins[r]))
    expected = torch.cat([torch.full((chunk,), float(r), device=dev) for r in range(P)])
    for r in range(P):
        assert torch.equal(outs[r], expected)


def test_pg_reduce_scatter_base(world, dev):
    # reference tests/test_processgroup.py:51-79
    chunk = 4
    ins = [torch.full((chunk * P,), float(r + 1), device=dev) for r in range(P)]
    outs = [torch.zeros(chunk, device=dev) for _ in range(P)]
    each_rank(world, lambda r, pg: pg._reduce_scatter_base(outs[r], ins[r]))
    for r in range(P):
        assert torch.equal(outs[r], torch.full((chunk,), P * (P + 1) / 2, device=dev))


def test_pg_allgather_varying_data(world, dev):
    # reference tests/test_processgroup.py:82-109
    chunk = 8
    ins = [torch.arange(r * 100, r * 100 + chunk, device=dev, dtype=torch.float32) for r in range(P)]
    outs = [torch.zeros(chunk * P, device=dev) for _ in range(P)]
    each_rank(world, lambda r, pg: pg._allgather_base(outs[r], ins[r]))
    for q in range(P):
        for r in range(P):
            assert torch.equal(outs[q][r * chunk:(r + 1) * chunk], ins[r])


def test_pg_large_allgather(world, dev):
    # reference tests/test_processgroup.py:112-146
    chunk = 256 * 1024
    ins = []
    for r in range(P):
        torch.manual_seed(r + 42)
        ins.append(torch.randn(chunk).to(dev))
    outs = [torch.zeros(chunk * P, device=dev) for _ in range(P)]
    each_rank(world, lambda r, pg: pg._allgather_base(outs[r], ins[r]))
    for q in range(P):
        for r in range(P):
            torch.manual_seed(r + 42)
            assert torch.equal(outs[q][r * chunk:(r + 1) * chunk].cpu(), torch.randn(chunk))


def test_pg_allreduce_sum_and_varying(world, dev):
    # reference tests/test_processgroup.py:201-248
    ts = [torch.full((8,), float(r + 1), device=dev) for r in range(P)]
    each_rank(world, lambda r, pg: pg.allreduce([ts[r]]))
    for t in ts:
        assert torch.equal(t, torch.full((8,), P * (P + 1) / 2, device=dev))
    ts = [torch.arange(r, r + 4, device=dev, dtype=torch.float32) for r in range(P)]
    each_rank(world, lambda r, pg: pg.allreduce([ts[r]]))
    want = torch.tensor([P * (P - 1) / 2 + i * P for i in range(4)], device=dev)
    for t in ts:  # 4 elements over 8 ranks: the padded-temporary path
        assert torch.equal(t, want)


def test_allreduce_matches_oracle_composition(world, dev):
    # allreduce = reduce_scatter into the rank's own chunk + all_gather (core/processgroup.cc:1674-1722):
    # chunk c of the result is the fold that starts at rank c
    for n in (8 * 1000, 8 * 1000 + 3):
        srcs = random_sources(P, n, torch.float32, seed=n)
        padded = (n + P - 1) // P * P
        chunk = padded // P
        full = [torch.cat([s, torch.zeros(padded - n)]) for s in srcs]
        want = np.concatenate([oracle.reduce([f[c * chunk:(c + 1) * chunk].numpy() for f in full], c, oracle.DT_F32,
                                             oracle.OP_SUM) for c in range(P)])[:n]
        ts = [s.to(dev) for s in srcs]
        each_rank(world, lambda r, pg: pg.allreduce([ts[r]]))
        for t in ts:
            assert same_bits(bits(t), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.int32, torch.int64, torch.bfloat16], ids=str)
def test_reduce_scatter_every_rank_matches_oracle_in_its_own_order(world, dev, dtype):
    n = 5000 + 3
    srcs = random_sources(P, P * n, dtype, seed=21)
    ins = [s.to(dev) for s in srcs]
    for name, c10d_op, code in (("SUM", dist.ReduceOp.SUM, oracle.OP_SUM), ("MIN", dist.ReduceOp.MIN, oracle.OP_MIN),
                                ("MAX", dist.ReduceOp.MAX, oracle.OP_MAX), ("AVG", dist.ReduceOp.AVG, oracle.OP_AVG)):
        if code == oracle.OP_AVG and not dtype.is_floating_point:
            continue
        outs = [torch.zeros(n, dtype=dtype, device=dev) for _ in range(P)]
        opts = dist.ReduceScatterOptions()
        opts.reduceOp = c10d_op
        each_rank(world, lambda r, pg: pg._reduce_scatter_base(outs[r], ins[r], opts))
        scale = float(np.float32(1.0) / np.float32(P))
        for q in range(P):
            want = oracle.reduce([bits(s[q * n:(q + 1) * n]) for s in srcs], q, TORCH_TO_CODE[dtype], code, scale)
            assert same_bits(bits(outs[q]), want), (name, q)


def test_reduce_scatter_premul_sum(world, dev):
    n = 4096
    srcs = random_sources(P, P * n, torch.float32, seed=5)
    ins = [s.to(dev) for s in srcs]
    outs = [torch.zeros(n, device=dev) for _ in range(P)]
    opts = dist.ReduceScatterOptions()
    opts.reduceOp = dist._make_nccl_premul_sum(0.37)
    each_rank(world, lambda r, pg: pg._reduce_scatter_base(outs[r], ins[r], opts))
    f = float(np.float32(0.37))
    for q in range(P):
        want = oracle.reduce([s[q * n:(q + 1) * n].numpy() for s in srcs], q, oracle.DT_F32, oracle.OP_PREMUL_SUM, f)
        assert same_bits(bits(outs[q]), want)


def test_unsupported_requests_raise(world, dev):
    x = torch.zeros(P * 4, device=dev)
    o = torch.zeros(4, device=dev)
    opts = dist.ReduceScatterOptions()
    opts.reduceOp = dist.ReduceOp.PRODUCT
    with pytest.raises(RuntimeError, match="Unsupported reduce operation"):
        world.groups[0]._reduce_scatter_base(o, x, opts)
    with pytest.raises(RuntimeError, match="Unsupported dtype for reduce operation"):
        world.groups[0]._reduce_scatter_base(o.to(torch.uint8), x.to(torch.uint8))
    with pytest.raises(RuntimeError, match="must be contiguous"):
        world.groups[0]._reduce_scatter_base(o, torch.zeros(P * 4, 2, device=dev)[:, 0])
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        world.groups[0]._reduce_scatter_base(o.cpu(), x.cpu())


def test_work_before_all_ranks_called_is_incomplete(world, dev):
    ins = [torch.ones(P * 4, device=dev) for _ in range(P)]
    outs = [torch.zeros(4, device=dev) for _ in range(P)]
    works = [world.groups[r]._reduce_scatter_base(outs[r], ins[r]) for r in range(P - 1)]
    assert not works[0].is_completed()
    with pytest.raises(RuntimeError, match="7 of 8 have"):
        works[0].wait()
    last = world.groups[P - 1]._reduce_scatter_base(outs[P - 1], ins[P - 1])
    for w in works + [last]:
        assert w.is_completed()
        w.wait()
    torch.cuda.synchronize()
    assert all(torch.equal(o, torch.full((4,), float(P), device=dev)) for o in outs)


def test_one_ranks_share_with_staged_peers(world, dev):
    # the benchmark's shape: only rank 0 wants its output; ranks 1..7 are staged contributions
    n = 100000
    srcs = random_sources(P, P * n, torch.float32, seed=8)
    ins = [s.to(dev) for s in srcs]
    out = torch.zeros(n, device=dev)
    for r in range(1, P):
        world.groups[r].stage_input("reduce_scatter", ins[r])
    world.groups[0]._reduce_scatter_base(out, ins[0]).wait()
    torch.cuda.synchronize()
    want = oracle.reduce([s[:n].numpy() for s in srcs], 0, oracle.DT_F32, oracle.OP_SUM)
    assert same_bits(bits(out), want)
    # and the gather
    shards = [s[:n].contiguous().to(dev) for s in srcs]
    g = torch.zeros(P * n, device=dev)
    for r in range(1, P):
        world.groups[r].stage_input("all_gather", shards[r])
    world.groups[0]._allgather_base(g, shards[0]).wait()
    torch.cuda.synchronize()
    assert torch.equal(g.cpu(), torch.cat([s[:n] for s in srcs]))


def test_coalesced_variants(world, dev):
    sizes = (4, 1000, 33)
    ins = [[torch.full((n,), float(r + 1), device=dev) for n in sizes] for r in range(P)]
    outs = [[torch.zeros(n * P, device=dev) for n in sizes] for _ in range(P)]
    each_rank(world, lambda r, pg: pg.allgather_into_tensor_coalesced(outs[r], ins[r]))
    for r in range(P):
        for k, n in enumerate(sizes):
            assert torch.equal(outs[r][k], torch.arange(1, P + 1, device=dev).float().repeat_interleave(n))
    rins = [[torch.full((n * P,), float(r + 1), device=dev) for n in sizes] for r in range(P)]
    routs = [[torch.zeros(n, device=dev) for n in sizes] for _ in range(P)]
    each_rank(world, lambda r, pg: pg.reduce_scatter_tensor_coalesced(routs[r], rins[r]))
    for r in range(P):
        for k, n in enumerate(sizes):
            assert torch.equal(routs[r][k], torch.full((n,), 36.0, device=dev))


@pytest.mark.parametrize("kernel_less", [False, True])
def test_allgather_coalesced_many_tensors_of_awkward_sizes_and_types(world, dev, kernel_less):
    # a list of tensors is ONE collective whose copies share launches (the reference loops,
    # wrapper/processgroup_wrapper.cc:139-148): 40 tensors, sizes with and without whole vectors,
    # three element types, one tensor already in place in its rank's output
    for pg in world:
        pg.options().force_kernel_less = kernel_less
    try:
        g = torch.Generator().manual_seed(4)
        sizes = [1, 2, 3, 7, 8, 15, 16, 17, 31, 64, 100, 255, 1000, 1023, 4096, 4099, 65536, 70001, 5, 9] * 2
        dtypes = [torch.float32, torch.bfloat16, torch.int64]
        ins = [[(torch.randn(n, generator=g) * 100).to(dtypes[k % 3]).to(dev) for k, n in enumerate(sizes)]
               for r in range(P)]
        outs = [[torch.zeros(n * P, dtype=dtypes[k % 3], device=dev) for k, n in enumerate(sizes)] for _ in range(P)]
        for r in range(P):  # tensor 14 of every rank already sits in its slot of that rank's output
            outs[r][14][r * sizes[14]:(r + 1) * sizes[14]] = ins[r][14]
            ins[r][14] = outs[r][14][r * sizes[14]:(r + 1) * sizes[14]]
        each_rank(world, lambda r, pg: pg.allgather_into_tensor_coalesced(outs[r], ins[r]))
        torch.cuda.synchronize()
        for k in range(len(sizes)):
            want = torch.cat([ins[j][k] for j in range(P)])
            for r in range(P):
                assert torch.equal(outs[r][k], want), (k, sizes[k], r)
    finally:
        for pg in world:
            pg.options().force_kernel_less = False


@pytest.mark.parametrize("kernel_less", [False, True])
def test_allgather_into_a_list_of_tensors(world, dev, kernel_less):
    # c10d's list form (reference wrapper/processgroup_wrapper.cc:112-129): outputs[j] = rank j's input.
    # Sizes with and without a 16-byte body and tail; one output is the rank's own input (in place).
    for pg in world:
        pg.options().force_kernel_less = kernel_less
    for n in (1, 7, 4096, 100003):
        g = torch.Generator().manual_seed(n)
        ins = [torch.randn(n, generator=g).to(dev) for _ in range(P)]
        outs = [[ins[r] if j == r else torch.zeros(n, device=dev) for j in range(P)] for r in range(P)]
        each_rank(world, lambda r, pg: pg.allgather([outs[r]], [ins[r]]))
        for r in range(P):
            for j in range(P):
                assert torch.equal(outs[r][j], ins[j]), (n, r, j)


def test_allgather_list_through_torch_distributed_api_shapes(world, dev):
    # 2-d inputs, bf16: the list form keeps each output's own shape
    ins = [torch.full((3, 5), float(r), device=dev, dtype=torch.bfloat16) for r in range(P)]
    outs = [[torch.empty(3, 5, device=dev, dtype=torch.bfloat16) for _ in range(P)] for _ in range(P)]
    each_rank(world, lambda r, pg: pg.allgather([outs[r]], [ins[r]]))
    for r in range(P):
        for j in range(P):
            assert torch.equal(outs[r][j], ins[j])
    with pytest.raises(RuntimeError, match="one output tensor per rank"):
        world.groups[0].allgather([outs[0][:3]], [ins[0]])


def test_allreduce_coalesced(world, dev):
    # reference wrapper/processgroup_wrapper.cc:182-191: one allreduce per tensor, in order
    sizes = (8, 1001, 4096)  # 1001 is not a multiple of 8: padded temporary
    ts = [[torch.arange(n, device=dev, dtype=torch.float32) * (r + 1) for n in sizes] for r in range(P)]
    each_rank(world, lambda r, pg: pg.allreduce_coalesced(ts[r]))
    for r in range(P):
        for k, n in enumerate(sizes):
            assert torch.equal(ts[r][k], torch.arange(n, device=dev, dtype=torch.float32) * 36.0)


@pytest.mark.parametrize("snapshot", [False, True])
def test_allreduce_coalesced_divisible_tensors_share_one_gather(world, dev, snapshot):
    # tensors whose sizes divide by the group size are reduced one by one and gathered together
    # (moodist_pg_allreduce_many); the others, and a tensor of another element type, take one
    # allreduce each.  Random values against the oracle's composition: chunk q of a tensor is
    # folded starting at rank q (reference core/processgroup.cc:1674-1722).
    for pg in world:
        pg.options().snapshot_inputs = snapshot
    g = torch.Generator().manual_seed(9)
    sizes = [8, 16, 1001, 4096, 8 * 1000, 24, 7, 65536, 8 * 12345, 40]
    dtypes = [torch.float32] * 9 + [torch.bfloat16]
    for name, code, op in (("SUM", oracle.OP_SUM, dist.ReduceOp.SUM), ("MAX", oracle.OP_MAX, dist.ReduceOp.MAX),
                           ("AVG", oracle.OP_AVG, dist.ReduceOp.AVG)):
        host = [[(torch.randn(n, generator=g) * 3).to(dt) for n, dt in zip(sizes, dtypes)] for _ in range(P)]
        ts = [[t.to(dev) for t in row] for row in host]
        opts = dist.AllreduceCoalescedOptions()
        opts.reduceOp = op
        works = []
        for r, pg in enumerate(world):
            works.append(pg.allreduce_coalesced(ts[r], opts))
        for w in works:
            w.wait()
        torch.cuda.synchronize()
        for k, (n, dt) in enumerate(zip(sizes, dtypes)):
            padded = (n + P - 1) // P * P
            c = padded // P
            pin = [torch.cat([host[r][k], torch.zeros(padded - n, dtype=dt)]) for r in range(P)]
            want = np.concatenate([oracle.reduce([bits(t[q * c:(q + 1) * c]) for t in pin], q, TORCH_TO_CODE[dt], code,
                                                 1.0 / P if code == oracle.OP_AVG else 1.0) for q in range(P)])[:n]
            for r in range(P):
                assert same_bits(bits(ts[r][k]), want), (name, k, n, r)
    for pg in world:
        pg.options().snapshot_inputs = False


def test_ranks_on_different_streams(world, dev):
    # each rank posts on its own stream; the launches must still see every rank's input
    n = 1 << 20
    streams = [torch.cuda.Stream(device=dev) for _ in range(P)]
    ins, outs = [None] * P, [None] * P
    torch.cuda.synchronize()
    works = []
    for r, pg in enumerate(world):
        with torch.cuda.stream(streams[r]):
            ins[r] = torch.full((P * n,), float(r + 1), device=dev)  # produced on the rank's own stream
            outs[r] = torch.zeros(n, device=dev)
            works.append(pg._reduce_scatter_base(outs[r], ins[r]))
    for w in works:
        w.wait()
    for r in range(P):
        streams[r].synchronize()
        assert torch.equal(outs[r], torch.full((n,), 36.0, device=dev))


@pytest.mark.parametrize("n", [1000, 100_000, 600_000])
def test_ranks_on_two_streams_share_launches_stream_by_stream(world, dev, n):
    # ranks 0-3 post on one stream, ranks 4-7 on another: short collectives (the first two sizes)
    # go out as one launch per stream with a job per rank, long ones as one launch per rank; either
    # way every rank's data is produced on its own stream and must be seen by all launches
    streams = [torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)]
    host = [torch.stack(random_sources(P, n, torch.float32, seed=7 * r + n)).reshape(-1) for r in range(P)]
    ins, outs, full, sums = [None] * P, [None] * P, [None] * P, [None] * P
    torch.cuda.synchronize()
    works = []
    for r, pg in enumerate(world):
        with torch.cuda.stream(streams[r // 4]):
            ins[r] = host[r].to(dev, non_blocking=False) * 1.0  # produced on the rank's stream
            outs[r] = torch.zeros(n, device=dev)
            works.append(pg._reduce_scatter_base(outs[r], ins[r]))
    for r, pg in enumerate(world):
        with torch.cuda.stream(streams[r // 4]):
            full[r] = torch.zeros(P * n, device=dev)
            works.append(pg._allgather_base(full[r], outs[r]))
    for r, pg in enumerate(world):
        with torch.cuda.stream(streams[r // 4]):
            sums[r] = ins[r].clone()
            works.append(pg.allreduce([sums[r]]))
    for w in works:
        w.wait()
    torch.cuda.synchronize()
    chunks = [oracle.reduce([bits(host[j][q * n:(q + 1) * n]) for j in range(P)], q, oracle.DT_F32, oracle.OP_SUM)
              for q in range(P)]
    for q in range(P):
        assert same_bits(bits(outs[q]), chunks[q]), q
        assert same_bits(bits(full[q]), np.concatenate(chunks)), q
        assert same_bits(bits(sums[q]), np.concatenate(chunks)), q


# ---- reference tests/test_stress.py ----

def test_stress_rapid_collectives(world, dev):
    # :16-82: 100 iterations, pre-allocated tensors, tight loop
    iters, chunk = 100, 256
    ag_in = [[torch.full((chunk,), float(r), device=dev) for _ in range(iters)] for r in range(P)]
    ag_out = [[torch.zeros(chunk * P, device=dev) for _ in range(iters)] for _ in range(P)]
    rs_in = [[torch.full((chunk * P,), float(r + 1), device=dev) for _ in range(iters)] for r in range(P)]
    rs_out = [[torch.zeros(chunk, device=dev) for _ in range(iters)] for _ in range(P)]
    for i in range(iters):
        for r, pg in enumerate(world):
            pg._allgather_base(ag_out[r][i], ag_in[r][i])
        for r, pg in enumerate(world):
            pg._reduce_scatter_base(rs_out[r][i], rs_in[r][i])
    torch.cuda.synchronize()
    want = torch.arange(P, device=dev).float().repeat_interleave(chunk)
    for r in range(P):
        for i in range(iters):
            assert torch.equal(ag_out[r][i], want)
            assert torch.equal(rs_out[r][i], torch.full((chunk,), 36.0, device=dev))


def test_stress_mixed_collectives(world, dev):
    # :146-232 without the broadcast (outside this path): all_gather, reduce_scatter, allreduce and
    # barrier interleaved in a tight loop
    iters, chunk = 50, 32
    ag_in = [[torch.full((chunk,), float(r), device=dev) for _ in range(iters)] for r in range(P)]
    ag_out = [[torch.zeros(chunk * P, device=dev) for _ in range(iters)] for _ in range(P)]
    rs_in = [[torch.full((chunk * P,), float(r + 1), device=dev) for _ in range(iters)] for r in range(P)]
    rs_out = [[torch.zeros(chunk, device=dev) for _ in range(iters)] for _ in range(P)]
    ar = [[torch.full((chunk,), float(r + 1), device=dev) for _ in range(iters)] for r in range(P)]
    for i in range(iters):
        each_rank(world, lambda r, pg: pg._allgather_base(ag_out[r][i], ag_in[r][i]))
        each_rank(world, lambda r, pg: pg._reduce_scatter_base(rs_out[r][i], rs_in[r][i]))
        each_rank(world, lambda r, pg: pg.allreduce([ar[r][i]]))
        each_rank(world, lambda r, pg: pg.barrier())
    want = torch.arange(P, device=dev).float().repeat_interleave(chunk)
    for r in range(P):
        for i in range(iters):
            assert torch.equal(ag_out[r][i], want)
            assert torch.equal(rs_out[r][i], torch.full((chunk,), 36.0, device=dev))
            assert torch.equal(ar[r][i], torch.full((chunk,), 36.0, device=dev))
    with pytest.raises(RuntimeError, match="broadcast .* is not supported"):
        world.groups[0].broadcast([ar[0][0]])


def test_stress_varying_sizes(world, dev):
    # :235-280
    for size in (1, 7, 64, 255, 1024, 4096, 65536):
        ag_in = [torch.full((size,), float(r), device=dev) for r in range(P)]
        ag_out = [torch.zeros(size * P, device=dev) for _ in range(P)]
        rs_in = [torch.full((size * P,), float(r + 1), device=dev) for r in range(P)]
        rs_out = [torch.zeros(size, device=dev) for _ in range(P)]
        each_rank(world, lambda r, pg: pg._allgather_base(ag_out[r], ag_in[r]))
        each_rank(world, lambda r, pg: pg._reduce_scatter_base(rs_out[r], rs_in[r]))
        for q in range(P):
            for r in range(P):
                assert (ag_out[q][r * size:(r + 1) * size] == float(r)).all()
            assert torch.equal(rs_out[q], torch.full((size,), 36.0, device=dev))


def test_stress_large_tensors(world, dev):
    # :283-313: 4 MiB per rank
    chunk = 1024 * 1024
    ins = [torch.full((chunk,), float(r), device=dev) for r in range(P)]
    outs = [torch.zeros(chunk * P, device=dev) for _ in range(P)]
    for _ in range(3):
        each_rank(world, lambda r, pg: pg._allgather_base(outs[r], ins[r]))
    for q in range(P):
        assert torch.equal(outs[q], torch.arange(P, device=dev).float().repeat_interleave(chunk))


# ---- through the plugin entry: the core's table, torch.distributed's own functions, lifetimes ----


def test_reduce_scatter_through_the_core_api_table_matches_the_oracle(world, dev):
    # _C resolves one symbol, moodistGetApi, and calls processGroupReduceScatter through the table it
    # returns (reference: wrapper/moodist_loader.cc:363-386, wrapper/processgroup_wrapper.cc:150-157);
    # here via torch.distributed's own function with the group passed as group=
    from moodist_amd import _C

    assert _C.core_api_info()["entry"] == "moodistGetApi"
    n = 40000 + 3  # ragged: not a multiple of 16 bytes
    srcs = random_sources(P, P * n, torch.float32, seed=11)
    ins = [s.to(dev) for s in srcs]
    outs = [torch.zeros(n, device=dev) for _ in range(P)]
    # async_op=True: the blocking form waits on the work at once, which a single thread playing
    # every rank cannot do before the other ranks have called
    works = []
    for r, pg in enumerate(world):
        assert isinstance(pg, dist.ProcessGroup)
        works.append(dist.reduce_scatter_tensor(outs[r], ins[r], group=pg, async_op=True))
    for w in works:
        w.wait()
    torch.cuda.synchronize()
    for r in range(P):
        chunks = [bits(s[r * n:(r + 1) * n]) for s in srcs]
        assert same_bits(bits(outs[r]), oracle.reduce(chunks, r, oracle.DT_F32, oracle.OP_SUM))


def test_all_gather_and_all_reduce_through_torch_distributed(world, dev):
    n = 1000
    ins = [torch.arange(r * n, (r + 1) * n, device=dev, dtype=torch.float32) for r in range(P)]
    outs = [torch.zeros(P * n, device=dev) for _ in range(P)]
    works = [dist.all_gather_into_tensor(outs[r], ins[r], group=pg, async_op=True) for r, pg in enumerate(world)]
    ts = [torch.full((P * 13 + 5,), float(r + 1), device=dev) for r in range(P)]  # needs the padded temporary
    works += [dist.all_reduce(ts[r], group=pg, async_op=True) for r, pg in enumerate(world)]
    for w in works:
        w.wait()
    torch.cuda.synchronize()
    for r in range(P):
        assert torch.equal(outs[r], torch.arange(P * n, device=dev, dtype=torch.float32))
        assert torch.equal(ts[r], torch.full((P * 13 + 5,), P * (P + 1) / 2, device=dev))


def test_posted_tensors_outlive_their_python_references(world, dev):
    # A rank posts and drops every reference to its tensors; many other allocations follow before
    # the peers arrive.  The core holds the posted tensors until the launch (the reference ties
    # their lifetime to the operation, core/processgroup.cc:3239-3245), so the caching allocator
    # cannot hand their memory out in between.
    n = 1 << 16
    srcs = random_sources(P, P * n, torch.float32, seed=5)
    outs = [torch.zeros(n, device=dev) for _ in range(P)]

    def post_and_forget(r):
        t = srcs[r].to(dev)
        world.groups[r]._reduce_scatter_base(outs[r], t)

    post_and_forget(0)
    torch.cuda.synchronize()
    churn = [torch.full((P * n,), 7.0, device=dev) for _ in range(100)]  # would reuse a freed input's block
    del churn
    for r in range(1, P):
        post_and_forget(r)
    torch.cuda.synchronize()
    for r in range(P):
        chunks = [bits(s[r * n:(r + 1) * n]) for s in srcs]
        assert same_bits(bits(outs[r]), oracle.reduce(chunks, r, oracle.DT_F32, oracle.OP_SUM))


def test_allreduce_coalesced_many_tensors_of_awkward_sizes(world, dev):
    # 48 tensors none of whose sizes divides by the group size: every one goes through a padded
    # temporary that must live until the LAST rank has made its call
    sizes = [P * k + 1 + (k % (P - 1)) for k in range(1, 49)]
    assert all(s % P for s in sizes)
    per_rank = [[torch.full((s,), float(r + 1) + 0.25 * i, device=dev) for i, s in enumerate(sizes)] for r in range(P)]
    works = [pg.allreduce_coalesced(per_rank[r]) for r, pg in enumerate(world)]
    for w in works:
        w.wait()
    torch.cuda.synchronize()
    for r in range(P):
        for i, s in enumerate(sizes):
            want = sum(float(q + 1) + 0.25 * i for q in range(P))
            assert torch.equal(per_rank[r][i], torch.full((s,), want, device=dev)), (r, i)


def test_input_changed_between_a_ranks_call_and_the_launch(world, dev):
    # The collective is launched when the last rank calls, on stream order at THAT moment: what a
    # rank does to its input after its own call but before the last rank's call is seen by the
    # collective (c10d and the reference see the value at call time).  snapshot_inputs copies
    # every posted input at the call's position in the stream and restores c10d's meaning.
    n = 4096
    for snapshot in (False, True):
        for pg in world:
            pg.options().snapshot_inputs = snapshot
        ins = [torch.full((P * n,), float(r + 1), device=dev) for r in range(P)]
        outs = [torch.zeros(n, device=dev) for _ in range(P)]
        works = []
        for r, pg in enumerate(world):
            works.append(pg._reduce_scatter_base(outs[r], ins[r]))
            if r == 0:
                ins[0].fill_(100.0)  # after rank 0's call, before the launch
        for w in works:
            w.wait()
        torch.cuda.synchronize()
        first = 1.0 if snapshot else 100.0
        want = first + sum(float(q + 1) for q in range(1, P))
        for r in range(P):
            assert torch.equal(outs[r], torch.full((n,), want, device=dev)), (snapshot, r)
    for pg in world:
        pg.options().snapshot_inputs = False


def test_snapshot_inputs_with_allreduce_and_allgather(world, dev):
    for pg in world:
        pg.options().snapshot_inputs = True
    n = 999  # not divisible: padded temporary
    ts = [torch.full((n,), float(r + 1), device=dev) for r in range(P)]
    ev = [torch.full((P * 64,), float(r + 1), device=dev) for r in range(P)]
    ins = [torch.full((100,), float(r), device=dev) for r in range(P)]
    outs = [torch.zeros(P * 100, device=dev) for _ in range(P)]
    for r, pg in enumerate(world):
        pg.allreduce([ts[r]])
        pg.allreduce([ev[r]])
        pg._allgather_base(outs[r], ins[r])
        ins[r].fill_(-1.0)  # after the call: must not be seen
    # a coalesced list is snapshotted tensor by tensor
    cins = [[torch.full((k + 5,), float(10 * r + k), device=dev) for k in range(3)] for r in range(P)]
    couts = [[torch.zeros(P * (k + 5), device=dev) for k in range(3)] for _ in range(P)]
    for r, pg in enumerate(world):
        pg.allgather_into_tensor_coalesced(couts[r], cins[r])
        for t in cins[r]:
            t.fill_(-1.0)
    torch.cuda.synchronize()
    for r in range(P):
        assert torch.equal(ts[r], torch.full((n,), P * (P + 1) / 2, device=dev))
        assert torch.equal(ev[r], torch.full((P * 64,), P * (P + 1) / 2, device=dev))
        assert torch.equal(outs[r], torch.arange(P, device=dev, dtype=torch.float32).repeat_interleave(100))
        for k in range(3):
            want = torch.cat([torch.full((k + 5,), float(10 * j + k), device=dev) for j in range(P)])
            assert torch.equal(couts[r][k], want), (r, k)


def test_kernel_less_gather_from_padded_staging_equals_the_kernel_path(world, dev):
    # The ranks' inputs are rows of ONE padded staging buffer (pitch > row bytes): with
    # force_kernel_less the core groups them into a single hipMemcpy2DAsync (the reference's Copy2d +
    # cuMemcpy2DAsync form, core/processgroup.cc:114-119, :618-704, :806-820); the kernel path
    # moves the same rows as strided boxes.  Same bytes either way.
    n, pad = 50000 + 3, 29
    g = torch.Generator().manual_seed(3)
    staging = torch.randn(P, n + pad, generator=g).to(dev)
    ins = [staging[r, :n] for r in range(P)]
    assert all(t.is_contiguous() for t in ins)
    results = {}
    for kernel_less in (False, True):
        for pg in world:
            pg.options().force_kernel_less = kernel_less
        before = (world.groups[0]._get_option("kernel_less_copies_1d"), world.groups[0]._get_option("kernel_less_copies_2d"))
        outs = [torch.full((P * n,), -1.0, device=dev) for _ in range(P)]
        each_rank(world, lambda r, pg: pg._allgather_base(outs[r], ins[r]))
        after = (world.groups[0]._get_option("kernel_less_copies_1d"), world.groups[0]._get_option("kernel_less_copies_2d"))
        results[kernel_less] = outs
        # one 2-D copy per rank's output in the kernel-less form, none in the kernel form
        assert (after[0] - before[0], after[1] - before[1]) == ((0, P) if kernel_less else (0, 0))
    want = staging[:, :n].reshape(-1)
    for r in range(P):
        assert torch.equal(results[False][r], want) and torch.equal(results[True][r], want)
    # dense staging (pitch == row bytes): one 1-D copy of everything; separate allocations: one per rank
    dense = torch.randn(P, n, generator=g).to(dev)
    separate = [torch.randn(n, generator=g).to(dev) for _ in range(P)]
    for ins2, want2, expect in (([dense[r] for r in range(P)], dense.reshape(-1), (P, 0)),
                                (separate, torch.cat(separate), None)):
        before = (world.groups[0]._get_option("kernel_less_copies_1d"), world.groups[0]._get_option("kernel_less_copies_2d"))
        outs = [torch.zeros(P * n, device=dev) for _ in range(P)]
        each_rank(world, lambda r, pg: pg._allgather_base(outs[r], ins2[r]))
        after = (world.groups[0]._get_option("kernel_less_copies_1d"), world.groups[0]._get_option("kernel_less_copies_2d"))
        if expect:
            assert (after[0] - before[0], after[1] - before[1]) == expect
        for r in range(P):
            assert torch.equal(outs[r], want2)
    for pg in world:
        pg.options().force_kernel_less = False


def test_kernel_less_gather_of_rows_far_apart(world, dev):
    # Rows of 75,002 bytes at a pitch of 3,669,242 bytes: a shape the runtime's 2-D copy has been
    # seen to refuse when it checks its arguments.  Whether it takes it (one 2-D copy per rank's
    # output) or not (the run then goes rank by rank), the bytes must be the gather's.
    width, pitch = 75002, 3669242
    g = torch.Generator().manual_seed(8)
    staging = torch.randint(0, 256, (P * pitch,), dtype=torch.uint8, generator=g).to(dev)
    ins = [staging[r * pitch:r * pitch + width] for r in range(P)]
    for pg in world:
        pg.options().force_kernel_less = True
    try:
        c = lambda: (world.groups[0]._get_option("kernel_less_copies_1d"), world.groups[0]._get_option("kernel_less_copies_2d"))
        before = c()
        outs = [torch.zeros(P * width, dtype=torch.uint8, device=dev) for _ in range(P)]
        each_rank(world, lambda r, pg: pg._allgather_base(outs[r], ins[r]))
        after = c()
        want = torch.cat(ins)
        for r in range(P):
            assert torch.equal(outs[r], want), r
        # per rank's output: one 2-D copy, or eight copies of one row each
        assert (after[0] - before[0], after[1] - before[1]) in ((0, P), (P * P, 0))
    finally:
        for pg in world:
            pg.options().force_kernel_less = False


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.int64], ids=str)
def test_reduce_scatter_coalesced_is_one_collective_and_matches_the_oracle(world, dev, dtype):
    # reference wrapper/processgroup_wrapper.cc:159-170 runs one reduce_scatter per tensor; here a
    # list of one element type is one collective whose reductions share launches.  Rank q's
    # output k is the fold of every rank's chunk q of tensor k, starting at rank q.
    g = torch.Generator().manual_seed(17)
    chunk_sizes = [1, 7, 64, 255, 1031, 4096 + 5, 70001, 3, 100000, 12, 513, 8191] * 4  # 48 tensors
    ops = [("SUM", oracle.OP_SUM, dist.ReduceOp.SUM), ("MAX", oracle.OP_MAX, dist.ReduceOp.MAX)]
    if dtype.is_floating_point:
        ops.append(("AVG", oracle.OP_AVG, dist.ReduceOp.AVG))
    for name, code, op in ops:
        if dtype.is_floating_point:
            host = [[(torch.randn(n * P, generator=g) * 3).to(dtype) for n in chunk_sizes] for _ in range(P)]
        else:
            host = [[torch.randint(-2 ** 40, 2 ** 40, (n * P,), generator=g) for n in chunk_sizes] for _ in range(P)]
        ins = [[t.to(dev) for t in row] for row in host]
        outs = [[torch.zeros(n, dtype=dtype, device=dev) for n in chunk_sizes] for _ in range(P)]
        opts = dist.ReduceScatterOptions()
        opts.reduceOp = op
        each_rank(world, lambda r, pg: pg.reduce_scatter_tensor_coalesced(outs[r], ins[r], opts))
        for k, n in enumerate(chunk_sizes):
            for q in range(P):
                want = oracle.reduce([bits(host[j][k][q * n:(q + 1) * n]) for j in range(P)], q, TORCH_TO_CODE[dtype], code,
                                     1.0 / P if code == oracle.OP_AVG else 1.0)
                assert same_bits(bits(outs[q][k]), want), (name, k, n, q)
        for r in range(P):  # inputs untouched
            assert torch.equal(ins[r][5].cpu(), host[r][5])


def test_reduce_scatter_coalesced_of_mixed_element_types_goes_tensor_by_tensor(world, dev):
    dtypes = [torch.float32, torch.int32, torch.float32]
    n = 1000
    ins = [[torch.full((n * P,), r + 1, device=dev).to(dt) for dt in dtypes] for r in range(P)]
    outs = [[torch.zeros(n, dtype=dt, device=dev) for dt in dtypes] for _ in range(P)]
    each_rank(world, lambda r, pg: pg.reduce_scatter_tensor_coalesced(outs[r], ins[r]))
    for r in range(P):
        for k, dt in enumerate(dtypes):
            assert torch.equal(outs[r][k], torch.full((n,), 36, device=dev).to(dt))


@pytest.mark.parametrize("option,value", [("num_chunks", 3), ("num_chunks", 64), ("chunk_size", 8192), ("chunk_size", 100000),
                                          ("method", 2)])
def test_chunk_options_cut_a_reduce_scatter_into_pieces_with_the_same_bits(world, dev, option, value):
    # The options the reference stores for its direct method (core/processgroup.cc:334-340) are
    # honoured here: the rank's chunk is reduced in pieces -- chunk_size bytes, or num_chunks
    # pieces by the reference's arithmetic (:1494-1503), or with method 2 the reference's own
    # count -- and the result is the unchunked fold, bit for bit.
    for pg in world:
        setattr(pg.options(), option, value)
    try:
        for dtype, n in ((torch.float32, 200003), (torch.bfloat16, 333337), (torch.float32, 1000), (torch.float64, 70001)):
            host = [torch.stack(random_sources(P, n, dtype, seed=31 * r + n)).reshape(-1) for r in range(P)]
            ins = [t.to(dev) for t in host]
            outs = [torch.zeros(n, dtype=dtype, device=dev) for _ in range(P)]
            each_rank(world, lambda r, pg: pg._reduce_scatter_base(outs[r], ins[r]))
            for q in range(P):
                want = oracle.reduce([bits(host[j][q * n:(q + 1) * n]) for j in range(P)], q, TORCH_TO_CODE[dtype],
                                     oracle.OP_SUM)
                assert same_bits(bits(outs[q]), want), (option, value, dtype, n, q)
    finally:
        for pg in world:
            setattr(pg.options(), option, None)
    with pytest.raises(RuntimeError, match=r"method 1 \(copy\)"):
        world.groups[0].options().method = 1


def test_init_process_group_with_the_moodist_backend(dev):
    # reference py/moodist/backend.py:112-116: torch.distributed finds the backend by name.  In a
    # process of its own: the default group is process-wide state.
    import os
    import subprocess
    import sys

    code = """
import torch, torch.distributed as dist
import moodist_amd
dist.init_process_group("moodist", store=dist.HashStore(), rank=0, world_size=1)
assert dist.get_backend() == "moodist"
x = torch.arange(1000, dtype=torch.float32, device="cuda") + 1
dist.all_reduce(x)
out = torch.zeros(1000, device="cuda")
dist.all_gather_into_tensor(out, x)
shard = torch.zeros(1000, device="cuda")
dist.reduce_scatter_tensor(shard, x)
torch.cuda.synchronize()
want = torch.arange(1000, dtype=torch.float32, device="cuda") + 1
assert torch.equal(x, want) and torch.equal(out, want) and torch.equal(shard, want)
assert moodist_amd.find_process_group(dist.group.WORLD.moodist_name()) is dist.group.WORLD
dist.destroy_process_group()
print("ok")
"""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300, cwd=root)
    assert r.returncode == 0 and "ok" in r.stdout, (r.stdout[-1000:], r.stderr[-3000:])


# ---------------------------------------------------------------- allreduce: one launch, or its two halves


def allreduce_want(srcs, n, dtype, op, scale):
    """What allreduce leaves in every rank's tensor: chunk c is the fold that starts at rank c
    (core/processgroup.cc:1674-1722 with core/group.cc:567-570), over zero padding if needed."""
    padded = (n + P - 1) // P * P
    chunk = padded // P
    full = [torch.cat([s, torch.zeros(padded - n, dtype=dtype)]) for s in srcs]
    return np.concatenate([oracle.reduce([bits(f[c * chunk:(c + 1) * chunk]) for f in full], c, TORCH_TO_CODE[dtype], op,
                                         scale) for c in range(P)])[:n]


ALLREDUCE_ROUTES = ["one_launch", "own_streams", "two_streams", "num_chunks", "kernel_less", "snapshot"]


@pytest.mark.parametrize("route", ALLREDUCE_ROUTES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.int64], ids=str)
def test_allreduce_routes_agree_with_the_oracle_bit_for_bit(world, dev, dtype, route):
    """Ranks that share a stream get ONE launch that reduces every chunk and stores it into every
    rank's tensor; ranks on different streams, pieces, the copy-engine gather and input snapshots
    get reduce_scatter + all_gather.  Every route must leave the same bits: the oracle's."""
    streams = {"own_streams": [torch.cuda.Stream(device=dev) for _ in range(P)],
               "two_streams": [torch.cuda.Stream(device=dev) for _ in range(2)] * (P // 2)}.get(route)
    for pg in world:
        if route == "num_chunks":
            pg.options().num_chunks = 3
        elif route == "kernel_less":
            pg.options().force_kernel_less = True
        elif route == "snapshot":
            pg.options().snapshot_inputs = True
    try:
        for n in (8, 8 * 1000, 8 * 1000 + 3, 5, 8 * 40001, 300007):
            for name, code in (("SUM", oracle.OP_SUM), ("MAX", oracle.OP_MAX), ("AVG", oracle.OP_AVG)):
                if code == oracle.OP_AVG and not dtype.is_floating_point:
                    continue
                srcs = random_sources(P, n, dtype, seed=n + code)
                want = allreduce_want(srcs, n, dtype, code, 1.0 / P if code == oracle.OP_AVG else 1.0)
                o = dist.AllreduceOptions()
                o.reduceOp = getattr(dist.ReduceOp, name)
                ts = [None] * P
                works = []
                torch.cuda.synchronize()
                for r, pg in enumerate(world):
                    if streams:
                        with torch.cuda.stream(streams[r]):
                            ts[r] = srcs[r].to(dev)  # produced on the rank's own stream
                            works.append(pg.allreduce([ts[r]], o))
                    else:
                        ts[r] = srcs[r].to(dev)
                        works.append(pg.allreduce([ts[r]], o))
                for w in works:
                    w.wait()
                torch.cuda.synchronize()
                for r in range(P):
                    assert same_bits(bits(ts[r]), want), (route, dtype, n, name, r)
    finally:
        for pg in world:
            pg.options().num_chunks = -1
            pg.options().force_kernel_less = False
            pg.options().snapshot_inputs = False


@pytest.mark.parametrize("own_streams", [False, True])
def test_allreduce_coalesced_routes_agree_with_the_oracle(world, dev, own_streams):
    # a list of divisible tensors (one collective) with two that need padding (an allreduce each)
    sizes = [8, 8 * 7, 8 * 1000, 8 * 12345, 13, 8 * 3, 1001]
    streams = [torch.cuda.Stream(device=dev) for _ in range(P)] if own_streams else None
    srcs = [random_sources(P, n, torch.float32, seed=3 * n) for n in sizes]  # [tensor][rank]
    wants = [allreduce_want(srcs[k], n, torch.float32, oracle.OP_SUM, 1.0) for k, n in enumerate(sizes)]
    ts = [None] * P
    works = []
    torch.cuda.synchronize()
    for r, pg in enumerate(world):
        if streams:
            with torch.cuda.stream(streams[r]):
                ts[r] = [srcs[k][r].to(dev) for k in range(len(sizes))]
                works.append(pg.allreduce_coalesced(ts[r]))
        else:
            ts[r] = [srcs[k][r].to(dev) for k in range(len(sizes))]
            works.append(pg.allreduce_coalesced(ts[r]))
    for w in works:
        w.wait()
    torch.cuda.synchronize()
    for r in range(P):
        for k in range(len(sizes)):
            assert same_bits(bits(ts[r][k]), wants[k]), (own_streams, r, k)


def test_allreduce_of_a_large_tensor_in_one_launch(world, dev):
    # 8 ranks x 72 MiB: chunks of 9 MiB, jobs that fill more than one launch of the list kernel
    n = 8 * (9 << 18) + 8
    g = torch.Generator().manual_seed(77)
    host = [torch.randint(-1000, 1000, (n,), dtype=torch.int32, generator=g) for _ in range(P)]
    ts = [h.to(dev) for h in host]
    each_rank(world, lambda r, pg: pg.allreduce([ts[r]]))
    want = host[0].clone()
    for h in host[1:]:
        want += h
    for t in ts:
        assert torch.equal(t.cpu(), want)
