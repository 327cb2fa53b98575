"""Seeded randomized differential tests on the GPU, through the C ABI.

The reduction is compared bit for bit with the CPU oracle over random element types, ops, source
counts, sizes, fold starts, element misalignments of every buffer, in-place destinations, special
values (NaN, infinities, -0) and launch-shape knobs; guard elements round the destination must
stay untouched.  The box copy is compared with torch slicing on the CPU over random N-d boxes
(1..6 dims, four element sizes, ragged inner runs, padded destinations, several boxes per call in
random order) and knobs.
"""

import random

import numpy as np
import pytest
import torch

import torch.distributed as dist

import moodist_amd
import oracle
from moodist_amd import _abi as abi
from util import ALL_DTYPES, TORCH_TO_CODE, bits, same_bits

pytestmark = pytest.mark.gpu
OPS = [oracle.OP_SUM, oracle.OP_MIN, oracle.OP_MAX, oracle.OP_AVG, oracle.OP_PREMUL_SUM]
KNOBS = ("reduce_unroll", "reduce_max_blocks", "reduce_wg_per_cu", "box_unroll", "copy_unroll", "copy_max_blocks",
         "copy_wg_per_cu", "box_preload")


@pytest.fixture()
def knobs():
    yield
    for k in KNOBS:
        abi.set_tuning(k, 0)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_reduce_random_cases_match_the_oracle(dev, knobs, seed):
    st = torch.cuda.current_stream().cuda_stream
    rng = random.Random(seed)
    for case in range(120):
        dtype = rng.choice(ALL_DTYPES)
        op = rng.choice(OPS)
        if op in (oracle.OP_AVG, oracle.OP_PREMUL_SUM) and not dtype.is_floating_point:
            op = oracle.OP_SUM
        P = rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 15, 16, 17, 24, 31, 32, 33, 63, 64])
        n = rng.choice([1, 2, 3, 5, 8, 15, 16, 17, 100, 1023, 1024, 4099, 65536, 70001, rng.randint(1, 300000),
                        rng.randint(1, 2000000) // max(1, P // 8)])
        first = rng.randrange(P)
        offs = [rng.randrange(0, 9) for _ in range(P + 1)]  # element misalignment of every buffer
        abi.set_tuning("reduce_unroll", rng.choice([0, 0, 1, 2, 4, 8]))
        abi.set_tuning("reduce_max_blocks", rng.choice([0, 0, 1, 7, 300]))
        abi.set_tuning("reduce_wg_per_cu", rng.choice([0, 0, 1, 2, 3, 6, 9]))
        g = torch.Generator().manual_seed(seed * 100000 + case)
        srcs = []
        for _ in range(P):
            if dtype.is_floating_point:
                t = (torch.randn(n, generator=g) * 4).to(dtype)
                if rng.random() < 0.1 and n > 3:
                    t[rng.randrange(n)] = float("nan")
                    t[rng.randrange(n)] = float("inf")
                    t[rng.randrange(n)] = -0.0
            else:
                t = torch.randint(-2**30, 2**30, (n,), generator=g).to(dtype) * 3
            srcs.append(t)
        scale = float(np.float32(1.0) / np.float32(P)) if op == oracle.OP_AVG else \
            float(np.float32(rng.choice([0.37, 2.0, -1.5, 1e-3])))
        want = oracle.reduce([bits(s) for s in srcs], first, TORCH_TO_CODE[dtype], op, scale)
        dbuf = []
        for j in range(P):
            b = torch.zeros(n + 16, dtype=dtype, device=dev)
            b[offs[j]:offs[j] + n] = srcs[j].to(dev)
            dbuf.append(b)
        inplace = rng.random() < 0.2
        if inplace:
            out_full, o = dbuf[first], offs[first]
        else:
            out_full, o = torch.full((n + 16,), 5, dtype=dtype, device=dev), offs[P]
        isz = out_full.element_size()
        abi.reduce([dbuf[j].data_ptr() + offs[j] * isz for j in range(P)], first, out_full.data_ptr() + o * isz, n,
                   TORCH_TO_CODE[dtype], op, scale, st)
        torch.cuda.synchronize()
        what = (seed, case, dtype, op, P, n, first, offs, inplace)
        assert same_bits(bits(out_full[o:o + n]), want), what
        if not inplace:
            assert bool((torch.cat([out_full[:o], out_full[o + n:]]).cpu() == 5).all()), what


@pytest.mark.parametrize("seed", [1, 2])
def test_copy_random_boxes_match_torch_slicing(dev, knobs, seed):
    st = torch.cuda.current_stream().cuda_stream
    rng = random.Random(seed)
    dtypes = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}
    for case in range(250):
        itemsize = rng.choice([1, 2, 4, 8])
        dtype = dtypes[itemsize]
        ndim = rng.randint(1, 6)
        big = rng.random() < 0.3
        full = [rng.randint(1, 6 if ndim > 3 else (40 if not big else 300)) for _ in range(ndim)]
        full[-1] = rng.choice([1, 2, 3, 7, 8, 16, 17, 33, 64, 100, 257, 1024, 1030]) if ndim < 4 else rng.randint(1, 40)
        while np.prod(full) > 3_000_000:
            k = rng.randrange(ndim)
            full[k] = max(1, full[k] // 2)
        g = torch.Generator().manual_seed(seed * 100000 + case)
        src = torch.randint(0, 120, tuple(full), generator=g).to(dtype)
        dstfull = [f + rng.choice([0, 0, 1, 3]) for f in full]
        sd = src.to(dev)
        out = torch.full(tuple(dstfull), 7, dtype=dtype, device=dev)
        want = torch.full(tuple(dstfull), 7, dtype=dtype)
        # dimension d is cut into slabs, so the boxes cannot overlap in the destination
        d = rng.randrange(ndim)
        cuts = sorted(set([0, full[d]] + [rng.randint(0, full[d]) for _ in range(rng.randint(0, 4))]))
        boxes = []
        for a, b in zip(cuts[:-1], cuts[1:]):
            lo = [rng.randint(0, f - 1) for f in full]
            hi = [rng.randint(l + 1, f) for l, f in zip(lo, full)]
            lo[d], hi[d] = a, b
            shape = [h - l for l, h in zip(lo, hi)]
            dlo = [rng.randint(0, df - s) for df, s in zip(dstfull, shape)]
            dlo[d] = a
            sidx = tuple(slice(l, h) for l, h in zip(lo, hi))
            didx = tuple(slice(l, l + s) for l, s in zip(dlo, shape))
            want[didx] = src[sidx]
            sview, dview = sd[sidx], out[didx]
            boxes.append(abi.make_box(sview.data_ptr(), dview.data_ptr(), shape, list(sview.stride()),
                                      list(dview.stride())))
        abi.set_tuning("box_unroll", rng.choice([0, 0, 1, 2, 4, 8]))
        abi.set_tuning("copy_unroll", rng.choice([0, 0, 1, 2, 4, 8]))
        abi.set_tuning("copy_max_blocks", rng.choice([0, 0, 1, 9]))
        abi.set_tuning("copy_wg_per_cu", rng.choice([0, 0, 2, 4, 9]))
        rng.shuffle(boxes)
        abi.copy_boxes(boxes, itemsize, st)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), want), (seed, case, itemsize, full, dstfull, d, cuts)


@pytest.mark.parametrize("seed", [1, 2])
def test_gather_random_shapes_match_numpy(dev, knobs, seed):
    # 1..70 shards, 1..300 rows, widths with and without a 16-byte body (among them the powers of
    # two whose tiles are all full: the forms started from preloaded arguments), independent row
    # pitches, byte misalignment of every shard and of the output, guard bytes between and after shards
    st = torch.cuda.current_stream().cuda_stream
    rng = random.Random(seed)
    for case in range(200):
        P = rng.choice([1, 2, 3, 8, 9, 33, 70])
        rows = rng.choice([1, 1, 2, 5, 32, 64, 128, 300])
        width = rng.choice([1, 3, 15, 16, 17, 100, 256, 1000, 2048, 4096, 4100, 8192, rng.randint(1, 20000)])
        if rows * width * P > 10_000_000:
            rows = max(1, 10_000_000 // (width * P))
        sp = width + rng.choice([0, 0, 1, 16, 100])
        dp = width + rng.choice([0, 0, 3, 16, 128])
        if rows == 1:
            sp = dp = width
        stride = rows * dp + rng.choice([0, 0, 5, 256])
        soff = [rng.randrange(0, 17) for _ in range(P)]
        doff = rng.randrange(0, 17)
        if rng.random() < 0.3:  # everything on the 16-byte grid
            soff, doff = [0] * P, 0
        g = torch.Generator().manual_seed(seed * 100000 + case)
        shards = [torch.randint(0, 255, (rows * sp + 32,), generator=g, dtype=torch.uint8) for _ in range(P)]
        d = [s.to(dev) for s in shards]
        out = torch.full((P * stride + 64,), 7, dtype=torch.uint8, device=dev)
        for k in ("copy_unroll", "box_unroll"):
            abi.set_tuning(k, rng.choice([0, 0, 1, 2, 4, 8]))
        abi.set_tuning("copy_max_blocks", rng.choice([0, 0, 1, 11]))
        abi.set_tuning("copy_wg_per_cu", rng.choice([0, 0, 2, 5, 9]))
        abi.set_tuning("box_preload", rng.choice([0, 0, 0, 1]))
        abi.gather([d[s].data_ptr() + soff[s] for s in range(P)], out.data_ptr() + doff, width, rows, sp, dp, stride, st)
        torch.cuda.synchronize()
        want = np.full(P * stride + 64, 7, dtype=np.uint8)
        for s in range(P):
            src = shards[s].numpy()[soff[s]:soff[s] + rows * sp]
            for r in range(rows):
                lo = doff + s * stride + r * dp
                want[lo:lo + width] = src[r * sp:r * sp + width]
        assert np.array_equal(out.cpu().numpy(), want), (seed, case, P, rows, width, sp, dp, stride, soff, doff)


def test_process_group_random_sequences_match_the_oracle(dev):
    # random worlds (1..16 ranks) running random sequences of reduce_scatter, all_gather (flat and
    # list form) and allreduce (sizes that do and do not divide by the world) on random dtypes
    rng = random.Random(5)
    dts = [torch.float32, torch.float64, torch.int32, torch.int64, torch.bfloat16, torch.float16]
    ops = {"SUM": (dist.ReduceOp.SUM, oracle.OP_SUM), "MIN": (dist.ReduceOp.MIN, oracle.OP_MIN),
           "MAX": (dist.ReduceOp.MAX, oracle.OP_MAX), "AVG": (dist.ReduceOp.AVG, oracle.OP_AVG)}
    for case in range(60):
        P = rng.choice([1, 2, 3, 4, 5, 8, 16])
        world = moodist_amd.LocalWorld(P, dev)
        for step in range(rng.randint(1, 5)):
            kind = rng.choice(["rs", "ag", "ar", "agl"])
            dtype = rng.choice(dts)
            n = rng.choice([1, 3, 16, 100, 1000, 4097, rng.randint(1, 50000)])
            g = torch.Generator().manual_seed(case * 100 + step)

            def rnd(m):
                if dtype.is_floating_point:
                    return (torch.randn(m, generator=g) * 3).to(dtype)
                return torch.randint(-1000, 1000, (m,), generator=g).to(dtype)

            what = (case, step, kind, P, dtype, n)
            if kind == "rs":
                name = rng.choice(list(ops))
                if name == "AVG" and not dtype.is_floating_point:
                    name = "SUM"
                ins = [rnd(n * P) for _ in range(P)]
                d_in = [t.to(dev) for t in ins]
                outs = [torch.zeros(n, dtype=dtype, device=dev) for _ in range(P)]
                opts = dist.ReduceScatterOptions()
                opts.reduceOp = ops[name][0]
                for w in [pg._reduce_scatter_base(outs[r], d_in[r], opts) for r, pg in enumerate(world)]:
                    w.wait()
                torch.cuda.synchronize()
                scale = float(np.float32(1.0) / np.float32(P))
                for r in range(P):
                    want = oracle.reduce([bits(t[r * n:(r + 1) * n]) for t in ins], r, TORCH_TO_CODE[dtype],
                                         ops[name][1], scale)
                    assert same_bits(bits(outs[r]), want), what + (name, r)
            elif kind in ("ag", "agl"):
                ins = [rnd(n) for _ in range(P)]
                d_in = [t.to(dev) for t in ins]
                if kind == "ag":
                    outs = [torch.zeros(n * P, dtype=dtype, device=dev) for _ in range(P)]
                    works = [pg._allgather_base(outs[r], d_in[r]) for r, pg in enumerate(world)]
                else:
                    lists = [[torch.zeros(n, dtype=dtype, device=dev) for _ in range(P)] for _ in range(P)]
                    works = [pg.allgather([lists[r]], [d_in[r]]) for r, pg in enumerate(world)]
                for w in works:
                    w.wait()
                torch.cuda.synchronize()
                want = bits(torch.cat(ins))
                for r in range(P):
                    got = outs[r] if kind == "ag" else torch.cat(lists[r])
                    assert same_bits(bits(got), want), what + (r,)
            else:
                name = rng.choice(["SUM", "MAX", "MIN"])
                ins = [rnd(n) for _ in range(P)]
                ts = [t.to(dev) for t in ins]
                opts = dist.AllreduceOptions()
                opts.reduceOp = ops[name][0]
                for w in [pg.allreduce([ts[r]], opts) for r, pg in enumerate(world)]:
                    w.wait()
                torch.cuda.synchronize()
                # chunk q of the (padded) tensor is folded starting at rank q (core/processgroup.cc:1674-1722)
                padded = (n + P - 1) // P * P
                c = padded // P
                pin = [torch.cat([t, torch.zeros(padded - n, dtype=dtype)]) for t in ins]
                want = np.concatenate([oracle.reduce([bits(t[q * c:(q + 1) * c]) for t in pin], q,
                                                     TORCH_TO_CODE[dtype], ops[name][1], 1.0) for q in range(P)])[:n]
                for r in range(P):
                    assert same_bits(bits(ts[r]), want), what + (name, r)


def test_process_group_random_coalesced_sequences_match_the_oracle(dev):
    # random worlds running random sequences of the coalesced collectives (lists of 1..12 tensors of
    # random sizes, one or two element types), with random chunk options on the groups and the ranks
    # spread over one, two or as many streams as ranks: results against the oracle's composition,
    # tensor by tensor
    rng = random.Random(11)
    dts = [torch.float32, torch.float64, torch.int32, torch.int64, torch.bfloat16, torch.float16]
    ops = {"SUM": (dist.ReduceOp.SUM, oracle.OP_SUM), "MIN": (dist.ReduceOp.MIN, oracle.OP_MIN),
           "MAX": (dist.ReduceOp.MAX, oracle.OP_MAX), "AVG": (dist.ReduceOp.AVG, oracle.OP_AVG)}
    for case in range(40):
        P = rng.choice([1, 2, 3, 4, 8, 16])
        world = moodist_amd.LocalWorld(P, dev)
        nstreams = rng.choice([1, 1, 2, P])
        streams = [torch.cuda.Stream(device=dev) for _ in range(nstreams)]
        option = rng.choice([None, None, ("num_chunks", rng.choice([2, 3, 7])), ("chunk_size", rng.choice([4096, 65536])),
                             ("method", 2)])
        if option:
            for pg in world:
                setattr(pg.options(), option[0], option[1])
        for step in range(rng.randint(1, 4)):
            kind = rng.choice(["rsc", "agc", "arc"])
            T = rng.randint(1, 12)
            dtypes = [rng.choice(dts)] * T
            if rng.random() < 0.25 and T > 1:
                dtypes[rng.randrange(T)] = rng.choice(dts)  # a second element type somewhere in the list
            sizes = [rng.choice([1, 2, 5, 64, 1000, 4097, rng.randint(1, 30000)]) for _ in range(T)]
            g = torch.Generator().manual_seed(case * 1000 + step)

            def rnd(m, dtype):
                if dtype.is_floating_point:
                    return (torch.randn(m, generator=g) * 3).to(dtype)
                return torch.randint(-1000, 1000, (m,), generator=g).to(dtype)

            name = rng.choice(list(ops))
            if name == "AVG" and not all(dt.is_floating_point for dt in dtypes):
                name = "SUM"
            scale = float(np.float32(1.0) / np.float32(P))
            what = (case, step, kind, P, nstreams, option, T, name)
            torch.cuda.synchronize()
            works = []
            if kind == "rsc":
                ins = [[rnd(n * P, dt) for n, dt in zip(sizes, dtypes)] for _ in range(P)]
                d_in = [[t.to(dev) for t in row] for row in ins]
                outs = [[torch.zeros(n, dtype=dt, device=dev) for n, dt in zip(sizes, dtypes)] for _ in range(P)]
                opts = dist.ReduceScatterOptions()
                opts.reduceOp = ops[name][0]
                torch.cuda.synchronize()
                for r, pg in enumerate(world):
                    with torch.cuda.stream(streams[r % nstreams]):
                        works.append(pg.reduce_scatter_tensor_coalesced(outs[r], d_in[r], opts))
                for w in works:
                    w.wait()
                torch.cuda.synchronize()
                for k, (n, dt) in enumerate(zip(sizes, dtypes)):
                    for r in range(P):
                        want = oracle.reduce([bits(ins[j][k][r * n:(r + 1) * n]) for j in range(P)], r, TORCH_TO_CODE[dt],
                                             ops[name][1], scale)
                        assert same_bits(bits(outs[r][k]), want), what + (k, r)
            elif kind == "agc":
                ins = [[rnd(n, dt) for n, dt in zip(sizes, dtypes)] for _ in range(P)]
                d_in = [[t.to(dev) for t in row] for row in ins]
                outs = [[torch.zeros(n * P, dtype=dt, device=dev) for n, dt in zip(sizes, dtypes)] for _ in range(P)]
                torch.cuda.synchronize()
                for r, pg in enumerate(world):
                    with torch.cuda.stream(streams[r % nstreams]):
                        works.append(pg.allgather_into_tensor_coalesced(outs[r], d_in[r]))
                for w in works:
                    w.wait()
                torch.cuda.synchronize()
                for k in range(T):
                    want = bits(torch.cat([ins[j][k] for j in range(P)]))
                    for r in range(P):
                        assert same_bits(bits(outs[r][k]), want), what + (k, r)
            else:
                ins = [[rnd(n, dt) for n, dt in zip(sizes, dtypes)] for _ in range(P)]
                ts = [[t.to(dev) for t in row] for row in ins]
                opts = dist.AllreduceCoalescedOptions()
                opts.reduceOp = ops[name][0]
                torch.cuda.synchronize()
                for r, pg in enumerate(world):
                    with torch.cuda.stream(streams[r % nstreams]):
                        works.append(pg.allreduce_coalesced(ts[r], opts))
                for w in works:
                    w.wait()
                torch.cuda.synchronize()
                for k, (n, dt) in enumerate(zip(sizes, dtypes)):
                    padded = (n + P - 1) // P * P
                    c = padded // P
                    pin = [torch.cat([ins[j][k], torch.zeros(padded - n, dtype=dt)]) for j in range(P)]
                    want = np.concatenate([oracle.reduce([bits(t[q * c:(q + 1) * c]) for t in pin], q, TORCH_TO_CODE[dt],
                                                         ops[name][1], scale) for q in range(P)])[:n]
                    for r in range(P):
                        assert same_bits(bits(ts[r][k]), want), what + (k, r)
