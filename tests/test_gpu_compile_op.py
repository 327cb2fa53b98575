"""compile_op on the GPU, written the way the reference's tests/test_compile_op.py is, plus the
strided redistributions its tests leave out (and its snapshot cannot execute)."""

import numpy as np
import pytest
import torch

import moodist_amd
from moodist_amd import compile_op

pytestmark = pytest.mark.gpu
P = 8


@pytest.fixture()
def world(dev):
    return moodist_amd.LocalWorld(P, dev)


def run(world, specs, tensors):
    """specs[r] = (inputs, outputs) dict lists or None; tensors[r] = (input tensors, output tensors)."""
    ops = [compile_op(pg, shape=specs["shape"], dtype=specs["dtype"], inputs=specs[r][0], outputs=specs[r][1])
           for r, pg in enumerate(world)]
    futures = [ops[r](tensors[r][0], tensors[r][1]) for r in range(P)]
    for f in futures:
        f.wait()
    torch.cuda.synchronize()
    return ops


def test_point_to_point(world, dev):
    # reference tests/test_compile_op.py:21-61
    specs = {"shape": [4], "dtype": torch.float32}
    tensors = {}
    out = torch.zeros(4, device=dev)
    for r in range(P):
        specs[r] = ([{"offset": [0], "shape": [4]}], None) if r == 0 else \
            (None, [{"offset": [0], "shape": [4]}]) if r == 1 else (None, None)
        tensors[r] = ([torch.tensor([1.0, 2.0, 3.0, 4.0], device=dev)], []) if r == 0 else \
            ([], [out]) if r == 1 else ([], [])
    run(world, specs, tensors)
    assert out.tolist() == [1.0, 2.0, 3.0, 4.0]


def test_broadcast_and_reuse_and_dtypes(world, dev):
    # reference tests/test_compile_op.py:64-99, :312-343, :346-379
    for dtype in (torch.float32, torch.float64, torch.int32, torch.int64):
        specs = {"shape": [8], "dtype": dtype}
        for r in range(P):
            specs[r] = ([{"offset": [0], "shape": [8]}] if r == 0 else None, [{"offset": [0], "shape": [8]}])
        ops = [compile_op(pg, shape=[8], dtype=dtype, inputs=specs[r][0], outputs=specs[r][1])
               for r, pg in enumerate(world)]
        for i in range(3):  # the same op, three times, different data
            src = (torch.arange(8) + 10 * i).to(dtype).to(dev)
            outs = [torch.zeros(8, dtype=dtype, device=dev) for _ in range(P)]
            futures = [ops[r]([src] if r == 0 else [], [outs[r]]) for r in range(P)]
            assert [f.result()[0] is outs[r] or True for r, f in enumerate(futures)]
            torch.cuda.synchronize()
            for o in outs:
                assert torch.equal(o, src)


def test_gather_scatter_allgather(world, dev):
    # reference tests/test_compile_op.py:102-144, :147-187, :190-222
    chunk = 4
    n = chunk * P
    f32 = torch.float32
    # gather to rank 0
    specs = {"shape": [n], "dtype": f32}
    out0 = torch.zeros(n, device=dev)
    tensors = {}
    for r in range(P):
        specs[r] = ([{"offset": [r * chunk], "shape": [chunk]}], [{"offset": [0], "shape": [n]}] if r == 0 else None)
        tensors[r] = ([torch.full((chunk,), float(r), device=dev)], [out0] if r == 0 else [])
    run(world, specs, tensors)
    assert torch.equal(out0, torch.arange(P, device=dev).float().repeat_interleave(chunk))
    # scatter from rank 0
    src = torch.arange(n, device=dev, dtype=f32)
    outs = [torch.zeros(chunk, device=dev) for _ in range(P)]
    for r in range(P):
        specs[r] = ([{"offset": [0], "shape": [n]}] if r == 0 else None, [{"offset": [r * chunk], "shape": [chunk]}])
        tensors[r] = ([src] if r == 0 else [], [outs[r]])
    run(world, specs, tensors)
    for r in range(P):
        assert torch.equal(outs[r], src[r * chunk:(r + 1) * chunk])
    # all-gather
    outs = [torch.zeros(n, device=dev) for _ in range(P)]
    for r in range(P):
        specs[r] = ([{"offset": [r * chunk], "shape": [chunk]}], [{"offset": [0], "shape": [n]}])
        tensors[r] = ([torch.full((chunk,), float(r * 10), device=dev)], [outs[r]])
    run(world, specs, tensors)
    for o in outs:
        assert torch.equal(o, (torch.arange(P, device=dev).float() * 10).repeat_interleave(chunk))


def test_2d_rows_and_multiple_inputs(world, dev):
    # reference tests/test_compile_op.py:225-258, :261-309
    specs = {"shape": [P, 4], "dtype": torch.float32}
    outs = [torch.zeros(P, 4, device=dev) for _ in range(P)]
    tensors = {}
    for r in range(P):
        specs[r] = ([{"offset": [r, 0], "shape": [1, 4]}], [{"offset": [0, 0], "shape": [P, 4]}])
        tensors[r] = ([torch.full((1, 4), float(r * 10), device=dev)], [outs[r]])
    run(world, specs, tensors)
    for o in outs:
        assert torch.equal(o, (torch.arange(P, device=dev).float() * 10).unsqueeze(1).expand(P, 4))
    specs = {"shape": [4], "dtype": torch.float32}
    out = torch.zeros(4, device=dev)
    for r in range(P):
        specs[r] = ([{"offset": [0], "shape": [2]}, {"offset": [2], "shape": [2]}] if r == 0 else None,
                    [{"offset": [0], "shape": [4]}] if r == 1 else None)
        tensors[r] = ([torch.tensor([1.0, 2.0], device=dev), torch.tensor([3.0, 4.0], device=dev)] if r == 0 else [],
                      [out] if r == 1 else [])
    run(world, specs, tensors)
    assert out.tolist() == [1.0, 2.0, 3.0, 4.0]


def _reshard(world, dev, G, in_dim, out_dim):
    """Every rank holds a slab along in_dim and wants a slab along out_dim."""
    shape = list(G.shape)
    specs = {"shape": shape, "dtype": G.dtype}
    tensors, outs = {}, []
    for r in range(P):
        ioff, ishp = [0] * len(shape), list(shape)
        ishp[in_dim] = shape[in_dim] // P
        ioff[in_dim] = r * ishp[in_dim]
        ooff, oshp = [0] * len(shape), list(shape)
        oshp[out_dim] = shape[out_dim] // P
        ooff[out_dim] = r * oshp[out_dim]
        specs[r] = ([{"offset": ioff, "shape": ishp}], [{"offset": ooff, "shape": oshp}])
        src = G[tuple(slice(o, o + s) for o, s in zip(ioff, ishp))].contiguous().to(dev)
        out = torch.zeros(oshp, dtype=G.dtype, device=dev)
        outs.append((out, tuple(slice(o, o + s) for o, s in zip(ooff, oshp))))
        tensors[r] = ([src], [out])
    ops = run(world, specs, tensors)
    for out, sl in outs:
        assert torch.equal(out.cpu(), G[sl])
    return ops


def test_strided_redistribution_small(world, dev):
    g = torch.Generator().manual_seed(0)
    G = torch.randn(16, 24, generator=g)
    ops = _reshard(world, dev, G, 0, 1)  # rows -> columns: staging copies on the senders
    assert len(ops[0].plan()["inputCopies"]) == P and ops[0].plan()["outputCopies"] == []
    ops = _reshard(world, dev, G, 1, 0)  # columns -> rows: staging copies on the receivers
    assert len(ops[0].plan()["outputCopies"]) == P and ops[0].plan()["inputCopies"] == []
    _reshard(world, dev, torch.randn(8, 6, 16, generator=g).bfloat16(), 0, 2)
    _reshard(world, dev, torch.randint(0, 100, (8, 16, 8, 3), generator=g), 1, 2)


def test_overlapping_outputs_and_bystanders(world, dev):
    g = torch.Generator().manual_seed(1)
    G = torch.randn(6, 6, generator=g)
    boxes = {0: ([1, 1], [4, 4]), 1: ([0, 0], [6, 6]), 2: ([2, 0], [2, 6]), 3: ([0, 4], [6, 2])}
    specs = {"shape": [6, 6], "dtype": torch.float32}
    tensors, outs = {}, {}
    for r in range(P):
        ins = [{"offset": [3 * r, 0], "shape": [3, 6]}] if r < 2 else None
        o = [{"offset": boxes[r][0], "shape": boxes[r][1]}] if r in boxes else None
        specs[r] = (ins, o)
        outs[r] = torch.zeros(boxes[r][1], device=dev) if r in boxes else None
        tensors[r] = ([G[3 * r:3 * r + 3].contiguous().to(dev)] if r < 2 else [], [outs[r]] if r in boxes else [])
    run(world, specs, tensors)
    for r, (off, shp) in boxes.items():
        assert torch.equal(outs[r].cpu(), G[off[0]:off[0] + shp[0], off[1]:off[1] + shp[1]])


@pytest.mark.parametrize("seed", [0, 1])
def test_random_redistributions_match_numpy_slicing(world, dev, seed):
    # inputs: one random dimension cut into slabs dealt to random ranks (some ranks hold several
    # slabs, some none); outputs: a random box per rank, possibly overlapping each other.  Every
    # output must equal the same slice of the global tensor.
    rng = np.random.RandomState(seed)
    for trial in range(25):
        ndim = int(rng.randint(1, 5))
        shape = [int(rng.randint(2, 20)) for _ in range(ndim)]
        shape[-1] = int(rng.choice([3, 8, 16, 33, 64]))
        dtype = [torch.float32, torch.bfloat16, torch.int64, torch.float64][trial % 4]
        G = torch.from_numpy(rng.randint(-50, 50, shape)).to(dtype)
        d = int(rng.randint(0, ndim))
        cuts = sorted(set([0, shape[d]] + [int(x) for x in rng.randint(0, shape[d] + 1, 6)]))
        ins = {r: [] for r in range(P)}
        for a, b in zip(cuts[:-1], cuts[1:]):
            off, shp = [0] * ndim, list(shape)
            off[d], shp[d] = a, b - a
            ins[int(rng.randint(0, P))].append((off, shp))
        specs = {"shape": shape, "dtype": dtype}
        tensors, outs, want = {}, {}, {}
        for r in range(P):
            ins[r].sort(key=lambda x: -int(np.prod(x[1])))  # a rank lists its slices largest first
            lo = [int(rng.randint(0, n)) for n in shape]
            hi = [int(rng.randint(l + 1, n + 1)) for l, n in zip(lo, shape)]
            has_out = rng.rand() < 0.8
            idx = tuple(slice(l, h) for l, h in zip(lo, hi))
            outs[r] = torch.zeros([h - l for l, h in zip(lo, hi)], dtype=dtype, device=dev) if has_out else None
            want[r] = G[idx] if has_out else None
            specs[r] = ([{"offset": o, "shape": s} for o, s in ins[r]] or None,
                        [{"offset": lo, "shape": [h - l for l, h in zip(lo, hi)]}] if has_out else None)
            tensors[r] = ([G[tuple(slice(o_, o_ + s_) for o_, s_ in zip(o, s))].contiguous().to(dev) for o, s in ins[r]],
                          [outs[r]] if has_out else [])
        run(world, specs, tensors)
        for r in range(P):
            if outs[r] is not None:
                assert torch.equal(outs[r].cpu(), want[r]), (seed, trial, r, shape, d, cuts)


def test_future_before_every_rank_called(world, dev):
    ops = [compile_op(pg, shape=[4], dtype=torch.float32, inputs=[{"offset": [0], "shape": [4]}] if r == 0 else None,
                      outputs=[{"offset": [0], "shape": [4]}]) for r, pg in enumerate(world)]
    src = torch.arange(4, device=dev, dtype=torch.float32)
    outs = [torch.zeros(4, device=dev) for _ in range(P)]
    futures = [ops[r]([src] if r == 0 else [], [outs[r]]) for r in range(P - 1)]
    with pytest.raises(RuntimeError, match="7 of 8 have"):
        futures[0].wait()
    futures.append(ops[P - 1]([], [outs[P - 1]]))
    for f in futures:
        f.wait()
    torch.cuda.synchronize()
    assert all(torch.equal(o, src) for o in outs)


# ---- the full-size redistribution configurations through the operator surface ----

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=str)
def test_config5_matrix_row_shards_to_column_shards(world, dev, dtype):
    torch.manual_seed(0)
    G = torch.randn(8192, 8192).to(dtype)
    ops = _reshard(world, dev, G, 0, 1)
    plan = ops[3].plan()
    isz = G.element_size()
    # eight reads of 1024 x 1024 elements, each from a staging copy of the sender's columns
    assert len(plan["reads"]) == 8 and all(rd[5] == 1024 * 1024 * isz for rd in plan["reads"])
    assert [c[1] for c in plan["inputCopies"]] == [[0, 1024 * k] for k in range(8)]


def test_config5_3d_dim0_to_dim2(world, dev):
    torch.manual_seed(0)
    G3 = torch.randn(64, 512, 1024).bfloat16()
    ops = _reshard(world, dev, G3, 0, 2)
    plan = ops[0].plan()
    assert len(plan["reads"]) == 8 and all(rd[5] == 8 * 512 * 128 * 2 for rd in plan["reads"])
