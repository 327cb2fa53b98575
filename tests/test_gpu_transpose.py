"""Boxes that transpose (source contiguous along one dimension, destination along another) through
mdh_copy_boxes and through prepared plans, against numpy: byte-exact, nothing outside the box
touched.  These boxes take the LDS-staged tile kernel when both dimensions are at least 16
elements long; the knob box_transpose = 1 sends them through the plain strided kernel, and both
must give the same bytes."""

import numpy as np
import pytest
import torch

from moodist_amd import _abi as abi

pytestmark = pytest.mark.gpu

DTYPES = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}


def st():
    return torch.cuda.current_stream().cuda_stream


@pytest.fixture(params=[(0, 0), (3, 2), (7, 3)], ids=["default", "three_walkers_rows", "seven_walkers_diagonals"], autouse=True)
def walkers_and_order(request):
    """Every test of this file runs three times: as the library launches by itself (a workgroup per
    tile on matrices of this size), and with three and seven workgroups walking all the tiles of a
    launch -- many tiles per workgroup, ragged ones among them -- in either order of the tiles."""
    wgs, order = request.param
    old_wgs, old_order = abi.get_tuning("box_transpose_wgs"), abi.get_tuning("box_transpose")
    abi.set_tuning("box_transpose_wgs", wgs)
    abi.set_tuning("box_transpose", order)
    yield
    abi.set_tuning("box_transpose_wgs", old_wgs)
    abi.set_tuning("box_transpose", old_order)


def host_array(shape, itemsize, seed):
    rng = np.random.RandomState(seed)
    return rng.randint(0, 256, size=tuple(shape) + (itemsize,)).astype(np.uint8)


def as_tensor(a, dev):
    return torch.from_numpy(a.reshape(-1).copy()).to(dev)


@pytest.mark.parametrize("itemsize", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("knob", [None, 1])
def test_two_dimensional_transposes(dev, itemsize, knob):
    old = abi.get_tuning("box_transpose")
    try:
        if knob is not None:
            abi.set_tuning("box_transpose", knob)
        # whole tiles, ragged edges, extents just over the threshold, one long and one short side
        for R, C in ((64, 64), (128, 256), (100, 36), (16, 16), (17, 333), (1000, 24), (65, 129), (512, 1024)):
            src = host_array((R, C), itemsize, R * 7 + C)
            d_src = as_tensor(src, dev)
            d_dst = torch.full((C * R * itemsize + 64,), 0xAB, dtype=torch.uint8, device=dev)
            # out[c][r] = in[r][c], 32 guard bytes in front
            abi.copy_boxes([abi.make_box(d_src.data_ptr(), d_dst.data_ptr() + 32, [C, R], [1, C], [R, 1])], itemsize, st())
            torch.cuda.synchronize()
            got = d_dst.cpu().numpy()
            want = np.ascontiguousarray(src.transpose(1, 0, 2)).reshape(-1)
            assert np.array_equal(got[32:32 + want.size], want), (itemsize, R, C)
            assert (got[:32] == 0xAB).all() and (got[32 + want.size:] == 0xAB).all(), (itemsize, R, C)
    finally:
        abi.set_tuning("box_transpose", old)


@pytest.mark.parametrize("itemsize", [2, 4, 8])
def test_sub_boxes_pitches_offsets_and_batches(dev, itemsize):
    # [batch0, batch1, R, C] parents with padding on both sides; a box inside them, starting at odd
    # element offsets (16-byte accesses do not fit: the element-wise form) and at aligned ones
    for (b0, b1, R, C, r0, c0, nr, nc, spad, dpad) in (
            (2, 3, 80, 96, 0, 0, 80, 96, 0, 0),      # dense, aligned: 16-byte accesses
            (2, 3, 80, 96, 3, 5, 70, 81, 1, 3),      # odd offsets, extents and pitches
            (1, 5, 200, 40, 8, 8, 160, 32, 8, 16),   # aligned sub-box of padded parents
            (4, 1, 33, 47, 1, 2, 31, 44, 0, 5)):
        src = host_array((b0, b1, R, C + spad), itemsize, R + C + itemsize)
        d_src = as_tensor(src, dev)
        dst = np.full((b0, b1, nc, nr + dpad, itemsize), 0xCD, dtype=np.uint8)
        d_dst = as_tensor(dst, dev)
        sstr = [b1 * R * (C + spad), R * (C + spad), 1, C + spad]  # box dims: batch0, batch1, c, r
        dstr = [b1 * nc * (nr + dpad), nc * (nr + dpad), nr + dpad, 1]
        soff = (r0 * (C + spad) + c0) * itemsize
        abi.copy_boxes([abi.make_box(d_src.data_ptr() + soff, d_dst.data_ptr(), [b0, b1, nc, nr], sstr, dstr)], itemsize, st())
        torch.cuda.synchronize()
        want = dst.copy()
        want[:, :, :, :nr] = src[:, :, r0:r0 + nr, c0:c0 + nc].transpose(0, 1, 3, 2, 4)
        assert np.array_equal(d_dst.cpu().numpy(), want.reshape(-1)), (itemsize, b0, b1, R, C)


def test_transposing_redistribution_of_eight_slabs_through_a_prepared_plan(dev):
    # eight row slabs [128, 512] of a [1024, 512] fp32 matrix -> this rank's [512, 1024] transposed whole:
    # eight boxes in one launch of the tile kernel, prepared once, launched twice with other tensors
    P, rows, cols, isz = 8, 128, 512, 4
    boxes = [abi.make_box(0, s * rows * isz, [cols, rows], [1, cols], [P * rows, 1]) for s in range(P)]
    plan = abi.CopyPlan(boxes, list(range(P)), [P] * P, isz, P + 1)
    assert plan.launches == 1
    plan.verify([rows * cols * isz] * P + [cols * P * rows * isz])
    for seed in (1, 2):
        G = torch.randint(-1000, 1000, (P * rows, cols), dtype=torch.int32, generator=torch.Generator().manual_seed(seed))
        slabs = [G[s * rows:(s + 1) * rows].contiguous().to(dev) for s in range(P)]
        out = torch.zeros(cols, P * rows, dtype=torch.int32, device=dev)
        plan.launch([t.data_ptr() for t in slabs] + [out.data_ptr()], st())
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), G.t().contiguous())


def test_many_transposing_boxes_in_one_call(dev):
    # 40 boxes: more than one launch's table holds, of mixed sizes
    rng = np.random.RandomState(3)
    boxes, checks, keep = [], [], []
    for k in range(40):
        R, C = int(rng.randint(16, 200)), int(rng.randint(16, 200))
        src = torch.randint(-2 ** 31, 2 ** 31 - 1, (R, C), dtype=torch.int32, generator=torch.Generator().manual_seed(k))
        d_src = src.to(dev)
        d_dst = torch.zeros(C, R, dtype=torch.int32, device=dev)
        keep.append((d_src, d_dst))
        boxes.append(abi.make_box(d_src.data_ptr(), d_dst.data_ptr(), [C, R], [1, C], [R, 1]))
        checks.append((d_dst, src.t().contiguous()))
    abi.copy_boxes(boxes, 4, st())
    torch.cuda.synchronize()
    for k, (got, want) in enumerate(checks):
        assert torch.equal(got.cpu(), want), k


def test_random_permuted_boxes_against_the_oracle(dev):
    """Random boxes whose source is a permuted view of a padded parent (so that its contiguous
    dimension is any of the box's dimensions), extents 1..90, one to four dimensions, every element
    size, several boxes per call: the oracle's element-by-element copy decides, and bytes outside
    the boxes must stay as they were."""
    import oracle

    rng = np.random.RandomState(23)
    for trial in range(60):
        itemsize = int(rng.choice([1, 2, 4, 8, 16]))
        nboxes = int(rng.randint(1, 4))
        specs, dst_elems = [], 0
        for _ in range(nboxes):
            nd = int(rng.randint(2, 5))
            shape = [int(rng.choice([1, 2, 3, 17, 33, 64, 90])) for _ in range(nd)]
            big = rng.choice(nd, 2, replace=False)  # at least two long extents: a transposing pair is possible
            for d in big:
                shape[d] = int(rng.choice([16, 31, 64, 70, 90]))
            pshape = [s + int(rng.randint(0, 3)) for s in shape]
            perm = list(rng.permutation(nd))
            sstr = [0] * nd
            acc = 1
            for d in reversed(range(nd)):
                sstr[perm[d]] = acc
                acc *= pshape[perm[d]]
            soff = int(rng.randint(0, 3))
            dshape = [s + int(rng.randint(0, 2)) for s in shape]
            dstr = [0] * nd
            acc2 = 1
            for d in reversed(range(nd)):
                dstr[d] = acc2
                acc2 *= dshape[d]
            specs.append((shape, sstr, soff, acc + soff, dstr, dst_elems + int(rng.randint(0, 3)), acc2))
            dst_elems = specs[-1][5] + acc2
        dst_elems += 3
        dst_host = rng.randint(0, 256, dst_elems * itemsize).astype(np.uint8)
        want = dst_host.copy()
        dst_dev = torch.from_numpy(dst_host.copy()).to(dev)
        boxes, keep = [], []
        for shape, sstr, soff, src_numel, dstr, doff, _ in specs:
            src_host = rng.randint(0, 256, src_numel * itemsize).astype(np.uint8)
            src_dev = torch.from_numpy(src_host).to(dev)
            keep.append(src_dev)
            oracle.copy_box(src_host, soff, want, doff, shape, sstr, dstr, itemsize)
            boxes.append(abi.make_box(src_dev.data_ptr() + soff * itemsize, dst_dev.data_ptr() + doff * itemsize, shape,
                                      sstr, dstr))
        abi.copy_boxes(boxes, itemsize, st())
        torch.cuda.synchronize()
        assert np.array_equal(dst_dev.cpu().numpy(), want), (trial, itemsize, specs)
