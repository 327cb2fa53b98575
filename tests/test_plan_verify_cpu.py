"""Prepared copy plans checked on the CPU: mdh_copy_plan_verify replays a plan's kernels on the
host, tile by tile and slot by slot, through the same index functions the device code is compiled
from, and compares every destination byte with what the boxes ask for.  The three compiled
redistributions of the benchmark, the strided gather, ragged and awkward boxes, and random ones.
No GPU: this is the bounds check of the kernels' indexing that runs before anything is launched.
"""

import numpy as np
import pytest

from moodist_amd import _abi as abi


def plan_for(specs, itemsize):
    """specs: (src bytes, src offset elems, dst offset elems, shape, src strides, dst strides); one source
    base per box and one shared destination base (the last)."""
    boxes = [abi.make_box(so * itemsize, do * itemsize, shape, sstr, dstr) for _, so, do, shape, sstr, dstr in specs]
    n = len(specs)
    return abi.CopyPlan(boxes, list(range(n)), [n] * n, itemsize, n + 1)


def test_the_three_compiled_redistributions_of_the_benchmark():
    # fp32 / bf16 8192 x 8192 row-sharded over 8 -> this rank's column block; [64,512,1024] bf16 dim0 -> dim2
    for itemsize in (4, 2):
        for k in (0, 3, 7):
            specs = [(1024 * 8192 * itemsize, 1024 * k, s * 1024 * 1024, [1024, 1024], [8192, 1], [1024, 1])
                     for s in range(8)]
            p = plan_for(specs, itemsize)
            assert p.launches == 1
            p.verify([1024 * 8192 * itemsize] * 8 + [8192 * 1024 * itemsize])
    for k in (0, 5):
        specs = [(8 * 512 * 1024 * 2, 128 * k, s * 8 * 512 * 128, [8, 512, 128], [512 * 1024, 1024, 1], [512 * 128, 128, 1])
                 for s in range(8)]
        p = plan_for(specs, 2)
        assert p.launches == 1
        p.verify([8 * 512 * 1024 * 2] * 8 + [64 * 512 * 128 * 2])


def test_equal_boxes_of_full_tiles_start_from_leading_scalar_arguments():
    # The shards of a redistribution (at most eight boxes of one shape, full tiles only) are launched
    # with fourteen leading 4-byte arguments -- source row pitch, tile shape, eight 48-bit source
    # addresses -- in front of the table; anything else with the table alone.
    import struct

    specs = [(1024 * 8192 * 4, 1024 * 3, s * 1024 * 1024, [1024, 1024], [8192, 1], [1024, 1]) for s in range(8)]
    p = plan_for(specs, 4)
    bases = [0x7F12_3456_0000 + (s << 33) + 16 * s for s in range(8)] + [0x7E00_0000_1000]
    args, lead, gx, gy, block, lds = p.step_arguments(bases, 0)
    assert lead == 14 and gy == 8 and block == 256
    words = struct.unpack("<14I", args[:56])
    assert words[0] == 8192 * 4                       # source row pitch in bytes
    log2tc, nct = words[1] & 31, words[1] >> 5
    assert (1 << log2tc) == 64 and nct == 4            # a row of 4 KiB is four tiles of 64 vectors (1 KiB) wide
    assert gx % nct == 0 and 1024 % (gx // nct) == 0  # whole rows of tiles, each of the same number of rows
    for s in range(8):
        pair = words[10 + s // 2]
        address = ((pair >> 16 if s & 1 else pair & 0xFFFF) << 32) | words[2 + s]
        assert address == bases[s] + 1024 * 3 * 4
    # the table that follows holds the same boxes: source and destination address lead each entry
    src0, dst0 = struct.unpack("<QQ", args[56:72])
    assert src0 == bases[0] + 1024 * 3 * 4 and dst0 == bases[8]
    # nine boxes, rows that are not whole vectors, or a ragged last row of tiles: the table form
    for other in (
        [(1024 * 8192 * 4, 0, s * 1024 * 1024, [1024, 1024], [8192, 1], [1024, 1]) for s in range(9)],
        [(1024 * 8192 * 2, 0, s * 1024 * 1021, [1024, 1021], [8192, 1], [1021, 1]) for s in range(8)],
        [(1023 * 8192 * 4, 0, s * 1023 * 512, [1023, 512], [8192, 1], [512, 1]) for s in range(8)],
    ):
        q = plan_for(other, 2 if other[0][3][1] == 1021 else 4)
        n = len(other)
        b = [0x7F00_0000_0000 + (s << 33) for s in range(n + 1)]
        for step in range(q.launches):
            assert q.step_arguments(b, step)[1] == 0
    # an address beyond 48 bits cannot be packed: the same plan then takes the table form
    assert p.step_arguments([1 << 50] + bases[1:], 0)[1] == 0
    # a dense gather of eight equal shards: the segments' length and the packed source addresses
    shard = 1 << 20
    g = plan_for([(shard, 0, r * shard, [shard], [1], [1]) for r in range(8)], 1)
    assert g.launches == 1
    g.verify([shard] * 8 + [8 * shard])
    args, lead, gx, gy, block, lds = g.step_arguments(bases, 0)
    assert lead == 14 and gy == 8
    words = struct.unpack("<14I", args[:56])
    assert words[0] == shard and shard % gx == 0 and (shard // gx) % 4096 == 0   # whole sub-tiles of 4 KiB
    for r in range(8):
        pair = words[10 + r // 2]
        assert (((pair >> 16 if r & 1 else pair & 0xFFFF) << 32) | words[2 + r]) == bases[r]
    # unequal shards: the table form
    lens = [shard, shard, shard - 16, shard]
    at, specs = 0, []
    for n in lens:
        specs.append((n, 0, at, [n], [1], [1]))
        at += n
    u = plan_for(specs, 1)
    assert all(u.step_arguments(bases[:4] + [bases[8]], k)[1] == 0 for k in range(u.launches))
    # equal shards that are not a whole number of vectors: cut to one common length of whole
    # vectors, their heads and tails copied by workgroup 0 of every row of the grid
    r = plan_for([(shard + 2, 0, k * (shard + 2), [shard + 2], [1], [1]) for k in range(8)], 1)
    assert r.launches == 1
    r.verify([shard + 2] * 8 + [8 * (shard + 2)])
    args, lead, gx, gy, block, lds = r.step_arguments(bases, 0)
    assert lead == 14 and gy == 8
    common = struct.unpack("<I", args[:4])[0]
    assert common % 16 == 0 and shard + 2 - 64 - 16 < common <= shard + 2
    assert (gx - 1) * 4096 >= common > (gx - 2) * 4096   # one workgroup more than the tiles of 4 KiB


def test_strided_gather_and_dense_gather_shapes():
    # [8, rows, cols] bf16 gather into a padded row pitch, scaled down 4x per side from the benchmark's
    rows, cols, pad = 1024, 1024, 64
    specs = [(rows * cols * 2, 0, s * rows * (cols + pad), [rows, cols], [cols, 1], [cols + pad, 1]) for s in range(8)]
    plan_for(specs, 2).verify([rows * cols * 2] * 8 + [8 * rows * (cols + pad) * 2])
    # dense: eight flat segments of unequal length (ragged last tiles, the scanned segment table)
    lens = [100000, 65536, 16, 4096 * 3 + 16, 48, 1 << 20, 999984, 32]
    at, specs = 0, []
    for n in lens:
        specs.append((n, 0, at, [n], [1], [1]))
        at += n
    plan_for(specs, 1).verify(lens + [at])


def test_ragged_dense_gathers_are_one_launch_with_heads_and_tails():
    # shards whose byte length is not a multiple of 16 land at destinations off the 64-byte grid:
    # the whole vectors start on the grid, heads and tails go to the same launch's edge workgroups
    for shard, nshards in ((100000 * 2 + 2, 8), (4096 + 1, 64), (1 << 20 | 6, 3), (5000, 8), (33, 5)):
        specs = [(shard + 64, 1, r * shard + 3, [shard], [1], [1]) for r in range(nshards)]
        p = plan_for(specs, 1)
        assert p.launches == 1, (shard, nshards, p.launches)
        p.verify([shard + 64] * nshards + [nshards * shard + 64])
    # shorter than two vectors: the narrow kernel's, still verified
    specs = [(64, 1, r * 21 + 3, [21], [1], [1]) for r in range(4)]
    plan_for(specs, 1).verify([64] * 4 + [200])


@pytest.mark.parametrize("itemsize", [1, 2, 4, 8])
def test_ragged_rows_transposes_and_many_dimensions(itemsize):
    specs = [
        (40 * 1000 * itemsize, 7, 11, [37, 1001], [1003, 1], [1004, 1]),          # rows not a multiple of 16 bytes
        (5000 * itemsize, 3, 40000, [40, 50], [1, 60], [50, 1]),                   # transposing: one-element runs
        (16 * itemsize, 5, 69999, [], [], []),                                     # a scalar
        (9000 * itemsize, 0, 50000, [3, 4, 5, 6], [2000, 400, 60, 1], [130, 31, 6, 1]),  # four strided extents
        (3000 * itemsize, 1, 60000, [2, 2, 2, 2, 2, 3], [1000, 500, 200, 90, 40, 1], [96, 48, 24, 12, 6, 1]),
        (70000 * itemsize, 0, 62000, [17, 33], [37, 1], [33, 1]),                  # dense on one side only
    ]
    sizes = [s[0] + 64 for s in specs] + [80000 * itemsize]
    plan_for(specs, itemsize).verify(sizes)


@pytest.mark.parametrize("itemsize", [1, 2, 4, 8, 16])
def test_transposing_boxes_take_tiles_through_lds(itemsize):
    # out[c][r] = in[r][c]: source contiguous along one dimension, destination along the other.  With
    # both dimensions at least 16 long the box is copied in tiles turned round in LDS; the check
    # replays every tile through the kernel's own index function.
    import struct

    for R, C, soff, doff, spad, dpad in ((64, 64, 0, 0, 0, 0), (100, 36, 0, 0, 0, 0), (17, 333, 3, 5, 1, 2),
                                         (130, 70, 4, 8, 4, 12), (16, 16, 0, 1, 0, 0)):
        specs = [((R * (C + spad) + soff + 4) * itemsize, soff, doff, [C, R], [1, C + spad], [R + dpad, 1])]
        p = plan_for(specs, itemsize)
        assert p.launches == 1
        p.verify([specs[0][0], (C * (R + dpad) + doff + 4) * itemsize])
        args, lead, gx, gy, block, lds = p.step_arguments([0x7F00_0000_0000, 0x7E00_0000_0000], 0)
        tile = 64 if itemsize <= 4 else 32
        assert lead == 0 and gy == 1 and block == 256 and gx == -(-R // tile) * -(-C // tile)
        src0, dst0 = struct.unpack("<QQ", args[:16])
        assert src0 == 0x7F00_0000_0000 + soff * itemsize and dst0 == 0x7E00_0000_0000 + doff * itemsize
    # two batch dimensions around the transposed pair, and the pair in the middle of the box
    specs = [(3 * 4 * 50 * 40 * itemsize + 64, 0, 0, [3, 4, 40, 50], [4 * 50 * 40, 50 * 40, 1, 40], [4 * 40 * 50, 40 * 50, 50, 1]),
             (20 * 30 * 6 * itemsize + 64, 2, 3 * 4 * 50 * 40 + 7, [30, 6, 20], [1, 20 * 30, 30], [6 * 20, 20, 1])]
    plan_for(specs, itemsize).verify([specs[0][0], specs[1][0], (3 * 4 * 50 * 40 + 7 + 30 * 6 * 20 + 4) * itemsize])
    # below 16 elements on one side the plain strided kernel keeps the box (one launch of it)
    small = [(8 * 500 * itemsize + 64, 0, 0, [500, 8], [1, 500], [8, 1])]
    plan_for(small, itemsize).verify([small[0][0], 500 * 8 * itemsize + 64])


def test_random_permuted_boxes():
    # sources that are permuted views of padded parents, extents up to 90: transposing pairs with
    # batch dimensions around them, partial tiles, every element size, several boxes per plan
    rng = np.random.RandomState(23)
    for trial in range(150):
        itemsize = int(rng.choice([1, 2, 4, 8, 16]))
        nboxes = int(rng.randint(1, 4))
        boxes, sizes, dst_elems = [], [], 0
        for _ in range(nboxes):
            nd = int(rng.randint(2, 5))
            shape = [int(rng.choice([1, 2, 3, 7, 17, 33])) for _ in range(nd)]  # (every element is replayed on the host)
            for d in rng.choice(nd, 2, replace=False):
                shape[d] = int(rng.choice([16, 31, 64, 70, 90]))
            pshape = [s + int(rng.randint(0, 3)) for s in shape]
            perm = list(rng.permutation(nd))
            sstr, acc = [0] * nd, 1
            for d in reversed(range(nd)):
                sstr[perm[d]] = acc
                acc *= pshape[perm[d]]
            soff = int(rng.randint(0, 3))
            dstr, acc2 = [0] * nd, 1
            for d in reversed(range(nd)):
                dstr[d] = acc2
                acc2 *= shape[d] + int(rng.randint(0, 2))
            doff = dst_elems + int(rng.randint(0, 3))
            boxes.append(abi.make_box(soff * itemsize, doff * itemsize, shape, sstr, dstr))
            sizes.append((acc + soff + 4) * itemsize)
            dst_elems = doff + acc2
        plan = abi.CopyPlan(boxes, list(range(nboxes)), [nboxes] * nboxes, itemsize, nboxes + 1)
        plan.verify(sizes + [(dst_elems + 4) * itemsize])


def test_random_boxes():
    rng = np.random.RandomState(11)
    for trial in range(60):
        itemsize = int(rng.choice([1, 2, 4, 8, 16]))
        specs, sizes, dst_at = [], [], 0
        for _ in range(int(rng.randint(1, 7))):
            nd = int(rng.randint(1, 5))
            shape = [int(rng.randint(1, 12)) for _ in range(nd)]
            shape[-1] = int(rng.choice([1, 2, 5, 16, 64, 300]))
            sstr, dstr = [1] * nd, [1] * nd
            for d in range(nd - 2, -1, -1):
                sstr[d] = sstr[d + 1] * shape[d + 1] + int(rng.randint(0, 4)) * (d == nd - 2)
                dstr[d] = dstr[d + 1] * shape[d + 1] + int(rng.randint(0, 4)) * (d == nd - 2)
            so = int(rng.randint(0, 9))
            specs.append(((sstr[0] * shape[0] + so + 4) * itemsize, so, dst_at, shape, sstr, dstr))
            dst_at += dstr[0] * shape[0] + int(rng.randint(0, 9))
        plan_for(specs, itemsize).verify([s[0] for s in specs] + [(dst_at + 4) * itemsize])


def test_the_verifier_notices_what_it_is_there_to_notice():
    specs = [(4096, 0, 0, [16, 64], [64, 1], [64, 1])]
    p = plan_for(specs, 4)
    p.verify([4096, 4096])
    with pytest.raises(abi.MoodistError, match="reaches outside its bases"):
        p.verify([4095, 4096])  # source one byte short
    with pytest.raises(abi.MoodistError, match="reaches outside its bases"):
        p.verify([4096, 4000])
    # overlapping destinations are a caller error the check reports
    two = [(256, 0, 0, [64], [1], [1]), (256, 0, 32, [64], [1], [1])]
    with pytest.raises(abi.MoodistError, match="boxes overlap"):
        plan_for(two, 4).verify([256, 256, 1024])
    with pytest.raises(abi.MoodistError, match="takes 2 bases"):
        p.verify([4096])
