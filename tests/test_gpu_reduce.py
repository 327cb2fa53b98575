"""Parity of the HIP K-source reduction against the CPU oracle, through the C ABI.

Bar: bit-exact for fp32/fp64/int32/int64 in every op; bf16/fp16 are compared bit-exactly with
the oracle (same fp32-accumulate, round-once rule) and additionally within 1 ulp of an
fp32-accumulated torch result, the tolerance the task states for 16-bit sums.
"""

import os

import numpy as np
import pytest
import torch

import oracle
from moodist_amd import _abi as abi
from util import ALL_DTYPES, TORCH_TO_CODE, bits, from_bits, random_sources, same_bits

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def gpu_reduce(srcs_dev, first, out_dev, op, scale=1.0, numel=None):
    st = torch.cuda.current_stream().cuda_stream
    n = out_dev.numel() if numel is None else numel
    abi.reduce([s.data_ptr() for s in srcs_dev], first, out_dev.data_ptr(), n, TORCH_TO_CODE[out_dev.dtype], op,
               scale, st)
    torch.cuda.synchronize()


def scale_for(op, P):
    return float(np.float32(1.0) / np.float32(P)) if op == oracle.OP_AVG else float(np.float32(0.37))


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=str)
@pytest.mark.parametrize("P", [1, 2, 3, 7, 8, 9, 16, 17, 33, 64])
def test_parity_all_ops_ragged_sizes(dev, dtype, P):
    for n in (1, 7, 64, 255, 1031, 4096 + 5, 70001):  # sizes of the reference's stress test plus tails
        srcs = random_sources(P, n, dtype, seed=P * 1000 + n)
        d = [s.to(dev) for s in srcs]
        first = (P * 7 + n) % P
        for op in (oracle.OP_SUM, oracle.OP_MIN, oracle.OP_MAX, oracle.OP_AVG, oracle.OP_PREMUL_SUM):
            if op in (oracle.OP_AVG, oracle.OP_PREMUL_SUM) and not dtype.is_floating_point:
                continue
            scale = scale_for(op, P)
            want = oracle.reduce([bits(s) for s in srcs], first, TORCH_TO_CODE[dtype], op, scale)
            out = torch.zeros(n, dtype=dtype, device=dev)
            gpu_reduce(d, first, out, op, scale)
            assert same_bits(bits(out), want), (dtype, P, n, op, first)


@pytest.mark.parametrize("unroll", [1, 2, 4, 8])
@pytest.mark.parametrize("max_blocks", [0, 3, 256])
def test_parity_under_every_launch_shape(dev, unroll, max_blocks):
    old = abi.get_tuning("reduce_unroll"), abi.get_tuning("reduce_max_blocks")
    try:
        abi.set_tuning("reduce_unroll", unroll)
        abi.set_tuning("reduce_max_blocks", max_blocks)
        for dtype in (torch.float32, torch.bfloat16, torch.int64):
            for P, n in ((8, 300000 + 3), (8, 8192 * 4 + 4), (16, 65536), (5, 12345)):
                srcs = random_sources(P, n, dtype, seed=n + P)
                want = oracle.reduce([bits(s) for s in srcs], 1, TORCH_TO_CODE[dtype], oracle.OP_SUM)
                out = torch.zeros(n, dtype=dtype, device=dev)
                gpu_reduce([s.to(dev) for s in srcs], 1, out, oracle.OP_SUM)
                assert same_bits(bits(out), want), (dtype, P, n)
    finally:
        abi.set_tuning("reduce_unroll", old[0])
        abi.set_tuning("reduce_max_blocks", old[1])


@pytest.mark.parametrize("wg_per_cu", [1, 2, 3, 5, 8, 9])
def test_parity_under_every_residency_cap(dev, wg_per_cu):
    # the cap is an unused LDS allocation; 1 needs the kernel's dynamic-LDS limit raised
    old = abi.get_tuning("reduce_wg_per_cu")
    try:
        abi.set_tuning("reduce_wg_per_cu", wg_per_cu)
        for dtype, op in ((torch.float32, oracle.OP_SUM), (torch.bfloat16, oracle.OP_AVG), (torch.float16, oracle.OP_PREMUL_SUM),
                          (torch.int32, oracle.OP_MAX)):
            P, n = 8, 700000 + 5
            srcs = random_sources(P, n, dtype, seed=wg_per_cu)
            scale = scale_for(op, P)
            want = oracle.reduce([bits(s) for s in srcs], 2, TORCH_TO_CODE[dtype], op, scale)
            out = torch.zeros(n, dtype=dtype, device=dev)
            gpu_reduce([s.to(dev) for s in srcs], 2, out, op, scale)
            assert same_bits(bits(out), want), (dtype, op)
    finally:
        abi.set_tuning("reduce_wg_per_cu", old)


def test_large_sources_take_the_capped_shape_and_match(dev):
    # 64 MiB per source and 8..16 sources select one or two sub-tiles with two workgroups per CU
    for dtype, P in ((torch.float32, 8), (torch.bfloat16, 9), (torch.float16, 12)):
        n = (64 << 20) // torch.empty(0, dtype=dtype).element_size() + 3
        g = torch.Generator().manual_seed(P)
        srcs = [(torch.randn(n, generator=g) * 3).to(dtype) for _ in range(P)]
        want = oracle.reduce([bits(s) for s in srcs], 5, TORCH_TO_CODE[dtype], oracle.OP_SUM)
        out = torch.zeros(n, dtype=dtype, device=dev)
        gpu_reduce([s.to(dev) for s in srcs], 5, out, oracle.OP_SUM)
        assert same_bits(bits(out), want), (dtype, P)
        del srcs, want, out
    # PREMUL_SUM and AVG of 16-bit types on the longest tiles (16 MiB per source and more)
    for dtype in (torch.bfloat16, torch.float16):
        n = (16 << 20) // 2 + 3
        srcs = random_sources(3, n, dtype, seed=77)
        d = [s.to(dev) for s in srcs]
        for op in (oracle.OP_PREMUL_SUM, oracle.OP_AVG):
            scale = scale_for(op, 3)
            want = oracle.reduce([bits(s) for s in srcs], 1, TORCH_TO_CODE[dtype], op, scale)
            out = torch.zeros(n, dtype=dtype, device=dev)
            gpu_reduce(d, 1, out, op, scale)
            assert same_bits(bits(out), want), (dtype, op)


def test_long_reductions_cut_into_several_launches(dev):
    # Reductions of more tiles than reduce_split_tiles are run as several launches over
    # consecutive parts.  With the limit at one tile every input of a few MiB is cut: ragged
    # sizes, element tails, pointers that are not 16-byte aligned, guard elements around the output.
    old = abi.get_tuning("reduce_split_tiles")
    try:
        abi.set_tuning("reduce_split_tiles", 1)
        for dtype, P, n in ((torch.float32, 3, 786432 + 5), (torch.bfloat16, 5, 1572864 + 7), (torch.int64, 2, 400000 + 1),
                            (torch.float64, 4, 393216 + 3), (torch.float16, 9, 3000000 + 1)):
            raw = random_sources(P, n + 8, dtype, seed=n % 1000 + P)
            views = [r[1 + i % 3:][:n] for i, r in enumerate(raw)]
            dviews = [r.to(dev)[1 + i % 3:][:n] for i, r in enumerate(raw)]
            canvas = torch.full((n + 8,), 7, dtype=dtype, device=dev)
            out = canvas[3:3 + n]
            for op in (oracle.OP_SUM, oracle.OP_MAX) + ((oracle.OP_AVG,) if dtype.is_floating_point else ()):
                scale = scale_for(op, P)
                gpu_reduce(dviews, P - 1, out, op, scale)
                want = oracle.reduce([bits(v) for v in views], P - 1, TORCH_TO_CODE[dtype], op, scale)
                assert same_bits(bits(out), want), (dtype, P, n, op)
                assert (canvas[:3] == 7).all() and (canvas[3 + n:] == 7).all()
    finally:
        abi.set_tuning("reduce_split_tiles", old)
    # and at the library's own limit: 160 MiB per source is 10,240 tiles, three launches
    n = (160 << 20) // 4 + 3
    g = torch.Generator().manual_seed(3)
    srcs = [torch.randn(n, generator=g) for _ in range(2)]
    want = oracle.reduce([bits(s) for s in srcs], 1, TORCH_TO_CODE[torch.float32], oracle.OP_SUM)
    out = torch.zeros(n, dtype=torch.float32, device=dev)
    gpu_reduce([s.to(dev) for s in srcs], 1, out, oracle.OP_SUM)
    assert same_bits(bits(out), want)


def test_golden_fixtures(dev):
    z = np.load(os.path.join(HERE, "golden", "reduce_cases.npz"))
    code_to_torch = {v: k for k, v in TORCH_TO_CODE.items()}
    for k, g, dtype, P, first, op, scale in z["meta"]:
        dt = code_to_torch[int(dtype)]
        srcs = [from_bits(row, dt).to(dev) for row in z["g%d_src" % int(g)]]
        out = torch.zeros(srcs[0].numel(), dtype=dt, device=dev)
        gpu_reduce(srcs, int(first), out, int(op), float(scale))
        assert same_bits(bits(out), z["c%d_out" % int(k)]), (dt, int(P), int(first), int(op))


def test_hand_derived_known_answers(dev):
    z = np.load(os.path.join(HERE, "golden", "known_answers.npz"))
    srcs = [torch.from_numpy(r.copy()).to(dev) for r in z["order_src"]]
    for first in range(4):
        out = torch.zeros(1, device=dev)
        gpu_reduce(srcs, first, out, oracle.OP_SUM)
        assert out.item() == float(z["order_out_by_first"][first])
    srcs = [from_bits(r, torch.bfloat16).to(dev) for r in z["bf16_src"]]
    out = torch.zeros(1, dtype=torch.bfloat16, device=dev)
    gpu_reduce(srcs, 0, out, oracle.OP_SUM)
    assert np.array_equal(bits(out), z["bf16_out"])
    srcs = [torch.from_numpy(r.copy()).to(dev) for r in z["rs_src"]]
    for first in range(8):
        out = torch.zeros(4, device=dev)
        gpu_reduce(srcs, first, out, oracle.OP_SUM)
        assert np.array_equal(out.cpu().numpy(), z["rs_out"])


def test_special_values_min_max_and_denormals(dev):
    nan, inf = float("nan"), float("inf")
    a = torch.tensor([+0.0, -0.0, nan, 1.0, 2.0, -inf, 1e-40, -1e-45, 3e-39])
    b = torch.tensor([-0.0, +0.0, 1.0, nan, 2.0, inf, 1e-40, 1e-45, -1e-39])
    c = torch.tensor([+0.0, -0.0, 5.0, -5.0, nan, 0.0, 1e-40, 1e-45, 2e-39])
    for dtype in (torch.float32, torch.float64, torch.bfloat16, torch.float16):
        srcs = [x.to(dtype) for x in (a, b, c)]
        d = [s.to(dev) for s in srcs]
        for first in range(3):
            for op in (oracle.OP_SUM, oracle.OP_MIN, oracle.OP_MAX):
                want = oracle.reduce([bits(s) for s in srcs], first, TORCH_TO_CODE[dtype], op)
                out = torch.zeros(a.numel(), dtype=dtype, device=dev)
                gpu_reduce(d, first, out, op)
                got = bits(out)
                # NaN payloads aside, every bit must agree (signed zeros and denormals included)
                wn = np.isnan(bits(from_bits(want, dtype).float()))
                gn = np.isnan(bits(out.float()))
                assert np.array_equal(wn, gn), (dtype, first, op)
                assert same_bits(got[~wn], want[~wn]), (dtype, first, op)


def test_integer_wraparound(dev):
    big = torch.tensor([2 ** 31 - 1, -2 ** 31, 5], dtype=torch.int32)
    one = torch.tensor([1, -1, -7], dtype=torch.int32)
    out = torch.zeros(3, dtype=torch.int32, device=dev)
    gpu_reduce([big.to(dev), one.to(dev)], 0, out, oracle.OP_SUM)
    assert out.tolist() == [-2 ** 31, 2 ** 31 - 1, -2]
    b64 = torch.tensor([2 ** 63 - 1], dtype=torch.int64)
    out = torch.zeros(1, dtype=torch.int64, device=dev)
    gpu_reduce([b64.to(dev), torch.ones(1, dtype=torch.int64, device=dev)], 0, out, oracle.OP_SUM)
    assert out.item() == -2 ** 63


def test_unaligned_pointers_and_guard_bytes(dev):
    for dtype in (torch.float32, torch.bfloat16, torch.float64):
        n = 4999
        raw = random_sources(8, n + 8, dtype, seed=11)
        views = [r[1 + i % 3:][:n] for i, r in enumerate(raw)]  # element-aligned, not 16-byte aligned
        dviews = [r.to(dev)[1 + i % 3:][:n] for i, r in enumerate(raw)]
        canvas = torch.full((n + 8,), 7, dtype=dtype, device=dev)
        out = canvas[3:3 + n]
        gpu_reduce(dviews, 2, out, oracle.OP_SUM)
        want = oracle.reduce([bits(v) for v in views], 2, TORCH_TO_CODE[dtype], oracle.OP_SUM)
        assert same_bits(bits(out), want)
        assert (canvas[:3] == 7).all() and (canvas[3 + n:] == 7).all()  # nothing written outside


def test_aligned_tail_does_not_spill(dev):
    # 16-byte aligned pointers, byte size not a multiple of 16: the vector body plus an element tail
    for n in (1, 3, 5, 1027, 1024 * 4 * 2 + 1):
        srcs = random_sources(8, n, torch.float32, seed=n)
        canvas = torch.full((n + 64,), 7.0, device=dev)
        out = canvas[:n]
        gpu_reduce([s.to(dev) for s in srcs], 0, out, oracle.OP_SUM)
        want = oracle.reduce([bits(s) for s in srcs], 0, oracle.DT_F32, oracle.OP_SUM)
        assert same_bits(bits(out), want)
        assert (canvas[n:] == 7.0).all()


def test_in_place_on_own_chunk(dev):
    # allreduce reduces into the rank's own chunk of its input (core/processgroup.cc:1689-1692)
    P, n, rank = 8, 40000, 3
    srcs = random_sources(P, n, torch.float32, seed=4)
    d = [s.to(dev) for s in srcs]
    want = oracle.reduce([bits(s) for s in srcs], rank, oracle.DT_F32, oracle.OP_SUM)
    gpu_reduce(d, rank, d[rank], oracle.OP_SUM)
    assert same_bits(bits(d[rank]), want)
    for j in range(P):
        if j != rank:
            assert torch.equal(d[j].cpu(), srcs[j])  # sources untouched


def test_direct_method_chunk_loop_and_final_rows(dev):
    # The multi-node method (core/reduce_scatter_direct.cc:165-177): for every remote destination
    # `source`, send[n] = in_self[source] (+) peers' in[source], cut into at most four chunks of
    # chunkSize bytes (core/processgroup.cc:1496-1503); the receiver then reduces its K rows
    # (:1599-1616).  Each chunk is one mdh_reduce call on offset pointers; the result must equal
    # the unchunked fold bit for bit, and the final K-row reduction must equal a fold of folds.
    local, nodes, rank = 4, 3, 1
    n = 200000 + 3  # 800,012 bytes: four ragged chunks, the last one short
    itemsize = 4
    nbytes = n * itemsize
    chunks = max(min(nbytes // 131072, 4), 1)
    chunk_size = ((nbytes + chunks - 1) // chunks + 4095) // 4096 * 4096
    chunks = (nbytes + chunk_size - 1) // chunk_size
    assert chunks == 4 and chunk_size % 16 == 0
    world = local * nodes
    # inputs of this node's `local` ranks: [world, n] each
    ins = [torch.stack(random_sources(world, n, torch.float32, seed=100 + r)) for r in range(local)]
    d = [x.to(dev) for x in ins]
    send = torch.zeros(world, n, device=dev)
    for dest in range(world):
        for c in range(chunks):
            lo = c * chunk_size // itemsize
            hi = min((c + 1) * chunk_size // itemsize, n)
            gpu_reduce([x[dest, lo:hi] for x in d], rank, send[dest, lo:hi], oracle.OP_SUM)
        want = oracle.reduce([bits(x[dest]) for x in ins], rank, oracle.DT_F32, oracle.OP_SUM)
        assert same_bits(bits(send[dest]), want), dest
    # final step on a receiver: rows = [received partials..., own, local peers...], reduced in row order
    rows = send[:5]
    out = torch.zeros(n, device=dev)
    gpu_reduce([rows[k] for k in range(5)], 0, out, oracle.OP_SUM)
    want = oracle.reduce([bits(rows[k]) for k in range(5)], 0, oracle.DT_F32, oracle.OP_SUM)
    assert same_bits(bits(out), want)


def test_sources_are_not_modified_and_zero_numel_is_a_no_op(dev):
    srcs = random_sources(4, 1000, torch.float32, seed=9)
    d = [s.to(dev) for s in srcs]
    out = torch.full((1000,), 3.0, device=dev)
    gpu_reduce(d, 0, out, oracle.OP_SUM, numel=0)
    assert (out == 3.0).all()
    gpu_reduce(d, 0, out, oracle.OP_MAX)
    for a, b in zip(d, srcs):
        assert torch.equal(a.cpu(), b)


def test_bf16_within_one_ulp_of_fp32_accumulated_reference(dev):
    # the tolerance the task states: 1 bf16 ulp against an fp32-accumulated result
    P, n = 16, 200000
    g = torch.Generator().manual_seed(3)
    srcs = [(torch.randn(n, generator=g) * 1e-3).bfloat16() for _ in range(P)]
    out = torch.zeros(n, dtype=torch.bfloat16, device=dev)
    gpu_reduce([s.to(dev) for s in srcs], 0, out, oracle.OP_SUM)
    acc = srcs[0].float()
    for s in srcs[1:]:
        acc = acc + s.float()
    ref = acc.bfloat16()
    # ulp distance on the ordered integer line of bf16 patterns
    def ordered(t):
        b = bits(t).astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b)
    assert np.abs(ordered(out) - ordered(ref)).max() <= 1
    assert torch.equal(out.cpu(), ref)  # in fact identical: same order, same single rounding


# ---- the benchmark configurations at full size ----

def _seeded(r, n, kind):
    torch.manual_seed(r)
    if kind == "randn":
        return torch.randn(n)
    if kind == "rand":
        return torch.rand(n) * 2 - 1
    raise ValueError(kind)


def test_config1_fp32_p8_full_size(dev):
    # reduce_scatter_tensor SUM fp32, world 8: rank 0's chunk of each rank's 8 x 4,194,304 input
    P, N = 8, 4194304
    srcs = [_seeded(r, P * N, "randn")[:N].clone() for r in range(P)]
    out = torch.zeros(N, device=dev)
    gpu_reduce([s.to(dev) for s in srcs], 0, out, oracle.OP_SUM)
    want = oracle.reduce([s.numpy() for s in srcs], 0, oracle.DT_F32, oracle.OP_SUM)
    assert same_bits(bits(out), want)
    # second witness: torch-CPU element-wise adds in the same order
    acc = srcs[0].clone()
    for s in srcs[1:]:
        acc.add_(s)
    assert torch.equal(out.cpu(), acc)


def test_config3_bf16_p16_full_size(dev):
    P, N = 16, 33554432
    srcs = []
    for r in range(P):
        torch.manual_seed(r)
        srcs.append((torch.randn(N) * 1e-3).bfloat16())
    d = [s.to(dev) for s in srcs]
    out = torch.zeros(N, dtype=torch.bfloat16, device=dev)
    gpu_reduce(d, 0, out, oracle.OP_SUM)
    del d
    want = oracle.reduce([bits(s) for s in srcs], 0, oracle.DT_BF16, oracle.OP_SUM)
    assert same_bits(bits(out), want)


def test_config4_fp32_p64_sum_avg_max_full_size(dev):
    P, N = 64, 1048576
    srcs = [_seeded(r, N, "rand") for r in range(P)]
    d = [s.to(dev) for s in srcs]
    np_srcs = [s.numpy() for s in srcs]
    outs = {}
    for op in (oracle.OP_SUM, oracle.OP_AVG, oracle.OP_MAX):
        scale = float(np.float32(1.0) / np.float32(P))
        out = torch.zeros(N, device=dev)
        gpu_reduce(d, 0, out, op, scale)
        assert same_bits(bits(out), oracle.reduce(np_srcs, 0, oracle.DT_F32, op, scale)), op
        outs[op] = out.cpu()
    # properties: AVG by 2^-6 is SUM / 64 exactly; MAX equals torch's maximum over the stack
    assert torch.equal(outs[oracle.OP_AVG], outs[oracle.OP_SUM] / 64)
    assert torch.equal(outs[oracle.OP_MAX], torch.stack(srcs).amax(dim=0))


def test_reduce_beyond_4_gib_per_source(dev):
    # byte offsets past 2^32: compared on the GPU with torch's own element-wise add (IEEE, same order)
    n = (1 << 30) + 4099  # 4 GiB + 16 KiB + 12 B of fp32
    a = torch.empty(n, device=dev).uniform_(-1, 1)
    b = torch.empty(n, device=dev).uniform_(-1, 1)
    out = torch.zeros(n, device=dev)
    gpu_reduce([a, b], 1, out, oracle.OP_SUM)
    assert torch.equal(out, b + a)
    del out
    out = torch.zeros(n, device=dev)
    gpu_reduce([a, b], 0, out, oracle.OP_MAX)
    assert torch.equal(out, torch.maximum(a, b))


def test_bf16_narrowing_follows_the_rounding_rule_for_every_fp32_pattern(dev):
    # the library narrows with the hardware conversion of gfx950; a device program compares it
    # with the rule (nearest, ties to even, quiet NaN with its payload) on all 2^32 inputs
    import subprocess

    exe = os.path.join(os.path.dirname(HERE), "tests", "native", "bf16_narrow_check.bin")
    if not os.path.exists(exe):
        pytest.skip("tests/native/bf16_narrow_check.bin is not built (run __graft_entry__.build())")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(r.stdout)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "4294967296 fp32 patterns and 65536 bf16 patterns checked, 0 differ" in r.stdout
