"""Benchmark of the hot path on one MI355X.

A step is one pass of the local multi-source reduction over one batch of staged chunks:
reduce_scatter_tensor SUM, fp32, world size 8 seen from rank 0 -- eight staged 16 MiB chunks
folded in rank order into one 16 MiB output (4,194,304 elements).  Inputs are resident in HBM
before the timed region; the launches rotate over 4 GiB of distinct buffers, so that they are
not in the 256 MB Infinity Cache either.  Prints one JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]
                  [--headline-only] [--tuning KNOB=VALUE ...]
  Without --workload the headline (reduce_fp32_p8) is measured and reported as the line's top-level
  figures, and after it, in the same process, every other configuration of the benchmark --
  reduce_bf16_p16, reduce_fp32_p64_{sum,avg,max}, allgather_bf16_p8[_strided],
  redistribute_{fp32,bf16}_8192, redistribute_bf16_3d -- each with the same steps, warm-up, rotation
  and result check; their kernel times go into "configs" of the same JSON line.
  NAME is one of those or, for sweeps,
    reduce:<fp32|bf16|fp16|fp64|int32|int64>:<sources>:<elements>[:<sum|avg|max>]
    gather:<sources>:<bytes per shard>
    rows:<boxes>:<rows per box>:<run bytes>:<source pitch bytes>    strided rows into a dense destination
    transpose:<rows>:<cols>:<itemsize>                              2-D element transpose
    coalesced:<tensors>:<elements>[:loop|:halves]                   allreduce_coalesced of eight local ranks
    reduce_many:<jobs>:<sources>:<elements>[:single]                a list of reductions in shared launches
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
CLOCK_WARMUP_S = 0.3   # untimed launches before the first timed window
TIMED_WINDOWS = 11     # windows of `steps` launches; the median window is reported
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch), each
# scaled by what the same counter reads for the flat copy of exactly 256 MiB (FETCH_SIZE x 1.99992,
# WRITE_SIZE x 1.00000): profiles/hbm_traffic_pmc_reduce_and_copy_kernels.md.  E.g. the headline:
# 65,560.15 x 1.99992 + 16,384.00 KiB = 147,498.9 KiB.  Workloads without an entry were not measured.
MEASURED_TRAFFIC_BYTES = {
    "reduce_fp32_p8": 151038850,
    "reduce_bf16_p16": 1140907970,
    "reduce_fp32_p64_sum": 272676956,
    "reduce_fp32_p64_avg": 272677784,
    "reduce_fp32_p64_max": 272690521,
    "allgather_bf16_p8": 536870912,
    "allgather_bf16_p8_strided": 536897643,
    "redistribute_fp32_8192": 67145701,
    "redistribute_bf16_8192": 33591324,
    "redistribute_bf16_3d": 16799942,
}

DTYPE_NAMES = {"float32": "f32", "bfloat16": "bf16", "float16": "f16", "float64": "f64", "int32": "i32", "int64": "i64",
               "uint8": "u8"}

# every configuration of the benchmark; the first is the headline
ALL_WORKLOADS = ("reduce_fp32_p8", "reduce_bf16_p16", "reduce_fp32_p64_sum", "reduce_fp32_p64_avg", "reduce_fp32_p64_max",
                 "allgather_bf16_p8", "allgather_bf16_p8_strided", "redistribute_fp32_8192", "redistribute_bf16_8192",
                 "redistribute_bf16_3d")
# measured after them by a default run, reported under "others"
OTHER_WORKLOADS = ["transpose:4096:4096:4", "transpose:8192:8192:2", "coalesced:1:4194304", "coalesced:48:65536"]


def box_kernel(abi):
    """The strided-box kernel the benchmark's shapes run: equal boxes of full tiles are started from
    preloaded arguments (copy_rows16_kernel) unless the knob box_preload=1 asks for the table form."""
    return "copy_boxes16_kernel" if abi.get_tuning("box_preload") == 1 else "copy_rows16_kernel"


def flat_kernel(abi, sources, shard_bytes):
    """The dense-gather kernel: up to eight equal shards start from preloaded arguments
    (copy_flat8_kernel), anything else from the segment table."""
    early = 1 < sources <= 8 and shard_bytes >= 32 and abi.get_tuning("box_preload") != 1
    return "copy_flat8_kernel" if early else "copy_flat_kernel"


def build_workload(name, torch, abi, dev, rotation_bytes):
    """Returns (describe, algorithmic_bytes, launch(i), check(), kernel name) for a named workload.
    Every workload rotates over distinct buffer sets whose TOUCHED bytes add up to
    rotation_bytes (default 4 GiB, sixteen times the 256 MB Infinity Cache), so that neither the
    sources nor the outputs of a launch are still cached from an earlier one: a rotation of two
    or three times the cache is not enough on this chip (see the measurement notes)."""
    L = abi.lib()

    # torch's current stream, on which main() records its events; nothing here ever changes it,
    # so the handle is looked up once instead of in every launch
    stream = torch.cuda.current_stream().cuda_stream

    def current():
        return stream

    def nsets_for(touched_bytes):
        # at most 512 sets: launches that touch less than 8 MiB rotate over less than 4 GiB
        return min(512, max(2, -(-rotation_bytes // touched_bytes)))

    if name.startswith("reduce") and not name.startswith("reduce_many:"):
        # reduce_fp32_p8 (headline), reduce_bf16_p16, reduce_fp32_p64_{sum,avg,max}
        spec = {
            "reduce_fp32_p8": (8, 4194304, torch.float32, abi.DTYPE_FLOAT32, abi.OP_SUM, "randn", 1.0),
            "reduce_bf16_p16": (16, 33554432, torch.bfloat16, abi.DTYPE_BFLOAT16, abi.OP_SUM, "randn1e-3", 1.0),
            "reduce_fp32_p64_sum": (64, 1048576, torch.float32, abi.DTYPE_FLOAT32, abi.OP_SUM, "rand", 1.0),
            "reduce_fp32_p64_avg": (64, 1048576, torch.float32, abi.DTYPE_FLOAT32, abi.OP_AVG, "rand", 1.0 / 64),
            "reduce_fp32_p64_max": (64, 1048576, torch.float32, abi.DTYPE_FLOAT32, abi.OP_MAX, "rand", 1.0),
        }.get(name)
        if spec is None:
            # reduce:<fp32|bf16|fp16>:<sources>:<elements>[:<sum|avg|max>] -- any size, for sweeps
            parts = name.split(":")
            if parts[0] != "reduce" or len(parts) not in (4, 5):
                raise SystemExit("bench.py: unknown workload " + name)
            tdt, code = {"fp32": (torch.float32, abi.DTYPE_FLOAT32), "bf16": (torch.bfloat16, abi.DTYPE_BFLOAT16),
                         "fp16": (torch.float16, abi.DTYPE_FLOAT16), "fp64": (torch.float64, abi.DTYPE_FLOAT64),
                         "int32": (torch.int32, abi.DTYPE_INT32), "int64": (torch.int64, abi.DTYPE_INT64)}[parts[1]]
            P, N = int(parts[2]), int(parts[3])
            op = {"sum": abi.OP_SUM, "avg": abi.OP_AVG, "max": abi.OP_MAX}[parts[4] if len(parts) == 5 else "sum"]
            spec = (P, N, tdt, code, op, "rand", 1.0 / P if op == abi.OP_AVG else 1.0)
        P, N, tdt, code, op, dist, scale = spec
        isz = torch.empty(0, dtype=tdt).element_size()
        set_bytes = (P + 1) * N * isz
        nsets = nsets_for(set_bytes)
        base = []
        for r in range(P):
            torch.manual_seed(r)
            if dist == "randn":
                x = torch.randn(N)  # first N draws of rank r's 8*N-element input = its chunk for rank 0
            elif dist == "randn1e-3":
                x = (torch.randn(N) * 1e-3).to(tdt)
            elif tdt.is_floating_point:
                x = (torch.rand(N) * 2 - 1).to(tdt)
            else:
                x = torch.randint(-2 ** 30, 2 ** 30, (N,)).to(tdt)
            base.append(x)
        on_device = [b.to(dev) for b in base]
        sets = [on_device] + [[b.clone() for b in on_device] for _ in range(nsets - 1)]
        outs = [torch.empty(N, dtype=tdt, device=dev) for _ in range(nsets)]
        tabs = [abi.ptr_table([t.data_ptr() for t in s]) for s in sets]

        # one argument tuple per buffer set, made once: the launch loop does nothing but call
        calls = [(tabs[k], P, 0, outs[k].data_ptr(), N, code, op, scale, stream) for k in range(nsets)]
        reduce_fn = L.mdh_reduce

        def launch(i):
            rc = reduce_fn(*calls[i % nsets])
            if rc:
                abi.check(rc)

        def check():
            import numpy as np

            import oracle

            def b(t):
                t = t.cpu()
                return t.view(torch.int16).numpy().view(np.uint16) if isz == 2 else t.numpy()

            want = oracle.reduce([b(x) for x in base], 0, code, op, scale)
            for o in outs:
                if not np.array_equal(b(o).view(np.uint8), want.view(np.uint8)):
                    raise SystemExit("bench: result differs from the oracle")

        desc = {"workload": name, "op": "reduce_scatter_tensor local reduction", "sources": P, "numel": N,
                "dtype": str(tdt).replace("torch.", ""), "fold_first": 0, "buffer_sets": nsets}
        return desc, set_bytes, launch, check, "reduce_vec_kernel"


    if name.startswith("gather:"):
        # gather:<sources>:<bytes per shard> -- dense assembly of any size, for sweeps
        P, shard = (int(x) for x in name.split(":")[1:3])
        set_bytes = 2 * P * shard
        nsets = nsets_for(set_bytes)
        g = torch.Generator().manual_seed(1)
        base = [torch.randint(0, 256, (shard,), dtype=torch.uint8, generator=g) for _ in range(P)]
        sets = [[b.to(dev) for b in base] for _ in range(nsets)]
        outs = [torch.empty(P * shard, dtype=torch.uint8, device=dev) for _ in range(nsets)]
        tabs = [abi.ptr_table([t.data_ptr() for t in s]) for s in sets]
        out_ptrs = [o.data_ptr() for o in outs]

        def launch(i):
            k = i % nsets
            rc = L.mdh_gather(tabs[k], P, out_ptrs[k], shard, 1, shard, shard, shard, current())
            if rc:
                abi.check(rc)

        def check():
            want = torch.cat(base)
            for o in outs:
                if not torch.equal(o.cpu(), want):
                    raise SystemExit("bench: result differs from the expected gather")

        desc = {"workload": name, "op": "all_gather_into_tensor chunk assembly", "sources": P, "shard_bytes": shard,
                "dtype": "uint8", "buffer_sets": nsets}
        return desc, set_bytes, launch, check, flat_kernel(abi, P, shard)

    if name == "allgather_bf16_p8" or name == "allgather_bf16_p8_strided":
        P, n = 8, 16777216
        rows = cols = 4096
        pad = 64 if name.endswith("strided") else 0
        set_bytes = 2 * P * n * 2
        nsets = nsets_for(set_bytes)
        base = []
        for r in range(P):
            torch.manual_seed(r)
            base.append(torch.randn(n).bfloat16())
        sets = [[b.to(dev) for b in base] for _ in range(nsets)]
        outs = [torch.empty(P, rows, cols + pad, dtype=torch.bfloat16, device=dev) for _ in range(nsets)]
        tabs = [abi.ptr_table([t.data_ptr() for t in s]) for s in sets]

        def launch(i):
            k = i % nsets
            if pad:
                rc = L.mdh_gather(tabs[k], P, outs[k].data_ptr(), cols * 2, rows, cols * 2, (cols + pad) * 2,
                                  rows * (cols + pad) * 2, current())
            else:
                rc = L.mdh_gather(tabs[k], P, outs[k].data_ptr(), n * 2, 1, n * 2, n * 2, n * 2, current())
            if rc:
                abi.check(rc)

        def check():
            want = torch.stack(base).view(P, rows, cols)
            for o in outs:
                if not torch.equal(o[:, :, :cols].cpu(), want):
                    raise SystemExit("bench: result differs from the expected gather")

        desc = {"workload": name, "op": "all_gather_into_tensor chunk assembly", "sources": P, "numel": n,
                "dtype": "bfloat16", "buffer_sets": nsets}
        return desc, set_bytes, launch, check, box_kernel(abi) if pad else flat_kernel(abi, P, n * 2)

    if name.startswith("redistribute"):
        # redistribute_fp32_8192, redistribute_bf16_8192, redistribute_bf16_3d
        P = 8
        if name.endswith("3d"):
            tdt, shape, box = torch.bfloat16, (64, 512, 1024), [8, 512, 128]
            sstr, dstr = [512 * 1024, 1024, 1], [512 * 128, 128, 1]
            out_shape = (64, 512, 128)
        else:
            tdt = torch.float32 if "fp32" in name else torch.bfloat16
            shape, box = (8192, 8192), [1024, 1024]
            sstr, dstr = [8192, 1], [1024, 1]
            out_shape = (8192, 1024)
        isz = torch.empty(0, dtype=tdt).element_size()
        torch.manual_seed(0)
        G = torch.randn(*shape).to(tdt)
        per = shape[0] // P
        out_numel = 1
        for s in out_shape:
            out_numel *= s
        set_bytes = 2 * out_numel * isz
        # the slabs are read only in part (this rank's columns): what counts for the caches is
        # what a launch touches, not what the slabs occupy
        nsets = nsets_for(set_bytes)
        k = 0  # this rank
        on_device = [G[per * s:per * (s + 1)].contiguous().to(dev) for s in range(P)]
        sets = [on_device] + [[t.clone() for t in on_device] for _ in range(nsets - 1)]
        outs = [torch.empty(out_shape, dtype=tdt, device=dev) for _ in range(nsets)]
        blk = out_numel // P
        # what a compiled custom op runs: the launches prepared once (mdh_copy_plan_create), every
        # call patches the tensors' addresses in (mdh_copy_plan_launch)
        plan = abi.CopyPlan([abi.make_box(box[-1] * k * isz, s * blk * isz, box, sstr, dstr) for s in range(P)],
                            list(range(P)), [P] * P, isz, P + 1)
        tabs = [abi.ptr_table([t.data_ptr() for t in sets[i]] + [outs[i].data_ptr()]) for i in range(nsets)]

        def launch(i):
            rc = L.mdh_copy_plan_launch(plan._plan, tabs[i % nsets], P + 1, current())
            if rc:
                abi.check(rc)

        def check():
            want = G[..., box[-1] * k:box[-1] * (k + 1)]
            for o in outs:
                if not torch.equal(o.cpu(), want):
                    raise SystemExit("bench: result differs from the expected redistribution")

        desc = {"workload": name, "op": "compile_op redistribution copies (prepared plan)", "sources": P,
                "global_shape": list(shape), "dtype": str(tdt).replace("torch.", ""), "buffer_sets": nsets,
                # these kernels are shorter than the host's launch call: the timed launches are
                # enqueued behind a long blocker kernel so that the GPU runs them back to back
                "queue_prefilled": True}
        return desc, set_bytes, launch, check, box_kernel(abi)

    if name.startswith("reduce_many:"):
        # reduce_many:<jobs>:<sources>:<elements>[:single] -- a list of fp32 SUM reductions of that many
        # elements each in one call of mdh_reduce_many (shared launches); with ":single", the same
        # jobs as one mdh_reduce call each.  A step is the whole list.
        parts = name.split(":")
        J, P, N = int(parts[1]), int(parts[2]), int(parts[3])
        single = len(parts) > 4 and parts[4] == "single"
        set_bytes = J * (P + 1) * N * 4
        nsets = nsets_for(set_bytes)
        g = torch.Generator().manual_seed(6)
        base = [[torch.rand(N, generator=g) * 2 - 1 for _ in range(P)] for _ in range(J)]
        on_device = [[t.to(dev) for t in job] for job in base]
        sets = [on_device] + [[[t.clone() for t in job] for job in on_device] for _ in range(nsets - 1)]
        outs = [[torch.empty(N, device=dev) for _ in range(J)] for _ in range(nsets)]
        tables = [abi.reduce_jobs([([t.data_ptr() for t in sets[k][j]], j % P, outs[k][j].data_ptr(), N) for j in range(J)])
                  for k in range(nsets)]
        singles = [[(abi.ptr_table([t.data_ptr() for t in sets[k][j]]), P, j % P, outs[k][j].data_ptr(), N,
                     abi.DTYPE_FLOAT32, abi.OP_SUM, 1.0, stream) for j in range(J)] for k in range(nsets)]

        def launch(i):
            k = i % nsets
            if single:
                for call in singles[k]:
                    rc = L.mdh_reduce(*call)
                    if rc:
                        abi.check(rc)
            else:
                rc = L.mdh_reduce_many(tables[k][0], J, abi.DTYPE_FLOAT32, abi.OP_SUM, 1.0, stream)
                if rc:
                    abi.check(rc)

        def check():
            import numpy as np

            import oracle

            for j in range(J):
                want = oracle.reduce([t.numpy() for t in base[j]], j % P, oracle.DT_F32, oracle.OP_SUM)
                for k in range(nsets):
                    if not np.array_equal(outs[k][j].cpu().numpy().view(np.uint32), want.view(np.uint32)):
                        raise SystemExit("bench: result differs from the oracle")

        desc = {"workload": name, "op": "a list of reductions, " + ("one launch per job" if single else "shared launches"),
                "jobs": J, "sources": P, "numel": N, "dtype": "float32", "buffer_sets": nsets}
        return desc, set_bytes, launch, check, "reduce_vec_kernel" if single else "reduce_many_kernel"

    if name.startswith("coalesced:"):
        # coalesced:<tensors>:<elements>[:loop|:halves] -- allreduce_coalesced (MAX, fp32, in place) of a list of
        # tensors of about that many elements each, called by all eight ranks of a local group: what
        # a DDP or ZeRO bucket of many small tensors costs, host and GPU together.  With ":loop", one
        # allreduce per tensor instead, as the reference serves the call
        # (wrapper/processgroup_wrapper.cc:182-191).
        import torch.distributed as dist

        import moodist_amd

        parts = name.split(":")
        T, n = int(parts[1]), int(parts[2])
        loop = len(parts) > 3 and parts[3] == "loop"
        halves = len(parts) > 3 and parts[3] == "halves"
        P = 8
        world = moodist_amd.LocalWorld(P, dev)
        sizes = [n + 8 * k for k in range(T)]  # multiples of the group size when n is
        g = torch.Generator().manual_seed(4)
        host = [[torch.rand(m, generator=g) for m in sizes] for _ in range(P)]
        tensors = [[t.to(dev) for t in row] for row in host]
        opts = dist.AllreduceCoalescedOptions()
        opts.reduceOp = dist.ReduceOp.MAX  # idempotent: the launches can repeat on the same tensors
        one = dist.AllreduceOptions()
        one.reduceOp = dist.ReduceOp.MAX
        # every rank's tensor read once and written once (what reduce_scatter + all_gather move is
        # (3P - 1) / 2P of that again)
        set_bytes = sum(2 * P * m * 4 for m in sizes)
        # ":halves": the two coalesced collectives an allreduce_coalesced is composed of, called
        # one after the other on chunk views
        chunks = [[t[r * (t.numel() // P):(r + 1) * (t.numel() // P)] for t in tensors[r]] for r in range(P)]
        rs_opts = dist.ReduceScatterOptions()
        rs_opts.reduceOp = dist.ReduceOp.MAX

        def launch(i):
            if halves:
                for r in range(P):
                    world.groups[r].reduce_scatter_tensor_coalesced(chunks[r], tensors[r], rs_opts)
                for r in range(P):
                    world.groups[r].allgather_into_tensor_coalesced(tensors[r], chunks[r])
            elif loop:
                for k in range(T):
                    for r in range(P):
                        world.groups[r].allreduce([tensors[r][k]], one)
            else:
                for r in range(P):
                    world.groups[r].allreduce_coalesced(tensors[r], opts)

        def check():
            for k in range(T):
                want = host[0][k]
                for r in range(1, P):
                    want = torch.maximum(want, host[r][k])
                for r in range(P):
                    if not torch.equal(tensors[r][k].cpu(), want):
                        raise SystemExit("bench: result differs from the expected allreduce")

        desc = {"workload": name, "op": "allreduce_coalesced MAX, eight local ranks" + (", one allreduce per tensor" if loop else ", as reduce_scatter_tensor_coalesced + allgather_into_tensor_coalesced" if halves else ""),
                "tensors": T, "numel": n, "dtype": "float32", "buffer_sets": 1,
                "note": "a step is all eight ranks' calls; ms_per_step is host and GPU together"}
        return desc, set_bytes, launch, check, "reduce_many_kernel + copy_flat_kernel" if halves else "reduce_many_kernel"

    if name.startswith("rows:"):
        # rows:<boxes>:<rows per box>:<run bytes>:<source pitch bytes> -- every box is `rows` runs of
        # `run` bytes, `pitch` bytes apart in its source, packed densely into the destination: the
        # shape of a last-dimension shard (run = row bytes / ranks) at any run length
        P, rows, run, pitch = (int(x) for x in name.split(":")[1:5])
        if run > pitch or run < 1:
            raise SystemExit("bench.py: rows: the run must fit the pitch")
        isz = 1
        while isz < 16 and run % (isz * 2) == 0 and pitch % (isz * 2) == 0:
            isz *= 2
        set_bytes = 2 * P * rows * run
        nsets = nsets_for(set_bytes)
        g = torch.Generator().manual_seed(2)
        # only the runs are read, so only they need distinct memory per set; the slabs are whole
        base = [torch.randint(0, 256, (rows, pitch), dtype=torch.uint8, generator=g) for _ in range(P)]
        on_device = [b.to(dev) for b in base]
        sets = [on_device] + [[t.clone() for t in on_device] for _ in range(nsets - 1)]
        outs = [torch.empty(P * rows * run, dtype=torch.uint8, device=dev) for _ in range(nsets)]
        plan = abi.CopyPlan([abi.make_box(0, s_ * rows * run, [rows, run // isz], [pitch // isz, 1], [run // isz, 1])
                             for s_ in range(P)], list(range(P)), [P] * P, isz, P + 1)
        tabs = [abi.ptr_table([t.data_ptr() for t in sets[i]] + [outs[i].data_ptr()]) for i in range(nsets)]

        def launch(i):
            rc = L.mdh_copy_plan_launch(plan._plan, tabs[i % nsets], P + 1, current())
            if rc:
                abi.check(rc)

        def check():
            want = torch.cat([b[:, :run].reshape(-1) for b in base])
            for o in outs:
                if not torch.equal(o.cpu(), want):
                    raise SystemExit("bench: result differs from the expected rows")

        desc = {"workload": name, "op": "strided rows into a dense destination (prepared plan)", "sources": P,
                "rows": rows, "run_bytes": run, "source_pitch_bytes": pitch, "vector_bytes": isz, "dtype": "uint8",
                "buffer_sets": nsets, "queue_prefilled": True, "launches_per_step": plan.launches}
        return desc, set_bytes, launch, check, "strided-box kernels"

    if name.startswith("transpose:"):
        # transpose:<rows>:<cols>:<itemsize> -- out[c, r] = in[r, c], both dense: through mdh_copy_boxes
        R, C, isz = (int(x) for x in name.split(":")[1:4])
        tdt = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[isz]
        set_bytes = 2 * R * C * isz
        nsets = nsets_for(set_bytes)
        g = torch.Generator().manual_seed(3)
        base = torch.randint(0, 127, (R, C), dtype=tdt, generator=g)
        ins = [base.to(dev) for _ in range(nsets)]
        outs = [torch.empty(C, R, dtype=tdt, device=dev) for _ in range(nsets)]
        boxes = [(abi.Box * 1)(abi.make_box(ins[k].data_ptr(), outs[k].data_ptr(), [C, R], [1, C], [R, 1]))
                 for k in range(nsets)]

        def launch(i):
            rc = L.mdh_copy_boxes(boxes[i % nsets], 1, isz, current())
            if rc:
                abi.check(rc)

        def check():
            want = base.t().contiguous()
            for o in outs:
                if not torch.equal(o.cpu(), want):
                    raise SystemExit("bench: result differs from the expected transpose")

        desc = {"workload": name, "op": "2-D element transpose (mdh_copy_boxes)", "rows": R, "cols": C, "itemsize": isz,
                "dtype": "uint8", "buffer_sets": nsets}
        return desc, set_bytes, launch, check, "transpose_kernel (copy_boxes_kernel with the knob box_transpose=1)"

    raise SystemExit("bench: unknown workload %r" % name)


def cpu_baseline(seconds_budget=12.0):
    """The reference's CPU reduce-scatter, restated in oracle.c, timed on this host: eight
    rank-threads (one service thread per rank process in the reference), each folding its chunk of
    all eight inputs with the memcpy + scalar-loop passes of the reference."""
    import numpy as np

    import oracle

    P, N = 8, 4194304
    threads = min(P, os.cpu_count() or 1)
    rng = np.random.RandomState(0)
    inputs = [rng.standard_normal(P * N).astype(np.float32) for _ in range(P)]
    outputs = [np.empty(N, dtype=np.float32) for _ in range(P)]
    alg_bytes = threads * (P + 1) * N * 4
    oracle.cpu_reduce_scatter_seconds(inputs, outputs, threads, N, oracle.DT_F32, reps=1)  # warm-up, page faults
    # rank-threads live through a batch of repetitions, as the reference's service threads live
    # through the job; batches until the time budget is spent
    medians, best, reps = [], None, 0
    t_end = time.time() + seconds_budget
    while (time.time() < t_end and reps < 2000) or not medians:
        m, b = oracle.cpu_reduce_scatter_seconds(inputs, outputs, threads, N, oracle.DT_F32, reps=20)
        medians.append(m)
        best = b if best is None or b < best else best
        reps += 20
    medians.sort()
    median = medians[len(medians) // 2]
    single = oracle.cpu_reduce_scatter_seconds(inputs, outputs, 1, N, oracle.DT_F32, reps=5)[0]
    want = oracle.reduce([x[:N] for x in inputs], 0, oracle.DT_F32, oracle.OP_SUM)
    assert np.array_equal(outputs[0], want)
    return {
        "value": round(alg_bytes / median / 1e9, 2),
        "unit": "GB/s",
        "cores": threads,  # threads used (one per emulated rank)
        "host_cores": os.cpu_count(),
        "kind": "port",
        "sample": "full workload (8 ranks x 8 chunks of 4,194,304 fp32), %d rank-threads at once, median over %d "
                  "repetitions in batches of 20 (best %.2f GB/s); one rank-thread alone: %.2f GB/s"
                  % (threads, reps, alg_bytes / best / 1e9, (P + 1) * N * 4 / single / 1e9),
    }


def measure(name, args, torch, abi, dev):
    """Builds the workload, warms up, times it and checks its results; returns the JSON line's
    fields for it.  Everything the workload allocated is released before returning."""
    desc, alg_bytes, launch, check, kernel = build_workload(name, torch, abi, dev, args.rotation_mib << 20)
    desc["rotation_mib"] = args.rotation_mib
    if args.tuning:
        desc["tuning"] = dict(item.split("=") for item in args.tuning)

    for i in range(args.warmup):
        launch(i)
    torch.cuda.synchronize()
    # Clock warm-up: a fresh box takes a few hundred milliseconds of work to reach its steady
    # clocks, far longer than `warmup` launches of 25 us; keep launching until CLOCK_WARMUP_S of
    # wall time have passed.  These launches are not timed.
    clock_launches = 0
    enqueue_us = []  # the host's launch call, per batch of 50: sizes the spin in front of a pre-filled window
    t_warm = time.perf_counter()
    while time.perf_counter() - t_warm < args.clock_warmup or not enqueue_us:
        t_batch = time.perf_counter()
        for i in range(50):
            launch(clock_launches + i)
        enqueue_us.append((time.perf_counter() - t_batch) * 1e6 / 50)
        clock_launches += 50
        torch.cuda.synchronize()
    # TIMED_WINDOWS windows of exactly `steps` launches each, every one bracketed by a
    # synchronize on both sides and by two HIP events on the launch stream; the reported step
    # time is the median window's (one window of 20 launches is 0.5 ms: a single one is noise).
    #
    # Two kinds of window.  A plain one starts on an idle stream: the GPU waits for the host's
    # first launch call (several microseconds), and that wait is part of the step time -- this is
    # the job's throughput, `value`.  A pre-filled one is enqueued behind a spinning kernel, so
    # that the launches are back to back when the first one starts: its step
    # time is the kernel's own duration, what `roofline` is about and what a kernel trace shows.
    # Launches shorter than the host's launch call (the compiled redistributions) would measure
    # the host in a plain window: they get pre-filled windows only, and config.queue_prefilled
    # says so.
    # The work in front is a spin kernel that touches no memory (torch.cuda._sleep): a kernel
    # that streams through HBM would leave the caches full of its dirty lines, and writing those
    # back would be charged to the launches that follow.  Long enough to outlast the host's
    # enqueuing of one window: 12 us per launch, or three times what the launch call took during
    # the clock warm-up when that is more (under a profiler it takes 10 us there and 25-65 us
    # into a queue that is held up).
    def spin_ms(cycles):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        torch.cuda._sleep(cycles)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1)

    spin_ms(100_000)
    cycles_per_ms = 4_000_000 / max(spin_ms(4_000_000), 1e-3)
    per_launch_ms = max(12e-3, 3e-3 * sorted(enqueue_us)[len(enqueue_us) // 2])
    spin_cycles = int(cycles_per_ms * (0.2 + args.steps * per_launch_ms))
    done = 0

    def median(v):
        v = sorted(v)
        return v[len(v) // 2]

    def timed_windows(prefilled):
        nonlocal done, spin_cycles
        window_ms, enqueue_ms, wall_ms = [], [], []
        lengthened = 0
        while len(window_ms) < TIMED_WINDOWS:
            torch.cuda.synchronize()
            if prefilled:
                torch.cuda._sleep(spin_cycles)
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            e0.record()  # on torch's current stream, the stream every launch above and below uses
            for i in range(args.steps):
                launch(done + i)
            enqueued = (time.perf_counter() - t0) * 1e3
            e1.record()
            torch.cuda.synchronize()
            wall = (time.perf_counter() - t0) * 1e3
            done += args.steps
            if prefilled and enqueued > 0.9 * spin_cycles / cycles_per_ms and lengthened < 6:
                # the host was still enqueuing when the spin ended (a profiler slows the launch
                # call several times over): this window measured the host; again behind a longer spin
                spin_cycles = max(int(spin_cycles * 1.6), int(enqueued * 1.3 * cycles_per_ms))
                lengthened += 1
                continue
            enqueue_ms.append(enqueued)
            wall_ms.append(wall)
            window_ms.append(e0.elapsed_time(e1))
        return window_ms, median(enqueue_ms), median(wall_ms)

    prefilled_ms, enqueue_ms, wall_ms = timed_windows(True)
    desc["prefill_spin_ms"] = round(spin_cycles / cycles_per_ms, 3)
    kernel_ms = median(prefilled_ms) / args.steps
    desc["timed_windows"] = TIMED_WINDOWS
    if desc.get("queue_prefilled"):
        window_ms = prefilled_ms
    else:
        window_ms, enqueue_ms, wall_ms = timed_windows(False)
        desc["prefilled_window_ms_min_median_max"] = [round(min(prefilled_ms), 5), round(median(prefilled_ms), 5),
                                                      round(max(prefilled_ms), 5)]
    ms = median(window_ms)
    ms_per_step = ms / args.steps
    desc["window_ms_min_median_max"] = [round(min(window_ms), 5), round(ms, 5), round(max(window_ms), 5)]
    desc["clock_warmup_s"] = args.clock_warmup
    desc["clock_warmup_launches"] = clock_launches
    checked = False
    if not args.no_check:
        # every set's output is checked: make sure each has been written (a short run may not
        # have gone round the whole rotation)
        for i in range(desc["buffer_sets"]):
            launch(i)
        torch.cuda.synchronize()
        check()
        checked = True
    gbs = alg_bytes / (ms_per_step * 1e-3) / 1e9
    kernel_gbs = alg_bytes / (kernel_ms * 1e-3) / 1e9
    out = {
        "metric": "achieved HBM GB/s (% of peak) for 1-GPU local reduce-scatter, fp32 P=8"
        if name == "reduce_fp32_p8" else "achieved HBM GB/s (% of peak), " + name,
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": DTYPE_NAMES[desc["dtype"]],
        "data": "synthetic",
        "config": desc,
        "percent_of_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "host_wall_ms_per_step": round(wall_ms / args.steps, 6),
        "host_enqueue_ms_per_step": round(enqueue_ms / args.steps, 6),
        "result_checked": checked,
        "roofline": {
            "bound": "hbm",
            "kernel": kernel,
            # algorithmic bytes / the kernel's duration (back-to-back launches, pre-filled queue)
            "achieved": round(kernel_gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(kernel_gbs / HBM_PEAK_GBS, 4),
            "kernel_us": round(kernel_ms * 1e3, 3),
            "algorithmic_bytes_per_launch": alg_bytes,
            # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by the
            # same counter's reading on a copy of known size; null for a workload not measured
            "traffic": MEASURED_TRAFFIC_BYTES.get(name),
        },
    }
    # the closures hold every buffer of the workload: let go of them, then of the allocator's cache
    del launch, check
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default=None,
                    help="measure this workload alone (default: the headline, then every other configuration)")
    ap.add_argument("--headline-only", action="store_true", help="measure reduce_fp32_p8 alone")
    ap.add_argument("--rotation-mib", type=int, default=4096,
                    help="touched bytes of all buffer sets together (the launches rotate over them)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--clock-warmup", type=float, default=CLOCK_WARMUP_S, metavar="SECONDS",
                    help="untimed launches before the first timed window (0 under a counter-collecting profiler)")
    ap.add_argument("--tuning", action="append", default=[], metavar="KNOB=VALUE",
                    help="force a launch-shape knob of the kernel library (mdh_set_tuning), e.g. reduce_unroll=8")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py measures one GPU: the path is one rank's share with its peers staged in the "
                         "same GPU's HBM; run it with --gpus 1")

    import torch

    from moodist_amd import _abi as abi

    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    for item in args.tuning:  # before the workload is built: a prepared plan fixes its shape at create time
        knob, _, value = item.partition("=")
        abi.set_tuning(knob, int(value))
    first = args.workload or ALL_WORKLOADS[0]
    t_start = time.perf_counter()
    out = measure(first, args, torch, abi, dev)
    if not args.no_cpu_baseline and first == "reduce_fp32_p8":
        out["cpu_baseline"] = cpu_baseline()
    if args.workload is None and not args.headline_only:
        # every other configuration, same steps, warm-up, rotation and result check; the line's
        # top-level figures stay the headline's
        configs = {}
        for name in ALL_WORKLOADS:
            if name == first:
                r = out
            else:
                sys.stderr.write("bench: %s (%.0f s so far)\n" % (name, time.perf_counter() - t_start))
                sys.stderr.flush()
                r = measure(name, args, torch, abi, dev)
            rf = r["roofline"]
            configs[name] = {
                "kernel": rf["kernel"], "kernel_us": rf["kernel_us"], "frac": rf["frac"], "achieved": rf["achieved"],
                "algorithmic_bytes": rf["algorithmic_bytes_per_launch"], "traffic": rf["traffic"],
                "ms_per_step": r["ms_per_step"], "queue_prefilled": bool(r["config"].get("queue_prefilled")),
                "buffer_sets": r["config"]["buffer_sets"], "result_checked": r["result_checked"],
            }
        out["configs"] = configs
        # what the library serves beyond those configurations: boxes that transpose, and the
        # allreduce of eight local ranks (one collective, a step is all eight ranks' calls)
        others = {}
        for name in OTHER_WORKLOADS:
            sys.stderr.write("bench: %s (%.0f s so far)\n" % (name, time.perf_counter() - t_start))
            sys.stderr.flush()
            a = argparse.Namespace(**vars(args))
            if name.startswith("coalesced:"):
                a.steps, a.warmup = min(args.steps, 30), min(args.warmup, 5)
            try:
                r = measure(name, a, torch, abi, dev)
            except (Exception, SystemExit) as e:  # the line above all reports the configurations: it still goes out
                others[name] = {"error": str(e)}
                continue
            rf = r["roofline"]
            others[name] = {
                "kernel": rf["kernel"], "kernel_us": rf["kernel_us"], "frac": rf["frac"], "achieved": rf["achieved"],
                "algorithmic_bytes": rf["algorithmic_bytes_per_launch"], "ms_per_step": r["ms_per_step"],
                "steps": a.steps, "buffer_sets": r["config"]["buffer_sets"], "result_checked": r["result_checked"],
            }
        out["others"] = others
        out["bench_wall_s"] = round(time.perf_counter() - t_start, 1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
